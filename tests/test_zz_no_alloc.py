"""rfa_causal_forward_noalloc: the forward for callers that cannot allocate.  Its segment totals
live in the library's static device array instead of a caller workspace; output must be
bit-identical to rfa_causal_forward's, also on a second, smaller call that finds the array full
of the first call's totals."""
import pytest
import torch

from oracle import rfa_oracle as O

pytestmark = pytest.mark.gpu


def _inputs(T, N, K, d, seed):
    """phi(q), phi(k) of unit vectors and v ~ N(0, 1), as the benchmark draws them"""
    from rfa_amd import rfa_hip
    q, k, v, _ = O.make_qkv(T, N, 1, d, seed=seed)
    W = O.make_w(d, K // 2, 1).half().cuda()
    pq = rfa_hip.feature_map_forward(q.cuda(), W, O.SCALE).view(T, N, K)
    pk = rfa_hip.feature_map_forward(k.cuda(), W, O.SCALE).view(T, N, K)
    return pq, pk, v.cuda().view(T, N, d)


def test_noalloc_forward_equals_workspace_forward_on_two_calls_in_a_row():
    from rfa_amd import _lib, rfa_hip
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.rfa_static_scratch_bytes() == 16 << 20
    first = True
    for (T, N, K, d, seed) in ((1024, 64, 128, 64, 1), (448, 5, 128, 64, 2)):   # the second call is smaller
        q, k, v = _inputs(T, N, K, d, seed)
        need = lib.rfa_causal_forward_workspace_bytes(T, N, K, d)
        assert 0 < need <= lib.rfa_static_scratch_bytes() and lib.rfa_causal_num_segments(T, N, K, d) > 1
        want = rfa_hip.forward(q, k, v)                    # the existing entry point, caller-owned workspace
        got = torch.full_like(v, float("nan"))
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["num_alloc_retries"], torch.cuda.memory_allocated()
        print(f"noalloc forward T={T} N={N} K={K} d={d}", flush=True)
        _lib.check(lib.rfa_causal_forward_noalloc(q.data_ptr(), k.data_ptr(), v.data_ptr(), got.data_ptr(), T, N, K, d, stream))
        torch.cuda.synchronize()
        assert (torch.cuda.memory_stats()["num_alloc_retries"], torch.cuda.memory_allocated()) == before
        assert torch.equal(got, want)
        if first:                                          # and against the oracle, once
            ref = O.causal_forward_chunked(q[:, :2].float().cpu(), k[:, :2].float().cpu(), v[:, :2].float().cpu())
            assert (got[:, :2].float().cpu() - ref).abs().max().item() <= 2e-3
            first = False
    # a shape whose totals do not fit the static array is refused, with the limit in the message
    T, N, K, d = 16384, 32, 256, 128
    assert lib.rfa_causal_forward_workspace_bytes(T, N, K, d) > lib.rfa_static_scratch_bytes()
    rc = lib.rfa_causal_forward_noalloc(q.data_ptr(), q.data_ptr(), q.data_ptr(), q.data_ptr(), T, N, K, d, stream)
    assert rc == -5 and b"static scratch" in lib.rfa_last_error()
    # empty input: nothing to do
    assert lib.rfa_causal_forward_noalloc(None, None, None, None, 0, 4, 128, 64, stream) == 0
