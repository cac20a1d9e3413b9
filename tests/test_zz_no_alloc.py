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


def test_noalloc_forward_equals_workspace_forward_on_two_calls_in_a_row(knobs):
    from rfa_amd import _lib, rfa_hip
    lib = _lib.load()
    knobs(recompute=0)      # the existing entry point in the form this one always takes: state from segment totals
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
        free_before = torch.cuda.mem_get_info()[0]          # the driver's own count: sees a hipMalloc inside the library
        print(f"noalloc forward T={T} N={N} K={K} d={d}", flush=True)
        _lib.check(lib.rfa_causal_forward_noalloc(q.data_ptr(), k.data_ptr(), v.data_ptr(), got.data_ptr(), T, N, K, d, stream))
        torch.cuda.synchronize()
        assert (torch.cuda.memory_stats()["num_alloc_retries"], torch.cuda.memory_allocated()) == before
        assert torch.cuda.mem_get_info()[0] == free_before
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


def test_noalloc_forward_under_graph_capture_replays_the_eager_bits(knobs):
    """The callers the entry point is for: a HIP graph captured after one warm-up call (the first call
    on a device looks the static array's address up and sets kernel attributes, which must not
    happen under capture).  Every replay, with eager work and synchronisation in between and new
    input values in the same tensors, gives the bits of rfa_causal_forward on those values."""
    from rfa_amd import _lib, rfa_hip
    lib = _lib.load()
    knobs(recompute=0)
    T, N, K, d = 1024, 64, 128, 64
    q, k, v = _inputs(T, N, K, d, 3)
    got = torch.empty_like(v)
    _lib.check(lib.rfa_causal_forward_noalloc(q.data_ptr(), k.data_ptr(), v.data_ptr(), got.data_ptr(), T, N, K, d,
                                              torch.cuda.current_stream().cuda_stream))      # warm-up, outside capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    print("noalloc forward: capture", flush=True)
    with torch.cuda.graph(graph):
        _lib.check(lib.rfa_causal_forward_noalloc(q.data_ptr(), k.data_ptr(), v.data_ptr(), got.data_ptr(), T, N, K, d,
                                                  torch.cuda.current_stream().cuda_stream))
    for rep in range(3):
        q2, k2, v2 = _inputs(T, N, K, d, 10 + rep)
        q.copy_(q2), k.copy_(k2), v.copy_(v2)
        want = rfa_hip.forward(q, k, v)                    # eager work of the program between replays
        got.fill_(float("nan"))
        torch.cuda.synchronize()
        print(f"noalloc forward: replay {rep}", flush=True)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want), rep
