"""GPU parity of the causal kernels (through the C ABI) against the CPU oracle.

Tolerances are the ones the path is specified with: fp16 outputs within
max-abs 2e-3 of the fp32 oracle, gradients within 1e-2 relative Frobenius
error; the oracle sees the same fp16-rounded inputs.
"""
import os

import pytest
import torch

from oracle import rfa_oracle as O

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("binding")]

OUT_ATOL = 2e-3
GRAD_RTOL = 1e-2


def _features(T, B, H, d, D, seed):
    """phi(q), phi(k) [T, N, 2D], v, g [T, N, d] as fp16 CPU tensors."""
    q, k, v, g = O.make_qkv(T, B, H, d, seed)
    W = O.make_w(d, D, H)
    pq = O.random_project(q.float(), W).to(torch.float16).reshape(T, B * H, 2 * D)
    pk = O.random_project(k.float(), W).to(torch.float16).reshape(T, B * H, 2 * D)
    return pq, pk, v.reshape(T, B * H, d), g.reshape(T, B * H, d)


def _rel(a, b):
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def _oracle_fwd(pq, pk, v):
    T, N, K = pq.shape
    if T * N * K * v.shape[-1] <= (1 << 26):
        return O.causal_forward_cumsum(pq.float(), pk.float(), v.float())
    return O.causal_forward_chunked(pq.float(), pk.float(), v.float())


def _oracle_bwd(pq, pk, v, g):
    T, N, K = pq.shape
    if T * N * K * v.shape[-1] <= (1 << 25):
        return O.causal_backward_cumsum(pq.float(), pk.float(), v.float(), g.float())
    return O.causal_backward_chunked(pq.float(), pk.float(), v.float(), g.float())


SHAPES = [
    # T, B, H, d, D
    (128, 2, 4, 64, 64),     # the CPU-runnable configuration
    (1, 1, 1, 64, 64),
    (63, 1, 2, 64, 64),
    (65, 2, 1, 64, 64),
    (200, 1, 3, 64, 64),     # ragged tail
    (640, 1, 2, 64, 64),     # several segments
    (192, 1, 2, 64, 32),     # K = 64
    (160, 1, 2, 128, 64),    # d = 128
    (130, 1, 1, 64, 128),    # K = 256
    (70, 65, 8, 64, 64),     # many sequences (N = 520), two chunks each
    (3000, 1, 2, 64, 64),    # long ragged sequence: 16 segments, last one short
    (640, 1, 11, 64, 64),    # 11 sequences x 5 segments: one full group of 8 sequences and a rest of 3
    (1100, 1, 2, 128, 128),  # K = 256, d = 128: split dQ sweep, dK / dV in separate workgroups
]


@pytest.mark.parametrize("T,B,H,d,D", SHAPES)
def test_forward_matches_oracle(T, B, H, d, D):
    from rfa_amd import rfa_hip
    pq, pk, v, _ = _features(T, B, H, d, D, seed=1000 + T)
    print(f"causal fwd T={T} N={B*H} K={2*D} d={d}", flush=True)
    out = rfa_hip.forward(pq.cuda(), pk.cuda(), v.cuda()).float().cpu()
    ref = _oracle_fwd(pq, pk, v)
    assert torch.isfinite(out).all()
    assert (out - ref).abs().max().item() <= OUT_ATOL


@pytest.mark.parametrize("T,B,H,d,D", SHAPES)
def test_backward_matches_oracle(T, B, H, d, D):
    from rfa_amd import rfa_hip
    pq, pk, v, g = _features(T, B, H, d, D, seed=2000 + T)
    print(f"causal bwd T={T} N={B*H} K={2*D} d={d}", flush=True)
    dq, dk, dv = [t.float().cpu() for t in rfa_hip.backward(pq.cuda(), pk.cuda(), v.cuda(), g.cuda())]
    rq, rk, rv = _oracle_bwd(pq, pk, v, g)
    for name, got, want in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
        assert torch.isfinite(got).all(), name
        assert _rel(got, want) <= GRAD_RTOL, (name, _rel(got, want))


def test_selftest_layout():
    from rfa_amd import rfa_hip
    rfa_hip.selftest_layout()


@pytest.mark.parametrize("T,B,H,d,D", SHAPES + [(100, 2, 1, 64, 64), (1024, 2, 8, 64, 64), (300, 1, 2, 128, 64)])
def test_saved_pair_matches_oracle(T, B, H, d, D):
    """forward_save / backward_saved: the forward hands its segment totals and raw denominators
    to the backward, which also reads the forward output (g . num = (g . out) * den).  The
    forward output is bit-identical to the plain forward; the gradients meet the same
    tolerance against the oracle as the plain backward (they are not bit-identical to it:
    the plain backward recomputes num in fp32, the saved one uses the fp16 output)."""
    from rfa_amd import rfa_hip
    cpu = _features(T, B, H, d, D, seed=3000 + T)
    pq, pk, v, g = (t.cuda() for t in cpu)
    print(f"causal saved pair T={T} N={B*H} K={2*D} d={d}", flush=True)
    out, saved = rfa_hip.forward_save(pq, pk, v)
    assert torch.equal(out, rfa_hip.forward(pq, pk, v))
    got = [t.float().cpu() for t in rfa_hip.backward_saved(pq, pk, v, g, out, saved)]
    want = _oracle_bwd(*cpu)
    for name, a, b in zip(("dq", "dk", "dv"), got, want):
        assert torch.isfinite(a).all(), name
        assert _rel(a, b) <= GRAD_RTOL, (name, _rel(a, b))
    # dv does not depend on gz: it must agree with the plain backward to fp16 rounding of G/den
    plain = rfa_hip.backward(pq, pk, v, g)
    assert _rel(got[2], plain[2].float().cpu()) <= 2e-3


def test_saved_pair_clamped_and_unclamped_rows():
    """Rows with den_raw <= 1 take gz = 0 (strict >, cuda/utils.cu:31-40); rows above take
    -(g . out) / den.  Scaling phi_k moves every row across the clamp."""
    from rfa_amd import rfa_hip
    T, B, H, d, D = 256, 1, 2, 64, 64
    pq, pk, v, g = _features(T, B, H, d, D, seed=77)
    for scale in (0.25, 4.0):
        pk2 = (pk.float() * scale).to(torch.float16)
        cq, ck, cv, cg = pq.cuda(), pk2.cuda(), v.cuda(), g.cuda()
        out, saved = rfa_hip.forward_save(cq, ck, cv)
        got = [t.float().cpu() for t in rfa_hip.backward_saved(cq, ck, cv, cg, out, saved)]
        want = _oracle_bwd(pq, pk2, v, g)
        for name, a, b in zip(("dq", "dk", "dv"), got, want):
            assert _rel(a, b) <= GRAD_RTOL, (scale, name, _rel(a, b))


@pytest.mark.parametrize("nseg,scanned", [(1, None), (2, None), (3, None), (8, None), (16, None),
                                          (2, "1"), (3, "1"), (11, "1"), (8, "0"), (1, "1")])
def test_every_segment_count_gives_the_same_answer(nseg, scanned, knobs):
    """The "nseg" knob overrides the number of time segments per sequence; the plain pair, the
    saved pair and the prefill state must meet the oracle for any of them (ragged last segment,
    single-chunk segments, one segment for the whole sequence).  The "prefix" knob forces the
    consumers to add up the segment totals themselves ("0") or to read totals that a scan
    kernel turned into running sums first ("1"); unset, five segments or more take the scan."""
    from rfa_amd import rfa_hip
    # recompute=0: every forward of this test takes its state from segment totals (the form without
    # totals has its own test below)
    knobs(nseg=nseg, prefix=-1 if scanned is None else int(scanned), recompute=0)
    T, B, H, d, D = 700, 1, 3, 64, 64
    cpu = _features(T, B, H, d, D, seed=5000)
    pq, pk, v, g = (t.cuda() for t in cpu)
    print(f"causal nseg={nseg} scanned={scanned} T={T}", flush=True)
    ref = _oracle_fwd(*cpu[:3])
    want = _oracle_bwd(*cpu)
    out, saved = rfa_hip.forward_save(pq, pk, v)
    assert (out.float().cpu() - ref).abs().max().item() <= OUT_ATOL
    assert torch.equal(out, rfa_hip.forward(pq, pk, v))
    for pair in (rfa_hip.backward_saved(pq, pk, v, g, out, saved), rfa_hip.backward(pq, pk, v, g)):
        for name, a, b in zip(("dq", "dk", "dv"), pair, want):
            assert _rel(a.float().cpu(), b) <= GRAD_RTOL, (nseg, name)
    o2, s, z = rfa_hip.prefill(pq, pk, v)
    assert torch.equal(o2, out)
    _, s_ref, z_ref = O.causal_forward_loop(cpu[0].float(), cpu[1].float(), cpu[2].float())
    assert _rel(s.cpu(), s_ref) < 1e-5 and _rel(z.cpu(), z_ref) < 1e-5


@pytest.mark.parametrize("T,B,H,d,D,nseg,cost,cut", [
    (700, 1, 3, 64, 64, 2, -1, True), (700, 1, 3, 64, 64, 3, -1, True), (700, 1, 3, 64, 64, 4, 50, True),
    (1024, 2, 3, 64, 64, 4, -1, True), (641, 1, 2, 64, 64, 11, 0, True), (3000, 1, 2, 64, 32, 12, 3, True),
    (3000, 1, 2, 64, 32, 16, 5, False),      # no cut into 16 non-empty segments at this cost: the form with totals runs
    (520, 1, 2, 128, 64, 3, -1, True), (130, 1, 5, 64, 64, 2, 90, True), (65, 1, 1, 64, 64, 2, -1, True)])
def test_forward_without_segment_totals(T, B, H, d, D, nseg, cost, cut, knobs):
    """The forward whose workgroups rebuild the state at their segment's first step from the k, v rows
    before it (no totals pass, unequal segments; taken by itself for up to 4 segments, "recompute"
    = 1 forces it for any count, "prefix_cost" moves the cut).  Output, prefill state and the
    denominators handed to the sliced backward meet the oracle; the state is accumulated chunk
    by chunk in time order whatever the cut, so the output has the bits of the one-segment scan."""
    from rfa_amd import rfa_hip
    cpu = _features(T, B, H, d, D, seed=5400 + T)
    pq, pk, v, g = (t.cuda() for t in cpu)
    ref = _oracle_fwd(*cpu[:3])
    knobs(nseg=1, recompute=0)
    one = rfa_hip.forward(pq, pk, v)
    knobs(nseg=nseg, recompute=1, prefix_cost=cost, sliced=1)
    print(f"forward without totals T={T} N={B * H} K={2 * D} d={d} nseg={nseg} cost={cost}", flush=True)
    out = rfa_hip.forward(pq, pk, v)
    assert (out.float().cpu() - ref).abs().max().item() <= OUT_ATOL
    assert torch.equal(out, one) == cut
    o2, s, z = rfa_hip.prefill(pq, pk, v)
    assert torch.equal(o2, out)
    _, s_ref, z_ref = O.causal_forward_loop(cpu[0].float(), cpu[1].float(), cpu[2].float())
    assert _rel(s.cpu(), s_ref) < 1e-5 and _rel(z.cpu(), z_ref) < 1e-5
    o3, saved = rfa_hip.forward_save(pq, pk, v)        # final-state layout: the same launch, plus den_raw and S_T, z_T
    assert torch.equal(o3, out)
    for name, a, b in zip(("dq", "dk", "dv"), rfa_hip.backward_saved(pq, pk, v, g, o3, saved), _oracle_bwd(*cpu)):
        assert _rel(a.float().cpu(), b) <= GRAD_RTOL, name


@pytest.mark.parametrize("nseg,same", [(8, False), (4, False), (6, False), (8, True), (5, False)])
def test_wide_state_backward_on_half_as_many_segments(nseg, same, knobs):
    """K = 256, d = 128: with scanned totals the saved-pair backward runs on segments twice as long
    as the forward's (even segment counts; the "nseg_same" knob keeps them equal); out and gradients
    must meet the oracle either way, and the plain pair as well."""
    from rfa_amd import rfa_hip
    knobs(nseg=nseg, prefix=-1, nseg_same=1 if same else -1)
    T, B, H, d, D = 1100, 1, 2, 128, 128
    cpu = _features(T, B, H, d, D, seed=5100)
    pq, pk, v, g = (t.cuda() for t in cpu)
    print(f"causal wide nseg={nseg} same={same} T={T}", flush=True)
    ref = _oracle_fwd(*cpu[:3])
    want = _oracle_bwd(*cpu)
    out, saved = rfa_hip.forward_save(pq, pk, v)
    assert (out.float().cpu() - ref).abs().max().item() <= OUT_ATOL
    for pair in (rfa_hip.backward_saved(pq, pk, v, g, out, saved), rfa_hip.backward(pq, pk, v, g)):
        for name, a, b in zip(("dq", "dk", "dv"), pair, want):
            assert _rel(a.float().cpu(), b) <= GRAD_RTOL, (nseg, name)


def _random_cases(count, seed):
    g = torch.Generator().manual_seed(seed)
    dims = [(64, 32), (64, 64), (64, 128), (128, 32), (128, 64), (128, 128)]       # (d, D): K = 2D in {64, 128, 256}
    cases = []
    for i in range(count):
        T = int(torch.randint(1, 700, (1,), generator=g))
        B = int(torch.randint(1, 4, (1,), generator=g))
        H = int(torch.randint(1, 4, (1,), generator=g))
        d, D = dims[int(torch.randint(0, len(dims), (1,), generator=g))]
        cases.append((T, B, H, d, D, 7000 + i))
    return cases


@pytest.mark.parametrize("T,B,H,d,D,seed", _random_cases(16, 424242))
def test_seeded_random_shapes(T, B, H, d, D, seed, knobs):
    """Sixteen shapes drawn once from a fixed seed (lengths 1..699, 1..3 batch entries and heads, every
    supported width pair): output, saved-pair gradients in both layouts of the saved buffer (time
    segments; final state with the one-launch backward where it exists) and plain-pair gradients
    against the oracle."""
    from rfa_amd import rfa_hip
    cpu = _features(T, B, H, d, D, seed)
    pq, pk, v, g = (t.cuda() for t in cpu)
    print(f"causal random T={T} B={B} H={H} d={d} D={D}", flush=True)
    ref = _oracle_fwd(*cpu[:3])
    want = _oracle_bwd(*cpu)
    pairs = [rfa_hip.backward(pq, pk, v, g)]
    for sliced in (0, 1):
        knobs(sliced=sliced)
        out, saved = rfa_hip.forward_save(pq, pk, v)
        assert (out.float().cpu() - ref).abs().max().item() <= OUT_ATOL
        pairs.append(rfa_hip.backward_saved(pq, pk, v, g, out, saved))
    for pair in pairs:
        for name, a, b in zip(("dq", "dk", "dv"), pair, want):
            assert torch.isfinite(a).all(), name
            assert _rel(a.float().cpu(), b) <= GRAD_RTOL, (name, _rel(a.float().cpu(), b))


def test_two_threads_on_two_streams_agree_with_one():
    """The library keeps no state between calls and launches on the caller's stream (the reference
    launches on the legacy default stream, forward.cu:155): two host threads, each with its own
    non-default stream, tensors and workspace, run the training pair at the same time and must get
    the bits of the same calls made one after the other on the default stream."""
    import threading
    from rfa_amd import rfa_hip
    cases = [_features(700, 1, 5, 64, 64, seed=8100), _features(450, 2, 3, 64, 32, seed=8101)]
    gpu = [tuple(t.cuda() for t in c) for c in cases]
    want = []
    for pq, pk, v, g in gpu:
        out, saved = rfa_hip.forward_save(pq, pk, v)
        want.append((out, *rfa_hip.backward_saved(pq, pk, v, g, out, saved)))
    torch.cuda.synchronize()
    got = [None, None]
    errors = []

    def worker(i):
        try:
            stream = torch.cuda.Stream()
            pq, pk, v, g = gpu[i]
            with torch.cuda.stream(stream):
                for _ in range(20):
                    out, saved = rfa_hip.forward_save(pq, pk, v)
                    grads = rfa_hip.backward_saved(pq, pk, v, g, out, saved)
                got[i] = (out, *grads)
            stream.synchronize()
        except Exception as exc:      # surfaced in the main thread below
            errors.append(exc)

    print("causal two threads, two streams", flush=True)
    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for i in range(2):
        for a, b in zip(got[i], want[i]):
            assert torch.equal(a, b)


def test_saved_buffer_carries_the_plan_of_its_forward(knobs):
    """The forward writes its plan into the saved buffer and the library remembers it: a backward
    call runs with that plan whatever the knobs say by then; a buffer the library has no record
    of (here: a copy) whose header differs from the current plan yields NaN gradients, never
    numbers computed from totals laid out for another plan, and so does a call of another shape."""
    import ctypes
    from rfa_amd import _lib, rfa_hip
    T, B, H, d, D = 700, 1, 3, 64, 64
    cpu = _features(T, B, H, d, D, seed=5200)
    pq, pk, v, g = (t.cuda() for t in cpu)
    want = _oracle_bwd(*cpu)
    knobs(nseg=4, prefix=0)
    out, saved = rfa_hip.forward_save(pq, pk, v)
    words = (ctypes.c_int32 * 16)()
    _lib.check(_lib.load().rfa_causal_saved_describe(saved.data_ptr(), words, None))
    assert words[0] == 0x52464153 and (words[3], words[4], words[5], words[7]) == (2 * D, d, 4, 0)
    assert (words[8], words[10]) == (T, B * H) and saved.numel() == _lib.load().rfa_causal_saved_state_bytes(T, B * H, 2 * D, d)
    knobs(nseg=8, prefix=1)                     # the knobs move between forward and backward
    for name, a, b in zip(("dq", "dk", "dv"), rfa_hip.backward_saved(pq, pk, v, g, out, saved), want):
        assert _rel(a.float().cpu(), b) <= GRAD_RTOL, name
    stray = torch.empty(saved.numel() + 4096, dtype=torch.uint8, device="cuda")[:saved.numel()].copy_(saved)
    assert stray.data_ptr() != saved.data_ptr()
    big = torch.empty(1 << 24, dtype=torch.uint8, device="cuda")       # room for the 8-segment layout
    big[:saved.numel()].copy_(saved)
    grads = rfa_hip.backward_saved(pq, pk, v, g, out, big)
    assert all(torch.isnan(t.float()).all() for t in grads)
    knobs(nseg=4, prefix=0)                     # back on the forward's plan: the copy is as good as the original
    for name, a, b in zip(("dq", "dk", "dv"), rfa_hip.backward_saved(pq, pk, v, g, out, stray), want):
        assert _rel(a.float().cpu(), b) <= GRAD_RTOL, name
    # another shape than the forward's: the record of this address does not apply, the call runs with the current
    # plan and the kernels find a header written for T = 700
    grads = rfa_hip.backward_saved(pq[:640].contiguous(), pk[:640].contiguous(), v[:640].contiguous(), g[:640].contiguous(),
                                   out[:640].contiguous(), saved)
    assert all(torch.isnan(t.float()).all() for t in grads)


def _forward_save_into(saved, pq, pk, v):
    """rfa_causal_forward_save into a buffer the test owns (the wrappers allocate their own)."""
    from rfa_amd import _lib
    lib = _lib.load()
    T, N, K = pq.shape
    d = v.shape[2]
    out = torch.empty_like(v)
    nbytes = lib.rfa_causal_forward_workspace_bytes(T, N, K, d)
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device="cuda")
    assert lib.rfa_causal_saved_state_bytes(T, N, K, d) <= saved.numel()
    _lib.check(lib.rfa_causal_forward_save(pq.data_ptr(), pk.data_ptr(), v.data_ptr(), out.data_ptr(), saved.data_ptr(),
                                           saved.numel(), T, N, K, d, ws.data_ptr(), nbytes,
                                           torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return out


@pytest.mark.parametrize("stale", ["other_plan", "other_shape"])
def test_saved_buffer_at_an_address_the_library_has_a_stale_record_of(stale, knobs):
    """The caller's allocator hands the address of a freed saved buffer to another one.  The library's
    record of that address then describes a buffer that is gone.  A copy of a saved buffer of
    another shape placed there gives correct gradients (the record is dropped, the current plan is
    the copy's plan); one of the same shape and another plan gives NaN (the kernels compare the
    header in the buffer with the plan they run) -- never numbers read through the wrong layout."""
    from rfa_amd import rfa_hip
    T, B, H, d, D = 700, 1, 3, 64, 64
    cpu = _features(T, B, H, d, D, seed=5300)
    pq, pk, v, g = (t.cuda() for t in cpu)
    want = _oracle_bwd(*cpu)
    nbytes = 1 << 23                               # one size for every buffer, so the allocator reuses the block
    knobs(nseg=2, prefix=0, sliced=0)
    if stale == "other_plan":
        first = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        _forward_save_into(first, pq, pk, v)       # record: address -> (T, N, 2 segments)
    else:
        Ts = 300
        cs = [t.cuda() for t in _features(Ts, B, H, d, D, seed=5301)]
        first = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        _forward_save_into(first, cs[0], cs[1], cs[2])   # record: address -> (T = 300, ...)
    address = first.data_ptr()
    knobs(nseg=4, prefix=0, sliced=0)
    other = torch.empty(nbytes + 512, dtype=torch.uint8, device="cuda")[:nbytes]    # another block
    out = _forward_save_into(other, pq, pk, v)     # the buffer whose copy will land on the stale address
    assert other.data_ptr() != address
    del first
    reused = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    if reused.data_ptr() != address:
        pytest.skip("the allocator did not hand the freed block out again")
    reused.copy_(other)
    grads = rfa_hip.backward_saved(pq, pk, v, g, out, reused)
    if stale == "other_plan":
        assert all(torch.isnan(t.float()).all() for t in grads)
        # the address is written by a forward again: the record follows
        out2 = _forward_save_into(reused, pq, pk, v)
        grads = rfa_hip.backward_saved(pq, pk, v, g, out2, reused)
    for name, a, b in zip(("dq", "dk", "dv"), grads, want):
        assert _rel(a.float().cpu(), b) <= GRAD_RTOL, name


SLICED_SHAPES = [
    # T, B, H, d, D: the feature and value widths the sliced backward exists for, ragged tails, one step, sequence
    # counts that are no multiple of the 8 XCDs, a long sequence (many backward steps of the state)
    (128, 2, 4, 64, 64),
    (1, 1, 1, 64, 64),
    (63, 1, 2, 64, 64),
    (65, 3, 1, 64, 64),
    (200, 1, 3, 64, 64),
    (640, 1, 11, 64, 64),
    (192, 1, 2, 64, 32),     # K = 64: one feature slice
    (70, 65, 8, 64, 64),     # N = 520
    (4100, 1, 2, 64, 64),    # 65 chunks
    (200, 2, 3, 128, 64),    # d = 128: two value slices
    (130, 1, 5, 128, 32),
    (1, 2, 1, 128, 64),
    (1100, 1, 2, 128, 64),
]


@pytest.mark.parametrize("T,B,H,d,D", SLICED_SHAPES)
def test_sliced_backward_matches_oracle(T, B, H, d, D, knobs):
    """The "sliced" knob makes the saving forward leave its final state and the backward walk whole
    sequences backwards in state slices (one launch, every chunk read once).  Same tolerances as the
    segment sweeps; dv does not depend on the stepped-back state and agrees with the segment
    backward to fp16 rounding of G / den."""
    from rfa_amd import _lib, rfa_hip
    cpu = _features(T, B, H, d, D, seed=8000 + T)
    pq, pk, v, g = (t.cuda() for t in cpu)
    print(f"causal sliced backward T={T} N={B*H} K={2*D} d={d}", flush=True)
    knobs(sliced=0)
    out0, saved0 = rfa_hip.forward_save(pq, pk, v)
    seg = rfa_hip.backward_saved(pq, pk, v, g, out0, saved0)
    knobs(sliced=1)
    out, saved = rfa_hip.forward_save(pq, pk, v)
    assert torch.equal(out, out0)
    import ctypes
    words = (ctypes.c_int32 * 16)()
    _lib.check(_lib.load().rfa_causal_saved_describe(saved.data_ptr(), words, None))
    assert words[2] == 1                                    # the final-state layout
    assert _lib.load().rfa_causal_backward_saved_workspace_bytes(saved.data_ptr(), T, B * H, 2 * D, d) == 0
    got = rfa_hip.backward_saved(pq, pk, v, g, out, saved)
    want = _oracle_bwd(*cpu)
    for name, a, b in zip(("dq", "dk", "dv"), got, want):
        assert torch.isfinite(a.float()).all(), name
        assert _rel(a.float().cpu(), b) <= GRAD_RTOL, (name, _rel(a.float().cpu(), b))
    assert _rel(got[2].float(), seg[2].float()) <= 2e-3
    # deterministic, and the knob may move between forward and backward
    knobs(sliced=0)
    again = rfa_hip.backward_saved(pq, pk, v, g, out, saved)
    assert all(torch.equal(a, b) for a, b in zip(got, again))
