"""GPU parity (through the C ABI) of the feature map, the cross-attention
contractions and the decode step against the CPU oracle.

Tolerances: fp16 outputs max-abs <= 2e-3 vs the fp32 oracle on identical
fp16-rounded inputs; gradients <= 1e-2 relative Frobenius error; fp32 states
<= 1e-3 relative.
"""
import pytest
import torch

from oracle import rfa_oracle as O

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("binding")]

OUT_ATOL = 2e-3
GRAD_RTOL = 1e-2


def _rel(a, b):
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def _randn(*shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float32)


# ------------------------------------------------------------------ feature map
FEATURE_SHAPES = [(128, 2, 4, 64, 64), (3, 1, 2, 64, 32), (70, 3, 2, 128, 128), (1, 1, 1, 64, 128), (33, 2, 3, 128, 64),
                  (45, 2, 2, 128, 32)]


@pytest.mark.parametrize("L,B,H,d,D", FEATURE_SHAPES)
def test_feature_map_forward(L, B, H, d, D):
    from rfa_amd import rfa_hip
    x = (_randn(L, B, H, d, seed=10 + L) * 1.7).half()
    x[0, 0, 0] = 0                                  # zero row: phi = [0.., 0.1..]
    w = (_randn(H, D, d, seed=11) * 0.9).half()
    print(f"phi fwd L={L} B={B} H={H} d={d} D={D}", flush=True)
    got = rfa_hip.feature_map_forward(x.cuda(), w.cuda(), O.SCALE).float().cpu()
    want = O.random_project(x.float(), w.float())
    assert (got - want).abs().max().item() <= 7e-5     # |phi| <= 0.1: one fp16 ulp there is 6.1e-5
    assert torch.equal(got[0, 0, 0, :D], torch.zeros(D))


@pytest.mark.parametrize("L,B,H,d,D", FEATURE_SHAPES)
def test_feature_map_forward_pair(L, B, H, d, D):
    """phi(q) and phi(k) in one launch: the bits of the two single launches; through
    random_project_pair also the gradients of the two random_project calls (dW' summed)."""
    from rfa_amd import rfa_hip
    from rfa_amd.utils import random_project, random_project_pair
    x0 = (_randn(L, B, H, d, seed=30 + L) * 1.7).half().cuda()
    x1 = (_randn(L, B, H, d, seed=31 + L) * 0.6).half().cuda()
    w = (_randn(H, D, d, seed=32) * 0.9).half().cuda()
    print(f"phi fwd pair L={L} B={B} H={H} d={d} D={D}", flush=True)
    p0, p1 = rfa_hip.feature_map_forward_pair(x0, x1, w, O.SCALE)
    assert torch.equal(p0, rfa_hip.feature_map_forward(x0, w, O.SCALE))
    assert torch.equal(p1, rfa_hip.feature_map_forward(x1, w, O.SCALE))
    g0, g1 = _randn(L, B, H, 2 * D, seed=33).half().cuda(), _randn(L, B, H, 2 * D, seed=34).half().cuda()
    a0, a1, aw = (t.clone().requires_grad_(True) for t in (x0, x1, w))
    q0, q1 = random_project_pair(x0=a0, x1=a1, random_matrices=aw)
    torch.autograd.backward([q0, q1], [g0, g1])
    b0, b1, bw = (t.clone().requires_grad_(True) for t in (x0, x1, w))
    torch.autograd.backward([random_project(x=b0, random_matrices=bw), random_project(x=b1, random_matrices=bw)], [g0, g1])
    assert torch.equal(q0, p0) and torch.equal(q1, p1)
    assert torch.equal(a0.grad, b0.grad) and torch.equal(a1.grad, b1.grad)
    assert _rel(aw.grad.float().cpu(), bw.grad.float().cpu()) <= 2e-3     # one fp32 sum rounded once instead of two rounded sums added


@pytest.mark.parametrize("L,B,H,d,D", FEATURE_SHAPES)
def test_feature_map_backward(L, B, H, d, D):
    from rfa_amd import rfa_hip
    x = (_randn(L, B, H, d, seed=20 + L) * 1.3).half()
    if L > 1:
        x[1, 0, 0] = 0                              # ||x|| = 0 row must give dx = finite
    w = (_randn(H, D, d, seed=21) * 0.9).half()
    g = _randn(L, B, H, 2 * D, seed=22).half()
    print(f"phi bwd L={L} B={B} H={H} d={d} D={D}", flush=True)
    dx, dw = rfa_hip.feature_map_backward(x.cuda(), w.cuda(), g.cuda(), O.SCALE)
    dx, dw = dx.float().cpu(), dw.cpu()
    rx, rw = O.random_project_backward(x.float(), w.float(), g.float())
    assert torch.isfinite(dx).all() and torch.isfinite(dw).all()
    assert _rel(dx, rx) <= GRAD_RTOL, _rel(dx, rx)
    assert _rel(dw, rw) <= GRAD_RTOL, _rel(dw, rw)


@pytest.mark.parametrize("L,B,H,d,D", FEATURE_SHAPES)
def test_feature_map_backward_pair(L, B, H, d, D):
    """Two tensors through the same W' in one launch: dx of each as from its own call (same bits),
    dW' the sum of both (summed in another order, and checked against the oracle)."""
    from rfa_amd import rfa_hip
    x0 = (_randn(L, B, H, d, seed=30 + L) * 1.3).half().cuda()
    x1 = (_randn(L, B, H, d, seed=31 + L) * 0.7).half().cuda()
    w = (_randn(H, D, d, seed=32) * 0.9).half().cuda()
    g0 = _randn(L, B, H, 2 * D, seed=33).half().cuda()
    g1 = _randn(L, B, H, 2 * D, seed=34).half().cuda()
    print(f"phi bwd pair L={L} B={B} H={H} d={d} D={D}", flush=True)
    dx0, dx1, dw = rfa_hip.feature_map_backward_pair(x0, x1, w, g0, g1, O.SCALE)
    sx0, sw0 = rfa_hip.feature_map_backward(x0, w, g0, O.SCALE)
    sx1, sw1 = rfa_hip.feature_map_backward(x1, w, g1, O.SCALE)
    assert torch.equal(dx0, sx0) and torch.equal(dx1, sx1)
    assert _rel(dw.cpu(), (sw0 + sw1).cpu()) <= 1e-5
    _, rw0 = O.random_project_backward(x0.float().cpu(), w.float().cpu(), g0.float().cpu())
    _, rw1 = O.random_project_backward(x1.float().cpu(), w.float().cpu(), g1.float().cpu())
    assert _rel(dw.cpu(), rw0 + rw1) <= GRAD_RTOL


@pytest.mark.parametrize("L,B,H,d,D", FEATURE_SHAPES + [(300, 3, 4, 64, 64)])
@pytest.mark.parametrize("with_third", [True, False])
def test_feature_map_backward_pair_packed(L, B, H, d, D, with_third):
    """[dx0 | dx1 | third] side by side in one [R, 3 H d] matrix: every block carries the bits of
    the separate tensors, dW' those of the pair call, and without a third tensor its block is left
    as it was."""
    from rfa_amd import _lib, rfa_hip
    x0 = (_randn(L, B, H, d, seed=50 + L) * 1.3).half().cuda()
    x1 = (_randn(L, B, H, d, seed=51 + L) * 0.7).half().cuda()
    w = (_randn(H, D, d, seed=52) * 0.9).half().cuda()
    g0 = _randn(L, B, H, 2 * D, seed=53).half().cuda()
    g1 = _randn(L, B, H, 2 * D, seed=54).half().cuda()
    third = _randn(L, B, H, d, seed=55).half().cuda() if with_third else None
    want0, want1, want_dw = rfa_hip.feature_map_backward_pair(x0, x1, w, g0, g1, O.SCALE)
    print(f"phi bwd packed L={L} B={B} H={H} d={d} D={D} third={with_third}", flush=True)
    E = H * d
    if with_third:
        packed, dw = rfa_hip.feature_map_backward_pair_packed(x0, x1, w, g0, g1, third, O.SCALE)
        assert torch.equal(packed[:, 2 * E:], third.view(L * B, E))
    else:       # through the C ABI into a buffer of known contents
        lib = _lib.load()
        packed = torch.full((L * B, 3 * E), 7.0, dtype=torch.float16, device="cuda")
        dw = torch.empty(H, D, d, dtype=torch.float32, device="cuda")
        nbytes = lib.rfa_feature_map_backward_pair_workspace_bytes(L * B, H, D, d)
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
        _lib.check(lib.rfa_feature_map_backward_pair_packed(
            x0.data_ptr(), x1.data_ptr(), w.data_ptr(), g0.data_ptr(), g1.data_ptr(), None, packed.data_ptr(),
            dw.data_ptr(), L * B, H, D, d, O.SCALE, ws.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        assert bool((packed[:, 2 * E:] == 7.0).all())
    assert packed.shape == (L * B, 3 * E)
    assert torch.equal(packed[:, :E], want0.view(L * B, E)) and torch.equal(packed[:, E:2 * E], want1.view(L * B, E))
    assert torch.equal(dw, want_dw)


@pytest.mark.parametrize("L,B,H,d,D", FEATURE_SHAPES)
def test_feature_map_backward_without_dw(L, B, H, d, D):
    """Matrices that take no gradient: dx carries the bits of the full backward, dW' is neither
    formed nor reduced (None), no workspace is asked for; through the autograd Functions a frozen
    random_matrices tensor gets no gradient and x the same one."""
    from rfa_amd import _lib, rfa_hip
    from rfa_amd.utils import random_project, random_project_pair
    x0 = (_randn(L, B, H, d, seed=60 + L) * 1.3).half().cuda()
    x1 = (_randn(L, B, H, d, seed=61 + L) * 0.7).half().cuda()
    w = (_randn(H, D, d, seed=62) * 0.9).half().cuda()
    g0 = _randn(L, B, H, 2 * D, seed=63).half().cuda()
    g1 = _randn(L, B, H, 2 * D, seed=64).half().cuda()
    third = _randn(L, B, H, d, seed=65).half().cuda()
    print(f"phi bwd, dx only L={L} B={B} H={H} d={d} D={D}", flush=True)
    want, _ = rfa_hip.feature_map_backward(x0, w, g0, O.SCALE)
    got, dw = rfa_hip.feature_map_backward(x0, w, g0, O.SCALE, need_dw=False)
    assert dw is None and torch.equal(got, want)
    w0, w1, _ = rfa_hip.feature_map_backward_pair(x0, x1, w, g0, g1, O.SCALE)
    a0, a1, dw = rfa_hip.feature_map_backward_pair(x0, x1, w, g0, g1, O.SCALE, need_dw=False)
    assert dw is None and torch.equal(a0, w0) and torch.equal(a1, w1)
    wp, _ = rfa_hip.feature_map_backward_pair_packed(x0, x1, w, g0, g1, third, O.SCALE)
    gp, dw = rfa_hip.feature_map_backward_pair_packed(x0, x1, w, g0, g1, third, O.SCALE, need_dw=False)
    assert dw is None and torch.equal(gp, wp)
    # the C ABI with a NULL dw takes a NULL workspace
    lib = _lib.load()
    dx = torch.empty_like(x0)
    _lib.check(lib.rfa_feature_map_backward(x0.data_ptr(), w.data_ptr(), g0.data_ptr(), dx.data_ptr(), None, L * B, H, D, d,
                                            O.SCALE, None, 0, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.equal(dx, want)
    # autograd: frozen matrices
    xa, xb = x0.clone().requires_grad_(True), x1.clone().requires_grad_(True)
    wf = w.clone()                                   # requires_grad False
    p0, p1 = random_project_pair(x0=xa, x1=xb, random_matrices=wf, scale=O.SCALE)
    torch.autograd.backward([p0, p1], [g0, g1])
    assert wf.grad is None and torch.equal(xa.grad, w0) and torch.equal(xb.grad, w1)
    xc = x0.clone().requires_grad_(True)
    random_project(x=xc, random_matrices=wf, scale=O.SCALE).backward(g0)
    assert torch.equal(xc.grad, want)


@pytest.mark.parametrize("L,B,H,d,D,wgs", [(333, 2, 2, 64, 64, 4), (333, 2, 2, 64, 64, 2), (100, 3, 1, 128, 32, 1),
                                           (257, 1, 2, 64, 32, 6)])
def test_feature_map_waves_that_walk_many_row_groups(L, B, H, d, D, wgs, knobs):
    """With few workgroups every wave of the streaming kernels walks several groups of 16 rows
    (ragged: some waves one group more than others, odd and even counts, a last group that is not
    full): phi and dx carry the bits of the default launch, dW' is the same sum in another order."""
    from rfa_amd import rfa_hip
    x0 = (_randn(L, B, H, d, seed=40 + L) * 1.3).half().cuda()
    x1 = (_randn(L, B, H, d, seed=41 + L) * 0.7).half().cuda()
    w = (_randn(H, D, d, seed=42) * 0.9).half().cuda()
    g0 = _randn(L, B, H, 2 * D, seed=43).half().cuda()
    g1 = _randn(L, B, H, 2 * D, seed=44).half().cuda()
    want_phi = rfa_hip.feature_map_forward_pair(x0, x1, w, O.SCALE)
    want_dx0, want_dx1, want_dw = rfa_hip.feature_map_backward_pair(x0, x1, w, g0, g1, O.SCALE)
    want_sx, want_sw = rfa_hip.feature_map_backward(x0, w, g0, O.SCALE)
    knobs(feature_wg=wgs)
    print(f"phi with {wgs} workgroups L={L} B={B} H={H} d={d} D={D}", flush=True)
    p0, p1 = rfa_hip.feature_map_forward_pair(x0, x1, w, O.SCALE)
    assert torch.equal(p0, want_phi[0]) and torch.equal(p1, want_phi[1])
    assert torch.equal(rfa_hip.feature_map_forward(x1, w, O.SCALE), want_phi[1])
    dx0, dx1, dw = rfa_hip.feature_map_backward_pair(x0, x1, w, g0, g1, O.SCALE)
    assert torch.equal(dx0, want_dx0) and torch.equal(dx1, want_dx1)
    assert _rel(dw.cpu(), want_dw.cpu()) <= 1e-5
    sx, sw = rfa_hip.feature_map_backward(x0, w, g0, O.SCALE)
    assert torch.equal(sx, want_sx) and _rel(sw.cpu(), want_sw.cpu()) <= 1e-5
    _, rw0 = O.random_project_backward(x0.float().cpu(), w.float().cpu(), g0.float().cpu())
    assert _rel(sw.cpu(), rw0) <= GRAD_RTOL


@pytest.mark.parametrize("H,D,d,tau,with_sigma", [(8, 64, 64, 1.0, True), (3, 32, 128, 0.7, True),
                                                   (2, 128, 64, 2.0, False), (1, 5, 24, 1.3, True)])
def test_build_random_matrices_matches_the_aten_chain(H, D, d, tau, with_sigma):
    """W' = (sigma * W) / tau (reference utils.py:90-97): the one-launch form must give the bits of
    the two ATen launches on the same fp16 tensors, and gradients that agree with autograd through
    them (the column sums of dsigma are taken in another order, hence a tolerance there)."""
    from rfa_amd.utils import build_random_matrices
    print(f"build_random_matrices H={H} D={D} d={d} tau={tau} sigma={with_sigma}", flush=True)
    W = _randn(H, D, d, seed=900 + D).half().cuda()
    sigma = (1.0 + 0.3 * _randn(H, 1, d, seed=901 + d)).half().cuda() if with_sigma else None
    g = _randn(H, D, d, seed=902).half().cuda()
    # reference chain with autograd
    Wr = W.clone().requires_grad_(True)
    sr = sigma.clone().requires_grad_(True) if with_sigma else None
    ref = (sr * Wr if with_sigma else Wr) / tau
    ref.backward(g)
    # fused
    Wf = W.clone().requires_grad_(True)
    sf = sigma.clone().requires_grad_(True) if with_sigma else None
    got = build_random_matrices(random_matrices=Wf, tau=tau, sigma=sf, reparam_proj=with_sigma)
    assert type(got.grad_fn).__name__.startswith("_BuildRandomMatrices")
    assert torch.equal(got, ref)
    got.backward(g)
    assert torch.equal(Wf.grad, Wr.grad)
    if with_sigma:
        assert sf.grad.shape == sr.grad.shape
        assert _rel(sf.grad.float().cpu(), sr.grad.float().cpu()) <= 2e-3
    # without gradients asked for sigma only the matrix gradient is formed, and vice versa
    sf2 = sigma.clone().requires_grad_(True) if with_sigma else None
    out2 = build_random_matrices(random_matrices=W, tau=tau, sigma=sf2, reparam_proj=with_sigma)
    assert torch.equal(out2, ref)
    if with_sigma:
        out2.backward(g)
        assert torch.equal(sf2.grad, sf.grad)


# ------------------------------------------------------------------------ cross
def _cross_inputs(S, T, B, H, d, D, seed, lengths=None):
    W = O.make_w(d, D, H)
    k = O.unit_rows(_randn(S, B, H, d, seed=seed)).half()
    q = O.unit_rows(_randn(T, B, H, d, seed=seed + 1)).half()
    v = _randn(S, B, H, d, seed=seed + 2).half()
    g = _randn(T, B, H, d, seed=seed + 3).half()
    pk = O.random_project(k.float(), W).half()
    pq = O.random_project(q.float(), W).half()
    mask = None
    if lengths is not None:
        mask = torch.zeros(B, S, dtype=torch.bool)
        for b, L in enumerate(lengths):
            mask[b, L:] = True
    return pq, pk, v, g, mask


CROSS_SHAPES = [
    # S, T, B, H, d, D, lengths
    (96, 40, 2, 2, 64, 64, None),
    (130, 70, 3, 2, 64, 64, [130, 64, 7]),
    (64, 1, 1, 1, 64, 32, [33]),
    (200, 129, 1, 2, 128, 64, [150]),
    (70, 65, 2, 1, 64, 128, None),
]


@pytest.mark.parametrize("S,T,B,H,d,D,lengths", CROSS_SHAPES)
def test_cross_forward(S, T, B, H, d, D, lengths):
    from rfa_amd import rfa_hip
    pq, pk, v, g, mask = _cross_inputs(S, T, B, H, d, D, 300 + S, lengths)
    print(f"cross fwd S={S} T={T} B={B} H={H} d={d} D={D}", flush=True)
    s, z = rfa_hip.cross_state(pk.cuda(), v.cuda(), None if mask is None else mask.cuda())
    rs, rz = O.cross_state(pk.float(), v.float(), None if mask is None else mask.t())
    assert _rel(s.cpu(), rs) <= 1e-3 and _rel(z.cpu(), rz) <= 1e-3
    out = rfa_hip.cross_readout(pq.cuda(), s, z).float().cpu()
    want = O.cross_readout(pq.float(), rs, rz)
    assert (out - want).abs().max().item() <= OUT_ATOL


def test_cross_mask_dtypes_agree():
    """The padding mask may come as bool, as bytes (any non-zero value marks a padded key), as int64 or
    as float, contiguous or not: one-byte contiguous masks reach the kernels as they are, the
    others are reduced to 0/1 bytes first.  All of them must give the same bits."""
    from rfa_amd import rfa_hip
    pq, pk, v, g, mask = _cross_inputs(130, 70, 3, 2, 64, 64, 777, [130, 64, 7])
    pk_c, v_c = pk.cuda(), v.cuda()
    base_s, base_z = rfa_hip.cross_state(pk_c, v_c, mask.cuda())
    ds = torch.randn_like(base_s)
    dz = torch.randn_like(base_z)
    base_dk, base_dv = rfa_hip.cross_state_backward(pk_c, v_c, ds, dz, mask.cuda())
    wide = torch.zeros(3, 260, dtype=torch.bool)
    wide[:, ::2] = mask
    variants = {
        "uint8 ones": mask.to(torch.uint8),
        "uint8 sevens": mask.to(torch.uint8) * 7,
        "int64": mask.to(torch.int64),
        "float": mask.to(torch.float32),
        "strided bool": wide[:, ::2],
    }
    for name, m in variants.items():
        print(f"cross mask variant {name}", flush=True)
        m = m.cuda()
        if name == "strided bool":
            m = wide.cuda()[:, ::2]
            assert not m.is_contiguous()
        s, z = rfa_hip.cross_state(pk_c, v_c, m)
        assert torch.equal(s, base_s) and torch.equal(z, base_z), name
        dk, dv = rfa_hip.cross_state_backward(pk_c, v_c, ds, dz, m)
        assert torch.equal(dk, base_dk) and torch.equal(dv, base_dv), name


@pytest.mark.parametrize("pattern", ["left padded", "holes", "all but one", "everything"])
def test_cross_arbitrary_padding_patterns(pattern):
    """The source mask need not be a suffix: left-padded batches (fairseq's default for sources),
    masked keys in the middle, a single live key, and a fully masked sequence (zero state, zero
    gradients) against the oracle."""
    from rfa_amd import rfa_hip
    S, T, B, H, d, D = 200, 70, 3, 2, 64, 64
    pq, pk, v, g, _ = _cross_inputs(S, T, B, H, d, D, 880)
    gen = torch.Generator().manual_seed(881)
    mask = torch.zeros(B, S, dtype=torch.bool)
    if pattern == "left padded":
        for b, L in enumerate([0, 37, 150]):
            mask[b, :L] = True
    elif pattern == "holes":
        mask = torch.rand(B, S, generator=gen) < 0.4
    elif pattern == "all but one":
        mask[:] = True
        mask[0, 199] = mask[1, 0] = mask[2, 64] = False
    else:
        mask[1] = True
    print(f"cross mask pattern {pattern}", flush=True)
    omask = mask.t()
    rs, rz = O.cross_state(pk.float(), v.float(), omask)
    s, z = rfa_hip.cross_state(pk.cuda(), v.cuda(), mask.cuda())
    assert (s.cpu() - rs).abs().max().item() <= 1e-3 * max(1.0, rs.abs().max().item())
    assert (z.cpu() - rz).abs().max().item() <= 1e-3 * max(1.0, rz.abs().max().item())
    if pattern == "everything":
        assert (s[1] == 0).all() and (z[1] == 0).all()
    out = rfa_hip.cross_readout(pq.cuda(), s, z).float().cpu()
    assert (out - O.cross_readout(pq.float(), rs, rz)).abs().max().item() <= OUT_ATOL
    wq, wds, wdz = O.cross_readout_backward(pq.float(), rs, rz, g.float())
    wk, wv = O.cross_state_backward(pk.float(), v.float(), wds, wdz, omask)
    dq, ds, dz = rfa_hip.cross_readout_backward(pq.cuda(), s, z, g.cuda())
    dk, dv = rfa_hip.cross_state_backward(pk.cuda(), v.cuda(), ds, dz, mask.cuda())
    for name, got, want in (("dq", dq, wq), ("dk", dk, wk), ("dv", dv, wv)):
        got = got.float().cpu()
        assert torch.isfinite(got).all(), name
        assert _rel(got, want) <= GRAD_RTOL, (name, _rel(got, want))
    assert (dk.float().cpu()[omask] == 0).all()


def test_cross_readout_negative_denominator():
    """abs() in the denominator: flip the sign of z so that q.z < -1."""
    from rfa_amd import rfa_hip
    pq, pk, v, g, _ = _cross_inputs(256, 64, 1, 2, 64, 64, 400)
    rs, rz = O.cross_state(pk.float(), v.float())
    rz = -rz
    assert (torch.einsum("tbhk,bhk->tbh", pq.float(), rz) < -1).any()
    out = rfa_hip.cross_readout(pq.cuda(), rs.cuda().contiguous(), rz.cuda().contiguous()).float().cpu()
    assert (out - O.cross_readout(pq.float(), rs, rz)).abs().max().item() <= OUT_ATOL
    dq, ds, dz = rfa_hip.cross_readout_backward(pq.cuda(), rs.cuda().contiguous(), rz.cuda().contiguous(), g.cuda())
    wq, ws, wz = O.cross_readout_backward(pq.float(), rs, rz, g.float())
    assert _rel(dq.float().cpu(), wq) <= GRAD_RTOL
    assert _rel(ds.cpu(), ws) <= GRAD_RTOL and _rel(dz.cpu(), wz) <= GRAD_RTOL


@pytest.mark.parametrize("S,T,B,H,d,D,lengths", CROSS_SHAPES)
def test_cross_backward(S, T, B, H, d, D, lengths):
    from rfa_amd import rfa_hip
    pq, pk, v, g, mask = _cross_inputs(S, T, B, H, d, D, 500 + S, lengths)
    print(f"cross bwd S={S} T={T} B={B} H={H} d={d} D={D}", flush=True)
    omask = None if mask is None else mask.t()
    rs, rz = O.cross_state(pk.float(), v.float(), omask)
    wq, wds, wdz = O.cross_readout_backward(pq.float(), rs, rz, g.float())
    wk, wv = O.cross_state_backward(pk.float(), v.float(), wds, wdz, omask)
    cmask = None if mask is None else mask.cuda()
    s, z = rfa_hip.cross_state(pk.cuda(), v.cuda(), cmask)
    dq, ds, dz = rfa_hip.cross_readout_backward(pq.cuda(), s, z, g.cuda())
    dk, dv = rfa_hip.cross_state_backward(pk.cuda(), v.cuda(), ds, dz, cmask)
    for name, got, want in (("dq", dq, wq), ("ds", ds, wds), ("dz", dz, wdz), ("dk", dk, wk), ("dv", dv, wv)):
        got = got.float().cpu()
        assert torch.isfinite(got).all(), name
        assert _rel(got, want) <= GRAD_RTOL, (name, _rel(got, want))
    if mask is not None:
        assert (dk.float().cpu()[mask.t()] == 0).all()


# ----------------------------------------------------------------------- decode
@pytest.mark.parametrize("B,H,d,D,prefill,steps", [(2, 4, 64, 64, 0, 5), (3, 2, 64, 64, 40, 9), (1, 2, 128, 64, 17, 4),
                                                   (2, 1, 64, 128, 10, 3), (1, 1, 128, 128, 5, 3), (2, 2, 64, 32, 3, 4)])
def test_incremental_matches_oracle(B, H, d, D, prefill, steps):
    from rfa_amd import rfa_hip
    T = prefill + steps
    q, k, v, _ = O.make_qkv(T, B, H, d, 700 + T)
    W = O.make_w(d, D, H)
    N, K = B * H, 2 * D
    pq = O.random_project(q.float(), W).half().reshape(T, N, K)
    pk = O.random_project(k.float(), W).half().reshape(T, N, K)
    vv = v.reshape(T, N, d)
    want, ws, wz = O.causal_forward_loop(pq.float(), pk.float(), vv.float())
    _, s0, z0 = O.causal_forward_loop(pq[:prefill].float(), pk[:prefill].float(), vv[:prefill].float())
    print(f"decode B={B} H={H} d={d} D={D} prefill={prefill} steps={steps}", flush=True)
    # feature-level entry point
    s, z = s0.cuda().contiguous(), z0.cuda().contiguous()
    out = rfa_hip.incremental(pq[prefill:].cuda().contiguous(), pk[prefill:].cuda().contiguous(),
                              vv[prefill:].cuda().contiguous(), s, z).float().cpu()
    assert (out - want[prefill:]).abs().max().item() <= OUT_ATOL
    assert _rel(s.cpu(), ws) <= 1e-3 and _rel(z.cpu(), wz) <= 1e-3
    # fused entry point: raw q, k plus the random matrix
    s = s0.cuda().reshape(B, H, K, d).contiguous()
    z = z0.cuda().reshape(B, H, K).contiguous()
    out2 = rfa_hip.incremental_fused(q[prefill:].cuda().contiguous(), k[prefill:].cuda().contiguous(),
                                     v[prefill:].cuda().contiguous(), W.half().cuda(), O.SCALE, s, z).float().cpu()
    assert (out2.reshape(steps, N, d) - want[prefill:]).abs().max().item() <= OUT_ATOL
    assert _rel(s.cpu().reshape(N, K, d), ws) <= 2e-3


@pytest.mark.usefixtures("binding")
@pytest.mark.parametrize("B,H,d,D,steps", [(2, 4, 64, 64, 5), (3, 2, 128, 64, 3), (1, 3, 64, 128, 70), (64, 16, 64, 64, 2)])
def test_incremental_qkv_equals_the_step_on_separate_tensors(B, H, d, D, steps):
    """q, k, v as the three thirds of one projection's output rows ([steps, B, 3, H, d]): the bits of
    incremental_fused on contiguous copies of the thirds, in place and into a second state, over
    single-step calls and one multi-step call (which streams the packed rows ahead of the steps)."""
    from rfa_amd import rfa_hip
    K = 2 * D
    qkv = (_randn(steps, B, 3, H, d, seed=900 + steps) * 0.7).half().cuda()
    W = O.make_w(d, D, H).half().cuda()
    s0 = (_randn(B, H, K, d, seed=901) * 0.3).cuda()
    z0 = (_randn(B, H, K, seed=902).abs() * 2.0).cuda()
    q, k, v = (qkv[:, :, i].contiguous() for i in range(3))
    print(f"decode packed B={B} H={H} d={d} D={D} steps={steps}", flush=True)
    s1, z1 = s0.clone(), z0.clone()
    want = rfa_hip.incremental_fused(q, k, v, W, O.SCALE, s1, z1)
    s2, z2 = s0.clone(), z0.clone()
    got = rfa_hip.incremental_qkv(qkv, W, O.SCALE, s2, z2)
    assert torch.equal(got, want) and torch.equal(s2, s1) and torch.equal(z2, z1)
    s3, z3 = s0.clone(), z0.clone()
    so, zo = torch.empty_like(s0), torch.empty_like(z0)
    rows = []
    for t in range(min(steps, 4)):           # one call per token, state into a second pair of tensors
        rows.append(rfa_hip.incremental_qkv(qkv[t:t + 1].contiguous(), W, O.SCALE, s3, z3, so, zo))
        s3, z3, so, zo = so, zo, s3, z3
    assert torch.equal(torch.cat(rows), want[:len(rows)])
    with pytest.raises(Exception, match="3, heads"):
        rfa_hip.incremental_qkv(qkv[:, :, :2].contiguous(), W, O.SCALE, s2, z2)
