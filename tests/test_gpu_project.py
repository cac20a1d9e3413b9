"""GPU parity (through the C ABI) of the fused Linear -> heads -> feature map launch
against torch's fp64 matmul and the CPU oracle's feature map.

Tolerances: the projections y are fp16 roundings of an fp32-accumulated product, compared
with the fp64 product of the same fp16 inputs: |dy| <= 1.5e-3 * max(1, |y|) (one fp16 ulp
is 9.8e-4 relative).  phi is compared (a) with the oracle applied to the y the kernel itself
returned (<= 2e-3 absolute, the feature-map bar) and (b) with the oracle applied to the
fp64 product rounded to fp16 (<= 4e-3: an ulp of difference in y moves the angle).
"""
import pytest
import torch

from oracle import rfa_oracle as O

pytestmark = pytest.mark.gpu

# L, B, E, H, d, D
SHAPES = [(128, 2, 256, 4, 64, 64), (300, 2, 512, 8, 64, 64), (70, 3, 128, 2, 64, 64), (33, 1, 256, 2, 128, 128), (5, 2, 64, 1, 64, 32),
          (1, 1, 192, 3, 64, 128), (257, 1, 128, 1, 128, 64)]


def _randn(*shape, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=torch.float32)


def _inputs(L, B, E, H, d, seed, n):
    x = (_randn(L, B, E, seed=seed) * 0.8).half()
    ws = [(_randn(H * d, E, seed=seed + 1 + p) / E ** 0.5 * 1.5).half() for p in range(n)]
    bs = [(_randn(H * d, seed=seed + 11 + p) * 0.3).half() for p in range(n)]
    return x, ws, bs


def _linear64(x, w, b, H, d):
    y = x.double() @ w.double().t()
    if b is not None:
        y = y + b.double()
    return y.view(*x.shape[:2], H, d)


@pytest.mark.parametrize("streaming", [False, True])
@pytest.mark.parametrize("L,B,E,H,d,D", SHAPES)
def test_qkv_projection_with_feature_map(L, B, E, H, d, D, streaming, knobs):
    """Both kernels: the one that keeps its rows of x in LDS (picked when they fit) and the one
    that streams x and the weights together (forced by the "project_streaming" knob)."""
    from rfa_amd import rfa_hip
    knobs(project_streaming=1 if streaming else -1)
    x, ws, bs = _inputs(L, B, E, H, d, 900 + L, 3)
    bs[1] = None                                       # one projection without bias
    wf = (_randn(H, D, d, seed=77) * 0.9).half()
    print(f"project+phi L={L} B={B} E={E} H={H} d={d} D={D}", flush=True)
    dev = lambda t: None if t is None else t.cuda()
    ys, phis = rfa_hip.project_feature_map(x.cuda(), [w.cuda() for w in ws], [dev(b) for b in bs],
                                           [True, True, False], wf.cuda(), H, O.SCALE)
    assert phis[2] is None and phis[0].shape == (L, B, H, 2 * D)
    for p in range(3):
        want = _linear64(x, ws[p], bs[p], H, d)
        got = ys[p].double().cpu()
        assert ys[p].shape == (L, B, H, d)
        assert ((got - want).abs() <= 1.5e-3 * want.abs().clamp_min(1.0)).all(), (p, (got - want).abs().max().item())
        if p < 2:
            phi = phis[p].float().cpu()
            own = O.random_project(ys[p].float().cpu(), wf.float())
            assert (phi - own).abs().max().item() <= 2e-3
            ref = O.random_project(want.half().float(), wf.float())
            assert (phi - ref).abs().max().item() <= 4e-3


@pytest.mark.parametrize("streaming", [False, True])
def test_projection_without_keeping_y(streaming, knobs):
    """keep_y=False (what the modules ask for when nothing requires a gradient): phi and the plain
    projection come out bit-identical to the keeping call, y of the phi projections is not produced."""
    from rfa_amd import rfa_hip
    from rfa_amd.projection import project_heads
    knobs(project_streaming=1 if streaming else -1)
    L, B, E, H, d, D = 200, 3, 256, 4, 64, 64
    x, ws, bs = _inputs(L, B, E, H, d, 4321, 3)
    wf = (_randn(H, D, d, seed=78) * 0.9).half().cuda()
    args = (x.cuda(), [w.cuda() for w in ws], [b.cuda() for b in bs], [True, True, False], wf, H, O.SCALE)
    print(f"project+phi without y, streaming={streaming}", flush=True)
    ys, phis = rfa_hip.project_feature_map(*args)
    ys0, phis0 = rfa_hip.project_feature_map(*args, keep_y=False)
    assert ys0[0] is None and ys0[1] is None and phis0[2] is None
    assert torch.equal(ys0[2], ys[2]) and torch.equal(phis0[0], phis[0]) and torch.equal(phis0[1], phis[1])
    layers = []
    for w, b in zip(ws, bs):
        lin = torch.nn.Linear(E, H * d).cuda().half()
        lin.weight.data.copy_(w); lin.bias.data.copy_(b)
        layers.append(lin)
    # the modules' entry: trainable layers under no_grad must take the keep_y=False launch, and the keeping one
    # (with the same bits) when a gradient can be asked for
    seen = []
    real = rfa_hip.project_feature_map

    def spy(*a, **kw):
        seen.append(a[7] if len(a) > 7 else kw.get("keep_y", True))
        return real(*a, **kw)
    rfa_hip.project_feature_map = spy
    try:
        with torch.no_grad():
            outs = project_heads(x.cuda(), layers, (True, True, False), H, wf, O.SCALE)
        kept = project_heads(x.cuda(), layers, (True, True, False), H, wf, O.SCALE)
    finally:
        rfa_hip.project_feature_map = real
    assert seen == [False, True] and all(p.requires_grad for lin in layers for p in lin.parameters())
    assert torch.equal(outs[0], phis[0]) and torch.equal(outs[1], phis[1]) and torch.equal(outs[2], ys[2])
    assert all(torch.equal(a, b) for a, b in zip(outs, kept)) and kept[0].requires_grad
    with pytest.raises(Exception, match="neither y nor phi"):
        from rfa_amd import _lib
        import ctypes
        arr = ctypes.c_void_p * 1
        xx = x.cuda()
        _lib.check(_lib.load().rfa_project_feature_map(xx.data_ptr(), arr(ws[0].cuda().data_ptr()), None, arr(None), None, 1,
                                                       None, L * B, E, H, D, d, O.SCALE, None))


def test_plain_projection_is_a_linear_layer():
    """No phi requested: out_proj-style use, one projection, with and without bias."""
    from rfa_amd import rfa_hip
    L, B, E, H, d = 130, 2, 512, 8, 64
    x, ws, bs = _inputs(L, B, E, H, d, 950, 1)
    for b in (bs[0], None):
        ys, phis = rfa_hip.project_feature_map(x.cuda(), [ws[0].cuda()], [None if b is None else b.cuda()], [False],
                                               None, H, O.SCALE)
        assert phis == [None]
        want = _linear64(x, ws[0], b, H, d)
        got = ys[0].double().cpu()
        assert ((got - want).abs() <= 1.5e-3 * want.abs().clamp_min(1.0)).all()
        ref16 = torch.nn.functional.linear(x.cuda(), ws[0].cuda(), None if b is None else b.cuda()).view(L, B, H, d)
        assert (ys[0].float() - ref16.float()).abs().max().item() <= 4e-3      # the library GEMM, for reference


def test_zero_rows_and_argument_checks():
    from rfa_amd import rfa_hip
    H, d, D, E = 2, 64, 64, 128
    x, ws, bs = _inputs(4, 1, E, H, d, 960, 2)
    x[1] = 0
    ws = [w.cuda() for w in ws]
    wf = (_randn(H, D, d, seed=78)).half().cuda()
    ys, phis = rfa_hip.project_feature_map(x.cuda(), ws, [None, None], [True, True], wf, H, O.SCALE)
    # a zero input row without bias projects to zero, whose phi is [0.., scale..]
    assert (ys[0][1] == 0).all()
    assert (phis[0][1, 0, :, :D] == 0).all() and (phis[0][1, 0, :, D:].float() - O.SCALE).abs().max() <= 1e-4
    with pytest.raises(ValueError):
        rfa_hip.project_feature_map(x.cuda(), ws, [None], [True, True], wf, H, O.SCALE)
    with pytest.raises(ValueError):
        rfa_hip.project_feature_map(x.cuda(), ws, [None, None], [True, False], None, H, O.SCALE)
    with pytest.raises((RuntimeError, ValueError)):
        rfa_hip.project_feature_map(x[..., :100].contiguous().cuda(), [w[:, :100].contiguous() for w in ws],
                                    [None, None], [False, False], None, H, O.SCALE)    # E not a multiple of 64
    with pytest.raises((RuntimeError, TypeError)):
        rfa_hip.project_feature_map(x, [w.cpu() for w in ws], [None, None], [False, False], None, H, O.SCALE)


@pytest.mark.parametrize("with_pad", [False, True])
def test_causal_module_fused_projections_match_unfused_chain(with_pad):
    """CausalAttention with the q/k/v projections + phi as one launch vs the same module running
    nn.Linear + random_project: outputs within 4e-3, every gradient within 1e-2 (relative
    Frobenius norm) of the unfused module's, and within 2e-2 of an fp64 autograd run of the
    oracle chain."""
    from rfa_amd import CausalAttention
    torch.manual_seed(5)
    T, B, E, H, d, D = 200, 3, 256, 4, 64, 64
    m = CausalAttention(embed_dim=E, num_heads=H, head_dim=d, proj_dim=D).cuda().half()
    with torch.no_grad():
        m.sigma.mul_(1.0 + 0.1 * torch.randn_like(m.sigma))
        m.out_proj.bias.normal_(0, 0.1)
    W = O.make_w(d, D, H).cuda().half()
    x0 = (torch.randn(T, B, E) * 0.7).half()
    go = torch.randn(T, B, E).half().cuda()
    pad = None
    if with_pad:
        pad = torch.zeros(B, T, dtype=torch.bool)
        pad[1, 150:] = True
        pad = pad.cuda()

    def run(fused):
        m.fuse_projections = fused
        m.zero_grad(set_to_none=True)
        x = x0.clone().cuda().requires_grad_(True)
        y = m(x, W, key_padding_mask=pad)
        y.backward(go)
        return y.detach().float().cpu(), {"x": x.grad.float().cpu(),
                                          **{n: p.grad.float().cpu() for n, p in m.named_parameters()}}

    y_f, g_f = run(True)
    y_u, g_u = run(False)
    assert (y_f - y_u).abs().max().item() <= 4e-3
    rel = lambda a, b: ((a - b).norm() / b.norm().clamp_min(1e-30)).item()
    for name in g_u:
        assert torch.isfinite(g_f[name]).all(), name
        assert rel(g_f[name], g_u[name]) <= 1e-2, (name, rel(g_f[name], g_u[name]))

    # fp64 autograd through the oracle chain with the same fp16 parameters
    P = {n: p.detach().double().cpu().requires_grad_(True) for n, p in m.named_parameters()}
    x = x0.double().requires_grad_(True)
    lin = lambda n: x @ P[n + ".weight"].t() + P[n + ".bias"]
    q, k, v = (lin(n).reshape(T, B, H, d) for n in ("q_proj", "k_proj", "v_proj"))
    Wp = O.build_random_matrices(W.double().cpu(), 1.0, P["sigma"], True)
    pq, pk = O.random_project(q, Wp), O.random_project(k, Wp)
    if with_pad:
        pk = pk.masked_fill(pad.cpu().t()[:, :, None, None], 0.0)
    att = O.causal_forward_chunked(pq.reshape(T, B * H, 2 * D), pk.reshape(T, B * H, 2 * D), v.reshape(T, B * H, d))
    want = att.reshape(T, B, E) @ P["out_proj.weight"].t() + P["out_proj.bias"]
    assert (y_f.double() - want.detach()).abs().max().item() <= 1e-2
    want.backward(go.double().cpu())
    ref = {"x": x.grad, **{n: p.grad for n, p in P.items()}}
    for name in ref:
        assert rel(g_f[name].double(), ref[name]) <= 2e-2, (name, rel(g_f[name].double(), ref[name]))


@pytest.mark.parametrize("R,Eo,Ei,n", [(8192, 512, 512, 3), (300, 256, 512, 2), (70, 768, 256, 1), (200, 128, 256, 1), (1, 128, 128, 2), (4097, 256, 128, 3),
                                       (64, 384, 128, 1)])
def test_linear_weight_and_bias_gradients(R, Eo, Ei, n):
    """dW = dy^T x and db = column sums against fp64; fp16 outputs of fp32 sums: <= 1.5e-3 relative
    to max(1, |value|) per element, and <= 1e-3 relative Frobenius error."""
    from rfa_amd import rfa_hip
    x = (_randn(R, Ei, seed=970 + R) * 0.5).half()
    dys = [(_randn(R, Eo, seed=971 + p) * 0.05).half() for p in range(n)]
    want_bias = [p != 1 for p in range(n)]
    print(f"weight grad R={R} Eo={Eo} Ei={Ei} n={n}", flush=True)
    dws, dbs = rfa_hip.linear_weight_grad(x.cuda(), [d.cuda() for d in dys], want_bias)
    for p in range(n):
        ww = dys[p].double().t() @ x.double()
        got = dws[p].double().cpu()
        assert ((got - ww).abs() <= 1.5e-3 * ww.abs().clamp_min(1.0)).all(), (p, (got - ww).abs().max().item())
        assert ((got - ww).norm() / ww.norm()).item() <= 1e-3
        if want_bias[p]:
            wb = dys[p].double().sum(0)
            gb = dbs[p].double().cpu()
            assert ((gb - wb).abs() <= 1.5e-3 * wb.abs().clamp_min(1.0)).all()
        else:
            assert dbs[p] is None
    with pytest.raises(ValueError):
        rfa_hip.linear_weight_grad(x[:, :64].contiguous().cuda(), [d.cuda() for d in dys], want_bias)


def test_cross_modules_fused_projections_match_unfused_chain():
    """CrossAttentionProjectLayer + CrossAttention with their projections on the fused launch vs
    the same modules on nn.Linear + random_project: output within 4e-3, gradients within 1e-2."""
    from rfa_amd import CrossAttention, CrossAttentionProjectLayer
    torch.manual_seed(6)
    S, T, B, E, H, d, D = 150, 70, 2, 256, 4, 64, 64
    proj = CrossAttentionProjectLayer(embed_dim=E, num_heads=H, head_dim=d, proj_dim=D).cuda().half()
    att = CrossAttention(embed_dim=E, num_heads=H, head_dim=d, proj_dim=D).cuda().half()
    with torch.no_grad():
        proj.sigma.mul_(1.0 + 0.1 * torch.randn_like(proj.sigma))
        att.q_proj.bias.normal_(0, 0.1)
    W = O.make_w(d, D, H).cuda().half()
    enc0 = (torch.randn(S, B, E) * 0.7).half()
    q0 = (torch.randn(T, B, E) * 0.7).half()
    go = torch.randn(T, B, E).half().cuda()
    mask = torch.zeros(S, B, 1, 1, dtype=torch.bool)
    mask[120:, 1] = True
    mask = mask.cuda()

    def run(fused):
        proj.fuse_projections = att.fuse_projections = fused
        proj.zero_grad(set_to_none=True)
        att.zero_grad(set_to_none=True)
        enc = enc0.clone().cuda().requires_grad_(True)
        q = q0.clone().cuda().requires_grad_(True)
        y = att(q, proj(encoder_output=enc, random_matrices=W, mask=mask))
        y.backward(go)
        grads = {"enc": enc.grad, "q": q.grad}
        grads.update({"proj." + n: p.grad for n, p in proj.named_parameters()})
        grads.update({"att." + n: p.grad for n, p in att.named_parameters()})
        return y.detach().float().cpu(), {k: v.float().cpu() for k, v in grads.items()}

    y_f, g_f = run(True)
    y_u, g_u = run(False)
    assert (y_f - y_u).abs().max().item() <= 4e-3
    for name in g_u:
        r = ((g_f[name] - g_u[name]).norm() / g_u[name].norm().clamp_min(1e-30)).item()
        assert torch.isfinite(g_f[name]).all() and r <= 1e-2, (name, r)


def test_module_step_replays_from_a_hip_graph():
    """Forward + backward of CausalAttention captured once and replayed: every replay, with eager
    steps and synchronisations in between, gives bit-identical output and gradients to the eager step."""
    from rfa_amd import CausalAttention
    torch.manual_seed(7)
    T, B, E, H, d, D = 320, 2, 256, 4, 64, 64
    m = CausalAttention(embed_dim=E, num_heads=H, head_dim=d, proj_dim=D).cuda().half()
    W = O.make_w(d, D, H).cuda().half()
    x = (torch.randn(T, B, E) * 0.6).half().cuda().requires_grad_(True)
    go = torch.randn(T, B, E).half().cuda()

    def step():
        m.zero_grad(set_to_none=True)
        x.grad = None
        y = m(x, W)
        y.backward(go)
        return y

    y_e = step().detach().clone()
    want = {"x": x.grad.detach().clone(), **{n: p.grad.detach().clone() for n, p in m.named_parameters()}}
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    m.zero_grad(set_to_none=True)
    x.grad = None
    with torch.cuda.graph(graph):
        y_g = m(x, W)
        y_g.backward(go)
    captured = {"x": x.grad, **{n: p.grad for n, p in m.named_parameters()}}   # the graph's output buffers
    for rep in range(3):
        for t in captured.values():
            t.zero_()
        y_g.detach().zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_g, y_e), rep
        for name, t in captured.items():
            assert torch.equal(t, want[name]), (rep, name)
        # eager work between the replays; it rebinds .grad, the graph keeps writing its own buffers
        grads_before = {k: v for k, v in captured.items()}
        step()
        torch.cuda.synchronize()
        captured = grads_before


def test_projection_backward_on_the_packed_gradient(monkeypatch):
    """q, k through the feature map and v plain: the backward that forms [dy_q | dy_k | dv] in one
    matrix (one GEMM for dx, one contraction for the three dW) against the one with a GEMM per
    projection.  dW, db and dW' carry the same bits (the same row-split sums); dx is one sum of 3E
    products in place of three rounded partial sums."""
    from rfa_amd import projection
    torch.manual_seed(11)
    L, B, E, H, d, D = 130, 3, 256, 4, 64, 64
    layers = [torch.nn.Linear(E, H * d).cuda().half() for _ in range(3)]
    layers[1].bias = None
    wf = (torch.randn(H, D, d) * 0.9).half().cuda().requires_grad_(True)
    x = (torch.randn(L, B, E) * 0.7).half().cuda().requires_grad_(True)
    gs = [torch.randn(L, B, H, 2 * D).half().cuda(), torch.randn(L, B, H, 2 * D).half().cuda(),
          torch.randn(L, B, H, d).half().cuda()]

    def run():
        for t in [x, wf] + [p for l in layers for p in l.parameters()]:
            t.grad = None
        outs = projection.project_heads(x, layers, [True, True, False], H, wf, O.SCALE)
        torch.autograd.backward(outs, gs)
        return [x.grad.clone(), wf.grad.clone()] + [p.grad.clone() for l in layers for p in l.parameters()]

    used = []
    real = projection.rfa_hip.feature_map_backward_pair_packed
    monkeypatch.setattr(projection.rfa_hip, "feature_map_backward_pair_packed",
                        lambda *a, **kw: (used.append(1), real(*a, **kw))[1])
    print("projection backward, packed gradient", flush=True)
    packed = run()
    assert used, "the packed path was not taken"
    key = tuple(id(l.weight) for l in layers)           # the stack of the weights is kept between eager steps ...
    stack = projection._STACKED[key].value
    again = run()
    assert projection._STACKED[key].value is stack and all(torch.equal(a, b) for a, b in zip(packed, again))
    with torch.no_grad():
        layers[2].weight.mul_(1.5)                      # ... until a weight changes
    changed = run()
    assert projection._STACKED[key].value is not stack and not torch.equal(changed[0], packed[0])
    with torch.no_grad():
        layers[2].weight.div_(1.5)                      # exact in fp16
    used.clear()
    packed = run()
    monkeypatch.setattr(projection, "_packed_backward_ok", lambda *a: False)
    plain = run()
    assert len(used) == 1 and len(packed) == len(plain) == 2 + 5
    scale = plain[0].float().abs().max().item()
    assert (packed[0].float() - plain[0].float()).abs().max().item() <= 4e-3 * scale
    for a, b in zip(packed[1:], plain[1:]):
        assert torch.equal(a, b)


def test_packed_backward_in_a_graph_follows_weight_updates():
    """The stacked weights [Wq; Wk; Wv] of the packed backward are kept between eager steps but
    formed inside a captured graph: a replay after an in-place weight update gives the eager
    gradients of the updated weights."""
    from rfa_amd import CausalAttention
    torch.manual_seed(13)
    T, B, E, H, d, D = 192, 2, 256, 4, 64, 64
    m = CausalAttention(embed_dim=E, num_heads=H, head_dim=d, proj_dim=D).cuda().half()
    W = O.make_w(d, D, H).cuda().half()
    x = (torch.randn(T, B, E) * 0.6).half().cuda().requires_grad_(True)
    go = torch.randn(T, B, E).half().cuda()

    def step():
        m.zero_grad(set_to_none=True)
        x.grad = None
        m(x, W).backward(go)
        return x.grad.detach().clone()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()                      # also fills the eager cache of the stacked weights
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    m.zero_grad(set_to_none=True)
    x.grad = None
    print("packed backward: capture", flush=True)
    with torch.cuda.graph(graph):
        m(x, W).backward(go)
    gx = x.grad
    for rep in range(3):
        with torch.no_grad():
            for p in (m.q_proj.weight, m.k_proj.weight, m.v_proj.weight):
                p.mul_(1.0 + 0.25 * (rep + 1))
        gx.zero_()
        torch.cuda.synchronize()
        print(f"packed backward: replay {rep}", flush=True)
        graph.replay()
        torch.cuda.synchronize()
        got = gx.clone()
        want = step()                   # eager, on the updated weights (rebinds x.grad; the graph keeps gx)
        torch.cuda.synchronize()
        assert torch.equal(got, want), rep


def test_empty_input():
    """No rows: the projections come back empty, the weight and bias gradients as zeros."""
    from rfa_amd import rfa_hip
    H, d, D, E = 2, 64, 64, 128
    x = torch.empty(0, 3, E, dtype=torch.float16).cuda()
    ws = [torch.randn(H * d, E).half().cuda() for _ in range(2)]
    wf = torch.randn(H, D, d).half().cuda()
    ys, phis = rfa_hip.project_feature_map(x, ws, [None, None], [True, False], wf, H, O.SCALE)
    assert ys[0].shape == (0, 3, H, d) and phis[0].shape == (0, 3, H, 2 * D) and phis[1] is None
    dws, dbs = rfa_hip.linear_weight_grad(x.view(0, E), [torch.empty(0, H * d, dtype=torch.float16).cuda()], [True])
    assert dws[0].shape == (H * d, E) and (dws[0] == 0).all() and (dbs[0] == 0).all()
