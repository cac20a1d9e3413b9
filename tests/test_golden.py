"""Golden vectors: the oracle must keep reproducing tests/golden/rfa_small.npz
(CPU), and the HIP path must reproduce it on the GPU."""
import os

import numpy as np
import pytest
import torch

from oracle import rfa_oracle as O

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "rfa_small.npz")


@pytest.fixture(scope="module")
def gold():
    with np.load(PATH, allow_pickle=False) as f:
        return {k: torch.from_numpy(f[k]) for k in f.files}


def _rel(a, b):
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


def test_oracle_reproduces_golden(gold):
    T, S, B, H, d, D = gold["dims"].tolist()
    N = B * H
    f = lambda k: gold[k].double()
    assert torch.allclose(O.random_project(f("q"), f("W")), f("phi_q"), atol=1e-7)
    assert torch.equal(O.random_project(f("k"), f("W")).half(), gold["phi_k16"])
    cq, ck, cv, cg = (f(k).reshape(T, N, -1) for k in ("phi_q16", "phi_k16", "v", "g"))
    assert torch.allclose(O.causal_forward_chunked(cq, ck, cv, chunk=16), f("causal_out"), atol=1e-6)
    for got, key in zip(O.causal_backward_chunked(cq, ck, cv, cg, chunk=16), ("causal_dq", "causal_dk", "causal_dv")):
        assert torch.allclose(got, f(key), atol=1e-5, rtol=1e-5), key
    s, z = O.cross_state(f("phi_ks16"), f("vs"), gold["mask"])
    assert torch.allclose(s, f("cross_s"), atol=1e-6) and torch.allclose(z, f("cross_z"), atol=1e-6)
    assert torch.allclose(O.cross_readout(f("phi_q16"), s, z), f("cross_out"), atol=1e-6)
    dx, dW = O.random_project_backward(f("q"), f("W"), f("gphi"))
    assert torch.allclose(dx, f("phi_dx"), atol=1e-6) and torch.allclose(dW, f("phi_dW"), atol=1e-5)
    _, ps, pz = O.causal_forward_loop(cq[:30], ck[:30], cv[:30])
    assert torch.allclose(ps, f("prefill30_s"), atol=1e-6) and torch.allclose(pz, f("prefill30_z"), atol=1e-6)


@pytest.mark.gpu
def test_hip_path_reproduces_golden(gold):
    from rfa_amd import rfa_hip
    T, S, B, H, d, D = gold["dims"].tolist()
    N, K = B * H, 2 * D
    c = lambda k: gold[k].cuda().contiguous()
    phi = rfa_hip.feature_map_forward(c("q"), c("W"), O.SCALE)
    assert (phi.float().cpu() - gold["phi_q"]).abs().max().item() <= 3e-4
    dx, dW = rfa_hip.feature_map_backward(c("q"), c("W"), c("gphi"), O.SCALE)
    assert _rel(dx.float().cpu(), gold["phi_dx"]) <= 1e-2 and _rel(dW.cpu(), gold["phi_dW"]) <= 1e-2
    cq, ck = c("phi_q16").view(T, N, K), c("phi_k16").view(T, N, K)
    cv, cg = c("v").view(T, N, d), c("g").view(T, N, d)
    out = rfa_hip.forward(cq, ck, cv)
    assert (out.float().cpu() - gold["causal_out"]).abs().max().item() <= 2e-3
    for got, key in zip(rfa_hip.backward(cq, ck, cv, cg), ("causal_dq", "causal_dk", "causal_dv")):
        assert _rel(got.float().cpu(), gold[key]) <= 1e-2, key
    pad = gold["mask"].t().contiguous().cuda()
    s, z = rfa_hip.cross_state(c("phi_ks16"), c("vs"), pad)
    assert _rel(s.cpu(), gold["cross_s"]) <= 1e-3 and _rel(z.cpu(), gold["cross_z"]) <= 1e-3
    xo = rfa_hip.cross_readout(c("phi_q16"), s, z)
    assert (xo.float().cpu() - gold["cross_out"]).abs().max().item() <= 2e-3
    dq, ds, dz = rfa_hip.cross_readout_backward(c("phi_q16"), s, z, c("g"))
    dk, dv = rfa_hip.cross_state_backward(c("phi_ks16"), c("vs"), ds, dz, pad)
    for got, key in ((dq, "cross_dq"), (ds, "cross_ds"), (dz, "cross_dz"), (dk, "cross_dk"), (dv, "cross_dv")):
        assert _rel(got.float().cpu(), gold[key]) <= 1e-2, key
    # decode from the stored 30-step prefill state
    s0, z0 = c("prefill30_s"), c("prefill30_z")
    dec = rfa_hip.incremental(cq[30:].contiguous(), ck[30:].contiguous(), cv[30:].contiguous(), s0, z0)
    assert (dec.float().cpu() - gold["causal_out"][30:]).abs().max().item() <= 2e-3
