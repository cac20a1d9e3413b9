"""Writes tests/golden/rfa_small.npz: seeded fp16 inputs of a miniature workload and
the float64 oracle outputs for every part of the path.

    python tests/golden/make_golden.py

The reference ships no golden vectors for this path and cannot be imported
(missing modules, top-level import of its CUDA extension), so these vectors come
from the pinned CPU oracle (oracle/rfa_oracle.py, pinned by tests/test_oracle_pins.py).
They freeze the oracle and give the GPU tests fixed expected values.
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import rfa_oracle as O  # noqa: E402


def main():
    T, S, B, H, d, D = 48, 40, 1, 2, 64, 64
    N, K = B * H, 2 * D
    q, k, v, g = O.make_qkv(T, B, H, d, seed=4242)
    ks, vs = O.make_qkv(S, B, H, d, seed=4243)[1:3]
    W = O.make_w(d, D, H).to(torch.float16)
    f64 = lambda t: t.to(torch.float64)
    pq, pk = O.random_project(f64(q), f64(W)), O.random_project(f64(k), f64(W))
    pq16, pk16 = pq.to(torch.float16), pk.to(torch.float16)
    cq, ck, cv, cg = (f64(t).reshape(T, N, -1) for t in (pq16, pk16, v, g))
    out = O.causal_forward_cumsum(cq, ck, cv)
    dq, dk, dv = O.causal_backward_cumsum(cq, ck, cv, cg)
    gphi = (f64(g).repeat(1, 1, 1, 2) * 0.5).to(torch.float16)
    dx, dW = O.random_project_backward(f64(q), f64(W), f64(gphi))
    pks16 = O.random_project(f64(ks), f64(W)).to(torch.float16)
    mask = torch.zeros(S, B, dtype=torch.bool)
    mask[33:, 0] = True
    s, z = O.cross_state(f64(pks16), f64(vs), mask)
    xo = O.cross_readout(f64(pq16), s, z)
    xdq, xds, xdz = O.cross_readout_backward(f64(pq16), s, z, f64(g))
    xdk, xdv = O.cross_state_backward(f64(pks16), f64(vs), xds, xdz, mask)
    _, st_s, st_z = O.causal_forward_loop(cq[:30], ck[:30], cv[:30])
    n = lambda t: (t.to(torch.float32) if t.dtype == torch.float64 else t).numpy()
    np.savez_compressed(
        os.path.join(os.path.dirname(os.path.abspath(__file__)), "rfa_small.npz"),
        dims=np.array([T, S, B, H, d, D]),
        q=n(q), k=n(k), v=n(v), g=n(g), ks=n(ks), vs=n(vs), W=n(W), mask=n(mask), gphi=n(gphi),
        phi_q=n(pq), phi_k=n(pk), phi_q16=n(pq16), phi_k16=n(pk16), phi_ks16=n(pks16),
        phi_dx=n(dx), phi_dW=n(dW),
        causal_out=n(out), causal_dq=n(dq), causal_dk=n(dk), causal_dv=n(dv),
        cross_s=n(s), cross_z=n(z), cross_out=n(xo), cross_dq=n(xdq), cross_ds=n(xds), cross_dz=n(xdz),
        cross_dk=n(xdk), cross_dv=n(xdv),
        prefill30_s=n(st_s), prefill30_z=n(st_z))


if __name__ == "__main__":
    main()
