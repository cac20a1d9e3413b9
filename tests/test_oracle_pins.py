"""Pins for the CPU oracle: every check here is independent of the formula it
pins (another algebraic form, a closed-form answer, autograd, a library
routine, brute force, or a statistical identity)."""
import math

import numpy as np
import pytest
import torch

from oracle import rfa_oracle as O

DT = torch.float64


def _rand(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=DT) * scale


def _phi_like(T, N, K, seed):
    # signed features of magnitude ~0.1 with a positive-mean half, like phi
    x = _rand(T, N, K, seed=seed) * 0.1
    x[..., K // 2:] = x[..., K // 2:].abs()
    return x


# ---------------------------------------------------------------- feature map
def test_phi_norm_invariant():
    H, D, d = 3, 16, 8
    x = _rand(5, 2, H, d, seed=1)
    W = _rand(H, D, d, seed=2)
    phi = O.random_project(x, W)
    assert torch.allclose((phi ** 2).sum(-1), torch.full((5, 2, H), O.SCALE ** 2 * D, dtype=DT), atol=1e-12)


def test_phi_layout_known_answer():
    # W = first D rows of identity, x = a * e_j  ->  u_j = a/(a+1e-3), others 0
    H, D, d = 1, 4, 6
    W = torch.eye(d, dtype=DT)[:D].unsqueeze(0)
    a = 2.5
    x = torch.zeros(1, 1, H, d, dtype=DT)
    x[..., 2] = a
    phi = O.random_project(x, W)[0, 0, 0]
    u = a / (a + 1e-3)
    want = torch.tensor([0, 0, math.sin(u), 0, 1, 1, math.cos(u), 1], dtype=DT) * 0.1
    assert torch.allclose(phi, want, atol=1e-15)


def test_phi_zero_input_is_finite():
    W = _rand(2, 4, 8, seed=3)
    phi = O.random_project(torch.zeros(1, 1, 2, 8, dtype=DT), W)
    want = torch.cat([torch.zeros(4), torch.full((4,), 0.1)]).to(DT)
    assert torch.allclose(phi[0, 0, 0], want, atol=1e-16)


def test_phi_scale_near_invariance():
    W = _rand(2, 8, 8, seed=4)
    x = _rand(3, 1, 2, 8, seed=5)
    p1 = O.random_project(x, W)
    p2 = O.random_project(x * 1000.0, W)
    # only the +1e-3 in the normaliser distinguishes them
    assert (p1 - p2).abs().max() < 2e-3 * O.SCALE * 4
    assert not torch.equal(p1, p2)


def test_phi_softmax_kernel_monte_carlo():
    # exp(q.k/tau^2) ~= e^{1/tau^2} * phi(q).phi(k) / (scale^2 D)  for unit q,k
    # (reference: construct_random_matrices.py:40-57)
    d, D, tau, b = 16, 4096, 0.9, 64
    g = torch.Generator().manual_seed(7)
    W = torch.randn(1, D, d, generator=g, dtype=DT) / tau
    q = O.unit_rows(torch.randn(b, 1, 1, d, generator=g, dtype=DT))
    k = O.unit_rows(torch.randn(b, 1, 1, d, generator=g, dtype=DT))
    pq, pk = O.random_project(q, W), O.random_project(k, W)
    pred = (pq * pk).sum(-1).flatten() * math.exp(1 / tau ** 2) / (O.SCALE ** 2 * D)
    gold = torch.exp((q * k).sum(-1).flatten() / tau ** 2)
    rel = (pred - gold).norm() / gold.norm()
    assert rel < 0.08   # ~ D^-1/2 scaling, plus the 1e-3 normaliser bias


def test_build_random_matrices():
    W = _rand(2, 3, 4, seed=8)
    sigma = _rand(2, 1, 4, seed=9)
    assert torch.equal(O.build_random_matrices(W, 2.0), W / 2.0)
    got = O.build_random_matrices(W, 0.5, sigma, True)
    for h in range(2):
        for j in range(3):
            assert torch.allclose(got[h, j], sigma[h, 0] * W[h, j] / 0.5)


def test_phi_backward_vs_autograd():
    x = _rand(4, 2, 3, 8, seed=10).requires_grad_(True)
    W = _rand(3, 5, 8, seed=11).requires_grad_(True)
    g = _rand(4, 2, 3, 10, seed=12)
    phi = O.random_project(x, W)
    dx_a, dW_a = torch.autograd.grad(phi, (x, W), g)
    dx, dW = O.random_project_backward(x.detach(), W.detach(), g)
    assert torch.allclose(dx, dx_a, atol=1e-12)
    assert torch.allclose(dW, dW_a, atol=1e-12)


# ------------------------------------------------------------- causal forward
@pytest.mark.parametrize("T,N,K,d,chunk", [(1, 1, 4, 3, 64), (7, 2, 8, 5, 3), (37, 3, 16, 8, 16), (64, 2, 8, 4, 64), (130, 1, 8, 4, 64)])
def test_causal_forms_agree(T, N, K, d, chunk):
    q, k = _phi_like(T, N, K, 20), _phi_like(T, N, K, 21)
    v = _rand(T, N, d, seed=22)
    a = O.causal_forward_cumsum(q, k, v)
    b, s, z = O.causal_forward_loop(q, k, v)
    c = O.causal_forward_quadratic(q, k, v)
    e = O.causal_forward_chunked(q, k, v, chunk=chunk)
    for other in (b, c, e):
        assert torch.allclose(a, other, atol=1e-11, rtol=1e-11)
    assert torch.allclose(s, torch.einsum("tnk,tnd->nkd", k, v), atol=1e-12)
    assert torch.allclose(z, k.sum(0), atol=1e-12)


def test_causal_first_row_closed_form():
    # phi.phi <= scale^2 D < 1  =>  clamp active at t=0  =>  out_0 = (q0.k0) v0
    q, k = _phi_like(5, 3, 8, 30), _phi_like(5, 3, 8, 31)
    v = _rand(5, 3, 4, seed=32)
    out = O.causal_forward_cumsum(q, k, v)
    want = (q[0] * k[0]).sum(-1, keepdim=True) * v[0]
    assert torch.allclose(out[0], want, atol=1e-14)


def test_causal_constant_value_when_unclamped():
    T, N, K = 12, 2, 8
    q = torch.full((T, N, K), 0.5, dtype=DT)
    k = torch.full((T, N, K), 0.5, dtype=DT)       # q.k = 2 > 1 from t=0
    v = torch.full((T, N, 3), 1.75, dtype=DT)
    out = O.causal_forward_cumsum(q, k, v)
    assert torch.allclose(out, v, atol=1e-13)


def test_causal_prefix_property():
    q, k = _phi_like(20, 2, 8, 40), _phi_like(20, 2, 8, 41)
    v = _rand(20, 2, 4, seed=42)
    full = O.causal_forward_cumsum(q, k, v)
    part = O.causal_forward_cumsum(q[:11], k[:11], v[:11])
    assert torch.allclose(full[:11], part, atol=1e-13)


def test_causal_zeroed_key_equals_deleted_key():
    q, k = _phi_like(9, 1, 8, 50), _phi_like(9, 1, 8, 51)
    v = _rand(9, 1, 4, seed=52)
    k2 = k.clone()
    k2[4] = 0
    out = O.causal_forward_cumsum(q, k2, v)
    keep = [0, 1, 2, 3, 5, 6, 7, 8]
    out_del = O.causal_forward_cumsum(q[keep], k[keep], v[keep])
    # rows after the deleted key see the same prefix sums
    assert torch.allclose(out[5:], out_del[4:], atol=1e-13)


# ------------------------------------------------------------ causal backward
def _bwd_inputs(T, N, K, d, seed):
    q, k = _phi_like(T, N, K, seed), _phi_like(T, N, K, seed + 1)
    v, g = _rand(T, N, d, seed=seed + 2), _rand(T, N, d, seed=seed + 3)
    return q, k, v, g


@pytest.mark.parametrize("T,N,K,d", [(6, 2, 8, 4), (33, 2, 16, 8), (70, 1, 8, 4)])
def test_causal_backward_vs_autograd(T, N, K, d):
    q, k, v, g = _bwd_inputs(T, N, K, d, 60)
    qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
    out = O.causal_forward_cumsum(qa, ka, va)
    want = torch.autograd.grad(out, (qa, ka, va), g)
    got = O.causal_backward_cumsum(q, k, v, g)
    got_c = O.causal_backward_chunked(q, k, v, g, chunk=16)
    for a, b, c in zip(want, got, got_c):
        assert torch.allclose(a, b, atol=1e-11, rtol=1e-10)
        assert torch.allclose(a, c, atol=1e-11, rtol=1e-10)


def test_causal_backward_autograd_of_loop_and_quadratic_forms():
    q, k, v, g = _bwd_inputs(10, 2, 8, 4, 70)
    got = O.causal_backward_cumsum(q, k, v, g)
    for fwd in (lambda a, b, c: O.causal_forward_loop(a, b, c)[0], O.causal_forward_quadratic):
        qa, ka, va = (t.clone().requires_grad_(True) for t in (q, k, v))
        want = torch.autograd.grad(fwd(qa, ka, va), (qa, ka, va), g)
        for a, b in zip(want, got):
            assert torch.allclose(a, b, atol=1e-11, rtol=1e-10)


def test_causal_backward_finite_differences():
    q, k, v, g = _bwd_inputs(5, 1, 4, 3, 80)
    q = q + 0.6   # keep q.z well away from the clamp kink
    k = k.abs() + 0.4
    dq, dk, dv = O.causal_backward_cumsum(q, k, v, g)
    h = 1e-6
    for name, x, dx in (("q", q, dq), ("k", k, dk), ("v", v, dv)):
        for idx in [(0, 0, 0), (2, 0, 1), (4, 0, 2)]:
            xp, xm = x.clone(), x.clone()
            xp[idx] += h
            xm[idx] -= h
            args_p = {"q": q, "k": k, "v": v}
            args_m = dict(args_p)
            args_p[name], args_m[name] = xp, xm
            fp = (O.causal_forward_cumsum(**args_p) * g).sum()
            fm = (O.causal_forward_cumsum(**args_m) * g).sum()
            assert abs((fp - fm) / (2 * h) - dx[idx]) < 1e-6


def test_causal_backward_clamped_rows_have_zero_denominator_grad():
    # where the clamp is active the output is linear in q: dq_t = sum_s<=t (g_t.v_s) k_s
    q, k, v, g = _bwd_inputs(3, 1, 8, 4, 90)
    q, k = q * 0.1, k * 0.1        # all rows clamped
    dq, _, _ = O.causal_backward_cumsum(q, k, v, g)
    for t in range(3):
        want = sum((g[t, 0] * v[s, 0]).sum() * k[s, 0] for s in range(t + 1))
        assert torch.allclose(dq[t, 0], want, atol=1e-14)


# --------------------------------------------------------------------- decode
def test_decode_steps_equal_causal_rows_and_prefill_handoff():
    T, N, K, d = 14, 3, 8, 4
    q, k = _phi_like(T, N, K, 100), _phi_like(T, N, K, 101)
    v = _rand(T, N, d, seed=102)
    full = O.causal_forward_cumsum(q, k, v)
    _, s, z = O.causal_forward_loop(q[:9], k[:9], v[:9])
    for t in range(9, T):
        out, s, z = O.incremental_step(q[t], k[t], v[t], s, z)
        assert torch.allclose(out, full[t], atol=1e-13)
    assert torch.allclose(s, torch.einsum("tnk,tnd->nkd", k, v), atol=1e-12)
    assert torch.allclose(z, k.sum(0), atol=1e-12)


# ---------------------------------------------------------------------- cross
def test_cross_is_matmul_and_matches_last_causal_row():
    S, B, H, K, d = 11, 2, 2, 8, 4
    pk = _phi_like(S, B * H, K, 110).view(S, B, H, K)
    pq = _phi_like(S, B * H, K, 111).view(S, B, H, K)
    v = _rand(S, B, H, d, seed=112)
    s, z = O.cross_state(pk, v)
    for b in range(B):
        for h in range(H):
            assert torch.allclose(s[b, h], pk[:, b, h].T @ v[:, b, h], atol=1e-13)
    out = O.cross_readout(pq, s, z)
    causal = O.causal_forward_cumsum(pq.reshape(S, B * H, K), pk.reshape(S, B * H, K), v.reshape(S, B * H, d))
    qz_last = (pq[-1] * z).sum(-1)
    assert (qz_last > 0).all()      # abs is a no-op here, so the two must agree
    assert torch.allclose(out[-1].reshape(B * H, d), causal[-1], atol=1e-13)


def test_cross_abs_on_negative_denominator():
    pq = torch.tensor([[[[-3.0, 0.0]]]], dtype=DT)       # [1,1,1,2]
    s = torch.tensor([[[[2.0], [5.0]]]], dtype=DT)       # [1,1,2,1]
    z = torch.tensor([[[1.0, 7.0]]], dtype=DT)
    out = O.cross_readout(pq, s, z)
    assert torch.allclose(out, torch.tensor([[[[-6.0 / 3.0]]]], dtype=DT))


def test_cross_mask_equals_truncation():
    S, B, H, K, d = 9, 2, 1, 8, 4
    pk = _phi_like(S, B * H, K, 120).view(S, B, H, K)
    v = _rand(S, B, H, d, seed=121)
    lens = [5, 9]
    mask = torch.zeros(S, B, dtype=torch.bool)
    for b, L in enumerate(lens):
        mask[L:, b] = True
    s, z = O.cross_state(pk, v, mask)
    for b, L in enumerate(lens):
        sb, zb = O.cross_state(pk[:L, b:b + 1], v[:L, b:b + 1])
        assert torch.allclose(s[b], sb[0], atol=1e-13)
        assert torch.allclose(z[b], zb[0], atol=1e-13)


def test_cross_backward_vs_autograd():
    S, T, B, H, K, d = 7, 5, 2, 2, 8, 4
    pk = _phi_like(S, B * H, K, 130).view(S, B, H, K)
    pq = (_phi_like(T, B * H, K, 131) * 3).view(T, B, H, K)
    pq[0] = -pq[0]                     # exercise the sign branch
    v = _rand(S, B, H, d, seed=132)
    g = _rand(T, B, H, d, seed=133)
    mask = torch.zeros(S, B, dtype=torch.bool)
    mask[5:, 0] = True
    pka, va, pqa = (t.clone().requires_grad_(True) for t in (pk, v, pq))
    s, z = O.cross_state(pka, va, mask)
    out = O.cross_readout(pqa, s, z)
    want = torch.autograd.grad(out, (pqa, pka, va), g)
    s0, z0 = O.cross_state(pk, v, mask)
    dpq, ds, dz = O.cross_readout_backward(pq, s0, z0, g)
    dpk, dv = O.cross_state_backward(pk, v, ds, dz, mask)
    for a, b in zip(want, (dpq, dpk, dv)):
        assert torch.allclose(a, b, atol=1e-11, rtol=1e-10)


def test_gradcheck_small():
    q, k, v, _ = _bwd_inputs(4, 1, 4, 2, 140)
    q, k = (q + 0.7).requires_grad_(True), (k.abs() + 0.5).requires_grad_(True)
    v = v.requires_grad_(True)
    assert torch.autograd.gradcheck(O.causal_forward_chunked, (q, k, v, 2), eps=1e-6, atol=1e-5)


def test_masked_rfa_oracle_against_explicit_loops():
    """The masked quadratic form, element by element: weights over the unmasked, unpadded keys,
    divided by |their sum| clamped at 1e-3 (sign kept in the numerator), including a row whose
    weights sum to a negative number and a row whose sum is below the clamp."""
    g = torch.Generator().manual_seed(1)
    T, B, H, K, d = 6, 2, 2, 8, 4
    pq = torch.rand(T, B, H, K, generator=g, dtype=torch.float64) - 0.3
    pk = torch.rand(T, B, H, K, generator=g, dtype=torch.float64) - 0.3
    pq[2, 0, 0] = -pq[2, 0, 0].abs()          # a negative row sum
    pk[:, 0, 0] = pk[:, 0, 0].abs()
    pq[3, 1, 1] *= 1e-5                        # a row sum below the clamp
    v = torch.randn(T, B, H, d, generator=g, dtype=torch.float64)
    causal = torch.triu(torch.full((T, T), float("-inf"), dtype=torch.float64), 1)
    pad = torch.zeros(B, T, dtype=torch.uint8)
    pad[1, 4:] = 1
    out = O.masked_rfa(pq, pk, v, pad, causal)
    seen_negative = seen_clamped = False
    for b in range(B):
        for h in range(H):
            for t in range(T):
                keys = [s_ for s_ in range(t + 1) if not pad[b, s_]]
                wts = torch.stack([(pq[t, b, h] * pk[s_, b, h]).sum() for s_ in keys])
                rs = wts.sum()
                seen_negative |= bool(rs < -1e-3)
                seen_clamped |= bool(rs.abs() < 1e-3)
                want = (wts[:, None] * torch.stack([v[s_, b, h] for s_ in keys])).sum(0) / max(abs(rs.item()), 1e-3)
                assert torch.allclose(out[t, b, h], want, atol=1e-12)
    assert seen_negative and seen_clamped
    # a 0-dim / absent mask changes nothing; without any mask every key counts
    full = O.masked_rfa(pq, pk, v)
    w = torch.einsum("tbhk,sbhk->bhts", pq, pk)
    assert torch.allclose(full, torch.einsum("bhts,sbhd->tbhd", w / w.sum(-1, keepdim=True).abs().clamp(1e-3), v))


def test_masked_rfa_oracle_equals_scan_when_denominators_agree():
    """With the causal mask and row sums >= 1 the two normalisers coincide:
    masked quadratic form == causal scan (rfa.py:57-63)."""
    T, N, K, d = 12, 3, 8, 4
    g = torch.Generator().manual_seed(5)
    q = torch.rand(T, N, K, generator=g, dtype=torch.float64) + 0.5
    k = torch.rand(T, N, K, generator=g, dtype=torch.float64) + 0.5     # q.k > 1 for every pair
    v = torch.randn(T, N, d, generator=g, dtype=torch.float64)
    causal = torch.triu(torch.full((T, T), float("-inf"), dtype=torch.float64), 1)
    a = O.masked_rfa(q.view(T, N, 1, K), k.view(T, N, 1, K), v.view(T, N, 1, d), None, causal).view(T, N, d)
    assert torch.allclose(a, O.causal_forward_cumsum(q, k, v), atol=1e-12)
