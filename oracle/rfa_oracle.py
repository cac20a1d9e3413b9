"""CPU oracle for the Random Feature Attention kernel path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this module;
it is used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / the timed CPU baseline.

Every function restates, in plain ``torch`` on CPU tensors (the same ATen
routines the reference's Python path calls), one formula of the reference and
cites the reference lines it follows.  Functions work in whatever floating
dtype they are given (tests use float64, the fp32 "reference" of the parity
gates uses float32).

Pinning status (see tests/test_oracle_*.py): every function below is pinned by
checks that do not retype its formula -- mutual agreement of independent
forms (cumulative-sum, per-step loop, chunked, quadratic brute force),
closed-form known answers (element-by-element loops for the masked quadratic form), ``torch.autograd`` / ``gradcheck`` for the
backward formulas, library ``matmul`` for the contractions, and the
softmax-kernel Monte-Carlo identity for the feature map.  The reference ships
no golden vectors for this path, so none are checked.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
from torch import Tensor

EPS = 1.0     # reference: random_feature_attention/rfa.py:17, utils.py:9
SCALE = 0.1   # reference: random_feature_attention/utils.py:10


# --------------------------------------------------------------------------
# feature map
# --------------------------------------------------------------------------
def build_random_matrices(random_matrices: Tensor, tau: float,
                          sigma: Optional[Tensor] = None,
                          reparam_proj: bool = False) -> Tensor:
    """W' = (sigma * W if reparam) / tau.  reference: utils.py:90-97."""
    if reparam_proj:
        random_matrices = sigma * random_matrices
    return random_matrices / tau


def normalize(x: Tensor) -> Tuple[Tensor, Tensor]:
    """x / (||x||_2 + 1e-3) over the last dim.  reference: utils.py:100-102."""
    norm = torch.linalg.vector_norm(x, ord=2, dim=-1, keepdim=True)
    return x / (norm + 1e-3), norm


def random_project(x: Tensor, random_matrices: Tensor, scale: float = SCALE) -> Tensor:
    """phi(x) = scale * [sin(W x^), cos(W x^)], sin block first.

    x: [L, B, H, d]; random_matrices: [H, D, d] -> [L, B, H, 2D].
    reference: utils.py:105-120.
    """
    xh, _ = normalize(x)
    u = torch.einsum("sbhd,hkd->sbhk", xh, random_matrices)
    return torch.cat([torch.sin(u), torch.cos(u)], dim=-1) * scale


# --------------------------------------------------------------------------
# causal attention, forward: four independent forms
# --------------------------------------------------------------------------
def causal_forward_cumsum(q: Tensor, k: Tensor, v: Tensor) -> Tensor:
    """Cumulative-sum form.  q,k: [T, N, K]; v: [T, N, d] -> [T, N, d].

    reference: rfa.py:46-64 (RFA.forward_torch).  Materialises [T, N, K, d].
    """
    s = torch.cumsum(torch.einsum("tbk,tbd->tbkd", k, v), dim=0)
    qs = torch.einsum("tbkd,tbk->tbd", s, q)
    z = torch.cumsum(k, dim=0)
    qz = torch.einsum("tbk,tbk->tb", q, z).clamp_min(EPS)
    return qs / qz.unsqueeze(-1)


def causal_forward_loop(q: Tensor, k: Tensor, v: Tensor,
                        s: Optional[Tensor] = None, z: Optional[Tensor] = None):
    """Per-step recurrence.  Returns (attn [T,N,d], s [N,K,d], z [N,K]).

    reference: causal_attention.py:42-50 (incremental_rfa loop body), with the
    (bsz, heads) axes flattened to N.
    """
    T, N, K = q.shape
    d = v.shape[-1]
    if s is None:
        s = torch.zeros(N, K, d, dtype=v.dtype)
        z = torch.zeros(N, K, dtype=v.dtype)
    outs = []
    for t in range(T):
        s = s + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        z = z + k[t]
        qs = torch.einsum("nk,nkd->nd", q[t], s)
        qz = (q[t] * z).sum(-1).clamp_min(EPS)
        outs.append(qs / qz.unsqueeze(-1))
    out = torch.stack(outs, 0) if outs else torch.zeros(0, N, d, dtype=v.dtype)
    return out, s, z


def causal_forward_quadratic(q: Tensor, k: Tensor, v: Tensor) -> Tensor:
    """Brute force: tril(Q K^T) V / max(rowsum(tril(Q K^T)), 1).

    Algebraically identical to rfa.py:57-63 (the inclusive cumsum is a
    lower-triangular mask with the diagonal kept); O(T^2), tiny T only.
    """
    T = q.shape[0]
    a = torch.einsum("tnk,snk->nts", q, k)
    a = a * torch.tril(torch.ones(T, T, dtype=q.dtype))
    num = torch.einsum("nts,snd->tnd", a, v)
    den = a.sum(-1).transpose(0, 1).clamp_min(EPS)
    return num / den.unsqueeze(-1)


def masked_rfa(phi_q: Tensor, phi_k: Tensor, v: Tensor, key_padding_mask: Optional[Tensor] = None,
               attn_mask: Optional[Tensor] = None) -> Tensor:
    """Quadratic form with explicit masks (causal_attention.py:57-109, utils.py:123-130).

    phi_q, phi_k: [T, B, H, K]; v: [T, B, H, d]; key_padding_mask: [B, T], non-zero = padded key;
    attn_mask: [T, T], entries < 0 are masked.  Weights are zeroed where masked, then divided by
    |row sum|.clamp(1e-3); returns [T, B, H, d].  (The reference casts the normalised weights back
    to the input dtype before applying them to v; here everything stays in the given dtype.)
    """
    w = torch.einsum("tbhk,sbhk->bhts", phi_q, phi_k)
    if key_padding_mask is not None:
        w = w.masked_fill(key_padding_mask.to(torch.bool)[:, None, None, :], 0.0)
    if attn_mask is not None:
        w = w.masked_fill((attn_mask < 0.0)[None, None], 0.0)
    w = w / w.sum(-1, keepdim=True).abs().clamp(1e-3)
    return torch.einsum("bhts,sbhd->tbhd", w, v)


def causal_forward_chunked(q: Tensor, k: Tensor, v: Tensor, chunk: int = 64) -> Tensor:
    """Chunked scan: intra-chunk masked product plus carried state.

    Same mathematics as rfa.py:46-64 regrouped by chunks of ``chunk`` steps;
    memory O(N K d).  This is the algorithm the HIP kernels implement and the
    form used for shapes whose [T,N,K,d] tensor does not fit in memory.
    """
    T, N, K = q.shape
    d = v.shape[-1]
    S = torch.zeros(N, K, d, dtype=q.dtype)
    z = torch.zeros(N, K, dtype=q.dtype)
    out = torch.empty(T, N, d, dtype=q.dtype)
    for t0 in range(0, T, chunk):
        t1 = min(T, t0 + chunk)
        qc, kc, vc = q[t0:t1], k[t0:t1], v[t0:t1]
        C = t1 - t0
        a = torch.einsum("tnk,snk->nts", qc, kc) * torch.tril(torch.ones(C, C, dtype=q.dtype))
        num = torch.einsum("nts,snd->tnd", a, vc) + torch.einsum("tnk,nkd->tnd", qc, S)
        den = a.sum(-1).transpose(0, 1) + torch.einsum("tnk,nk->tn", qc, z)
        out[t0:t1] = num / den.clamp_min(EPS).unsqueeze(-1)
        S = S + torch.einsum("snk,snd->nkd", kc, vc)
        z = z + kc.sum(0)
    return out


# --------------------------------------------------------------------------
# causal attention, backward
# --------------------------------------------------------------------------
def _reverse_cumsum(x: Tensor, dim: int) -> Tensor:
    """reference: rfa.py:20-21."""
    return torch.flip(torch.cumsum(torch.flip(x, [dim]), dim), [dim])


def causal_backward_cumsum(q: Tensor, k: Tensor, v: Tensor, grad_attn: Tensor):
    """Closed-form gradients (dq, dk, dv).  reference: rfa.py:66-103.

    The mask on grad_qz is (qz > EPS) evaluated on the *clamped* qz with a
    strict comparison (rfa.py:91; cuda/utils.cu:37-40).
    """
    s = torch.cumsum(torch.einsum("tbk,tbd->tbkd", k, v), dim=0)
    qs = torch.einsum("tbkd,tbk->tbd", s, q)
    z = torch.cumsum(k, dim=0)
    qz = torch.einsum("tbk,tbk->tb", q, z).clamp_min(EPS)

    grad_qs = grad_attn / qz.unsqueeze(-1)
    grad_qz = -torch.einsum("tbd,tbd->tb", grad_attn, qs) / (qz ** 2)
    grad_qz = grad_qz * (qz > EPS)

    grad_q = torch.einsum("tbd,tbkd->tbk", grad_qs, s) + grad_qz.unsqueeze(-1) * z
    grad_s = _reverse_cumsum(torch.einsum("tbk,tbd->tbkd", q, grad_qs), 0)
    grad_k = torch.einsum("tbkd,tbd->tbk", grad_s, v)
    grad_v = torch.einsum("tbkd,tbk->tbd", grad_s, k)
    grad_k = grad_k + _reverse_cumsum(q * grad_qz.unsqueeze(-1), 0)
    return grad_q, grad_k, grad_v


def causal_backward_chunked(q: Tensor, k: Tensor, v: Tensor, grad_attn: Tensor,
                            chunk: int = 64):
    """rfa.py:66-103 regrouped by chunks (forward sweep for dq, reverse sweep
    for dk/dv); memory O(N K d).  Used where the cumsum form does not fit."""
    T, N, K = q.shape
    d = v.shape[-1]
    dt = q.dtype
    S = torch.zeros(N, K, d, dtype=dt)
    z = torch.zeros(N, K, dtype=dt)
    dq = torch.empty_like(q)
    gs_all = torch.empty_like(grad_attn)
    gz_all = torch.empty(T, N, dtype=dt)
    for t0 in range(0, T, chunk):
        t1 = min(T, t0 + chunk)
        qc, kc, vc, gc = q[t0:t1], k[t0:t1], v[t0:t1], grad_attn[t0:t1]
        C = t1 - t0
        tri = torch.tril(torch.ones(C, C, dtype=dt))
        a = torch.einsum("tnk,snk->nts", qc, kc) * tri
        num = torch.einsum("nts,snd->tnd", a, vc) + torch.einsum("tnk,nkd->tnd", qc, S)
        den_raw = a.sum(-1).transpose(0, 1) + torch.einsum("tnk,nk->tn", qc, z)
        den = den_raw.clamp_min(EPS)
        gs = gc / den.unsqueeze(-1)
        gz = -(gc * num).sum(-1) / den ** 2 * (den > EPS)
        p = (torch.einsum("tnd,snd->nts", gs, vc) + gz.transpose(0, 1).unsqueeze(-1)) * tri
        dq[t0:t1] = (torch.einsum("nts,snk->tnk", p, kc)
                     + torch.einsum("tnd,nkd->tnk", gs, S)
                     + gz.unsqueeze(-1) * z.unsqueeze(0))
        gs_all[t0:t1] = gs
        gz_all[t0:t1] = gz
        S = S + torch.einsum("snk,snd->nkd", kc, vc)
        z = z + kc.sum(0)
    R = torch.zeros(N, K, d, dtype=dt)
    r = torch.zeros(N, K, dtype=dt)
    dk = torch.empty_like(k)
    dv = torch.empty_like(v)
    starts = list(range(0, T, chunk))
    for t0 in reversed(starts):
        t1 = min(T, t0 + chunk)
        qc, kc, vc = q[t0:t1], k[t0:t1], v[t0:t1]
        gs, gz = gs_all[t0:t1], gz_all[t0:t1]
        C = t1 - t0
        tri = torch.tril(torch.ones(C, C, dtype=dt))
        a = torch.einsum("tnk,snk->nts", qc, kc) * tri
        p = (torch.einsum("tnd,snd->nts", gs, vc) + gz.transpose(0, 1).unsqueeze(-1)) * tri
        dk[t0:t1] = (torch.einsum("nts,tnk->snk", p, qc)
                     + torch.einsum("snd,nkd->snk", vc, R) + r.unsqueeze(0))
        dv[t0:t1] = torch.einsum("nts,tnd->snd", a, gs) + torch.einsum("snk,nkd->snd", kc, R)
        R = R + torch.einsum("tnk,tnd->nkd", qc, gs)
        r = r + torch.einsum("tnk,tn->nk", qc, gz)
    return dq, dk, dv


# --------------------------------------------------------------------------
# incremental decoding
# --------------------------------------------------------------------------
def incremental_step(phi_q: Tensor, phi_k: Tensor, v: Tensor, s: Tensor, z: Tensor):
    """One decode step for all heads.  phi_q, phi_k: [N, K]; v: [N, d];
    s: [N, K, d]; z: [N, K].  Returns (attn [N, d], s', z').

    reference: causal_attention.py:43-50.
    """
    s = s + phi_k.unsqueeze(-1) * v.unsqueeze(-2)
    z = z + phi_k
    qs = torch.einsum("nk,nkd->nd", phi_q, s)
    qz = (phi_q * z).sum(-1).clamp_min(EPS)
    return qs / qz.unsqueeze(-1), s, z


# --------------------------------------------------------------------------
# cross attention
# --------------------------------------------------------------------------
def cross_state(phi_k: Tensor, v: Tensor, mask: Optional[Tensor] = None):
    """S = sum_s phi_k[s] (x) v[s];  z = sum_s phi_k[s], padded positions zeroed.

    phi_k: [S, B, H, K]; v: [S, B, H, d]; mask: bool [S, B] (True = pad).
    Returns s [B, H, K, d], z [B, H, K].  reference: cross_attention.py:97-104.
    """
    if mask is not None:
        phi_k = phi_k.masked_fill(mask.unsqueeze(-1).unsqueeze(-1), 0.0)
    s = torch.einsum("sbhk,sbhd->bhkd", phi_k, v)
    z = phi_k.sum(0)
    return s, z


def cross_readout(phi_q: Tensor, s: Tensor, z: Tensor) -> Tensor:
    """attn = (phi_q S) / max(|phi_q z|, 1).  phi_q: [T, B, H, K] -> [T, B, H, d].

    reference: cross_attention.py:266-269 (note the abs, absent in the causal path).
    """
    qs = torch.einsum("tbhk,bhkd->tbhd", phi_q, s)
    qz = torch.einsum("tbhk,bhk->tbh", phi_q, z).abs().clamp_min(EPS)
    return qs / qz.unsqueeze(-1)


def cross_readout_backward(phi_q: Tensor, s: Tensor, z: Tensor, grad_attn: Tensor):
    """Closed-form gradients of cross_readout: (dphi_q, ds, dz).

    Derived from cross_attention.py:266-269 the way rfa.py:87-101 derives the
    causal ones: with den = max(|qz_raw|, 1),
    d qz_raw = -(g . qs) / den^2 * sign(qz_raw) * [|qz_raw| > 1].
    """
    qs = torch.einsum("tbhk,bhkd->tbhd", phi_q, s)
    qz_raw = torch.einsum("tbhk,bhk->tbh", phi_q, z)
    den = qz_raw.abs().clamp_min(EPS)
    gs = grad_attn / den.unsqueeze(-1)
    gz = -(grad_attn * qs).sum(-1) / den ** 2 * torch.sign(qz_raw) * (qz_raw.abs() > EPS)
    dphi_q = torch.einsum("tbhd,bhkd->tbhk", gs, s) + gz.unsqueeze(-1) * z.unsqueeze(0)
    ds = torch.einsum("tbhk,tbhd->bhkd", phi_q, gs)
    dz = torch.einsum("tbhk,tbh->bhk", phi_q, gz)
    return dphi_q, ds, dz


def cross_state_backward(phi_k: Tensor, v: Tensor, ds: Tensor, dz: Tensor,
                         mask: Optional[Tensor] = None):
    """Gradients of cross_state w.r.t. (phi_k, v) given (ds, dz).

    d phi_k[s] = v[s] . ds^T + dz (zero at padded positions); dv[s] = phi_k[s] . ds.
    """
    dphi_k = torch.einsum("sbhd,bhkd->sbhk", v, ds) + dz.unsqueeze(0)
    pk = phi_k
    if mask is not None:
        m = mask.unsqueeze(-1).unsqueeze(-1)
        dphi_k = dphi_k.masked_fill(m, 0.0)
        pk = phi_k.masked_fill(m, 0.0)
    dv = torch.einsum("sbhk,bhkd->sbhd", pk, ds)
    return dphi_k, dv


# --------------------------------------------------------------------------
# feature-map backward (closed form; pinned against autograd in the tests)
# --------------------------------------------------------------------------
def random_project_backward(x: Tensor, random_matrices: Tensor, grad_phi: Tensor,
                            scale: float = SCALE):
    """Gradients of random_project w.r.t. (x, random_matrices).

    With n = ||x||, xh = x/(n+1e-3), u = W xh:
      du = scale * (cos u * g_sin - sin u * g_cos)
      dW[h] = sum_{s,b} du (x) xh ;  dxh = du W
      dx = dxh/(n+1e-3) - x * (x . dxh) / (n * (n+1e-3)^2)
    (utils.py:100-120 differentiated by hand).
    """
    D = random_matrices.shape[1]
    xh, n = normalize(x)
    u = torch.einsum("sbhd,hkd->sbhk", xh, random_matrices)
    g_sin, g_cos = grad_phi[..., :D], grad_phi[..., D:]
    du = scale * (torch.cos(u) * g_sin - torch.sin(u) * g_cos)
    dW = torch.einsum("sbhk,sbhd->hkd", du, xh)
    dxh = torch.einsum("sbhk,hkd->sbhd", du, random_matrices)
    xdot = (x * dxh).sum(-1, keepdim=True)
    n_safe = torch.where(n > 0, n, torch.ones_like(n))
    dx = dxh / (n + 1e-3) - x * xdot / (n_safe * (n + 1e-3) ** 2)
    return dx, dW


# --------------------------------------------------------------------------
# synthetic workload generator shared by tests, smoke and bench
# --------------------------------------------------------------------------
def make_w(head_dim: int, proj_dim: int, num_heads: int, seed: int = 31415) -> Tensor:
    """Seeded Gaussian random matrix [H, D, d] (one [D, d] draw shared by all
    heads), the stand-in for the absent random_matrices/{d}_{D}.npy blob."""
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(proj_dim, head_dim, generator=g, dtype=torch.float32)
    return w.unsqueeze(0).expand(num_heads, -1, -1).contiguous()


def unit_rows(x: Tensor) -> Tensor:
    return x / torch.linalg.vector_norm(x, dim=-1, keepdim=True)


def make_qkv(T: int, B: int, H: int, d: int, seed: int, n_tensors: int = 4):
    """q,k,v,grad ~ N(0,1) fp32 [T,B,H,d]; q,k unit-normalised per head; all
    rounded to fp16 (returned as fp16 so both sides see identical inputs)."""
    g = torch.Generator().manual_seed(seed)
    xs = [torch.randn(T, B, H, d, generator=g, dtype=torch.float32) for _ in range(n_tensors)]
    xs[0] = unit_rows(xs[0])
    xs[1] = unit_rows(xs[1])
    return [x.to(torch.float16) for x in xs]
