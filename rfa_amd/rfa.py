"""Causal RFA as a torch.autograd.Function over the HIP kernels.

Mirror of random_feature_attention/rfa.py: same names (EPS, reverse_cumsum,
rfa_debug, class RFA with forward_torch / backward_torch / forward_cuda /
backward_cuda / forward / backward), same tensor layout

    q, k: [tgt_len, bsz * num_heads, 2 * proj_dim]   v: [tgt_len, bsz * num_heads, head_dim]

``RFA.apply`` runs the MI355X kernels (rfa_hip.forward / rfa_hip.backward) and
nothing else: CPU tensors raise.  ``forward_torch`` / ``backward_torch`` /
``rfa_debug`` are kept because the reference exposes them as the in-file
formula statement (rfa.py:24-103); no dispatch path calls them.
"""
from __future__ import annotations

import torch
from torch import Tensor

from . import rfa_hip

EPS = 1.0   # reference rfa.py:17 -- a clamp on the denominator, not a small epsilon


def reverse_cumsum(x: Tensor, dim: int) -> Tensor:
    """Suffix sums along ``dim`` (reference rfa.py:20-21)."""
    return x + x.sum(dim, keepdim=True) - torch.cumsum(x, dim)


def _prefix_terms(q: Tensor, k: Tensor, v: Tensor):
    s = torch.cumsum(k.unsqueeze(-1) * v.unsqueeze(-2), dim=0)        # [T, N, K, d]
    z = torch.cumsum(k, dim=0)
    qs = torch.einsum("tnk,tnkd->tnd", q, s)
    qz = (q * z).sum(-1).clamp_min(EPS)
    return s, z, qs, qz


def rfa_debug(q: Tensor, k: Tensor, v: Tensor) -> Tensor:
    """Formula statement of the causal forward (reference rfa.py:24-41)."""
    _, _, qs, qz = _prefix_terms(q, k, v)
    return qs / qz.unsqueeze(-1)


def _as_kernel_input(t: Tensor) -> Tensor:
    return t.to(torch.float16).contiguous()


class RFA(torch.autograd.Function):

    @staticmethod
    def forward_torch(q: Tensor, k: Tensor, v: Tensor) -> Tensor:
        """ATen statement of the forward (reference rfa.py:46-64); O(T N K d) memory."""
        return rfa_debug(q, k, v)

    @staticmethod
    def backward_torch(q: Tensor, k: Tensor, v: Tensor, grad_attn: Tensor):
        """ATen statement of the backward (reference rfa.py:66-103)."""
        s, z, qs, qz = _prefix_terms(q, k, v)
        g_qs = grad_attn / qz.unsqueeze(-1)
        g_qz = -(grad_attn * qs).sum(-1) / qz.square() * (qz > EPS)
        grad_q = torch.einsum("tnd,tnkd->tnk", g_qs, s) + g_qz.unsqueeze(-1) * z
        g_s = reverse_cumsum(q.unsqueeze(-1) * g_qs.unsqueeze(-2), 0)
        grad_k = torch.einsum("tnkd,tnd->tnk", g_s, v) + reverse_cumsum(q * g_qz.unsqueeze(-1), 0)
        grad_v = torch.einsum("tnkd,tnk->tnd", g_s, k)
        return grad_q, grad_k, grad_v

    @staticmethod
    def forward_hip(q: Tensor, k: Tensor, v: Tensor) -> Tensor:
        return rfa_hip.forward(q, k, v)

    @staticmethod
    def backward_hip(q: Tensor, k: Tensor, v: Tensor, grad_attn: Tensor):
        return rfa_hip.backward(q, k, v, grad_attn)

    # names the reference's callers use (rfa.py:105-111, grad_check.py:24,43)
    forward_cuda = forward_hip
    backward_cuda = backward_hip

    @staticmethod
    def forward(ctx, q: Tensor, k: Tensor, v: Tensor) -> Tensor:
        """attn [tgt_len, bsz*heads, head_dim]; saves (q, k, v) like rfa.py:124 (plus the forward products backward reuses)."""
        ctx.in_dtypes = (q.dtype, k.dtype, v.dtype)
        q, k, v = _as_kernel_input(q), _as_kernel_input(k), _as_kernel_input(v)
        if any(ctx.needs_input_grad):
            # also keep the forward's segment totals, denominators and output so that backward
            # need not rebuild them
            attn, fwd_saved = rfa_hip.forward_save(q, k, v)
            ctx.save_for_backward(q, k, v, attn, fwd_saved)
        else:
            attn = rfa_hip.forward(q, k, v)
        return attn.to(ctx.in_dtypes[2])

    @staticmethod
    def backward(ctx, grad_attn: Tensor):
        q, k, v, attn, fwd_saved = ctx.saved_tensors
        gq, gk, gv = rfa_hip.backward_saved(q, k, v, _as_kernel_input(grad_attn), attn, fwd_saved)
        dq, dk, dv = ctx.in_dtypes
        return gq.to(dq), gk.to(dk), gv.to(dv)
