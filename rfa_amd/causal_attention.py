"""Causal random feature attention; mirror of random_feature_attention/causal_attention.py.

Functional forms (keyword-only, as in the reference):
  incremental_rfa   decode loop                       -> HIP step kernel, fp32 state
  cuda_causal_rfa   training / prefill                -> HIP chunked-scan kernels via RFA.apply
  masked_rfa        quadratic form with explicit masks -> HIP quadratic-form kernels
and the ``CausalAttention`` module with the reference's parameter names
(q_proj, k_proj, v_proj, out_proj, sigma) and ``saved_state`` keys
("prev_s", "prev_z").
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch
import torch.nn.functional as F
from torch import Tensor, nn
from torch.nn import Parameter

from . import rfa_hip
from ._derived import derived
from .projection import fused_projection_supported, linear_out, project_heads
from .rfa import RFA
from .utils import (EPS, SCALE, build_random_matrices, random_project, random_project_pair,
                    upgrade_state_dict_named)


def _drop_scalar_mask(mask: Optional[Tensor]) -> Optional[Tensor]:
    # a 0-dim tensor stands for "no mask" (reference causal_attention.py:83-84,134-135)
    if mask is not None and mask.dim() == 0:
        return None
    return mask


def incremental_rfa(*, phi_q: Tensor, phi_k: Tensor, v: Tensor, s: Optional[Tensor] = None,
                    z: Optional[Tensor] = None, inplace: bool = False):
    """Per-step causal RFA (reference causal_attention.py:17-54).

    phi_q, phi_k: [tgt_len, bsz, heads, 2*proj_dim]; v: [tgt_len, bsz, heads, head_dim];
    s: [bsz, heads, 2*proj_dim, head_dim]; z: [bsz, heads, 2*proj_dim] (fp32; None = zeros).
    Returns (attn [tgt_len, bsz, heads*head_dim], s, z).  With ``inplace=False`` (the
    reference's behaviour) the given state is left untouched and new tensors are
    returned; ``inplace=True`` updates s and z where they are.  Inference only.
    """
    tgt_len, bsz, num_heads, feat = phi_q.size()
    head_dim = v.size(-1)
    if s is None:
        assert z is None
        s = torch.zeros((bsz, num_heads, feat, head_dim), device=v.device, dtype=torch.float32)
        z = torch.zeros((bsz, num_heads, feat), device=v.device, dtype=torch.float32)
        s_new, z_new = s, z
    else:
        assert z is not None
        s_in, z_in = s, z
        s, z = s.to(torch.float32).contiguous(), z.to(torch.float32).contiguous()
        if inplace or (s is not s_in and z is not z_in):
            s_new, z_new = s, z          # the caller's own tensors, or private fp32 copies: advance where they are
        else:
            # the kernel reads the caller's state and writes the advanced one elsewhere: no copy pass
            s_new, z_new = torch.empty_like(s), torch.empty_like(z)
    n = bsz * num_heads
    attn = rfa_hip.incremental(
        phi_q.detach().to(torch.float16).contiguous().view(tgt_len, n, feat),
        phi_k.detach().to(torch.float16).contiguous().view(tgt_len, n, feat),
        v.detach().to(torch.float16).contiguous().view(tgt_len, n, head_dim),
        s.view(n, feat, head_dim), z.view(n, feat),
        None if s_new is s else s_new.view(n, feat, head_dim), None if z_new is z else z_new.view(n, feat))
    return attn.to(v.dtype).view(tgt_len, bsz, num_heads * head_dim), s_new, z_new


class _MaskedRFA(torch.autograd.Function):
    """masked_rfa on the quadratic-form kernels (rfa_masked_forward / rfa_masked_backward)."""

    @staticmethod
    def forward(ctx, phi_q, phi_k, v, heads, key_padding_mask, mask_bytes, mask_t_bytes):
        ctx.in_dtypes = (phi_q.dtype, phi_k.dtype, v.dtype)
        q16, k16, v16 = (t.to(torch.float16).contiguous() for t in (phi_q, phi_k, v))
        attn, rsum = rfa_hip.masked_forward(q16, k16, v16, heads, key_padding_mask, mask_bytes)
        ctx.heads = heads
        ctx.masks = (key_padding_mask, mask_bytes, mask_t_bytes)
        ctx.save_for_backward(q16, k16, v16, attn, rsum)
        return attn.to(v.dtype)

    @staticmethod
    def backward(ctx, grad_attn):
        q16, k16, v16, attn, rsum = ctx.saved_tensors
        pad, mb, mtb = ctx.masks
        dq, dk, dv = rfa_hip.masked_backward(q16, k16, v16, grad_attn.to(torch.float16).contiguous(), attn, rsum,
                                             ctx.heads, pad, mb, mtb)
        tq, tk, tv = ctx.in_dtypes
        return dq.to(tq), dk.to(tk), dv.to(tv), None, None, None, None


def masked_rfa(*, phi_q: Tensor, phi_k: Tensor, v: Tensor, key_padding_mask: Optional[Tensor] = None,
               attn_mask: Optional[Tensor] = None) -> Tensor:
    """Quadratic-form RFA with explicit masks (reference causal_attention.py:57-109).

    phi_q, phi_k: [tgt_len, bsz, heads, 2*proj_dim]; v: [tgt_len, bsz, heads, head_dim];
    key_padding_mask: [bsz, tgt_len], 1 = padded key (a 0-dim tensor stands for None);
    attn_mask: [tgt_len, tgt_len], entries < 0 are masked (typically the causal mask).
    Note its normaliser, |row sum|.clamp(1e-3) (utils.py:123-130), is not the clamp-at-1 of
    the scan path.  Runs on the quadratic-form HIP kernels; tensors must be on a HIP device.
    """
    tgt_len, bsz, num_heads, feat = phi_q.size()
    head_dim = v.size(-1)
    key_padding_mask = _drop_scalar_mask(key_padding_mask)
    if key_padding_mask is not None:
        assert key_padding_mask.size(0) == bsz and key_padding_mask.size(1) == tgt_len
    mask_bytes = mask_t_bytes = None
    if attn_mask is not None:
        assert attn_mask.size(0) == tgt_len and attn_mask.size(1) == tgt_len
        mask_bytes, mask_t_bytes = rfa_hip.pack_attn_mask((attn_mask < 0.0).to(phi_q.device))
    n = bsz * num_heads
    attn = _MaskedRFA.apply(phi_q.contiguous().view(tgt_len, n, feat), phi_k.contiguous().view(tgt_len, n, feat),
                            v.contiguous().view(tgt_len, n, head_dim), num_heads, key_padding_mask, mask_bytes,
                            mask_t_bytes)
    return attn.contiguous().view(tgt_len, bsz, num_heads * head_dim)


def cuda_causal_rfa(*, phi_q: Tensor, phi_k: Tensor, v: Tensor,
                    key_padding_mask: Optional[Tensor] = None) -> Tensor:
    """Causal RFA through the fused kernels (reference causal_attention.py:112-151).

    key_padding_mask: [bsz, tgt_len], 1 = padded key, whose phi_k is zeroed.
    Returns attn [tgt_len, bsz, heads*head_dim].
    """
    tgt_len, bsz, num_heads, feat = phi_q.size()
    head_dim = v.size(-1)
    key_padding_mask = _drop_scalar_mask(key_padding_mask)
    if key_padding_mask is not None:
        assert key_padding_mask.size(0) == bsz and key_padding_mask.size(1) == tgt_len
        pad = key_padding_mask.to(torch.bool).transpose(0, 1)[:, :, None, None]
        phi_k = phi_k.masked_fill(pad, 0.0)
    n = bsz * num_heads
    attn = RFA.apply(phi_q.contiguous().view(tgt_len, n, feat),
                     phi_k.contiguous().view(tgt_len, n, feat),
                     v.contiguous().view(tgt_len, n, head_dim))
    return attn.contiguous().view(tgt_len, bsz, num_heads * head_dim)


# name without the vendor prefix
hip_causal_rfa = cuda_causal_rfa


def reorder_incremental_state(saved_state: Dict[str, Optional[Tensor]], new_order: Tensor) -> Dict[str, Optional[Tensor]]:
    """Beam-search reordering of a decode state: batch entry i of the result is entry
    ``new_order[i]`` of the input ("prev_s" [bsz, heads, 2*proj_dim, head_dim], "prev_z"
    [bsz, heads, 2*proj_dim]; reference state layout causal_attention.py:249-265).  The dict
    is updated in place and returned; an empty state is left alone."""
    for key in ("prev_s", "prev_z"):
        t = saved_state.get(key)
        if t is not None:
            saved_state[key] = t.index_select(0, new_order.to(device=t.device, dtype=torch.long))
    return saved_state


class CausalAttention(nn.Module):
    """Causal random feature self-attention (reference causal_attention.py:154-280)."""

    def __init__(self, *, embed_dim: int, num_heads: int, head_dim: int, proj_dim: int, tau: float = 1.0,
                 reparam_proj: bool = True, cuda_causal_rfa: bool = True):
        super().__init__()
        assert head_dim * num_heads == embed_dim, "embed_dim must be divisible by num_heads"
        self.embed_dim, self.num_heads, self.head_dim, self.proj_dim = embed_dim, num_heads, head_dim, proj_dim
        self.reparam_proj, self.cuda_causal_rfa, self.tau = reparam_proj, cuda_causal_rfa, tau
        self.q_proj = nn.Linear(embed_dim, embed_dim, bias=True)
        self.k_proj = nn.Linear(embed_dim, embed_dim, bias=True)
        self.v_proj = nn.Linear(embed_dim, embed_dim, bias=True)
        self.out_proj = nn.Linear(embed_dim, embed_dim, bias=True)
        if reparam_proj:
            self.sigma = Parameter(Tensor(num_heads, 1, head_dim))
        self.reset_parameters()
        self.upgrade_state_dict_named = upgrade_state_dict_named
        # q/k/v projections + view to heads + phi(q), phi(k) as one launch when the tensors allow it
        self.fuse_projections = True
        # Decoding: the reference builds a new state tensor every step (causal_attention.py:42-43), so
        # a caller may keep the tensors of an earlier step (a prefix shared between hypotheses, a
        # roll-back).  False keeps that: each step writes its state into fresh tensors (the kernel
        # reads one buffer and writes the other, no extra pass).  True advances the tensors under
        # "prev_s" / "prev_z" where they are -- what a captured HIP graph of the step needs.
        self.decode_inplace = False

    def reset_parameters(self):
        for proj in (self.q_proj, self.k_proj, self.v_proj, self.out_proj):
            nn.init.xavier_uniform_(proj.weight, gain=1 / math.sqrt(2))
        if self.reparam_proj:
            nn.init.constant_(self.sigma, 1.0)
        if self.out_proj.bias is not None:
            nn.init.constant_(self.out_proj.bias, 0.0)

    def _heads(self, t: Tensor, tgt_len: int, bsz: int) -> Tensor:
        return t.contiguous().view(tgt_len, bsz, self.num_heads, self.head_dim)

    # ---- inference-time caches ------------------------------------------------------------------
    # Decoding calls forward once per token with the same parameters: what depends on the parameters
    # alone is then kept between calls (only while autograd is off) for as long as every tensor it
    # was made from is the same object in the same state (version counter, address, dtype, shape),
    # so an optimizer step, load_state_dict, a replaced parameter or another random_matrices tensor
    # makes it anew.
    def _cached(self, name: str, sources, extra, make):
        return derived(self.__dict__.setdefault("_inference_cache", {}), name, sources, extra, make)

    def __getstate__(self):
        # copies and pickles of the module start without the cache (it holds weak references)
        state = self.__dict__.copy()
        state.pop("_inference_cache", None)
        return state

    def _scaled_matrices(self, random_matrices: Tensor) -> Tensor:
        sigma = self.sigma if self.reparam_proj else None
        make = lambda: build_random_matrices(random_matrices=random_matrices, tau=self.tau, sigma=sigma,
                                             reparam_proj=self.reparam_proj)
        if torch.is_grad_enabled():
            return make()
        return self._cached("w", (random_matrices, sigma), (self.tau, self.reparam_proj), make)

    def _stacked_qkv(self):
        """(weight [3E, E], bias [3E] or None) of one Linear layer that computes q_proj, k_proj and v_proj at once."""
        layers = (self.q_proj, self.k_proj, self.v_proj)

        def make():
            weight = torch.cat([layer.weight.detach() for layer in layers], 0).contiguous()
            biases = [layer.bias for layer in layers]
            bias = None if any(b is None for b in biases) else torch.cat([b.detach() for b in biases], 0).contiguous()
            return weight, bias
        return self._cached("qkv", tuple(t for layer in layers for t in (layer.weight, layer.bias)), None, make)

    def _packed_decode_ok(self, x: Tensor) -> bool:
        layers = (self.q_proj, self.k_proj, self.v_proj)
        with_bias = [layer.bias is not None for layer in layers]
        return (not torch.is_grad_enabled() and x.is_cuda and x.dtype == torch.float16
                and all(layer.weight.dtype == torch.float16 for layer in layers)
                and (all(with_bias) or not any(with_bias)))

    def forward(self, x: Tensor, random_matrices: Tensor, key_padding_mask: Optional[Tensor] = None,
                attn_mask: Optional[Tensor] = None,
                saved_state: Optional[Dict[str, Optional[Tensor]]] = None) -> Tensor:
        """x: [tgt_len, bsz, embed_dim]; random_matrices: [heads, proj_dim, head_dim] -> [tgt_len, bsz, embed_dim].

        With ``saved_state`` (a dict) the call is part of incremental decoding and the state under
        "prev_s" / "prev_z" is advanced (reference causal_attention.py:249-265, where tgt_len
        must be 1).  Here tgt_len > 1 is accepted as well: on an empty state the whole prompt
        goes through the chunked-scan kernels once and the state after its last step is kept
        (prefill); on a non-empty state the steps are taken one after the other.
        """
        tgt_len, bsz, embed_dim = x.size()
        assert embed_dim == self.embed_dim
        w = self._scaled_matrices(random_matrices)
        if saved_state is not None and saved_state.get("prev_s") is not None and self._packed_decode_ok(x):
            # a decoding step without autograd: q, k, v of the token(s) from one stacked projection (one
            # small-M GEMM instead of three), and feature map + state update + readout in one kernel per step
            feat = 2 * self.proj_dim
            s_in, z_in = saved_state["prev_s"], saved_state["prev_z"]
            assert z_in is not None
            s = s_in.to(torch.float32).contiguous()
            z = z_in.to(torch.float32).contiguous()
            s_out = z_out = None
            if not self.decode_inplace and (s is s_in or z is z_in):
                s_out, z_out = torch.empty_like(s), torch.empty_like(z)
            weight, bias = self._stacked_qkv()
            rows = F.linear(x, weight, bias).view(tgt_len, bsz, 3, self.num_heads, self.head_dim)
            attn = rfa_hip.incremental_qkv(rows, w.to(torch.float16).contiguous(), SCALE, s, z, s_out, z_out)
            if s_out is not None:
                s, z = s_out, z_out
            saved_state["prev_s"], saved_state["prev_z"] = s, z
            return linear_out(attn.view(tgt_len, bsz, embed_dim), self.out_proj)
        qkv = (self.q_proj, self.k_proj, self.v_proj)
        if self.fuse_projections and saved_state is None and fused_projection_supported(x, qkv, self.num_heads, w):
            # the three projections, the view to heads and phi of q and k in one launch
            phi_q, phi_k, v = project_heads(x, qkv, (True, True, False), self.num_heads, w, SCALE)
            if self.cuda_causal_rfa:
                attn = cuda_causal_rfa(phi_q=phi_q, phi_k=phi_k, v=v, key_padding_mask=key_padding_mask)
            else:
                attn = masked_rfa(phi_q=phi_q, phi_k=phi_k, v=v, attn_mask=attn_mask,
                                  key_padding_mask=key_padding_mask)
            return linear_out(attn, self.out_proj)
        q = self._heads(self.q_proj(x), tgt_len, bsz)
        k = self._heads(self.k_proj(x), tgt_len, bsz)
        v = self._heads(self.v_proj(x), tgt_len, bsz)
        if saved_state is not None:
            feat = 2 * self.proj_dim
            s, z = saved_state.get("prev_s"), saved_state.get("prev_z")
            if s is None and tgt_len > 1:
                # prefill: one pass of the training kernels over the prompt, final state kept
                with torch.no_grad():
                    phi_q, phi_k = random_project_pair(x0=q, x1=k, random_matrices=w)
                    pad = _drop_scalar_mask(key_padding_mask)
                    if pad is not None:
                        phi_k = phi_k.masked_fill(pad.to(torch.bool).transpose(0, 1)[:, :, None, None], 0.0)
                    n = bsz * self.num_heads
                    attn, s, z = rfa_hip.prefill(
                        phi_q.to(torch.float16).contiguous().view(tgt_len, n, feat),
                        phi_k.to(torch.float16).contiguous().view(tgt_len, n, feat),
                        v.detach().to(torch.float16).contiguous().view(tgt_len, n, self.head_dim))
                s = s.view(bsz, self.num_heads, feat, self.head_dim)
                z = z.view(bsz, self.num_heads, feat)
            else:
                s_out = z_out = None
                if s is None:
                    s = torch.zeros((bsz, self.num_heads, feat, self.head_dim), device=x.device, dtype=torch.float32)
                    z = torch.zeros((bsz, self.num_heads, feat), device=x.device, dtype=torch.float32)
                else:
                    assert z is not None
                    s_in, z_in = s, z
                    s = s.to(torch.float32).contiguous()
                    z = z.to(torch.float32).contiguous()
                    if not self.decode_inplace and (s is s_in or z is z_in):
                        s_out, z_out = torch.empty_like(s), torch.empty_like(z)
                # feature map + state update + readout in one kernel per step
                attn = rfa_hip.incremental_fused(
                    q.detach().to(torch.float16).contiguous(), k.detach().to(torch.float16).contiguous(),
                    v.detach().to(torch.float16).contiguous(), w.detach().to(torch.float16).contiguous(), SCALE, s, z,
                    s_out, z_out)
                if s_out is not None:
                    s, z = s_out, z_out
            attn = attn.to(x.dtype).view(tgt_len, bsz, embed_dim)
            saved_state["prev_s"], saved_state["prev_z"] = s, z
        else:
            phi_q, phi_k = random_project_pair(x0=q, x1=k, random_matrices=w)
            if self.cuda_causal_rfa:
                attn = cuda_causal_rfa(phi_q=phi_q, phi_k=phi_k, v=v, key_padding_mask=key_padding_mask)
            else:
                attn = masked_rfa(phi_q=phi_q, phi_k=phi_k, v=v, attn_mask=attn_mask,
                                  key_padding_mask=key_padding_mask)
        return linear_out(attn, self.out_proj)
