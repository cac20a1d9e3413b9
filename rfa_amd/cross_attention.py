"""Random feature cross attention; mirror of random_feature_attention/cross_attention.py.

The two contractions run as HIP kernels with their own backward:
  source side   s = sum_s phi_k (x) v, z = sum_s phi_k     (CrossAttentionProjectLayer)
  target side   attn = (phi_q s) / max(|phi_q z|, 1)        (CrossAttention.rfa)
The state (s, z) is kept in fp32.
"""
from __future__ import annotations

import math
from typing import List, Optional, Tuple

import torch
from torch import Tensor, nn
from torch.nn import Parameter

from . import rfa_hip
from .projection import fused_projection_supported, linear_out, project_heads
from .utils import (EPS, SCALE, CrossAttentionState, build_random_matrices, load_random_matrices, random_project,
                    sample_random_matrices, upgrade_state_dict_named)


class _CrossState(torch.autograd.Function):
    """(phi_k [S,B,H,K], v [S,B,H,d], pad [B,S] or None) -> (s [B,H,K,d], z [B,H,K]) fp32."""

    @staticmethod
    def forward(ctx, phi_k: Tensor, v: Tensor, pad: Optional[Tensor]):
        ctx.in_dtypes = (phi_k.dtype, v.dtype)
        pk, vv = phi_k.to(torch.float16).contiguous(), v.to(torch.float16).contiguous()
        ctx.save_for_backward(pk, vv)
        ctx.pad = pad
        return rfa_hip.cross_state(pk, vv, pad)

    @staticmethod
    def backward(ctx, ds: Tensor, dz: Tensor):
        pk, vv = ctx.saved_tensors
        dk, dv = rfa_hip.cross_state_backward(pk, vv, ds.to(torch.float32).contiguous(),
                                              dz.to(torch.float32).contiguous(), ctx.pad)
        return dk.to(ctx.in_dtypes[0]), dv.to(ctx.in_dtypes[1]), None


class _CrossReadout(torch.autograd.Function):
    """(phi_q [T,B,H,K], s, z) -> attn [T,B,H,d]."""

    @staticmethod
    def forward(ctx, phi_q: Tensor, s: Tensor, z: Tensor):
        ctx.in_dtypes = (phi_q.dtype, s.dtype, z.dtype)
        pq = phi_q.to(torch.float16).contiguous()
        s32, z32 = s.to(torch.float32).contiguous(), z.to(torch.float32).contiguous()
        ctx.save_for_backward(pq, s32, z32)
        return rfa_hip.cross_readout(pq, s32, z32).to(phi_q.dtype)

    @staticmethod
    def backward(ctx, grad_attn: Tensor):
        pq, s32, z32 = ctx.saved_tensors
        dq, ds, dz = rfa_hip.cross_readout_backward(pq, s32, z32, grad_attn.to(torch.float16).contiguous())
        tq, ts, tz = ctx.in_dtypes
        return dq.to(tq), ds.to(ts), dz.to(tz)


class CrossAttentionProjectLayer(nn.Module):
    """Source-side projection of one decoder layer (reference cross_attention.py:18-131)."""

    def __init__(self, *, embed_dim: int, num_heads: int, head_dim: int, proj_dim: int, tau: float = 1.0,
                 reparam_proj: bool = True):
        super().__init__()
        assert num_heads * head_dim == embed_dim
        self.embed_dim, self.num_heads, self.head_dim, self.proj_dim = embed_dim, num_heads, head_dim, proj_dim
        self.reparam_proj, self.tau = reparam_proj, tau
        self.k_proj = nn.Linear(embed_dim, embed_dim, bias=True)
        self.v_proj = nn.Linear(embed_dim, embed_dim, bias=True)
        if reparam_proj:
            self.sigma = Parameter(Tensor(num_heads, 1, head_dim))
        self.reset_parameters()
        self.upgrade_state_dict_named = upgrade_state_dict_named
        self.fuse_projections = True      # k/v projections + view to heads + phi(k) as one launch when possible

    def reset_parameters(self):
        nn.init.xavier_uniform_(self.k_proj.weight, gain=1 / math.sqrt(2))
        nn.init.xavier_uniform_(self.v_proj.weight, gain=1 / math.sqrt(2))
        if self.reparam_proj:
            nn.init.constant_(self.sigma, 1.0)

    def project_and_reshape(self, *, encoder_output: Tensor, random_matrices: Tensor,
                            mask: Optional[Tensor] = None) -> Tuple[Tensor, Tensor, Tensor, float]:
        """encoder_output [src_len, bsz, embed_dim]; mask [src_len, bsz, 1, 1] bool (True = pad).
        Returns (s [bsz, heads, 2*proj_dim, head_dim], z [bsz, heads, 2*proj_dim], W', tau)
        (reference cross_attention.py:52-106)."""
        src_len, bsz, _ = encoder_output.size()
        w = build_random_matrices(random_matrices=random_matrices, tau=self.tau,
                                  sigma=self.sigma if self.reparam_proj else None,
                                  reparam_proj=self.reparam_proj)
        kv = (self.k_proj, self.v_proj)
        if self.fuse_projections and fused_projection_supported(encoder_output, kv, self.num_heads, w):
            # both projections, the view to heads and phi(k) in one launch
            phi_k, v = project_heads(encoder_output, kv, (True, False), self.num_heads, w, SCALE)
        else:
            k = self.k_proj(encoder_output).contiguous().view(src_len, bsz, self.num_heads, self.head_dim)
            v = self.v_proj(encoder_output).contiguous().view(src_len, bsz, self.num_heads, self.head_dim)
            phi_k = random_project(x=k, random_matrices=w)
        pad = None
        if mask is not None:
            pad = mask.reshape(src_len, bsz).transpose(0, 1).contiguous()   # [bsz, src_len]
        s, z = _CrossState.apply(phi_k, v, pad)
        return s, z, w, self.tau

    def forward(self, *, encoder_output: Tensor, random_matrices: Tensor,
                mask: Optional[Tensor] = None) -> CrossAttentionState:
        assert encoder_output.size(2) == self.embed_dim
        s, z, w, tau = self.project_and_reshape(encoder_output=encoder_output,
                                                random_matrices=random_matrices, mask=mask)
        return CrossAttentionState(s, z, w, tau)


class CrossAttentionProject(nn.Module):
    """Encoder-output projection for all decoder layers (reference cross_attention.py:134-213)."""

    def __init__(self, *, num_layers: int, embed_dim: int, num_heads: int, head_dim: int, proj_dim: int,
                 tau: float = 1.0, reparam_proj: bool = True):
        super().__init__()
        assert num_heads * head_dim == embed_dim
        self.num_layers, self.embed_dim, self.num_heads = num_layers, embed_dim, num_heads
        self.head_dim, self.proj_dim = head_dim, proj_dim
        self.layers = nn.ModuleList([
            CrossAttentionProjectLayer(embed_dim=embed_dim, num_heads=num_heads, head_dim=head_dim,
                                       proj_dim=proj_dim, tau=tau, reparam_proj=reparam_proj)
            for _ in range(num_layers)])
        self.random_matrices = load_random_matrices(head_dim=head_dim, proj_dim=proj_dim, dtype=torch.float16)
        self.random_matrices_eval = nn.Parameter(
            sample_random_matrices(num_layers=num_layers, num_heads=num_heads,
                                   random_matrices=self.random_matrices, is_training=False),
            requires_grad=False)

    def forward(self, *, encoder_output: Tensor,
                key_padding_mask: Optional[Tensor] = None) -> List[CrossAttentionState]:
        """encoder_output [src_len, bsz, embed_dim]; key_padding_mask [bsz, src_len], 1 = pad."""
        src_len, bsz, embed_dim = encoder_output.size()
        assert embed_dim == self.embed_dim
        if self.training:
            mats = sample_random_matrices(num_layers=self.num_layers, num_heads=self.num_heads,
                                          random_matrices=self.random_matrices, is_training=True)
        else:
            mats = self.random_matrices_eval
        mask = key_padding_mask
        if mask is not None and mask.dim() == 0:
            mask = None
        if mask is not None:
            mask = mask.transpose(0, 1)
            assert mask.size(0) == src_len and mask.size(1) == bsz
            mask = mask.to(torch.bool)[:, :, None, None]
        return [layer(encoder_output=encoder_output, random_matrices=mats[i] if self.training else mats, mask=mask)
                for i, layer in enumerate(self.layers)]


class CrossAttention(nn.Module):
    """Target-side random feature cross attention (reference cross_attention.py:216-300)."""

    def __init__(self, *, embed_dim: int, num_heads: int, head_dim: int, proj_dim: int, tau: float = 1.0,
                 reparam_proj: bool = True):
        super().__init__()
        assert head_dim * num_heads == embed_dim, "embed_dim must be divisible by num_heads"
        self.embed_dim, self.num_heads, self.head_dim, self.proj_dim = embed_dim, num_heads, head_dim, proj_dim
        self.reparam_proj, self.tau = reparam_proj, tau
        self.q_proj = nn.Linear(embed_dim, embed_dim, bias=True)
        self.out_proj = nn.Linear(embed_dim, embed_dim, bias=True)
        self.reset_parameters()
        self.upgrade_state_dict_named = upgrade_state_dict_named
        self.fuse_projections = True      # q projection + view to heads + phi(q) as one launch when possible

    def reset_parameters(self):
        for proj in (self.q_proj, self.out_proj):
            nn.init.xavier_uniform_(proj.weight, gain=1 / math.sqrt(2))
            if proj.bias is not None:
                nn.init.constant_(proj.bias, 0.0)

    def rfa(self, query: Tensor, s: Tensor, z: Tensor, random_matrices: Tensor) -> Tensor:
        """query [tgt_len, bsz, heads, head_dim] -> attn [tgt_len, bsz, heads, head_dim]
        (reference cross_attention.py:254-270)."""
        phi_q = random_project(x=query, random_matrices=random_matrices)
        return _CrossReadout.apply(phi_q, s, z)

    def forward(self, query: Tensor, state: CrossAttentionState) -> Tensor:
        """query [tgt_len, bsz, embed_dim] -> [tgt_len, bsz, embed_dim]."""
        s, z, random_matrices, tau = state
        tgt_len, bsz, embed_dim = query.size()
        assert embed_dim == self.embed_dim
        if self.fuse_projections and fused_projection_supported(query, (self.q_proj,), self.num_heads, random_matrices):
            # q projection, the view to heads and phi(q) in one launch
            (phi_q,) = project_heads(query, (self.q_proj,), (True,), self.num_heads, random_matrices, SCALE)
            attn = _CrossReadout.apply(phi_q, s, z)
        else:
            q = self.q_proj(query).contiguous().view(tgt_len, bsz, self.num_heads, self.head_dim)
            attn = self.rfa(q, s, z, random_matrices)
        assert list(attn.size()) == [tgt_len, bsz, self.num_heads, self.head_dim]
        return linear_out(attn.contiguous().view(tgt_len, bsz, self.num_heads * self.head_dim), self.out_proj)
