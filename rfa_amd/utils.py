"""Feature map and helpers; mirror of random_feature_attention/utils.py.

``random_project`` runs the fused HIP feature-map kernel (forward and backward)
instead of the reference's chain of ATen ops.  Inputs are computed in fp16 (the
kernels' input type); other floating dtypes are rounded to fp16 on the way in
and the result is returned in the caller's dtype.
"""
from __future__ import annotations

import os
from typing import List, NamedTuple, Optional, Tuple

import numpy as np
import torch
from torch import Tensor

from . import rfa_hip

EPS = 1.0      # reference utils.py:9
SCALE = 0.1    # reference utils.py:10
RANDOM_MATRICES_PATH = os.path.join(os.path.dirname(__file__), "../random_matrices")


class CrossAttentionState(NamedTuple):
    """reference utils.py:14-18; s and z are fp32 here."""
    s: Tensor
    z: Tensor
    random_matrices: Tensor
    tau: float


def upgrade_state_dict_named(state_dict, name):
    """Checkpoint-upgrade hook the reference modules store (causal_attention.py:187,
    cross_attention.py:44,243) but never define; parameter names are unchanged here,
    so there is nothing to upgrade."""
    return state_dict


def load_random_matrices(*, head_dim: int, proj_dim: int, dtype: torch.dtype = torch.half) -> Tensor:
    """[num_random_matrices, proj_dim, head_dim] as a frozen Parameter (reference utils.py:49-59).

    Reads ``random_matrices/{head_dim}_{proj_dim}.npy`` when it exists; otherwise the
    matrices are generated in memory by the same recipe that wrote that file
    (construct_random_matrices.py: Gaussian features, numpy seed 31415, 500 matrices).
    """
    path = os.path.join(RANDOM_MATRICES_PATH, f"{head_dim}_{proj_dim}.npy")
    if os.path.exists(path):
        mats = np.load(path)
    else:
        from .construct_random_matrices import construct_random_matrices, rrf
        # a generator of its own: the caller's global numpy seed is left as it is
        mats = construct_random_matrices(rrf, 500, head_dim=head_dim, proj_dim=proj_dim,
                                         rng=np.random.RandomState(31415))
    return torch.nn.Parameter(torch.tensor(mats, dtype=dtype), requires_grad=False)


def sample_random_matrices(*, num_layers: int, num_heads: int, random_matrices: Tensor,
                           is_training: bool = True):
    """reference utils.py:62-87: training draws num_layers*num_heads distinct matrices and
    returns one [num_heads, proj_dim, head_dim] stack per layer; evaluation returns the
    first num_heads matrices (shared by all layers)."""
    if is_training:
        picks = np.random.choice(random_matrices.size(0), size=num_layers * num_heads, replace=False)
        chosen = random_matrices[picks]
        return [chosen[i * num_heads:(i + 1) * num_heads] for i in range(num_layers)]
    return random_matrices[list(range(num_heads))]


class _BuildRandomMatrices(torch.autograd.Function):
    """W' = (sigma * W if sigma) / tau and its gradient, one launch each."""

    @staticmethod
    def forward(ctx, random_matrices: Tensor, sigma: Optional[Tensor], tau: float) -> Tensor:
        w = random_matrices.contiguous()
        sg = None if sigma is None else sigma.contiguous()
        ctx.tau = tau
        ctx.has_sigma = sg is not None
        ctx.save_for_backward(w, *([sg] if sg is not None else []))
        return rfa_hip.build_random_matrices(w, sg, tau)

    @staticmethod
    def backward(ctx, grad_out: Tensor):
        w = ctx.saved_tensors[0]
        sg = ctx.saved_tensors[1] if ctx.has_sigma else None
        dsigma, dw = rfa_hip.build_random_matrices_backward(
            w, sg, grad_out.contiguous(), ctx.tau, ctx.has_sigma and ctx.needs_input_grad[1], ctx.needs_input_grad[0])
        return dw, dsigma, None


def build_random_matrices(random_matrices: Tensor, tau: float, sigma: Optional[Tensor] = None,
                          reparam_proj: bool = False) -> Tensor:
    """W' = (sigma * W if reparam_proj) / tau (reference utils.py:90-97).

    fp16 tensors on a HIP device ([H, D, d] matrices, [H, 1, d] sigma) take one kernel launch
    forward and one backward, in the arithmetic of the reference's two ATen launches; anything
    else takes those ATen launches."""
    sg = sigma if reparam_proj else None
    if (random_matrices.is_cuda and random_matrices.dtype == torch.float16 and random_matrices.dim() == 3
            and isinstance(tau, (int, float)) and tau != 0
            and (sg is None or (sg.is_cuda and sg.dtype == torch.float16 and sg.dim() == 3
                                and tuple(sg.shape) == (random_matrices.shape[0], 1, random_matrices.shape[2])))):
        return _BuildRandomMatrices.apply(random_matrices, sg, float(tau))
    if reparam_proj:
        random_matrices = sigma * random_matrices
    return random_matrices / tau


def _normalize(x: Tensor) -> Tuple[Tensor, Tensor]:
    """(x / (||x|| + 1e-3), ||x||) (reference utils.py:100-102)."""
    norm = torch.linalg.vector_norm(x, ord=2, dim=-1, keepdim=True)
    return x / (norm + 1e-3), norm


class _FeatureMap(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x: Tensor, w: Tensor, scale: float) -> Tensor:
        ctx.in_dtypes = (x.dtype, w.dtype)
        ctx.scale = scale
        xh = x.to(torch.float16).contiguous()
        wh = w.to(torch.float16).contiguous()
        ctx.save_for_backward(xh, wh)
        return rfa_hip.feature_map_forward(xh, wh, scale).to(x.dtype)

    @staticmethod
    def backward(ctx, grad_phi: Tensor):
        xh, wh = ctx.saved_tensors
        # matrices that take no gradient (not reparametrised, or frozen): dW' is neither formed nor reduced
        dx, dw = rfa_hip.feature_map_backward(xh, wh, grad_phi.to(torch.float16).contiguous(), ctx.scale,
                                              need_dw=ctx.needs_input_grad[1])
        return dx.to(ctx.in_dtypes[0]), None if dw is None else dw.to(ctx.in_dtypes[1]), None


class _FeatureMapPair(torch.autograd.Function):
    """phi of two tensors of one shape through the same matrices: one launch forward, one backward
    (with one reduction for the sum of both dW')."""

    @staticmethod
    def forward(ctx, x0: Tensor, x1: Tensor, w: Tensor, scale: float):
        ctx.in_dtypes = (x0.dtype, x1.dtype, w.dtype)
        ctx.scale = scale
        x0h, x1h = x0.to(torch.float16).contiguous(), x1.to(torch.float16).contiguous()
        wh = w.to(torch.float16).contiguous()
        ctx.save_for_backward(x0h, x1h, wh)
        phi0, phi1 = rfa_hip.feature_map_forward_pair(x0h, x1h, wh, scale)
        return phi0.to(x0.dtype), phi1.to(x1.dtype)

    @staticmethod
    def backward(ctx, g0: Tensor, g1: Tensor):
        x0h, x1h, wh = ctx.saved_tensors
        dx0, dx1, dw = rfa_hip.feature_map_backward_pair(x0h, x1h, wh, g0.to(torch.float16).contiguous(),
                                                         g1.to(torch.float16).contiguous(), ctx.scale,
                                                         need_dw=ctx.needs_input_grad[2])
        return dx0.to(ctx.in_dtypes[0]), dx1.to(ctx.in_dtypes[1]), None if dw is None else dw.to(ctx.in_dtypes[2]), None


def random_project_pair(*, x0: Tensor, x1: Tensor, random_matrices: Tensor, scale: float = SCALE):
    """(random_project(x=x0, ...), random_project(x=x1, ...)) for two tensors of one shape that go
    through the same matrices -- the q and k of causal_attention.py:241-248 -- in one launch each
    way.  Same values and gradients as the two calls."""
    if x0.shape != x1.shape or x0.device != x1.device:
        return (random_project(x=x0, random_matrices=random_matrices, scale=scale),
                random_project(x=x1, random_matrices=random_matrices, scale=scale))
    return _FeatureMapPair.apply(x0, x1, random_matrices, scale)


def random_project(*, x: Tensor, random_matrices: Tensor, scale: float = SCALE) -> Tensor:
    """phi(x) = scale * [sin(W x^), cos(W x^)] (reference utils.py:105-120).

    x: [seq_len, bsz, num_heads, head_dim]; random_matrices: [num_heads, proj_dim, head_dim]
    -> [seq_len, bsz, num_heads, 2 * proj_dim].  ``scale`` defaults to the reference's
    constant 0.1; pass proj_dim ** -0.5 for the variance-normalised map.
    """
    return _FeatureMap.apply(x, random_matrices, scale)


def normalize_attn_weights(x: Tensor, dim: int = -1, dtype: torch.dtype = torch.float32) -> Tensor:
    """x / |sum(x)|.clamp(1e-3) in fp32 (reference utils.py:123-130)."""
    x = x.to(torch.float32)
    denom = x.sum(dim=dim, keepdim=True).abs().clamp(1e-3)
    return (x / denom).to(dtype)
