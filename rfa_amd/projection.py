"""Input projections of the attention modules on the fused projection + feature-map launch.

The reference modules run ``q_proj / k_proj / v_proj`` (torch.nn.Linear), view the results as
heads and call ``random_project`` on q and k (causal_attention.py:228-247;
cross_attention.py:66-76, :279-283).  ``project_heads`` does that chain in one kernel launch
(``rfa_project_feature_map``) and differentiates it with the feature-map backward kernel plus
library GEMMs for the Linear layers.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import torch
from torch import Tensor, nn

from . import rfa_hip
from ._derived import derived


def linear_param_grads(x2: Tensor, dys: Sequence[Tensor], has_bias: Sequence[bool]):
    """(dW, db) lists of Linear layers sharing the input x2 [R, E_in], given dy [R, E_out] each:
    one row-split MFMA launch when the sizes allow it, library GEMMs and column sums otherwise."""
    e_out, e_in = dys[0].shape[1], x2.shape[1]
    if (x2.is_cuda and x2.dtype == torch.float16 and all(d.dtype == torch.float16 for d in dys)
            and rfa_hip.linear_weight_grad_supported(e_out, e_in) and 1 <= len(dys) <= 3):
        return rfa_hip.linear_weight_grad(x2.contiguous(), [d.contiguous() for d in dys], list(has_bias))
    return ([torch.mm(d.t(), x2) for d in dys], [d.sum(0) if b else None for d, b in zip(dys, has_bias)])


_STACKED: dict = {}      # ids of the three weights -> their [3 * E_out, E_in] stack


def _stacked_weights(weights: Sequence[Tensor]) -> Tensor:
    """[Wq; Wk; Wv] as one matrix.  Outside stream capture the stack is kept for as long as the
    three weights are the same tensor objects in the same state (an optimizer step moves their
    version counters); under capture it is always formed, so that a replayed graph reads the
    weights of the day."""
    make = lambda: torch.cat(list(weights), 0)
    if torch.cuda.is_current_stream_capturing():
        return make()
    return derived(_STACKED, tuple(id(w) for w in weights), tuple(weights), None, make, limit=8)


def _packed_backward_ok(ctx, grads, weights) -> bool:
    """q and k through the feature map, v plain, an input gradient wanted, equal fp16 weights: the
    three dx products can be one over the packed gradient."""
    return (len(ctx.want_phi) == 3 and tuple(ctx.want_phi) == (True, True, False) and ctx.needs_input_grad[0]
            and all(g is not None and g.is_cuda and g.dtype == torch.float16 for g in grads)
            and all(w.dtype == torch.float16 and w.shape == weights[0].shape for w in weights))


class _ProjectHeads(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x: Tensor, w_feat: Optional[Tensor], scale: float, heads: int, want_phi: Tuple[bool, ...],
                grad_mode: bool, *params: Optional[Tensor]):
        n = len(want_phi)
        weights, biases = list(params[0::2]), list(params[1::2])
        wf = None if w_feat is None else w_feat.contiguous()
        # y of a projection that goes through the feature map is only kept for the backward pass
        # (needs_input_grad does not see grad mode -- under no_grad it still names the trainable
        # parameters -- and inside forward() grad mode is always off: the caller passes its own)
        keep_y = grad_mode and any(ctx.needs_input_grad)
        ys, phis = rfa_hip.project_feature_map(x.contiguous(), [w.contiguous() for w in weights], biases, list(want_phi),
                                               wf, heads, scale, keep_y)
        ctx.scale, ctx.heads, ctx.want_phi = scale, heads, want_phi
        ctx.has_bias = tuple(b is not None for b in biases)
        ctx.has_wf = w_feat is not None
        if keep_y:
            ctx.save_for_backward(x, *([wf] if wf is not None else []), *weights, *[y for y, f in zip(ys, want_phi) if f])
        return tuple(phis[p] if want_phi[p] else ys[p] for p in range(n))

    @staticmethod
    def backward(ctx, *grads: Tensor):
        saved = list(ctx.saved_tensors)
        x = saved.pop(0)
        wf = saved.pop(0) if ctx.has_wf else None
        n = len(ctx.want_phi)
        weights, ys = saved[:n], saved[n:]
        L, B, E = x.shape
        x2 = x.reshape(L * B, E)
        dx = None
        dwf = None
        dys = []
        yi = 0
        if _packed_backward_ok(ctx, grads, weights):
            # [dy_q | dy_k | dv] side by side, written by the feature-map backward launch itself: one
            # GEMM for dx and one contraction for the three weight gradients
            e_out = weights[0].shape[0]
            packed, dwf = rfa_hip.feature_map_backward_pair_packed(ys[0], ys[1], wf, grads[0].contiguous(),
                                                                   grads[1].contiguous(), grads[2].contiguous(), ctx.scale,
                                                                   need_dw=ctx.needs_input_grad[1])
            dx = torch.mm(packed, _stacked_weights(weights)).view(L, B, E)
            dws, dbs = linear_param_grads(x2, [packed], [any(ctx.has_bias)])
            dparams = []
            for p in range(n):
                dparams += [dws[0][p * e_out:(p + 1) * e_out],
                            dbs[0][p * e_out:(p + 1) * e_out] if ctx.has_bias[p] else None]
            return (dx, None if dwf is None else dwf.to(wf.dtype), None, None, None, None, *dparams)
        phi_idx = [p for p in range(n) if ctx.want_phi[p]]
        pair = {}
        if len(phi_idx) == 2:       # phi(q) and phi(k): both through the same w, one launch for the two
            p0, p1 = phi_idx
            dy0, dy1, dwf = rfa_hip.feature_map_backward_pair(ys[0], ys[1], wf, grads[p0].contiguous(),
                                                              grads[p1].contiguous(), ctx.scale,
                                                              need_dw=ctx.needs_input_grad[1])
            pair = {p0: dy0, p1: dy1}
        for p in range(n):
            g = grads[p].contiguous()
            if p in pair:
                dy = pair[p]
            elif ctx.want_phi[p]:
                dy, dw = rfa_hip.feature_map_backward(ys[yi], wf, g, ctx.scale, need_dw=ctx.needs_input_grad[1])
                yi += 1
                if dw is not None:
                    dwf = dw if dwf is None else dwf + dw
            else:
                dy = g
            dy2 = dy.reshape(L * B, -1)
            dys.append(dy2)
            if ctx.needs_input_grad[0]:
                dx = torch.mm(dy2, weights[p]) if dx is None else dx.addmm_(dy2, weights[p])
        dws, dbs = linear_param_grads(x2, dys, ctx.has_bias)
        dparams = []
        for p in range(n):
            dparams += [dws[p], dbs[p]]
        if dx is not None:
            dx = dx.view(L, B, E)
        if dwf is not None:
            dwf = dwf.to(wf.dtype)
        return (dx, dwf, None, None, None, None, *dparams)


def fused_projection_supported(x: Tensor, layers: Sequence[nn.Linear], heads: int,
                               w_feat: Optional[Tensor] = None) -> bool:
    """True when the fused launch can stand in for ``[layer(x) for layer in layers]``: fp16 HIP
    tensors, a common [out, in] weight shape with ``in`` a multiple of 64 and a head width of
    64 or 128 (and a supported proj_dim if a feature map is asked for)."""
    if not (x.is_cuda and x.dtype == torch.float16 and x.dim() == 3 and 1 <= len(layers) <= 3):
        return False
    out_dim, in_dim = layers[0].weight.shape
    if in_dim != x.shape[-1] or in_dim % 64 != 0 or out_dim % heads != 0 or out_dim // heads not in (64, 128):
        return False
    for layer in layers:
        if tuple(layer.weight.shape) != (out_dim, in_dim) or layer.weight.dtype != torch.float16:
            return False
        if layer.bias is not None and layer.bias.dtype != torch.float16:
            return False
    if w_feat is not None:
        if w_feat.dtype != torch.float16 or w_feat.dim() != 3 or w_feat.shape[1] not in (32, 64, 128):
            return False
    return True


def project_heads(x: Tensor, layers: Sequence[nn.Linear], want_phi: Sequence[bool], heads: int,
                  w_feat: Optional[Tensor], scale: float):
    """``[phi(layer(x)) if flag else layer(x)]`` viewed as [L, B, heads, .], in one launch.

    x: [L, B, E] fp16 on a HIP device; layers: 1..3 ``nn.Linear`` with equal weight shapes;
    w_feat: [heads, proj_dim, head_dim] (None when no flag is set).
    """
    params = []
    for layer in layers:
        params += [layer.weight, layer.bias]
    return _ProjectHeads.apply(x, w_feat, scale, heads, tuple(bool(f) for f in want_phi), torch.is_grad_enabled(),
                               *params)


class _LinearOut(torch.autograd.Function):
    """y = x W^T + b with the library GEMM forward and the row-split weight/bias-gradient kernel
    backward (the library's choice for dy^T x with a long row count is several times slower)."""

    @staticmethod
    def forward(ctx, x: Tensor, weight: Tensor, bias: Optional[Tensor]):
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        return torch.nn.functional.linear(x, weight, bias)

    @staticmethod
    def backward(ctx, dy: Tensor):
        x, weight = ctx.saved_tensors
        dy2 = dy.reshape(-1, dy.shape[-1])
        x2 = x.reshape(-1, x.shape[-1])
        dx = torch.mm(dy2, weight).view(x.shape) if ctx.needs_input_grad[0] else None
        dws, dbs = linear_param_grads(x2, [dy2], [ctx.has_bias])
        return dx, dws[0], dbs[0]


def linear_out(x: Tensor, layer: nn.Linear) -> Tensor:
    """``layer(x)`` (the modules' out_proj, causal_attention.py:278, cross_attention.py:298); fp16 HIP
    tensors with widths that are multiples of 128 take the row-split gradient kernel in backward."""
    w = layer.weight
    if (x.is_cuda and x.dtype == torch.float16 and w.dtype == torch.float16 and torch.is_grad_enabled()
            and (w.requires_grad or x.requires_grad) and rfa_hip.linear_weight_grad_supported(*w.shape)
            and (layer.bias is None or layer.bias.dtype == torch.float16)):
        return _LinearOut.apply(x, w, layer.bias)
    return layer(x)
