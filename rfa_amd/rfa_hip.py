"""Python face of the kernel library: the module that stands where the
reference's pybind extension ``rfa_cuda`` stood
(random_feature_attention/cuda/rfa_cuda.cpp:39-42), with the same two entry
points ``forward(q, k, v)`` and ``backward(q, k, v, grad_attn)`` and the same
argument order and return arity, plus the entry points for the other parts of
the path.  Tensors are validated (the reference validated nothing,
cuda/forward.cu:156-159) and handed to the C ABI as raw device pointers; the
work is enqueued on the current torch stream.

Two bindings of the same library stand behind these names.  ``_rfa_hip_ext`` is a PyTorch C++
extension (csrc/rfa_torch_ext.cpp: TORCH_CHECK, device guard, current HIP stream, outputs from
torch's allocator, a few microseconds of host time per call) and is used when it has been built;
the functions written out in this file do the same through ctypes and need nothing but the
shared library.  ``use_binding("ext" | "ctypes")`` switches, ``binding()`` tells which is active;
the environment variable RFA_AMD_BINDING picks the initial one.
"""
from __future__ import annotations

from typing import List, Optional

import torch
from torch import Tensor

from . import _lib


def _require(cond: bool, exc, msg):
    # msg is a callable so that the text is only built when the check fails
    if not cond:
        raise exc(msg())


_HALF = torch.float16


def _check_half_cuda(name: str, t: Tensor, ndim: int):
    # one cheap test for the common case; the individual checks below only name what is wrong
    try:
        if t.is_cuda and t.dtype is _HALF and t.dim() == ndim and t.is_contiguous():
            return
    except AttributeError:
        pass
    _require(isinstance(t, Tensor), TypeError, lambda: f"{name} must be a torch.Tensor")
    _require(t.is_cuda, RuntimeError,
             lambda: f"{name} must live on a HIP device (got {t.device}); the kernels have no CPU path")
    _require(t.dtype == torch.float16, TypeError, lambda: f"{name} must be float16 (got {t.dtype})")
    _require(t.dim() == ndim, ValueError, lambda: f"{name} must have {ndim} dims (got {tuple(t.shape)})")
    _require(t.is_contiguous(), ValueError, lambda: f"{name} must be contiguous")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_ptr(device) -> int:
    # the raw-stream accessor skips the Stream object; same value as current_stream(device).cuda_stream
    if _raw_stream is not None:
        index = device if isinstance(device, int) else device.index
        if index is not None:
            return _raw_stream(index)
    return torch.cuda.current_stream(device).cuda_stream


class _on_device:
    """``with _on_device(dev):`` makes dev the current device for the launch; a no-op (no context
    switch, no driver call) when it already is, which is the common case."""
    __slots__ = ("ctx",)

    def __init__(self, device):
        self.ctx = None if device.index == torch.cuda.current_device() else torch.cuda.device(device)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            return self.ctx.__exit__(*exc)
        return False


def _workspace(nbytes: int, device) -> Tensor:
    # torch's caching allocator: no hipMalloc on the steady-state path
    return torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)


def supported(K: int, d: int) -> bool:
    return bool(_lib.load().rfa_shape_supported(int(K), int(d)))


def selftest_layout() -> None:
    lib = _lib.load()
    _lib.check(lib.rfa_selftest_layout(_stream_ptr(torch.cuda.current_device())))


def _check_qkv(q: Tensor, k: Tensor, v: Tensor):
    _check_half_cuda("q", q, 3)
    _check_half_cuda("k", k, 3)
    _check_half_cuda("v", v, 3)
    _require(q.shape == k.shape, ValueError, lambda: f"q {tuple(q.shape)} and k {tuple(k.shape)} differ")
    _require(v.shape[:2] == q.shape[:2], ValueError,
             lambda: f"v {tuple(v.shape)} does not match q {tuple(q.shape)} in [tgt_len, bsz*heads]")
    _require(q.device == k.device == v.device, RuntimeError, lambda: "q, k, v must be on one device")


def forward(q: Tensor, k: Tensor, v: Tensor) -> Tensor:
    """attn[T, N, d] of causal RFA.  q, k: fp16 [T, N, K]; v: fp16 [T, N, d].

    Same contract as rfa_cuda.forward (reference cuda/rfa_cuda.cpp:22-27).
    """
    _check_qkv(q, k, v)
    lib = _lib.load()
    T, N, K = q.shape
    d = v.shape[2]
    out = torch.empty_like(v)
    with _on_device(q.device):
        nbytes = lib.rfa_causal_forward_workspace_bytes(T, N, K, d)
        ws = _workspace(nbytes, q.device)
        _lib.check(lib.rfa_causal_forward(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                          T, N, K, d, ws.data_ptr(), nbytes, _stream_ptr(q.device)))
    return out


def prefill(q: Tensor, k: Tensor, v: Tensor):
    """(attn, s, z): causal forward over a prompt plus the state after its last step.

    s: fp32 [N, K, d], z: fp32 [N, K] -- what ``incremental`` / ``incremental_fused`` continue from.
    """
    _check_qkv(q, k, v)
    lib = _lib.load()
    T, N, K = q.shape
    d = v.shape[2]
    out = torch.empty_like(v)
    s = torch.empty((N, K, d), dtype=torch.float32, device=q.device)
    z = torch.empty((N, K), dtype=torch.float32, device=q.device)
    with _on_device(q.device):
        nbytes = lib.rfa_causal_forward_workspace_bytes(T, N, K, d)
        ws = _workspace(nbytes, q.device)
        _lib.check(lib.rfa_causal_prefill(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), s.data_ptr(),
                                          z.data_ptr(), T, N, K, d, ws.data_ptr(), nbytes, _stream_ptr(q.device)))
    return out, s, z


def forward_save(q: Tensor, k: Tensor, v: Tensor):
    """(attn, saved): forward that also returns the buffer backward_saved reuses (segment totals, denominators)."""
    _check_qkv(q, k, v)
    lib = _lib.load()
    T, N, K = q.shape
    d = v.shape[2]
    out = torch.empty_like(v)
    with _on_device(q.device):
        nbytes = lib.rfa_causal_forward_workspace_bytes(T, N, K, d)
        sbytes = lib.rfa_causal_saved_state_bytes(T, N, K, d)
        ws = _workspace(nbytes, q.device)
        saved = _workspace(sbytes, q.device)
        _lib.check(lib.rfa_causal_forward_save(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                               saved.data_ptr(), sbytes, T, N, K, d, ws.data_ptr(), nbytes,
                                               _stream_ptr(q.device)))
    return out, saved


def backward_saved(q: Tensor, k: Tensor, v: Tensor, grad_attn: Tensor, out: Tensor, saved: Tensor) -> List[Tensor]:
    """backward() that reuses what forward_save returned for the same q, k, v: its output and saved buffer."""
    _check_qkv(q, k, v)
    _check_half_cuda("grad_attn", grad_attn, 3)
    _check_half_cuda("out", out, 3)
    _require(grad_attn.shape == v.shape, ValueError,
             lambda: f"grad_attn {tuple(grad_attn.shape)} must match v {tuple(v.shape)}")
    _require(out.shape == v.shape, ValueError, lambda: f"out {tuple(out.shape)} must match v {tuple(v.shape)}")
    _require(saved.is_cuda and saved.dtype == torch.uint8 and saved.is_contiguous(), TypeError,
             lambda: "saved must be the byte buffer returned by forward_save")
    lib = _lib.load()
    T, N, K = q.shape
    d = v.shape[2]
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    with _on_device(q.device):
        # sized for the plan of the forward call that wrote `saved`
        nbytes = lib.rfa_causal_backward_saved_workspace_bytes(saved.data_ptr(), T, N, K, d)
        ws = _workspace(nbytes, q.device)
        _lib.check(lib.rfa_causal_backward_saved(q.data_ptr(), k.data_ptr(), v.data_ptr(), grad_attn.data_ptr(),
                                                 out.data_ptr(), saved.data_ptr(), saved.numel(), dq.data_ptr(), dk.data_ptr(),
                                                 dv.data_ptr(), T, N, K, d, ws.data_ptr(), nbytes,
                                                 _stream_ptr(q.device)))
    return [dq, dk, dv]


def backward(q: Tensor, k: Tensor, v: Tensor, grad_attn: Tensor) -> List[Tensor]:
    """[grad_q, grad_k, grad_v] of causal RFA.

    Same contract as rfa_cuda.backward (reference cuda/rfa_cuda.cpp:30-36).
    """
    _check_qkv(q, k, v)
    _check_half_cuda("grad_attn", grad_attn, 3)
    _require(grad_attn.shape == v.shape, ValueError,
             lambda: f"grad_attn {tuple(grad_attn.shape)} must match v {tuple(v.shape)}")
    lib = _lib.load()
    T, N, K = q.shape
    d = v.shape[2]
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    with _on_device(q.device):
        nbytes = lib.rfa_causal_backward_workspace_bytes(T, N, K, d)
        ws = _workspace(nbytes, q.device)
        _lib.check(lib.rfa_causal_backward(q.data_ptr(), k.data_ptr(), v.data_ptr(), grad_attn.data_ptr(),
                                           dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                           T, N, K, d, ws.data_ptr(), nbytes, _stream_ptr(q.device)))
    return [dq, dk, dv]


# ---------------------------------------------------------------------------
# feature map
# ---------------------------------------------------------------------------
def feature_map_supported(D: int, d: int) -> bool:
    return bool(_lib.load().rfa_feature_map_supported(int(D), int(d)))


def _check_feature_args(x: Tensor, w: Tensor):
    _check_half_cuda("x", x, 4)
    _check_half_cuda("random_matrices", w, 3)
    _require(w.shape[0] == x.shape[2] and w.shape[2] == x.shape[3], ValueError,
             lambda: f"random_matrices {tuple(w.shape)} must be [num_heads, proj_dim, head_dim] for x {tuple(x.shape)}")
    _require(x.device == w.device, RuntimeError, lambda: "x and random_matrices must be on one device")


def build_random_matrices(w: Tensor, sigma: Optional[Tensor], tau: float) -> Tensor:
    """W' = (sigma * w if sigma is not None) / tau in one launch; w fp16 [H, D, d], sigma fp16 [H, 1, d]."""
    _check_half_cuda("random_matrices", w, 3)
    H, D, d = w.shape
    if sigma is not None:
        _check_half_cuda("sigma", sigma, 3)
        _require(tuple(sigma.shape) == (H, 1, d), ValueError, lambda: f"sigma must be [{H}, 1, {d}] (got {tuple(sigma.shape)})")
    out = torch.empty_like(w)
    with _on_device(w.device):
        _lib.check(_lib.load().rfa_build_random_matrices(
            w.data_ptr(), None if sigma is None else sigma.data_ptr(), float(tau), out.data_ptr(), H, D, d,
            _stream_ptr(w.device)))
    return out


def build_random_matrices_backward(w: Tensor, sigma: Optional[Tensor], grad_out: Tensor, tau: float,
                                   want_dsigma: bool, want_dw: bool):
    """(dsigma fp16 [H, 1, d] or None, dw fp16 [H, D, d] or None) for grad_out fp16 [H, D, d]."""
    _check_half_cuda("random_matrices", w, 3)
    _check_half_cuda("grad_out", grad_out, 3)
    _require(grad_out.shape == w.shape, ValueError, lambda: "grad_out must have the shape of random_matrices")
    H, D, d = w.shape
    want_dsigma = bool(want_dsigma and sigma is not None)
    dsigma = torch.empty((H, 1, d), dtype=torch.float16, device=w.device) if want_dsigma else None
    dw = torch.empty_like(w) if want_dw else None
    with _on_device(w.device):
        _lib.check(_lib.load().rfa_build_random_matrices_backward(
            w.data_ptr(), None if sigma is None else sigma.data_ptr(), grad_out.data_ptr(), float(tau),
            None if dsigma is None else dsigma.data_ptr(), None if dw is None else dw.data_ptr(), H, D, d,
            _stream_ptr(w.device)))
    return dsigma, dw


def feature_map_forward(x: Tensor, w: Tensor, scale: float) -> Tensor:
    """phi [L, B, H, 2D] for x fp16 [L, B, H, d] and w fp16 [H, D, d]."""
    _check_feature_args(x, w)
    L, B, H, d = x.shape
    D = w.shape[1]
    phi = torch.empty((L, B, H, 2 * D), dtype=torch.float16, device=x.device)
    with _on_device(x.device):
        _lib.check(_lib.load().rfa_feature_map_forward(
            x.data_ptr(), w.data_ptr(), phi.data_ptr(), L * B, H, D, d, float(scale), _stream_ptr(x.device)))
    return phi


def feature_map_forward_pair(x0: Tensor, x1: Tensor, w: Tensor, scale: float):
    """(phi(x0), phi(x1)) through the same w in one launch; x0, x1 fp16 of one shape [L, B, H, d]."""
    _check_feature_args(x0, w)
    _check_feature_args(x1, w)
    _require(x0.shape == x1.shape and x0.device == x1.device, ValueError,
             lambda: f"x0 {tuple(x0.shape)} and x1 {tuple(x1.shape)} must have one shape and device")
    L, B, H, d = x0.shape
    D = w.shape[1]
    phi0 = torch.empty((L, B, H, 2 * D), dtype=torch.float16, device=x0.device)
    phi1 = torch.empty_like(phi0)
    with _on_device(x0.device):
        _lib.check(_lib.load().rfa_feature_map_forward_pair(
            x0.data_ptr(), x1.data_ptr(), w.data_ptr(), phi0.data_ptr(), phi1.data_ptr(), L * B, H, D, d, float(scale),
            _stream_ptr(x0.device)))
    return phi0, phi1


def project_feature_map(x: Tensor, weights, biases, want_phi, w: Optional[Tensor], heads: int, scale: float,
                        keep_y: bool = True):
    """Linear projections of x to heads, with the feature map applied to some of them, in one launch.

    x fp16 [L, B, E]; weights: 1..3 fp16 [heads*d, E] (torch.nn.Linear.weight); biases: a matching
    list of fp16 [heads*d] or None entries; want_phi: one bool per projection; w fp16 [heads, D, d]
    (None allowed when no phi is wanted).  Returns (ys, phis): ys[p] fp16 [L, B, heads, d];
    phis[p] fp16 [L, B, heads, 2D] or None.  keep_y=False: ys[p] is None (and never written) where
    phis[p] is produced -- for callers that will not differentiate through the feature map.
    """
    import ctypes
    _check_half_cuda("x", x, 3)
    L, B, E = x.shape
    n = len(weights)
    _require(1 <= n <= 3 and len(biases) == n and len(want_phi) == n, ValueError,
             lambda: "1..3 projections with one bias entry and one want_phi flag each")
    out_dim = weights[0].shape[0]
    _require(out_dim % heads == 0, ValueError, lambda: f"output width {out_dim} is not a multiple of heads={heads}")
    d = out_dim // heads
    for wt, b in zip(weights, biases):
        _check_half_cuda("weight", wt, 2)
        _require(tuple(wt.shape) == (out_dim, E), ValueError, lambda: f"weight {tuple(wt.shape)} must be {(out_dim, E)}")
        _require(wt.device == x.device, RuntimeError, lambda: "x and weights must be on one device")
        if b is not None:
            _check_half_cuda("bias", b, 1)
            _require(b.shape[0] == out_dim and b.device == x.device, ValueError, lambda: f"bias must be [{out_dim}] on x's device")
    if any(want_phi):
        _require(w is not None, ValueError, lambda: "feature matrices are needed when a phi is wanted")
        _check_half_cuda("random_matrices", w, 3)
        _require(w.shape[0] == heads and w.shape[2] == d and w.device == x.device, ValueError,
                 lambda: f"random_matrices {tuple(w.shape)} must be [{heads}, D, {d}] on x's device")
        D = w.shape[1]
    else:
        D = 32
    ys = [torch.empty((L, B, heads, d), dtype=torch.float16, device=x.device) if keep_y or not f else None
          for f in want_phi]
    phis = [torch.empty((L, B, heads, 2 * D), dtype=torch.float16, device=x.device) if f else None for f in want_phi]
    arr = ctypes.c_void_p * n
    ptr = lambda t: None if t is None else t.data_ptr()
    with _on_device(x.device):
        _lib.check(_lib.load().rfa_project_feature_map(
            x.data_ptr(), arr(*[wt.data_ptr() for wt in weights]), arr(*[ptr(b) for b in biases]),
            arr(*[ptr(t) for t in ys]), arr(*[ptr(t) for t in phis]), n, ptr(w) if any(want_phi) else None,
            L * B, E, heads, D, d, float(scale), _stream_ptr(x.device)))
    return ys, phis


def linear_weight_grad_supported(e_out: int, e_in: int) -> bool:
    return e_out % 128 == 0 and e_in % 128 == 0


def linear_weight_grad(x: Tensor, dys, want_bias):
    """(dWs, dbs) of 1..3 Linear layers that share the input: dW_p = dy_p^T x, db_p = dy_p.sum(0).

    x fp16 [R, E_in]; dys: fp16 [R, E_out] each; want_bias: one bool per layer.  dWs[p] fp16
    [E_out, E_in]; dbs[p] fp16 [E_out] or None.  E_out and E_in must be multiples of 128.
    """
    import ctypes
    _check_half_cuda("x", x, 2)
    R, e_in = x.shape
    n = len(dys)
    _require(1 <= n <= 3 and len(want_bias) == n, ValueError, lambda: "1..3 layers with one want_bias flag each")
    e_out = dys[0].shape[1]
    for dy in dys:
        _check_half_cuda("dy", dy, 2)
        _require(tuple(dy.shape) == (R, e_out) and dy.device == x.device, ValueError,
                 lambda: f"dy {tuple(dy.shape)} must be {(R, e_out)} on x's device")
    _require(linear_weight_grad_supported(e_out, e_in), ValueError,
             lambda: f"E_out={e_out} and E_in={e_in} must be multiples of 128")
    lib = _lib.load()
    dws = [torch.empty((e_out, e_in), dtype=torch.float16, device=x.device) for _ in range(n)]
    dbs = [torch.empty((e_out,), dtype=torch.float16, device=x.device) if f else None for f in want_bias]
    arr = ctypes.c_void_p * n
    with _on_device(x.device):
        nbytes = lib.rfa_linear_weight_grad_workspace_bytes(max(R, 1), e_out, e_in, n)
        ws = _workspace(nbytes, x.device)
        _lib.check(lib.rfa_linear_weight_grad(
            x.data_ptr(), arr(*[t.data_ptr() for t in dys]), arr(*[t.data_ptr() for t in dws]),
            arr(*[None if t is None else t.data_ptr() for t in dbs]), n, R, e_out, e_in, ws.data_ptr(), nbytes,
            _stream_ptr(x.device)))
    return dws, dbs


def feature_map_backward(x: Tensor, w: Tensor, grad_phi: Tensor, scale: float, need_dw: bool = True):
    """(dx fp16 [L,B,H,d], dw fp32 [H,D,d]); with ``need_dw=False`` w counts as a constant: dw is None
    and neither formed nor reduced."""
    _check_feature_args(x, w)
    L, B, H, d = x.shape
    D = w.shape[1]
    _check_half_cuda("grad_phi", grad_phi, 4)
    _require(tuple(grad_phi.shape) == (L, B, H, 2 * D), ValueError,
             lambda: f"grad_phi {tuple(grad_phi.shape)} must be {(L, B, H, 2 * D)}")
    lib = _lib.load()
    dx = torch.empty_like(x)
    dw = torch.empty((H, D, d), dtype=torch.float32, device=x.device) if need_dw else None
    with _on_device(x.device):
        nbytes = lib.rfa_feature_map_backward_workspace_bytes(L * B, H, D, d) if need_dw else 0
        ws = _workspace(nbytes, x.device) if need_dw else None
        _lib.check(lib.rfa_feature_map_backward(
            x.data_ptr(), w.data_ptr(), grad_phi.data_ptr(), dx.data_ptr(), dw.data_ptr() if need_dw else None,
            L * B, H, D, d, float(scale), ws.data_ptr() if need_dw else None, nbytes, _stream_ptr(x.device)))
    return dx, dw


def feature_map_backward_pair(x0: Tensor, x1: Tensor, w: Tensor, grad_phi0: Tensor, grad_phi1: Tensor, scale: float,
                              need_dw: bool = True):
    """Two tensors that went through the same w in one launch: (dx0, dx1 fp16 [L,B,H,d], dw fp32 [H,D,d]
    = the sum of both contributions, or None with ``need_dw=False``)."""
    _check_feature_args(x0, w)
    _check_feature_args(x1, w)
    _require(x0.shape == x1.shape, ValueError, lambda: "the two tensors must have one shape")
    L, B, H, d = x0.shape
    D = w.shape[1]
    for name, g in (("grad_phi0", grad_phi0), ("grad_phi1", grad_phi1)):
        _check_half_cuda(name, g, 4)
        _require(tuple(g.shape) == (L, B, H, 2 * D), ValueError, lambda: f"{name} {tuple(g.shape)} must be {(L, B, H, 2 * D)}")
    lib = _lib.load()
    dx0, dx1 = torch.empty_like(x0), torch.empty_like(x1)
    dw = torch.empty((H, D, d), dtype=torch.float32, device=x0.device) if need_dw else None
    with _on_device(x0.device):
        nbytes = lib.rfa_feature_map_backward_pair_workspace_bytes(L * B, H, D, d) if need_dw else 0
        ws = _workspace(nbytes, x0.device) if need_dw else None
        _lib.check(lib.rfa_feature_map_backward_pair(
            x0.data_ptr(), x1.data_ptr(), w.data_ptr(), grad_phi0.data_ptr(), grad_phi1.data_ptr(), dx0.data_ptr(),
            dx1.data_ptr(), dw.data_ptr() if need_dw else None, L * B, H, D, d, float(scale),
            ws.data_ptr() if need_dw else None, nbytes, _stream_ptr(x0.device)))
    return dx0, dx1, dw


def feature_map_backward_pair_packed(x0: Tensor, x1: Tensor, w: Tensor, grad_phi0: Tensor, grad_phi1: Tensor,
                                     third: Optional[Tensor], scale: float, need_dw: bool = True):
    """feature_map_backward_pair that leaves [dx0 | dx1 | third] side by side in one fp16 [L*B, 3*H*d]
    matrix (third: [L, B, H, d] or [L*B, H*d], copied by the same launch; None leaves that block
    unset) and returns (packed, dw): the operand of one GEMM for the three input projections.
    ``need_dw=False``: dw is None, w counts as a constant."""
    _check_feature_args(x0, w)
    _check_feature_args(x1, w)
    _require(x0.shape == x1.shape, ValueError, lambda: "the two tensors must have one shape")
    L, B, H, d = x0.shape
    D = w.shape[1]
    for name, g in (("grad_phi0", grad_phi0), ("grad_phi1", grad_phi1)):
        _check_half_cuda(name, g, 4)
        _require(tuple(g.shape) == (L, B, H, 2 * D), ValueError, lambda: f"{name} {tuple(g.shape)} must be {(L, B, H, 2 * D)}")
    if third is not None:
        _check_half_cuda("third", third, third.dim())
        _require(third.numel() == x0.numel(), ValueError, lambda: f"third {tuple(third.shape)} must hold {L * B} rows of {H * d}")
    lib = _lib.load()
    packed = torch.empty((L * B, 3 * H * d), dtype=torch.float16, device=x0.device)
    dw = torch.empty((H, D, d), dtype=torch.float32, device=x0.device) if need_dw else None
    with _on_device(x0.device):
        nbytes = lib.rfa_feature_map_backward_pair_workspace_bytes(L * B, H, D, d) if need_dw else 0
        ws = _workspace(nbytes, x0.device) if need_dw else None
        _lib.check(lib.rfa_feature_map_backward_pair_packed(
            x0.data_ptr(), x1.data_ptr(), w.data_ptr(), grad_phi0.data_ptr(), grad_phi1.data_ptr(),
            None if third is None else third.data_ptr(), packed.data_ptr(), dw.data_ptr() if need_dw else None, L * B, H,
            D, d, float(scale), ws.data_ptr() if need_dw else None, nbytes, _stream_ptr(x0.device)))
    return packed, dw


# ---------------------------------------------------------------------------
# cross attention
# ---------------------------------------------------------------------------
def _check_f32_cuda(name: str, t: Tensor, shape):
    _require(isinstance(t, Tensor) and t.is_cuda, RuntimeError, lambda: f"{name} must live on a HIP device")
    _require(t.dtype == torch.float32, TypeError, lambda: f"{name} must be float32 (got {t.dtype})")
    _require(tuple(t.shape) == tuple(shape), ValueError, lambda: f"{name} must have shape {tuple(shape)} (got {tuple(t.shape)})")
    _require(t.is_contiguous(), ValueError, lambda: f"{name} must be contiguous")


def _mask_arg(mask, B: int, S: int, device):
    """key_padding_mask [B, S] (non-zero = pad) -> (uint8 tensor kept alive, pointer)."""
    if mask is None:
        return None, None
    _require(tuple(mask.shape) == (B, S), ValueError, lambda: f"key_padding_mask must be [{B}, {S}] (got {tuple(mask.shape)})")
    _require(mask.device == device, RuntimeError, lambda: "key_padding_mask must be on the tensors' device")
    # the kernels test the bytes for non-zero: a contiguous one-byte mask goes in as it is (no
    # conversion kernels in front of the launch), anything else is reduced to 0/1 bytes first
    if mask.dtype == torch.bool and mask.is_contiguous():
        m = mask.view(torch.uint8)
    elif mask.dtype == torch.uint8 and mask.is_contiguous():
        m = mask
    else:
        m = (mask != 0).to(torch.uint8).contiguous()
    return m, m.data_ptr()


def cross_state(phi_k: Tensor, v: Tensor, key_padding_mask=None):
    """phi_k fp16 [S, B, H, K], v fp16 [S, B, H, d], mask [B, S] -> (s fp32 [B,H,K,d], z fp32 [B,H,K])."""
    _check_half_cuda("phi_k", phi_k, 4)
    _check_half_cuda("v", v, 4)
    _require(phi_k.shape[:3] == v.shape[:3], ValueError, lambda: "phi_k and v must agree in [src_len, bsz, heads]")
    S, B, H, K = phi_k.shape
    d = v.shape[3]
    s = torch.empty((B, H, K, d), dtype=torch.float32, device=v.device)
    z = torch.empty((B, H, K), dtype=torch.float32, device=v.device)
    keep, mptr = _mask_arg(key_padding_mask, B, S, v.device)
    with _on_device(v.device):
        _lib.check(_lib.load().rfa_cross_state(phi_k.data_ptr(), v.data_ptr(), mptr, s.data_ptr(), z.data_ptr(),
                                               S, B, H, K, d, _stream_ptr(v.device)))
    return s, z


def cross_state_backward(phi_k: Tensor, v: Tensor, ds: Tensor, dz: Tensor, key_padding_mask=None):
    _check_half_cuda("phi_k", phi_k, 4)
    _check_half_cuda("v", v, 4)
    S, B, H, K = phi_k.shape
    d = v.shape[3]
    _check_f32_cuda("ds", ds, (B, H, K, d))
    _check_f32_cuda("dz", dz, (B, H, K))
    dphi_k, dv = torch.empty_like(phi_k), torch.empty_like(v)
    keep, mptr = _mask_arg(key_padding_mask, B, S, v.device)
    with _on_device(v.device):
        _lib.check(_lib.load().rfa_cross_state_backward(
            phi_k.data_ptr(), v.data_ptr(), mptr, ds.data_ptr(), dz.data_ptr(), dphi_k.data_ptr(), dv.data_ptr(),
            S, B, H, K, d, _stream_ptr(v.device)))
    return dphi_k, dv


def cross_readout(phi_q: Tensor, s: Tensor, z: Tensor) -> Tensor:
    """phi_q fp16 [T, B, H, K], s fp32 [B,H,K,d], z fp32 [B,H,K] -> attn fp16 [T, B, H, d]."""
    _check_half_cuda("phi_q", phi_q, 4)
    T, B, H, K = phi_q.shape
    _require(s.dim() == 4, ValueError, lambda: "s must be [bsz, heads, 2*proj_dim, head_dim]")
    d = s.shape[3]
    _check_f32_cuda("s", s, (B, H, K, d))
    _check_f32_cuda("z", z, (B, H, K))
    out = torch.empty((T, B, H, d), dtype=torch.float16, device=phi_q.device)
    with _on_device(phi_q.device):
        _lib.check(_lib.load().rfa_cross_readout(phi_q.data_ptr(), s.data_ptr(), z.data_ptr(), out.data_ptr(),
                                                 T, B * H, K, d, _stream_ptr(phi_q.device)))
    return out


def cross_readout_backward(phi_q: Tensor, s: Tensor, z: Tensor, grad_attn: Tensor):
    _check_half_cuda("phi_q", phi_q, 4)
    T, B, H, K = phi_q.shape
    d = s.shape[3]
    _check_f32_cuda("s", s, (B, H, K, d))
    _check_f32_cuda("z", z, (B, H, K))
    _check_half_cuda("grad_attn", grad_attn, 4)
    _require(tuple(grad_attn.shape) == (T, B, H, d), ValueError, lambda: "grad_attn must be [tgt_len, bsz, heads, head_dim]")
    dphi_q = torch.empty_like(phi_q)
    ds, dz = torch.empty_like(s), torch.empty_like(z)
    with _on_device(phi_q.device):
        _lib.check(_lib.load().rfa_cross_readout_backward(
            phi_q.data_ptr(), s.data_ptr(), z.data_ptr(), grad_attn.data_ptr(), dphi_q.data_ptr(),
            ds.data_ptr(), dz.data_ptr(), T, B * H, K, d, _stream_ptr(phi_q.device)))
    return dphi_q, ds, dz


# ---------------------------------------------------------------------------
# incremental decoding (state updated in place)
# ---------------------------------------------------------------------------
def incremental(phi_q: Tensor, phi_k: Tensor, v: Tensor, s: Tensor, z: Tensor, s_out: Optional[Tensor] = None,
                z_out: Optional[Tensor] = None) -> Tensor:
    """phi_q, phi_k fp16 [steps, N, K]; v fp16 [steps, N, d]; s fp32 [N,K,d], z fp32 [N,K].

    Without s_out / z_out the state is advanced in place; with them s and z are only read and the
    advanced state is written to s_out, z_out (same shapes, fp32)."""
    _check_qkv(phi_q, phi_k, v)
    steps, N, K = phi_q.shape
    d = v.shape[2]
    _check_f32_cuda("s", s, (N, K, d))
    _check_f32_cuda("z", z, (N, K))
    _require((s_out is None) == (z_out is None), ValueError, lambda: "s_out and z_out go together")
    if s_out is None:
        s_out, z_out = s, z
    else:
        _check_f32_cuda("s_out", s_out, (N, K, d))
        _check_f32_cuda("z_out", z_out, (N, K))
    out = torch.empty_like(v)
    with _on_device(v.device):
        _lib.check(_lib.load().rfa_incremental_out(phi_q.data_ptr(), phi_k.data_ptr(), v.data_ptr(), s.data_ptr(),
                                                   z.data_ptr(), s_out.data_ptr(), z_out.data_ptr(), out.data_ptr(),
                                                   steps, N, K, d, _stream_ptr(v.device)))
    return out


def incremental_fused(q: Tensor, k: Tensor, v: Tensor, w: Tensor, scale: float, s: Tensor, z: Tensor,
                      s_out: Optional[Tensor] = None, z_out: Optional[Tensor] = None) -> Tensor:
    """q, k, v fp16 [steps, B, H, d]; w fp16 [H, D, d]; s fp32 [B,H,2D,d], z fp32 [B,H,2D]: advanced in
    place, or only read when s_out / z_out (same shapes) are given to receive the advanced state."""
    for name, t in (("q", q), ("k", k), ("v", v)):
        _check_half_cuda(name, t, 4)
    _require(q.shape == k.shape == v.shape, ValueError, lambda: "q, k, v must have one shape [steps, bsz, heads, head_dim]")
    _check_half_cuda("random_matrices", w, 3)
    steps, B, H, d = q.shape
    D = w.shape[1]
    _require(w.shape[0] == H and w.shape[2] == d, ValueError, lambda: "random_matrices must be [heads, proj_dim, head_dim]")
    _check_f32_cuda("s", s, (B, H, 2 * D, d))
    _check_f32_cuda("z", z, (B, H, 2 * D))
    _require((s_out is None) == (z_out is None), ValueError, lambda: "s_out and z_out go together")
    if s_out is None:
        s_out, z_out = s, z
    else:
        _check_f32_cuda("s_out", s_out, (B, H, 2 * D, d))
        _check_f32_cuda("z_out", z_out, (B, H, 2 * D))
    out = torch.empty_like(v)
    with _on_device(v.device):
        _lib.check(_lib.load().rfa_incremental_fused_out(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), w.data_ptr(), float(scale), s.data_ptr(), z.data_ptr(),
            s_out.data_ptr(), z_out.data_ptr(), out.data_ptr(), steps, B, H, D, d, _stream_ptr(v.device)))
    return out


def incremental_qkv(qkv: Tensor, w: Tensor, scale: float, s: Tensor, z: Tensor,
                    s_out: Optional[Tensor] = None, z_out: Optional[Tensor] = None) -> Tensor:
    """incremental_fused for q, k, v that are the three thirds of one projection's output rows:
    qkv fp16 [steps, B, 3, H, d] (one Linear layer with the q, k, v weights stacked).  Returns
    attn fp16 [steps, B, H, d]."""
    _check_half_cuda("qkv", qkv, 5)
    _check_half_cuda("random_matrices", w, 3)
    steps, B, three, H, d = qkv.shape
    D = w.shape[1]
    _require(three == 3, ValueError, lambda: f"qkv must be [steps, bsz, 3, heads, head_dim] (got {tuple(qkv.shape)})")
    _require(w.shape[0] == H and w.shape[2] == d, ValueError, lambda: "random_matrices must be [heads, proj_dim, head_dim]")
    _check_f32_cuda("s", s, (B, H, 2 * D, d))
    _check_f32_cuda("z", z, (B, H, 2 * D))
    _require((s_out is None) == (z_out is None), ValueError, lambda: "s_out and z_out go together")
    if s_out is None:
        s_out, z_out = s, z
    else:
        _check_f32_cuda("s_out", s_out, (B, H, 2 * D, d))
        _check_f32_cuda("z_out", z_out, (B, H, 2 * D))
    out = torch.empty((steps, B, H, d), dtype=torch.float16, device=qkv.device)
    with _on_device(qkv.device):
        _lib.check(_lib.load().rfa_incremental_qkv(
            qkv.data_ptr(), w.data_ptr(), float(scale), s.data_ptr(), z.data_ptr(), s_out.data_ptr(), z_out.data_ptr(),
            out.data_ptr(), steps, B, H, D, d, _stream_ptr(qkv.device)))
    return out


# ---------------------------------------------------------------------------
# quadratic form with explicit masks (masked_rfa)
# ---------------------------------------------------------------------------
def pack_attn_mask(masked: Tensor):
    """bool [T, S] (True = masked) -> (bytes [T, Sp], bytes of the transpose [S, Tp]), rows padded
    to a multiple of 64 with ones, as rfa_masked_forward / rfa_masked_backward read them."""
    _require(masked.dim() == 2 and masked.shape[0] == masked.shape[1], ValueError,
             lambda: f"attn_mask must be [tgt_len, tgt_len] (got {tuple(masked.shape)})")
    T = masked.shape[0]
    Tp = (T + 63) // 64 * 64
    m = torch.ones((T, Tp), dtype=torch.uint8, device=masked.device)
    m[:, :T] = masked.to(torch.uint8)
    mt = torch.ones((T, Tp), dtype=torch.uint8, device=masked.device)
    mt[:, :T] = masked.t().to(torch.uint8)
    return m, mt


def masked_forward(phi_q: Tensor, phi_k: Tensor, v: Tensor, H: int, key_padding_mask=None, attn_mask_bytes=None):
    """(attn [T, N, d], rsum fp32 [T, N]).  phi_q, phi_k fp16 [T, N, K], v fp16 [T, N, d], N = B * H;
    key_padding_mask [B, T] (non-zero = pad) or None; attn_mask_bytes from pack_attn_mask()[0] or None."""
    _check_qkv(phi_q, phi_k, v)
    T, N, K = phi_q.shape
    d = v.shape[2]
    _require(N % H == 0, ValueError, lambda: f"N={N} is not a multiple of heads={H}")
    B = N // H
    Tp = (T + 63) // 64 * 64
    out = torch.empty_like(v)
    rsum = torch.empty((T, N), dtype=torch.float32, device=v.device)
    keep, mptr = _mask_arg(key_padding_mask, B, T, v.device)
    if attn_mask_bytes is not None:
        _require(attn_mask_bytes.is_cuda and attn_mask_bytes.dtype == torch.uint8 and attn_mask_bytes.is_contiguous()
                 and tuple(attn_mask_bytes.shape) == (T, Tp), ValueError, lambda: "attn_mask_bytes must come from pack_attn_mask")
    with _on_device(v.device):
        _lib.check(_lib.load().rfa_masked_forward(
            phi_q.data_ptr(), phi_k.data_ptr(), v.data_ptr(), mptr,
            attn_mask_bytes.data_ptr() if attn_mask_bytes is not None else None, out.data_ptr(), rsum.data_ptr(),
            T, Tp, B, H, K, d, _stream_ptr(v.device)))
    return out, rsum


def masked_backward(phi_q: Tensor, phi_k: Tensor, v: Tensor, grad_attn: Tensor, out: Tensor, rsum: Tensor, H: int,
                    key_padding_mask=None, attn_mask_bytes=None, attn_mask_t_bytes=None) -> List[Tensor]:
    """[dphi_q, dphi_k, dv] of masked_forward."""
    _check_qkv(phi_q, phi_k, v)
    _check_half_cuda("grad_attn", grad_attn, 3)
    _check_half_cuda("out", out, 3)
    T, N, K = phi_q.shape
    d = v.shape[2]
    B = N // H
    Tp = (T + 63) // 64 * 64
    _require(grad_attn.shape == v.shape and out.shape == v.shape, ValueError, lambda: "grad_attn and out must match v")
    _check_f32_cuda("rsum", rsum, (T, N))
    dq, dk, dv = torch.empty_like(phi_q), torch.empty_like(phi_k), torch.empty_like(v)
    keep, mptr = _mask_arg(key_padding_mask, B, T, v.device)
    lib = _lib.load()
    with _on_device(v.device):
        nbytes = lib.rfa_masked_backward_workspace_bytes(T, N, d)
        ws = _workspace(nbytes, v.device)
        _lib.check(lib.rfa_masked_backward(
            phi_q.data_ptr(), phi_k.data_ptr(), v.data_ptr(), grad_attn.data_ptr(), out.data_ptr(), rsum.data_ptr(),
            mptr, attn_mask_bytes.data_ptr() if attn_mask_bytes is not None else None,
            attn_mask_t_bytes.data_ptr() if attn_mask_t_bytes is not None else None,
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), T, Tp, B, H, K, d, ws.data_ptr(), nbytes,
            _stream_ptr(v.device)))
    return [dq, dk, dv]


# ---------------------------------------------------------------------------
# binding selection
# ---------------------------------------------------------------------------
_BOUND = ("supported", "feature_map_supported", "selftest_layout", "forward", "backward", "prefill", "forward_save",
          "backward_saved", "build_random_matrices", "build_random_matrices_backward", "feature_map_forward",
          "feature_map_forward_pair",
          "feature_map_backward", "feature_map_backward_pair", "feature_map_backward_pair_packed", "project_feature_map", "linear_weight_grad", "cross_state",
          "cross_state_backward", "cross_readout", "cross_readout_backward", "incremental", "incremental_fused",
          "incremental_qkv",
          "masked_forward", "masked_backward")
_CTYPES_IMPL = {name: globals()[name] for name in _BOUND}
_active = "ctypes"

_ext = None


def _resolve_ext():
    """Imports the torch binding if it is there.  Retried on every query while it is missing, so a
    process that imported this package before the binding was built (the build entry point does)
    finds it afterwards."""
    global _ext
    if _ext is None:
        import importlib
        try:
            mod = importlib.import_module(__package__ + "._rfa_hip_ext")   # built by rfa_amd.build.build_ext
        except ImportError:
            mod = None
        if mod is not None and not all(hasattr(mod, n) for n in _BOUND):
            # built from older sources than this file (the build itself imports the package first):
            # unusable until rebuilt, and a rebuilt file needs a fresh process to be loaded
            import warnings
            warnings.warn("rfa_amd._rfa_hip_ext is older than rfa_hip.py (missing entry points); using the ctypes "
                          "binding -- rebuild with `python -m rfa_amd.build`", RuntimeWarning)
            mod = None
        _ext = mod
    return _ext


def ext_available() -> bool:
    return _resolve_ext() is not None


def binding() -> str:
    """"ext" or "ctypes": which binding the functions of this module currently go through."""
    return _active


def use_binding(name: str) -> None:
    global _active
    if name == "ext":
        if _resolve_ext() is None:
            raise ImportError("the torch binding _rfa_hip_ext has not been built (python -m rfa_amd.build)")
        impl = {n: getattr(_ext, n) for n in _BOUND}
    elif name == "ctypes":
        impl = _CTYPES_IMPL
    else:
        raise ValueError(f"binding must be 'ext' or 'ctypes' (got {name!r})")
    globals().update(impl)
    _active = name


def _initial_binding() -> None:
    import os
    want = os.environ.get("RFA_AMD_BINDING", "ext" if _resolve_ext() is not None else "ctypes")
    use_binding(want)


_initial_binding()
