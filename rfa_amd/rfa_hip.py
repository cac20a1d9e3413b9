"""Python face of the kernel library: the module that stands where the
reference's pybind extension ``rfa_cuda`` stood
(random_feature_attention/cuda/rfa_cuda.cpp:39-42), with the same two entry
points ``forward(q, k, v)`` and ``backward(q, k, v, grad_attn)`` and the same
argument order and return arity, plus the entry points for the other parts of
the path.  Tensors are validated here (the reference validated nothing,
cuda/forward.cu:156-159) and handed to the C ABI as raw device pointers; the
work is enqueued on the current torch stream.
"""
from __future__ import annotations

from typing import List

import torch
from torch import Tensor

from . import _lib


def _require(cond: bool, exc, msg: str):
    if not cond:
        raise exc(msg)


def _check_half_cuda(name: str, t: Tensor, ndim: int):
    _require(isinstance(t, Tensor), TypeError, f"{name} must be a torch.Tensor")
    _require(t.is_cuda, RuntimeError,
             f"{name} must live on a HIP device (got {t.device}); the kernels have no CPU path")
    _require(t.dtype == torch.float16, TypeError, f"{name} must be float16 (got {t.dtype})")
    _require(t.dim() == ndim, ValueError, f"{name} must have {ndim} dims (got {tuple(t.shape)})")
    _require(t.is_contiguous(), ValueError, f"{name} must be contiguous")


def _stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


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
    _require(q.shape == k.shape, ValueError, f"q {tuple(q.shape)} and k {tuple(k.shape)} differ")
    _require(v.shape[:2] == q.shape[:2], ValueError,
             f"v {tuple(v.shape)} does not match q {tuple(q.shape)} in [tgt_len, bsz*heads]")
    _require(q.device == k.device == v.device, RuntimeError, "q, k, v must be on one device")


def forward(q: Tensor, k: Tensor, v: Tensor) -> Tensor:
    """attn[T, N, d] of causal RFA.  q, k: fp16 [T, N, K]; v: fp16 [T, N, d].

    Same contract as rfa_cuda.forward (reference cuda/rfa_cuda.cpp:22-27).
    """
    _check_qkv(q, k, v)
    lib = _lib.load()
    T, N, K = q.shape
    d = v.shape[2]
    out = torch.empty_like(v)
    with torch.cuda.device(q.device):
        nbytes = lib.rfa_causal_forward_workspace_bytes(T, N, K, d)
        ws = _workspace(nbytes, q.device)
        _lib.check(lib.rfa_causal_forward(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                          T, N, K, d, ws.data_ptr(), nbytes, _stream_ptr(q.device)))
    return out


def backward(q: Tensor, k: Tensor, v: Tensor, grad_attn: Tensor) -> List[Tensor]:
    """[grad_q, grad_k, grad_v] of causal RFA.

    Same contract as rfa_cuda.backward (reference cuda/rfa_cuda.cpp:30-36).
    """
    _check_qkv(q, k, v)
    _check_half_cuda("grad_attn", grad_attn, 3)
    _require(grad_attn.shape == v.shape, ValueError,
             f"grad_attn {tuple(grad_attn.shape)} must match v {tuple(v.shape)}")
    lib = _lib.load()
    T, N, K = q.shape
    d = v.shape[2]
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    with torch.cuda.device(q.device):
        nbytes = lib.rfa_causal_backward_workspace_bytes(T, N, K, d)
        ws = _workspace(nbytes, q.device)
        _lib.check(lib.rfa_causal_backward(q.data_ptr(), k.data_ptr(), v.data_ptr(), grad_attn.data_ptr(),
                                           dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                           T, N, K, d, ws.data_ptr(), nbytes, _stream_ptr(q.device)))
    return [dq, dk, dv]
