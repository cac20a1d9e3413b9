"""Random-matrix generator; mirror of random_feature_attention/construct_random_matrices.py.

    python -m rfa_amd.construct_random_matrices {rrf|orf} HEAD_DIM PROJ_DIM [OUT_DIR]

writes OUT_DIR/{HEAD_DIM}_{PROJ_DIM}.npy holding 500 matrices [proj_dim, head_dim]
drawn with numpy seed 31415 (construct_random_matrices.py:66-80).
"""
from __future__ import annotations

import os
import sys

import numpy as np


def rrf(*, head_dim: int, proj_dim: int, rng=np.random) -> np.ndarray:
    """Gaussian random features (reference :10-11)."""
    return rng.normal(loc=0.0, scale=1.0, size=(proj_dim, head_dim))


def orf(*, head_dim: int, proj_dim: int, rng=np.random) -> np.ndarray:
    """Orthogonal random features: QR of a Gaussian, rows rescaled by chi(proj_dim) draws (reference :14-21)."""
    assert proj_dim >= head_dim
    basis, _ = np.linalg.qr(rng.normal(loc=0.0, scale=1.0, size=(proj_dim, head_dim)))
    lengths = np.sqrt(rng.chisquare(df=proj_dim, size=proj_dim))
    return basis * lengths[: basis.shape[0], None]


def construct_random_matrices(feature_func, num_random_matrices: int, *, head_dim: int, proj_dim: int,
                              seed=None, rng=None) -> np.ndarray:
    """Stack of num_random_matrices draws.  ``rng`` (a numpy RandomState) keeps the draws off the
    global numpy generator; RandomState(s) yields the stream that np.random.seed(s) followed by the
    module-level functions yields.  ``seed`` without ``rng`` seeds the global generator, which is
    what the reference script does (construct_random_matrices.py:77)."""
    if rng is None:
        if seed is not None:
            np.random.seed(seed)
        rng = np.random
    return np.stack([feature_func(head_dim=head_dim, proj_dim=proj_dim, rng=rng) for _ in range(num_random_matrices)],
                    axis=0)


def softmax_kernel_error(head_dim: int, proj_dim: int, random_matrix: np.ndarray, tau: float = 0.7,
                         batch: int = 100, iters: int = 100) -> float:
    """Mean relative error of exp(q.k/tau^2) ~= e^{1/tau^2} phi(q).phi(k) with scale D^-1/2
    (the check in reference :40-57)."""
    w = random_matrix / tau
    err = 0.0
    for _ in range(iters):
        q = 3 * (np.random.normal(size=(batch, head_dim)) - 0.5)
        k = 10 * (np.random.normal(size=(batch, head_dim)) - 0.7)
        q /= np.linalg.norm(q, axis=-1, keepdims=True)
        k /= np.linalg.norm(k, axis=-1, keepdims=True)
        gold = np.exp((q * k).sum(-1) / tau ** 2)
        uq, uk = q @ w.T, k @ w.T
        pq = np.concatenate([np.sin(uq), np.cos(uq)], -1) * proj_dim ** -0.5
        pk = np.concatenate([np.sin(uk), np.cos(uk)], -1) * proj_dim ** -0.5
        pred = (pq * pk).sum(-1) * np.exp(1.0 / tau ** 2)
        err += np.linalg.norm(gold - pred) / np.linalg.norm(gold)
    return err / iters


if __name__ == "__main__":
    kind, head_dim, proj_dim = sys.argv[1], int(sys.argv[2]), int(sys.argv[3])
    out_dir = sys.argv[4] if len(sys.argv) > 4 else os.path.join(os.path.dirname(__file__), "../random_matrices")
    func = {"rrf": rrf, "orf": orf}[kind]
    mats = construct_random_matrices(func, 500, head_dim=head_dim, proj_dim=proj_dim, seed=31415)
    os.makedirs(out_dir, exist_ok=True)
    np.save(os.path.join(out_dir, f"{head_dim}_{proj_dim}"), mats)
