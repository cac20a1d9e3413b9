"""rfa_amd: Random Feature Attention kernel path for AMD MI355X (gfx950).

Public names follow the reference package random_feature_attention: the ``RFA``
autograd Function, ``CausalAttention``, ``CrossAttention``,
``CrossAttentionProject`` and ``CrossAttentionState``.  All compute runs in
librfa_hip.so (see include/rfa_hip.h); build it with ``python -m rfa_amd.build``.
"""
from .causal_attention import CausalAttention, cuda_causal_rfa, incremental_rfa, masked_rfa
from .cross_attention import CrossAttention, CrossAttentionProject, CrossAttentionProjectLayer
from .rfa import RFA
from .utils import CrossAttentionState, build_random_matrices, random_project

__all__ = [
    "RFA", "CausalAttention", "CrossAttention", "CrossAttentionProject", "CrossAttentionProjectLayer",
    "CrossAttentionState", "build_random_matrices", "random_project", "cuda_causal_rfa",
    "incremental_rfa", "masked_rfa",
]
