"""Fastmax polynomial-kernel linear attention on MI355X (gfx950).

    from fastmax_amd import FASTMultiHeadAttention, fastmax_custom

mirrors the reference's operator API; the C ABI underneath is include/fastmax_amd.h.
"""
from .attention import (FASTMultiHeadAttention, FASTMultiHeadAttention_Function, FASTMultiHeadAttentionRPE,
                        fastmax_custom, fastmax_function, rpe_matrix_creator)
from ._ext import install_as_fastmax_cuda
from .rope import qkv_attention, qkv_rope_split

__all__ = ["FASTMultiHeadAttention", "FASTMultiHeadAttention_Function", "FASTMultiHeadAttentionRPE",
           "fastmax_custom", "fastmax_function", "install_as_fastmax_cuda", "qkv_attention", "qkv_rope_split", "rpe_matrix_creator"]
