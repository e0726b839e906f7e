"""Kernel-level ops under the names the reference exports from ``kernels/sparse_attn/triton/__init__.py:1-5``
(``csp_attn``, ``dense_attn``, ``dense_colsum_attn``), so that

    import lvar_amd.sattn_kernels as sattn_triton

replaces ``import kernels.sparse_attn.triton as sattn_triton`` (kernels/sparse_attn/sparse_attn_ops.py:7) and
the provider branches of the reference's wrappers run unedited.  All three launch the HIP library.
"""
from __future__ import annotations

from . import sparse_attn_ops as _ops

__all__ = ["csp_attn", "dense_attn", "dense_colsum_attn"]


def dense_attn(q, k, v, scale=None):
    """``(o, (M, L))`` (kernels/sparse_attn/triton/attn_dense.py:186-231)."""
    return _ops.dense_attn(q, k, v, scale)


def dense_colsum_attn(q, k, v, scale=None):
    """``(o, blocksums, (M, L))`` (kernels/sparse_attn/triton/attn_dense_colsum.py:237-296)."""
    return _ops.dense_colsum_attn(q, k, v, scale)


def csp_attn(q, k, v, sparsity_indices, sparsity_counts, O_scale=1.0, scale=None):
    """``(O_scale * delta, (M, L))``: the token-list attention accumulated onto zeros
    (kernels/sparse_attn/triton/attn_csp.py:215-265)."""
    return _ops.csp_attn_delta(q, k, v, sparsity_indices, sparsity_counts, O_scale, scale)
