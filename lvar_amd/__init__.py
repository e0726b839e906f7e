"""MI355X-native (gfx950) drop-in for the ``kernels.sparse_attn`` hot path of Lvar/SparVAR:
dense / block-sparse / column-sparse flash-attention forward and the colsum kernel, as
hand-written HIP kernels behind a C-ABI shared library (see ``include/lvar_sparse_attn.h``).

The operator API mirrors ``kernels/sparse_attn/sparse_attn_ops.py`` of the reference:

    from lvar_amd.sparse_attn_ops import dense_attn, dense_colsum_attn_s, dense_colsum_attn_q, csp_attn
"""
from . import sparse_attn_config  # noqa: F401

__all__ = ["sparse_attn_config", "sparse_attn_ops", "mask_build", "build"]
__version__ = "0.1.0"
