"""ctypes binding of the C ABI declared in ``include/lvar_sparse_attn.h``.

The library is loaded from the source tree; there is no fallback path: if it is missing
the import of the operator module fails with instructions to build it.
"""
from __future__ import annotations

import ctypes as C
import os

from .build import LIB_PATH

EXPORTED_SYMBOLS = (
    "lvar_version", "lvar_target_arch", "lvar_status_string",
    "lvar_dense_attn_fwd", "lvar_dense_attn_rcp_fwd", "lvar_colsum_fwd", "lvar_csp_attn_fwd", "lvar_csp_attn_upsample_fwd",
    "lvar_block_sparse_attn_fwd",
    "lvar_attn_workspace_bytes", "lvar_attn_balanced_workgroups", "lvar_dense_attn_ws_fwd", "lvar_csp_attn_ws_fwd", "lvar_csp_attn_upsample_ws_fwd",
    "lvar_block_sparse_attn_ws_fwd", "lvar_block_sparse_attn_static_fwd",
    "lvar_block_topk_lists", "lvar_topk_token_lists", "lvar_remap_concat_lists", "lvar_mask_to_lists",
    "lvar_window_key_scores",
)


class LvarTensor(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("stride_b", C.c_int64), ("stride_h", C.c_int64), ("stride_row", C.c_int64)]


class LvarWorkspace(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("bytes", C.c_int64), ("min_share_tiles", C.c_int), ("min_piece_tiles", C.c_int)]


class LvarError(RuntimeError):
    def __init__(self, status: int, where: str, text: str):
        super().__init__(f"{where} failed with status {status}: {text}")
        self.status = status


_lib = None


def load() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    path = os.environ.get("LVAR_AMD_LIB", LIB_PATH)  # override for debug builds of the same ABI
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `python -m lvar_amd.build` (needs hipcc). "
            "lvar_amd has no CPU or PyTorch fallback.")
    lib = C.CDLL(path)
    T, P, I, I64, F = LvarTensor, C.c_void_p, C.c_int, C.c_int64, C.c_float
    lib.lvar_version.restype = I
    lib.lvar_version.argtypes = []
    lib.lvar_target_arch.restype = C.c_char_p
    lib.lvar_target_arch.argtypes = []
    lib.lvar_status_string.restype = C.c_char_p
    lib.lvar_status_string.argtypes = [I]
    lib.lvar_dense_attn_fwd.restype = I
    lib.lvar_dense_attn_fwd.argtypes = [T, T, T, T, P, P, P, I, I, I, I, I, I, F, P]
    lib.lvar_dense_attn_rcp_fwd.restype = I
    lib.lvar_dense_attn_rcp_fwd.argtypes = [T, T, T, T, P, I, I, I, I, I, I, F, P]
    lib.lvar_colsum_fwd.restype = I
    lib.lvar_colsum_fwd.argtypes = [T, T, P, P, P, I, I, I, I, I, I, I, F, P]
    lib.lvar_csp_attn_fwd.restype = I
    lib.lvar_csp_attn_fwd.argtypes = [T, T, T, T, T, P, P, P, P, I, I64, I, I, I, I, I, I, F, F, P]
    lib.lvar_csp_attn_upsample_fwd.restype = I
    lib.lvar_csp_attn_upsample_fwd.argtypes = [T, T, T, T, I, I, T, P, P, P, P, I, I64, I, I, I, I, I, I, F, F, P]
    lib.lvar_block_sparse_attn_fwd.restype = I
    lib.lvar_block_sparse_attn_fwd.argtypes = [T, T, T, T, P, P, P, I64, I64, P, I64, I64, I64, I, I, I, I, I, I, I, I, F, P]
    W = LvarWorkspace
    lib.lvar_attn_workspace_bytes.restype = I64
    lib.lvar_attn_workspace_bytes.argtypes = [I]
    lib.lvar_attn_balanced_workgroups.restype = I
    lib.lvar_attn_balanced_workgroups.argtypes = [I, I, I, I, I, I, I, I, I, W]
    lib.lvar_dense_attn_ws_fwd.restype = I
    lib.lvar_dense_attn_ws_fwd.argtypes = lib.lvar_dense_attn_fwd.argtypes[:-1] + [W, P]
    lib.lvar_csp_attn_ws_fwd.restype = I
    lib.lvar_csp_attn_ws_fwd.argtypes = lib.lvar_csp_attn_fwd.argtypes[:-1] + [W, P]
    lib.lvar_csp_attn_upsample_ws_fwd.restype = I
    lib.lvar_csp_attn_upsample_ws_fwd.argtypes = lib.lvar_csp_attn_upsample_fwd.argtypes[:-1] + [W, P]
    lib.lvar_block_sparse_attn_ws_fwd.restype = I
    lib.lvar_block_sparse_attn_ws_fwd.argtypes = lib.lvar_block_sparse_attn_fwd.argtypes[:-1] + [W, P]
    lib.lvar_block_sparse_attn_static_fwd.restype = I
    lib.lvar_block_sparse_attn_static_fwd.argtypes = lib.lvar_block_sparse_attn_fwd.argtypes
    lib.lvar_block_topk_lists.restype = I
    lib.lvar_block_topk_lists.argtypes = [P, P, P, P, I, I, I, I, I, P]
    lib.lvar_topk_token_lists.restype = I
    lib.lvar_topk_token_lists.argtypes = [P, I64, P, I64, P, I, I, I, I, P]
    lib.lvar_remap_concat_lists.restype = I
    lib.lvar_remap_concat_lists.argtypes = [P, I64, I, P, I64, I, P, I64, P, I, I, I, I, I, I, P]
    lib.lvar_mask_to_lists.restype = I
    lib.lvar_mask_to_lists.argtypes = [P, I64, P, I64, P, I, I, I, P]
    lib.lvar_window_key_scores.restype = I
    lib.lvar_window_key_scores.argtypes = [T, T, P, I, P, I, I, I, I, I, I, I, F, P]
    _lib = lib
    return lib


def check(status: int, where: str) -> None:
    if status != 0:
        raise LvarError(status, where, load().lvar_status_string(status).decode())


_binding = False      # False: not tried yet; None: not available


def torch_binding():
    """The compiled torch binding (``_lvar_torch.so`` next to this file), bound to the loaded C-ABI library, or
    None when it is not built, does not load, or ``LVAR_AMD_NO_TORCH_BINDING`` is set.  It only shortens the
    host side of ``dense_attn``; every call it declines goes through the ctypes path."""
    global _binding
    if _binding is not False:
        return _binding
    _binding = None
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_lvar_torch.so")
    if os.environ.get("LVAR_AMD_NO_TORCH_BINDING") or not os.path.exists(path):
        return None
    try:
        import importlib.util
        import torch  # noqa: F401  (the module links against libtorch)
        spec = importlib.util.spec_from_file_location("_lvar_torch", path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        lib = load()
        mod.bind(C.cast(lib.lvar_dense_attn_fwd, C.c_void_p).value, C.cast(lib.lvar_dense_attn_rcp_fwd, C.c_void_p).value)
        _binding = mod
    except Exception as e:     # a stale or incompatible module must not take the ctypes path down with it
        import warnings
        warnings.warn(f"lvar_amd: the compiled torch binding {path} did not load ({type(e).__name__}: {e}); "
                      "dense_attn runs through the slower ctypes path.  Rebuild it with `python -m lvar_amd.build`.",
                      RuntimeWarning, stacklevel=2)
        _binding = None
    return _binding
