"""Operator API of the sparse-attention path, signature-compatible with the reference's
``kernels/sparse_attn/sparse_attn_ops.py`` (``dense_attn`` :21-59, ``dense_colsum_attn_s`` :65-113,
``dense_colsum_attn_q`` :119-149, ``csp_attn`` :273-292) and with the kernel-level functions of
``kernels/sparse_attn/triton/__init__.py`` (``dense_colsum_attn``, ``csp_attn_delta``; under the reference's own
names in :mod:`lvar_amd.sattn_kernels`).

Tensor contract: q ``[B,H,Lq,d]``, k/v ``[B,H,Lk,d]`` bf16 on a HIP device, unit stride on d;
``cs`` fp32 ``[B,H,ceil(Lq/bm),Lk]``; ``indices`` int32 ``[B,H,G,Lk]`` (valid prefix ``counts``),
``counts`` int32 ``[B,H,G]``; ``(M, L)`` fp32 ``[B,H,Lq,1]`` in the base-2 convention
``M = max(qk*scale*log2e)``, ``L = sum exp2(qk*scale*log2e - M)``.  Outputs are freshly allocated;
inputs are never written.  Work is enqueued on the current torch stream of the tensors' device.

All compute runs in the HIP library; there is no PyTorch or CPU fallback.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from . import _lib
from .sparse_attn_config import get_kernel_config_attn

__all__ = [
    "dense_attn", "dense_colsum_attn", "dense_colsum_attn_s", "dense_colsum_attn_q", "colsum",
    "csp_attn", "csp_attn_delta", "block_sparse_attn", "block_topk_lists", "mask_to_indices", "topk_indices", "ShapeError",
]


class ShapeError(AssertionError, ValueError):
    """Shape / dtype contract violation (the reference raises AssertionError at the same places)."""


def _require(cond: bool, msg) -> None:
    """``msg`` is a string or a zero-argument callable that builds it (so that hot paths do not
    format messages that are never shown)."""
    if not cond:
        raise ShapeError(msg() if callable(msg) else msg)


def _scale(q: torch.Tensor, scale) -> float:
    return 1.0 / math.sqrt(q.shape[-1]) if scale is None else float(scale)


def _pad_head_dim(q, k, v=None):
    """Head dimensions 16 and 32 (the reference's Triton kernels take {16, 32, 64, 128, 256},
    kernels/sparse_attn/triton/attn_dense_colsum.py:246) run on the 64-wide kernels with zero padding: zero
    columns add nothing to q.k, and the padded output columns (zero) are cut off again.  Returns the padded
    tensors and the original head_dim, or the inputs and None when no padding applies."""
    d = q.shape[-1]
    if d not in (16, 32) or q.dim() != 4:
        return q, k, v, None
    pad = (0, 64 - d)
    f = torch.nn.functional.pad
    return f(q, pad), f(k, pad), (None if v is None else f(v, pad)), d


def _scale_for(d: int, scale) -> float:
    return 1.0 / math.sqrt(d) if scale is None else float(scale)


def _prep(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.dtype is torch.bfloat16 and t.is_cuda and t.dim() == 4 and t.is_contiguous() and t.shape[-1] % 8 == 0 \
            and t.data_ptr() % 16 == 0:
        return t                                   # the common case, checked without walking the strides
    _require(t.dim() == 4, lambda: f"{name} must be [B,H,L,d], got {tuple(t.shape)}")
    if t.dtype != torch.bfloat16:
        raise TypeError(f"{name} must be bfloat16, got {t.dtype}")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on a HIP device; lvar_amd has no CPU path")
    if t.stride(-1) != 1 or any(s % 8 for s in t.stride()[:-1]) or t.data_ptr() % 16:
        t = t.contiguous()
    return t


def _view(t: Optional[torch.Tensor]) -> _lib.LvarTensor:
    if t is None:
        return _lib.LvarTensor(None, 0, 0, 0)
    return _lib.LvarTensor(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


def _check_qkv(q, k, v, gqa: bool = False):
    """``gqa``: the op supports grouped-query attention (fewer K/V heads than query heads, query head ``h`` reads
    K/V head ``h // (H // Hkv)``: the expansion of the reference's naive_dense_colsum_attn2,
    kernels/sparse_attn/sparse_attn_ops.py:228-233)."""
    # messages are only formatted on failure: these checks run on every call
    qs, ks = q.shape, k.shape
    if ks != v.shape:
        raise ShapeError(f"k/v shape mismatch: {tuple(k.shape)} vs {tuple(v.shape)}")
    if qs[0] != ks[0] or qs[3] != ks[3] or (qs[1] != ks[1] and not (gqa and ks[1] > 0 and qs[1] % ks[1] == 0)):
        raise ShapeError(f"q/k batch, head or head_dim mismatch: {tuple(q.shape)} vs {tuple(k.shape)}"
                         + ("" if gqa or qs[1] == ks[1] else " (this op takes as many K/V heads as query heads)"))
    if qs[3] != 128 and qs[3] != 64 and qs[3] != 256:
        raise ShapeError(f"head_dim must be 16, 32, 64, 128 or 256, got {q.shape[-1]}")
    if not (q.device == k.device == v.device):
        raise ShapeError("q, k, v must be on the same device")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor) -> int:
    """Raw handle of torch's current stream on the tensor's device."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index if t.device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


class _on_device:
    """``with _on_device(t):`` makes the tensor's device current for the launch, and does nothing
    (no guard object, no runtime calls) when it already is."""
    __slots__ = ("guard",)

    def __init__(self, t: torch.Tensor):
        idx = t.device.index
        self.guard = None if idx is None or idx == torch.cuda.current_device() else torch.cuda.device(idx)

    def __enter__(self):
        if self.guard is not None:
            self.guard.__enter__()

    def __exit__(self, *exc):
        if self.guard is not None:
            self.guard.__exit__(*exc)
        return False


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


# Partial-result workspaces of the balanced launches (``lvar_workspace_t``): one per (device, stream), allocated
# zero-filled on first use and kept for the life of the process (launches that share one must not overlap).
_workspaces = {}
_balanced = False
_NO_WORKSPACE = _lib.LvarWorkspace(None, 0, 0, 0)


def _set_balanced_launch(enabled: bool, min_share_tiles: int = 0, min_piece_tiles: int = 0) -> None:
    """Test and measurement hook, not part of the operator API: routes the attention operators through the
    ``*_ws_fwd`` entry points with a workspace, so that launches whose plain grid would fill the chip unevenly are cut
    into pieces (the balanced launch of the C ABI).  The operators themselves always take the plain launch: on a
    256-CU part the balanced one measures within +-10 % of it at the Infinity-2B shapes and mostly slower.  Callers
    that want it (few query tiles with very long lists) call the ``*_ws_fwd`` entry points with their own workspace.
    ``min_share_tiles`` / ``min_piece_tiles`` override the library defaults (0 = default)."""
    global _balanced
    _balanced = bool(enabled)
    for ws, _ in _workspaces.values():
        ws.min_share_tiles, ws.min_piece_tiles = int(min_share_tiles), int(min_piece_tiles)
    _workspaces_defaults[:] = [int(min_share_tiles), int(min_piece_tiles)]


_workspaces_defaults = [0, 0]


def _workspace(t: torch.Tensor, stream: int):
    if not _balanced:
        return _NO_WORKSPACE
    key = (t.device.index, stream)
    hit = _workspaces.get(key)
    if hit is None:
        if torch.cuda.is_current_stream_capturing():
            return _NO_WORKSPACE                     # no allocation inside a graph capture: plain launch
        with _on_device(t):
            nbytes = int(_lib.load().lvar_attn_workspace_bytes(128))
            if nbytes <= 0:
                return _NO_WORKSPACE
            buf = torch.zeros(nbytes, dtype=torch.uint8, device=t.device)
        hit = (_lib.LvarWorkspace(buf.data_ptr(), nbytes, _workspaces_defaults[0], _workspaces_defaults[1]), buf)
        _workspaces[key] = hit
    return hit[0]


def _dense_launch(q, k, v, scale, want_o=True, want_ml=True, want_lse2=False):
    B, H, Lq, d = q.shape
    Lk = k.shape[2]
    o = torch.empty((B, H, Lq, d), dtype=q.dtype, device=q.device) if want_o else None
    M = L = None
    if want_ml:
        M, L = torch.empty((2, B, H, Lq, 1), dtype=torch.float32, device=q.device).unbind(0)   # one allocation
    lse2 = torch.empty((B, H, Lq), dtype=torch.float32, device=q.device) if want_lse2 else None
    with _on_device(q):
        stream = _stream(q)
        st = _lib.load().lvar_dense_attn_ws_fwd(_view(q), _view(k), _view(v if want_o else None), _view(o), _ptr(M), _ptr(L),
                                               _ptr(lse2), B, H, k.shape[1], Lq, Lk, d, _scale(q, scale),
                                               _workspace(q, stream) if want_o else _NO_WORKSPACE, stream)
    _lib.check(st, "lvar_dense_attn_ws_fwd")
    return o, M, L, lse2


def dense_attn(q, k, v, scale=None):
    """Dense flash attention, ``(o, (M, L))`` (reference ``dense_attn``, sparse_attn_ops.py:21-59,
    Triton-provider return convention: ``lse`` is the tuple ``(M, L)``, each ``[B,H,Lq,1]``)."""
    fast = None if _balanced else _lib.torch_binding()   # (the compiled path takes no workspace)
    if fast is not None:
        # None unless the inputs are the plain contiguous bf16 case
        r = fast.fast_dense_attn(q, k, v, None if scale is None else float(scale)) if isinstance(q, torch.Tensor) else None
        if r is not None:
            return r[0], (r[1], r[2])
    q, k, v, d_small = _pad_head_dim(q, k, v)
    if d_small is not None:
        scale = _scale_for(d_small, scale)
    q, k, v = _prep(q, "q"), _prep(k, "k"), _prep(v, "v")
    _check_qkv(q, k, v, gqa=True)
    o, M, L, _ = _dense_launch(q, k, v, scale)
    return (o if d_small is None else o[..., :d_small].contiguous()), (M, L)


def _lse_only(q, k, scale):
    """Statistics sweep without the PV product: base-2 log-sum-exp ``M + log2(L)``, fp32 [B,H,Lq]."""
    return _dense_launch(q, k, None, scale, want_o=False, want_ml=False, want_lse2=True)[3]


def _colsum_given_lse(q, k, lse2, scale, q_group_size, want_block_sums=False):
    B, H, Lq, d = q.shape
    Lk = k.shape[2]
    G = (Lq + q_group_size - 1) // q_group_size
    cs = torch.empty((B, H, G, Lk), dtype=torch.float32, device=q.device)
    bs = torch.empty((B, H, G, (Lk + 63) // 64), dtype=torch.float32, device=q.device) if want_block_sums else None
    with _on_device(q):
        st = _lib.load().lvar_colsum_fwd(_view(q), _view(k), lse2.data_ptr(), cs.data_ptr(), _ptr(bs),
                                        B, H, k.shape[1], Lq, Lk, d, q_group_size, _scale(q, scale), _stream(q))
    _lib.check(st, "lvar_colsum_fwd")
    return (cs, bs) if want_block_sums else cs


def colsum(q, k, scale=None, q_group_size: Optional[int] = None, lse: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
           return_block_sums: bool = False):
    """Column sums of the softmax probabilities per group of ``q_group_size`` query rows
    (default: the kernel config's ``bm`` = 192), fp32 ``[B,H,G,Lk]``.  Self-contained two-pass form
    (statistics sweep, then column sweep) unless ``lse=(M, L)`` from a previous dense pass is given.
    With ``return_block_sums`` also returns the sums over blocks of 64 keys, ``[B,H,G,ceil(Lk/64)]``."""
    q, k, _, d_small = _pad_head_dim(q, k)
    if d_small is not None:
        scale = _scale_for(d_small, scale)
    q, k = _prep(q, "q"), _prep(k, "k")
    _check_qkv(q, k, k, gqa=True)
    if q_group_size is None:
        q_group_size = get_kernel_config_attn()["bm"]
    _require(q_group_size > 0 and q_group_size % 32 == 0, "q_group_size must be a positive multiple of 32")
    if lse is None:
        lse2 = _lse_only(q, k, scale)
    else:
        M, L = lse
        _require(M.numel() == q.shape[0] * q.shape[1] * q.shape[2] == L.numel(), "lse must be ([B,H,Lq,1], [B,H,Lq,1])")
        lse2 = (M.to(torch.float32) + torch.log2(L.to(torch.float32))).reshape(q.shape[:3]).contiguous()
    return _colsum_given_lse(q, k, lse2, scale, q_group_size, return_block_sums)


def dense_colsum_attn(q, k, v, scale=None):
    """Kernel-level op ``(o, blocksums, (M, L))`` (reference Triton ``dense_colsum_attn``,
    kernels/sparse_attn/triton/attn_dense_colsum.py:237-296): dense attention, then the column
    sweep that reuses its row statistics."""
    q, k, v, d_small = _pad_head_dim(q, k, v)
    if d_small is not None:
        scale = _scale_for(d_small, scale)
    q, k, v = _prep(q, "q"), _prep(k, "k"), _prep(v, "v")
    _check_qkv(q, k, v, gqa=True)
    o, M, L, lse2 = _dense_launch(q, k, v, scale, want_lse2=True)
    cs = _colsum_given_lse(q, k, lse2, scale, get_kernel_config_attn()["bm"])
    return (o if d_small is None else o[..., :d_small].contiguous()), cs, (M, L)


def dense_colsum_attn_s(q, k, v, scale=None):
    """``(o, cs)`` (reference ``dense_colsum_attn_s``, sparse_attn_ops.py:65-113)."""
    o, cs, (M, L) = dense_colsum_attn(q, k, v, scale)
    pad_to = get_kernel_config_attn()["bm"]
    assert M.shape == (q.shape[0], q.shape[1], q.shape[2], 1), "L shape mismatch"
    assert o.shape == q.shape, "Output shape mismatch"
    assert cs.shape == (q.shape[0], q.shape[1], (q.shape[-2] + pad_to - 1) // pad_to, k.shape[2]), "CS shape mismatch"
    return o, cs


def dense_colsum_attn_q(q, k, v, scale=None):
    """``(o, cs)`` (reference ``dense_colsum_attn_q``, sparse_attn_ops.py:119-149).  The reference
    keeps a separate "quality" variant because its CUDA colsum is bf16 and ignores ``scale``; here
    both variants are the same fp32, scale-honouring kernels."""
    return dense_colsum_attn_s(q, k, v, scale)


def _csp_launch(q, k, v, indices, counts, o_accum, o_scale, scale, want_stats, upsample_from=None, out=None):
    q, k, v, d_small = _pad_head_dim(q, k, v)
    if d_small is not None:
        if out is not None:
            raise ShapeError("the in-place op needs head_dim 64 or 128")
        scale = _scale_for(d_small, scale)
        if o_accum is not None:
            o_accum = torch.nn.functional.pad(o_accum, (0, 64 - d_small))
        res = _csp_launch(q, k, v, indices, counts, o_accum, o_scale, scale, want_stats, upsample_from)
        return (res[0][..., :d_small].contiguous(),) + tuple(res[1:])
    q, k, v = _prep(q, "q"), _prep(k, "k"), _prep(v, "v")
    _check_qkv(q, k, v)
    B, H, Lq, d = q.shape
    Lk = k.shape[2]
    bm = get_kernel_config_attn()["bm"]
    _require(indices.dim() == 4 and indices.shape[0] == B and indices.shape[1] == H,
             lambda: f"Indices shape mismatch - indices: {tuple(indices.shape)}, q: {tuple(q.shape)}")
    G = indices.shape[2]
    _require(G * bm >= Lq, lambda: f"indices has {G} query groups of {bm} rows, fewer than Lq={Lq}")
    _require(tuple(counts.shape) == tuple(indices.shape[:-1]),
             lambda: f"Indices counts shape mismatch - indices_counts: {tuple(counts.shape)}, indices: {tuple(indices.shape)}")
    if indices.dtype != torch.int32 or counts.dtype != torch.int32:
        raise TypeError("indices and indices_counts must be int32")
    _require(indices.device == q.device and counts.device == q.device, "indices / counts must be on q's device")
    if indices.stride(3) != 1 or indices.stride(1) != G * indices.stride(2) or indices.stride(0) != H * indices.stride(1):
        indices = indices.contiguous()
    counts = counts.contiguous()
    if o_accum is not None:
        if o_accum is not out:
            o_accum = _prep(o_accum, "o")
        if upsample_from is None:
            _require(o_accum.shape == q.shape, lambda: f"Output shape mismatch - o: {tuple(o_accum.shape)}, q: {tuple(q.shape)}")
        else:
            src, dst = upsample_from
            _require(dst * dst == Lq and tuple(o_accum.shape) == (B, H, src * src, d),
                     lambda: f"O-cache shape mismatch - o_cache: {tuple(o_accum.shape)}, expected {(B, H, src * src, d)} "
                     f"for a {src}x{src} -> {dst}x{dst} grid, q: {tuple(q.shape)}")
    # `out` (the in-place op): the caller's tensor is the destination; it may alias o_accum
    o = torch.empty((B, H, Lq, d), dtype=q.dtype, device=q.device) if out is None else out
    M = L = None
    if want_stats:
        M = torch.empty((B, H, Lq, 1), dtype=torch.float32, device=q.device)
        L = torch.empty_like(M)
    with _on_device(q):
        stream = _stream(q)
        if upsample_from is None:
            st = _lib.load().lvar_csp_attn_ws_fwd(_view(q), _view(k), _view(v), _view(o_accum), _view(o), _ptr(M), _ptr(L),
                                                 indices.data_ptr(), counts.data_ptr(), G, indices.stride(2), bm,
                                                 B, H, Lq, Lk, d, float(o_scale), _scale(q, scale), _workspace(q, stream), stream)
        else:
            st = _lib.load().lvar_csp_attn_upsample_ws_fwd(
                _view(q), _view(k), _view(v), _view(o_accum), int(upsample_from[0]), int(upsample_from[1]), _view(o),
                _ptr(M), _ptr(L), indices.data_ptr(), counts.data_ptr(), G, indices.stride(2), bm,
                B, H, Lq, Lk, d, float(o_scale), _scale(q, scale), _workspace(q, stream), stream)
    _lib.check(st, "lvar_csp_attn_ws_fwd" if upsample_from is None else "lvar_csp_attn_upsample_ws_fwd")
    return o, M, L


def csp_attn(q, k, v, scale, indices, indices_counts, o, o_scale):
    """``o + o_scale * softmax(q k[idx]^T scale) v[idx]`` with per-192-row-group key-token lists
    (reference ``csp_attn``, sparse_attn_ops.py:273-292).  Returns a new tensor; ``o`` is not
    modified (the reference's Triton behaviour).  The sum is formed in fp32 and rounded once."""
    _require(indices.dim() == 4 and indices.shape[-1] == k.shape[-2] and indices.shape[:2] == q.shape[:2],
             lambda: f"Indices shape mismatch - indices: {tuple(indices.shape)}, q: {tuple(q.shape)}, k: {tuple(k.shape)}")
    _require(tuple(o.shape) == tuple(q.shape), lambda: f"Output shape mismatch - o: {tuple(o.shape)}, q: {tuple(q.shape)}")
    out, _, _ = _csp_launch(q, k, v, indices, indices_counts, o, o_scale, scale, False)
    return out


def csp_attn_upsampled(q, k, v, scale, indices, indices_counts, o_cache, o_scale=1):
    """Sparse step with the O-cache resampled inside the attention epilogue:
    ``upsample(o_cache) + o_scale * softmax(q k[idx]^T scale) v[idx]`` where ``o_cache`` ``[B,H,h*h,d]``
    is the cached output of a coarser ``h x h`` scale and the queries form an ``h' x h'`` grid
    (``Lq = h'*h'``); the resampling is bilinear with half-pixel centres (``align_corners=False``).
    One launch and one rounding for ``upsample_Ocache(...).to(v.dtype)`` followed by ``csp_attn``
    (models/sparvar/sparse_attn.py:324-362, 1129-1142); the upsampled cache never goes to memory."""
    _require(indices.dim() == 4 and indices.shape[-1] == k.shape[-2] and indices.shape[:2] == q.shape[:2],
             lambda: f"Indices shape mismatch - indices: {tuple(indices.shape)}, q: {tuple(q.shape)}, k: {tuple(k.shape)}")
    _require(o_cache.dim() == 4, "o_cache must be [B,H,h*h,d]")
    src, dst = math.isqrt(o_cache.shape[-2]), math.isqrt(q.shape[-2])
    _require(src * src == o_cache.shape[-2] and dst * dst == q.shape[-2], "o_cache and q must hold square token grids")
    out, _, _ = _csp_launch(q, k, v, indices, indices_counts, o_cache, o_scale, scale, False, upsample_from=(src, dst))
    return out


def csp_attn_delta(q, k, v, sparsity_indices, sparsity_counts, O_scale=1.0, scale=None):
    """Kernel-level op ``(O_scale * delta, (M, L))`` (reference Triton ``csp_attn``,
    kernels/sparse_attn/triton/attn_csp.py:215-265, which accumulates onto zeros)."""
    out, M, L = _csp_launch(q, k, v, sparsity_indices, sparsity_counts, None, O_scale, scale, True)
    return out, (M, L)


def block_sparse_attn(q, k, v, kv_num_blocks, kv_indices, block_q: int = 128, block_k: int = 64, scale=None):
    """Block-sparse attention over a compacted per-query-block list of key blocks in the flex
    ``BlockMask`` layout consumed by ``SparseFlexAttn`` (models/sparvar/basic_sparvar.py:55-72,187-194):
    ``kv_num_blocks`` int32 ``[B|1,H|1,nQ]``, ``kv_indices`` int32 ``[B|1,H|1,nQ,nKmax]``.
    Returns ``(o, (M, L))``."""
    q, k, v, d_small = _pad_head_dim(q, k, v)
    if d_small is not None:
        o, ml = block_sparse_attn(q, k, v, kv_num_blocks, kv_indices, block_q, block_k, _scale_for(d_small, scale))
        return o[..., :d_small].contiguous(), ml
    q, k, v = _prep(q, "q"), _prep(k, "k"), _prep(v, "v")
    _check_qkv(q, k, v)
    B, H, Lq, d = q.shape
    Lk = k.shape[2]
    _require((block_q == 64 or (block_q > 0 and block_q % 128 == 0)) and block_k in (64, 128, 256),
             "block_q must be 64 or a multiple of 128, block_k 64, 128 or 256")
    nQ = (Lq + block_q - 1) // block_q
    _require(kv_num_blocks.dim() == 3 and kv_indices.dim() == 4, "kv_num_blocks must be [B,H,nQ], kv_indices [B,H,nQ,nKmax]")
    _require(kv_num_blocks.shape[2] == nQ and kv_indices.shape[2] == nQ,
             lambda: f"block list has {kv_num_blocks.shape[2]} query blocks, expected {nQ}")
    _require(kv_num_blocks.shape[0] in (1, B) and kv_num_blocks.shape[1] in (1, H)
             and tuple(kv_indices.shape[:2]) == tuple(kv_num_blocks.shape[:2]), "block list batch/head dims must be 1 or B/H")
    if kv_num_blocks.dtype != torch.int32 or kv_indices.dtype != torch.int32:
        raise TypeError("kv_num_blocks and kv_indices must be int32")
    kv_num_blocks = kv_num_blocks.contiguous()
    kv_indices = kv_indices.contiguous()
    nb_sb = kv_num_blocks.stride(0) if kv_num_blocks.shape[0] == B and B > 1 else 0
    nb_sh = kv_num_blocks.stride(1) if kv_num_blocks.shape[1] == H and H > 1 else 0
    ki_sb = kv_indices.stride(0) if kv_indices.shape[0] == B and B > 1 else 0
    ki_sh = kv_indices.stride(1) if kv_indices.shape[1] == H and H > 1 else 0
    o = torch.empty((B, H, Lq, d), dtype=q.dtype, device=q.device)
    M = torch.empty((B, H, Lq, 1), dtype=torch.float32, device=q.device)
    L = torch.empty_like(M)
    with _on_device(q):
        stream = _stream(q)
        st = _lib.load().lvar_block_sparse_attn_ws_fwd(
            _view(q), _view(k), _view(v), _view(o), M.data_ptr(), L.data_ptr(),
            kv_num_blocks.data_ptr(), nb_sb, nb_sh, kv_indices.data_ptr(), ki_sb, ki_sh, kv_indices.stride(2), kv_indices.shape[3],
            block_q, block_k, B, H, Lq, Lk, d, _scale(q, scale), _workspace(q, stream), stream)
    _lib.check(st, "lvar_block_sparse_attn_ws_fwd")
    return o, (M, L)


def block_topk_lists(block_scores, target: int, base_mask=None):
    """Block lists from block scores on the GPU: per ``[B,H,nQ]`` row keep the blocks of ``base_mask``
    (bool/uint8 ``[nQ,nK]``, optional) plus the best-scoring others up to ``target`` blocks; returns
    ``(kv_num_blocks int32 [B,H,nQ], kv_indices int32 [B,H,nQ,nK])`` in ascending block order with a
    zero tail, ready for :func:`block_sparse_attn`.  Ties go to the smaller block index."""
    _require(block_scores.dim() == 4, "block_scores must be [B,H,nQ,nK]")
    if not block_scores.is_cuda:
        raise RuntimeError("block_scores must live on a HIP device; lvar_amd has no CPU path")
    bs = block_scores.to(torch.float32).contiguous()
    B, H, nQ, nK = bs.shape
    _require(nK <= 2048, "at most 2048 key blocks per row")
    base = None
    if base_mask is not None:
        _require(tuple(base_mask.shape) == (nQ, nK), lambda: f"base_mask must be [nQ,nK] = {(nQ, nK)}")
        base = base_mask.to(device=bs.device, dtype=torch.uint8).contiguous()
    num = torch.empty((B, H, nQ), dtype=torch.int32, device=bs.device)
    idx = torch.empty((B, H, nQ, nK), dtype=torch.int32, device=bs.device)
    with _on_device(bs):
        st = _lib.load().lvar_block_topk_lists(bs.data_ptr(), _ptr(base), num.data_ptr(), idx.data_ptr(),
                                              B, H, nQ, nK, int(target), _stream(bs))
    _lib.check(st, "lvar_block_topk_lists")
    return num, idx


def topk_token_lists(scores, k: int, out_len: Optional[int] = None, order: str = "index", zero_tail: bool = True):
    """Exact top-``k`` key columns of every row of ``scores`` (fp32 ``[..., Lk]``, e.g. the column sums
    ``[B,H,G,Lk]``) on the GPU: returns ``(indices int32 [..., out_len], counts int32 [...])`` with the
    selected columns in the first ``k`` entries (``out_len`` defaults to ``Lk``, the width the list
    attention op expects; entries beyond ``k`` are zero, or left as allocated with ``zero_tail=False``: nothing reads
    them).  ``order="index"`` (default, one kernel)
    lists them in ascending column order, which is also the best order for the gather kernel;
    ``order="value"`` re-orders them by descending score like ``torch.topk``
    (models/sparvar/sparse_attn.py:1016).  Ties at the k-th value go to the smaller column."""
    _require(scores.dim() >= 1, "scores must have a key axis")
    if not scores.is_cuda:
        raise RuntimeError("scores must live on a HIP device; lvar_amd has no CPU path")
    _require(order in ("index", "value"), "order must be 'index' or 'value'")
    sc = scores.to(torch.float32).contiguous()
    Lk = sc.shape[-1]
    rows = sc.numel() // Lk if Lk else 0
    k = int(k)
    _require(0 <= k <= Lk, lambda: f"k = {k} must lie in [0, Lk = {Lk}]")
    out_len = Lk if out_len is None else int(out_len)
    _require(out_len >= k, "out_len must be at least k")
    idx = torch.empty(sc.shape[:-1] + (out_len,), dtype=torch.int32, device=sc.device)   # the kernel zeroes the tail
    cnt = torch.empty(sc.shape[:-1], dtype=torch.int32, device=sc.device)
    with _on_device(sc):
        st = _lib.load().lvar_topk_token_lists(sc.data_ptr(), Lk, idx.data_ptr(), out_len, cnt.data_ptr(),
                                              rows, Lk, k, out_len if zero_tail else k, _stream(sc))
    _lib.check(st, "lvar_topk_token_lists")
    if order == "value" and k > 0:
        sel = idx[..., :k].long()
        vals = sc.gather(-1, sel)
        perm = torch.sort(vals, dim=-1, descending=True, stable=True).indices
        idx[..., :k] = sel.gather(-1, perm).to(torch.int32)
    return idx, cnt


def remap_concat_lists(src_indices, src_count: int, cur_q_len: int, cur_k_len: int, local_indices=None,
                       bm: int = 192, indices_pad_to: int = 1, out_len: Optional[int] = None, zero_tail: bool = True):
    """One-launch sparse-step key list: the decision-scale lists ``src_indices`` int32 ``[B,H,Gs,Ks]``
    (first ``src_count`` columns valid) are mapped to the ``Gk = ceil(cur_q_len / bm)`` query groups of the
    current scale (nearest group centre, half-to-even), clamped to ``[0, cur_k_len)``, and followed by
    the rows of ``local_indices`` int64 ``[Gk, L]`` (optional).  Returns ``(indices int32 [B,H,Gk,out_len],
    counts int32 [B,H,Gk])``; ``out_len`` defaults to ``cur_k_len``.  The columns behind the list are zero unless
    ``zero_tail`` is false: then they are left as allocated (the reference pads with ``torch.empty``,
    models/sparvar/sparse_attn.py:1113-1117; nothing reads them), which saves writing the full-width rows.  Equals
    ``append_local_run(map_inds_counts_across_scales(...))`` of :mod:`lvar_amd.mask_build`
    (models/sparvar/sparse_attn.py:366-421, 1096-1121)."""
    _require(src_indices.dim() == 4, "src_indices must be [B,H,Gs,Ks]")
    if not src_indices.is_cuda:
        raise RuntimeError("src_indices must live on a HIP device; lvar_amd has no CPU path")
    src = src_indices.to(torch.int32).contiguous()
    B, H, Gs, Ks = src.shape
    Gk = (int(cur_q_len) + bm - 1) // bm
    raw = int(src_count)
    cnt = max(indices_pad_to, (raw + indices_pad_to - 1) // indices_pad_to * indices_pad_to)
    L = 0
    loc = None
    if local_indices is not None:
        _require(local_indices.dim() == 2 and local_indices.shape[0] == Gk, lambda: f"local_indices must be [Gk = {Gk}, L]")
        loc = local_indices.to(device=src.device, dtype=torch.int64).contiguous()
        L = loc.shape[1]
    out_len = int(cur_k_len) if out_len is None else int(out_len)
    _require(cnt + L <= out_len, lambda: f"list length {cnt + L} exceeds the output width {out_len}")
    out = torch.empty((B, H, Gk, out_len), dtype=torch.int32, device=src.device)    # the kernel zeroes the tail (zero_tail)
    counts = torch.empty((B, H, Gk), dtype=torch.int32, device=src.device)
    with _on_device(src):
        st = _lib.load().lvar_remap_concat_lists(src.data_ptr(), Ks, Ks, _ptr(loc), L, L, out.data_ptr(), out_len,
                                                counts.data_ptr(), B * H, Gs, Gk, cnt, int(cur_k_len),
                                                out_len if zero_tail else cnt + L, _stream(src))
    _lib.check(st, "lvar_remap_concat_lists")
    return out, counts


def mask_to_lists(mask, multiple_of: int = 1):
    """Compaction of a boolean mask ``[..., n]`` on the GPU: ``(counts int32 [...], indices int32 [..., n])``
    with the ascending set columns first, the count rounded up to ``multiple_of`` with the lowest unset
    columns as padding, and a zero tail.  For a block mask ``[B,H,nQ,nK]`` and ``multiple_of = 1`` these are
    the flex ``BlockMask`` lists ``(kv_num_blocks, kv_indices)`` taken by :func:`block_sparse_attn`.
    Counterpart of the reference's ``mask_to_indices`` (kernels/chipmunk/csrc/indexed_io/mask_to_indices.cu:21-97):
    the same set, but in ascending order (the reference's order is thread-strided) and with the padded count
    capped at ``n`` (the reference's rounded count can exceed the row)."""
    if not mask.is_cuda:
        raise RuntimeError("mask must live on a HIP device; lvar_amd has no CPU path")
    # a bool tensor is one byte per entry with the values 0 / 1: viewed, not converted
    m = (mask.contiguous().view(torch.uint8) if mask.dtype == torch.bool else mask.ne(0).view(torch.uint8).contiguous())
    n = m.shape[-1]
    rows = m.numel() // n if n else 0
    idx = torch.empty(m.shape, dtype=torch.int32, device=m.device)
    cnt = torch.empty(m.shape[:-1], dtype=torch.int32, device=m.device)
    with _on_device(m):
        st = _lib.load().lvar_mask_to_lists(m.data_ptr(), n, idx.data_ptr(), n, cnt.data_ptr(), rows, n,
                                           int(multiple_of), _stream(m))
    _lib.check(st, "lvar_mask_to_lists")
    return cnt, idx


def mask_to_indices(mask, multiple_of: int, pad_to_multiple_of: int = 192):
    """``[indices, counts]`` of a boolean mask ``[b,h,m,n]`` (reference ``mask_to_indices``, sparse_attn_ops.py:402-407,
    kernels/chipmunk/csrc/indexed_io/mask_to_indices.cu:96-141): ``indices`` int32 ``[b,h,m,pad_n]`` with ``pad_n`` =
    ``n`` rounded up to ``pad_to_multiple_of``, ``counts`` int32 ``[b,h,m]`` = the number of set columns rounded up to
    ``multiple_of``, the padding entries being the lowest unset columns.  The set columns come in ascending order
    (the reference's order is thread-strided) and the padded count is capped at ``n``; columns from the count on are
    zero up to ``n`` and left as allocated beyond (the reference leaves all of them as allocated)."""
    _require(mask.dim() == 4, "mask must be 4-dimensional [b, h, m, n]")
    if mask.dtype != torch.bool:
        raise TypeError("mask must be bool type")
    if not mask.is_cuda:
        raise RuntimeError("mask must live on a HIP device; lvar_amd has no CPU path")
    _require(multiple_of >= 1 and pad_to_multiple_of >= 1, "multiple_of and pad_to_multiple_of must be positive")
    m = mask.contiguous().view(torch.uint8)
    b, h, rows_m, n = m.shape
    pad_n = (n + pad_to_multiple_of - 1) // pad_to_multiple_of * pad_to_multiple_of
    idx = torch.empty((b, h, rows_m, pad_n), dtype=torch.int32, device=m.device)
    cnt = torch.empty((b, h, rows_m), dtype=torch.int32, device=m.device)
    if n > 0 and cnt.numel() > 0:
        with _on_device(m):
            st = _lib.load().lvar_mask_to_lists(m.data_ptr(), n, idx.data_ptr(), pad_n, cnt.data_ptr(), b * h * rows_m, n,
                                               int(multiple_of), _stream(m))
        _lib.check(st, "lvar_mask_to_lists")
    return [idx, cnt]


def topk_indices(activations, indices_out, counts_out, sparsity_amount: float, multiple_of: int, rk: float = 0.0) -> None:
    """In-place counterpart of the reference's ``topk_indices`` (sparse_attn_ops.py:381-389,
    kernels/chipmunk/csrc/indexed_io/topk_indices.cu:26-175): for every row of ``activations`` ``[batch, rows, cols]``
    keep the columns at or above the ``sparsity_amount`` quantile, plus each other column with probability ``rk``,
    pad the count to a multiple of ``multiple_of`` with the lowest unselected columns, and write the list into
    ``indices_out`` int32 ``[batch, rows, cols]`` (entries beyond the count are left as the caller filled them) and the
    count into ``counts_out`` int32 ``[batch, rows]``.  ``sparsity_amount`` 0 keeps every column, 1 none.
    The reference estimates the quantile from the first 1024 entries of a row with a block sort; here it is exact over
    the whole row (radix select: the ``cols - int(cols * sparsity_amount)`` largest entries, ties to the smaller
    column), and the list is in ascending column order."""
    _require(activations.dim() == 3, "activation must be 3-dimensional [batch, rows, cols]")
    _require(indices_out.dim() == 3 and tuple(indices_out.shape) == tuple(activations.shape),
             "indices must be 3-dimensional [batch, rows, cols]")
    _require(counts_out.dim() == 2 and tuple(counts_out.shape) == tuple(activations.shape[:2]),
             "counts must be 2-dimensional [batch, rows]")
    _require(0.0 <= sparsity_amount <= 1.0, "sparsity_amount must be between 0 and 1")
    _require(multiple_of >= 1, "multiple_of must be positive")
    if not activations.is_cuda:
        raise RuntimeError("activation must live on a HIP device; lvar_amd has no CPU path")
    if indices_out.dtype != torch.int32 or counts_out.dtype != torch.int32 or not indices_out.is_contiguous() \
            or not counts_out.is_contiguous():
        raise TypeError("indices and counts must be contiguous int32 tensors")
    batch, rows, cols = activations.shape
    if sparsity_amount == 1.0:
        indices_out.fill_(-1)
        counts_out.zero_()
        return
    keep = cols - int(cols * float(sparsity_amount))
    sel, _ = topk_token_lists(activations, keep, out_len=cols, zero_tail=False)
    if rk <= 0.0 and keep % multiple_of == 0:
        indices_out[..., :keep] = sel[..., :keep]
        counts_out.fill_(keep)
        return
    mask = torch.zeros((1, batch, rows, cols), dtype=torch.bool, device=activations.device)
    mask[0].scatter_(-1, sel[..., :keep].long(), True)
    if rk > 0.0:
        mask |= torch.rand(mask.shape, device=mask.device) < float(rk)
    idx, cnt = mask_to_indices(mask, multiple_of, 1)
    width = torch.arange(cols, device=mask.device) < cnt[0].unsqueeze(-1)
    indices_out.copy_(torch.where(width, idx[0], indices_out))
    counts_out.copy_(cnt[0])


def window_key_scores(q, k, window_keys, kernel_size: int = 5, pooling: str = "avgpool", scale=None):
    """Scores of all keys against a small set of window queries, as ScaleKV's cache selection computes them
    (models/scalekv/scale_kv.py:233-262): the logits of the window's queries are summed per key (scaled by
    ``1/sqrt(d)`` unless ``scale`` is given), the window's own keys are set to ``-inf``, the result is pooled
    along the key axis (``avgpool`` with zero padding or ``maxpool``, odd ``kernel_size``, stride 1) and masked
    again.  ``q`` ``[B,H,Lq,d]`` are the queries of the newest ``Lq`` keys of ``k`` ``[B,H,Lk,d]``;
    ``window_keys`` int64 ``[B,H,W]`` are key positions.  Returns fp32 ``[B,H,Lk]``.  One pass over K."""
    q, k = _prep(q, "q"), _prep(k, "k")
    _check_qkv(q, k, k)
    B, H, Lq, d = q.shape
    Lk = k.shape[2]
    _require(Lq <= Lk, "q holds the queries of the newest keys: Lq must not exceed Lk")
    _require(pooling in ("avgpool", "maxpool"), "pooling must be 'avgpool' or 'maxpool'")
    _require(kernel_size % 2 == 1 and 1 <= kernel_size <= 33, "kernel_size must be odd and at most 33")
    _require(window_keys.dim() == 3 and tuple(window_keys.shape[:2]) == (B, H), "window_keys must be [B,H,W]")
    win = window_keys.to(device=q.device, dtype=torch.int64).contiguous()
    out = torch.empty((B, H, Lk), dtype=torch.float32, device=q.device)
    with _on_device(q):
        st = _lib.load().lvar_window_key_scores(_view(q), _view(k), win.data_ptr(), win.shape[2], out.data_ptr(),
                                               B, H, Lq, Lk, d, int(kernel_size), 1 if pooling == "maxpool" else 0,
                                               _scale(q, scale), _stream(q))
    _lib.check(st, "lvar_window_key_scores")
    return out


def scalekv_keep_indices(q, k, window_keys, max_capacity: int, kernel_size: int = 5, pooling: str = "avgpool"):
    """Key positions a ScaleKV-style cache keeps (models/scalekv/scale_kv.py:229-282): the window keys plus
    the ``max_capacity - W`` best-scoring other keys, ascending; int64 ``[B,H,min(max_capacity, Lk)]``.
    Scores and the top-k selection run in the HIP library (ties go to the smaller key position)."""
    B, H, W = window_keys.shape
    Lk = k.shape[2]
    keep = min(max(0, int(max_capacity) - W), Lk - W)
    if keep <= 0:
        return torch.sort(window_keys.to(torch.int64), dim=-1).values
    scores = window_key_scores(q, k, window_keys, kernel_size, pooling)
    rest, _ = topk_token_lists(scores, keep, out_len=keep)
    combined = torch.cat([rest.to(torch.int64), window_keys.to(device=rest.device, dtype=torch.int64)], dim=-1)
    return torch.sort(combined, dim=-1).values
