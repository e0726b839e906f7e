"""Mask / key-list construction around the sparse-attention kernels (host-side policy code).

Counterparts of the arithmetic in the reference's ``SparseDiffAttn`` and ``SparseFlexAttn``
(models/sparvar/sparse_attn.py, models/sparvar/basic_sparvar.py); every function works on the
device its inputs live on and is vectorised with torch, so it can run on the GPU between the
colsum kernel and the sparse-attention kernel without a host round trip.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F

from .sparse_attn_config import get_kernel_config_attn

INFINITY_SCALES = (1, 2, 4, 6, 8, 12, 16, 20, 24, 32, 40, 48, 64)

__all__ = [
    "INFINITY_SCALES", "scale_offsets", "indices_count", "topk_index_list", "map_inds_counts_across_scales",
    "local_group_runs", "append_local_run", "upsample_ocache", "flex_block_mask", "block_mask_to_lists",
    "key_block_sums", "topk_block_lists", "block_keep_count", "sink_window_base_mask", "sink_window_topk_block_mask",
    "video_window_base_mask", "video_window_topk_block_lists",
]


def scale_offsets(scales: Sequence[int] = INFINITY_SCALES) -> List[int]:
    """Start offset of every scale on the concatenated key axis (``cum`` of
    models/sparvar/sparse_attn.py:908-909): [0, 1, 5, 21, ..., 10521]."""
    offs = [0]
    for s in scales:
        offs.append(offs[-1] + s * s)
    return offs


def indices_count(top_keys: float, k_len: int, multiple_of: Optional[int] = None) -> int:
    """Number of keys kept per query group: ``m * round(top_keys * Lk / m)``, half-to-even
    (models/sparvar/sparse_attn.py:1012)."""
    m = get_kernel_config_attn()["counts_multiple_of"] if multiple_of is None else multiple_of
    return int(m * round((top_keys * k_len) / m))


def topk_index_list(bs: torch.Tensor, top_keys: float, multiple_of: Optional[int] = None,
                    indices_pad_to: Optional[int] = None, order: str = "value", zero_tail: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
    """Full-step list build (models/sparvar/sparse_attn.py:1012-1036): top-k of the colsum ``bs``
    [B,H,G,Lk] -> ``inds`` int32 [B,H,G,Lk] whose first ``count`` columns are valid, and ``counts``
    int32 [B,H,G].  Padding columns are zero-filled unless ``zero_tail`` is false (the reference leaves them
    uninitialised, sparse_attn.py:1031-1034; they are never read).  ``order="value"`` lists the keys by descending score as ``torch.topk`` does,
    ``order="index"`` by ascending key (same set; the attention kernels do not depend on the order
    and gather ascending lists faster).  The selection is the radix-select kernel
    (:func:`lvar_amd.sparse_attn_ops.topk_token_lists`, ties to the smaller key): ``bs`` must live on a HIP device."""
    cfg = get_kernel_config_attn()
    m = cfg["counts_multiple_of"] if multiple_of is None else multiple_of
    B, H, G, Lk = bs.shape
    cnt = indices_count(top_keys, Lk, m)
    if cnt > Lk:
        raise ValueError(f"top-k count {cnt} exceeds key length {Lk}")
    if order not in ("value", "index"):
        raise ValueError("order must be 'value' or 'index'")
    from . import sparse_attn_ops as ops
    return ops.topk_token_lists(bs, cnt, out_len=Lk, order=order, zero_tail=zero_tail)   # HIP tensors only


def map_inds_counts_across_scales(inds_S: torch.Tensor, counts_S, cur_q_len: int, cur_k_len: int,
                                  bm: int = 192, indices_pad_to: int = 1, add_sink: bool = False, sink_len: int = 0,
                                  sink_quota_frac: float = 0.2) -> Tuple[torch.Tensor, torch.Tensor]:
    """Nearest query-group remap of a key list from the decision scale to the current scale
    (models/sparvar/sparse_attn.py:366-469).  ``counts_S`` may be a tensor (its [0,0,0] element is read, one host
    sync as in the reference) or a Python int.  ``add_sink`` (the branch at :423-469, which no shipped
    configuration switches on): the first ``min(round(count*sink_quota_frac), count, sink_len)`` entries are the keys
    from 0 on, the others the smallest entries >= ``sink_len`` of the whole source row in ascending order.  The
    default path also exists as one kernel fused with the local-run append
    (:func:`lvar_amd.sparse_attn_ops.remap_concat_lists`); the sink path is torch on the lists' device."""
    B, H, Gs, Ks = inds_S.shape
    Gk = (cur_q_len + bm - 1) // bm
    raw = int(counts_S[0, 0, 0]) if torch.is_tensor(counts_S) else int(counts_S)
    cnt = max(indices_pad_to, (raw + indices_pad_to - 1) // indices_pad_to * indices_pad_to)
    centers = torch.arange(Gk, device=inds_S.device, dtype=torch.float32) + 0.5
    src = torch.round(centers / Gk * Gs - 0.5).to(torch.int64).clamp_(0, Gs - 1)
    templ = inds_S.index_select(2, src)
    counts = torch.full((B, H, Gk), cnt, dtype=torch.int32, device=inds_S.device)
    if not add_sink or sink_len <= 0 or cnt == 0:
        if Ks >= cnt:
            out = templ[..., :cnt].to(torch.int32)
        else:
            out = templ.repeat_interleave(math.ceil(cnt / Ks), dim=-1)[..., :cnt].to(torch.int32)
        return out.clamp(0, max(0, cur_k_len - 1)).contiguous(), counts
    sink_quota = min(int(round(cnt * sink_quota_frac)), cnt, sink_len)
    quota = cnt - sink_quota
    big = torch.iinfo(torch.int32).max
    vals = torch.where(templ >= sink_len, templ.to(torch.int64), torch.full_like(templ, big, dtype=torch.int64))
    vals = vals.sort(dim=-1).values                    # the smallest surviving entries first
    if quota > Ks:
        vals = vals.repeat_interleave(math.ceil(quota / Ks), dim=-1)
    head = torch.arange(sink_quota, device=inds_S.device, dtype=torch.int64).expand(B, H, Gk, sink_quota)
    out = torch.cat([head, vals[..., :quota]], dim=-1).clamp(0, max(0, cur_k_len - 1)).to(torch.int32)
    return out.contiguous(), counts


def local_group_runs(scale_idx: int, win: int, bm: int = 192, counts_multiple_of: Optional[int] = None,
                     scales: Sequence[int] = INFINITY_SCALES, device=None) -> Tuple[torch.Tensor, int]:
    """Local-window key run of every query group of scale ``scale_idx`` (the composition of
    ``local_window_indices``, ``build_crossscale_indices`` with ``{0: (win, win)}`` and
    ``aggregate_group_indices``, models/sparvar/sparse_attn.py:620-674, 678-768, 778-857, as used at
    :921-938): the union of the clamp-padded win x win windows of the group's queries fixes a
    first key and a count; the count, rounded up to ``counts_multiple_of`` and maximised over
    groups, gives ONE contiguous run ``[tail-(L-1), tail]``, ``tail = min(first+L-1, Lk-1)``.
    Returns (int64 [G, L], L)."""
    m = get_kernel_config_attn()["counts_multiple_of"] if counts_multiple_of is None else counts_multiple_of
    offs = scale_offsets(scales)
    S = scales[scale_idx]
    base, kv_len, q_len = offs[scale_idx], offs[scale_idx + 1], S * S
    ry = (win - 1) // 2
    d = torch.arange(-ry, win - ry, device=device)
    y = torch.arange(S, device=device)
    ny = (y[:, None] + d[None, :]).clamp_(0, S - 1)                        # [S, win]
    lin = (ny[:, None, :, None] * S + ny[None, :, None, :]).reshape(q_len, win * win) + base
    G = (q_len + bm - 1) // bm
    firsts, cnts = [], []
    for g in range(G):
        u = torch.unique(lin[g * bm:min((g + 1) * bm, q_len)])
        c = int(u.numel())
        if m and m > 1:
            c = (c + m - 1) // m * m
        firsts.append(int(u[0]))
        cnts.append(c)
    run = max(cnts)
    first = torch.tensor(firsts, device=device, dtype=torch.int64)
    tail = torch.clamp(first + (run - 1), max=kv_len - 1)
    out = (tail[:, None] - (run - 1)) + torch.arange(run, device=device, dtype=torch.int64)[None, :]
    return out, run


def append_local_run(inds: torch.Tensor, count: int, local_inds: torch.Tensor, local_count: int, k_len: int,
                     multiple_of: Optional[int] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Sparse-step list: remapped top-k keys followed by the scale's local run
    (models/sparvar/sparse_attn.py:1096-1121).  ``inds`` [B,H,G,count], ``local_inds`` [G,local_count]
    -> (int32 [B,H,G,k_len] zero-padded, counts int32 [B,H,G] = count + local_count)."""
    m = get_kernel_config_attn()["counts_multiple_of"] if multiple_of is None else multiple_of
    B, H, G, _ = inds.shape
    total = count + local_count
    assert total % m == 0, f"after add local sparse index, mismatch multiple_of={m}"
    if total > k_len:
        raise ValueError(f"list length {total} exceeds key length {k_len}")
    out = torch.zeros((B, H, G, k_len), dtype=torch.int32, device=inds.device)
    out[..., :count] = inds[..., :count]
    out[..., count:total] = local_inds.to(device=inds.device, dtype=torch.int32).expand(B, H, G, local_count)
    counts = torch.full((B, H, G), total, dtype=torch.int32, device=inds.device)
    return out, counts


def upsample_ocache(o_cache: torch.Tensor, L_src: int, L_tgt: int) -> torch.Tensor:
    """Bilinear (align_corners=False) upsample of an O-cache stored as an h x h token grid
    (``upsample_Ocache``, models/sparvar/sparse_attn.py:324-362)."""
    B, H, _, Dh = o_cache.shape
    hs, ht = int(L_src ** 0.5), int(L_tgt ** 0.5)
    x = o_cache.view(B, H, hs, hs, Dh).permute(0, 1, 4, 2, 3).reshape(B * H, Dh, hs, hs)
    x = F.interpolate(x, size=(ht, ht), mode="bilinear", align_corners=False)
    return x.view(B, H, Dh, ht, ht).permute(0, 1, 3, 4, 2).reshape(B, H, ht * ht, Dh)


def _hw(scales) -> List[Tuple[int, int]]:
    return [(int(s), int(s)) if isinstance(s, int) else (int(s[0]), int(s[1])) for s in scales]


def flex_block_mask(q_scale_idx: int, kernel_schedule: Sequence[int], attn_sink_scale: int, block_size: int = 128,
                    block_k: Optional[int] = None, scales: Sequence = INFINITY_SCALES, device=None) -> torch.Tensor:
    """Attention-sink + local-window block mask of ``SparseFlexAttn``
    (models/sparvar/basic_sparvar.py:74-185): a key is attended if it lies below
    ``cum[attn_sink_scale]`` or inside the square window (per-key-scale kernel size, negative =
    never) around the query position rescaled to the key's grid; a block is kept if any of its
    elements is.  ``scales`` holds side lengths or ``(h, w)`` pairs (the reference's
    ``scale_schedule``).  Returns bool [nQ, nK] for (block_size x block_k) blocks."""
    bq, bk = block_size, (block_size if block_k is None else block_k)
    hw = _hw(scales)[:q_scale_idx + 1]
    offs = [0]
    for h_, w_ in hw:
        offs.append(offs[-1] + h_ * w_)
    Hq, Wq = hw[q_scale_idx]
    Sq, Sk = Hq * Wq, offs[-1]
    sink = offs[attn_sink_scale] if attn_sink_scale > 0 else 0
    kv = torch.arange(Sk, device=device)
    bounds = torch.tensor(offs, device=device)
    si = torch.searchsorted(bounds, kv, right=True) - 1
    Hk = torch.tensor([h_ for h_, _ in hw], device=device)[si]
    Wk = torch.tensor([w_ for _, w_ in hw], device=device)[si]
    ksz = torch.tensor(list(kernel_schedule[:q_scale_idx + 1]), device=device)[si]
    rel = kv - bounds[si]
    ky, kx = rel // Wk, rel % Wk
    qi = torch.arange(Sq, device=device)
    qy, qx = (qi // Wq).float(), (qi % Wq).float()
    cy = torch.round((qy / Hq)[:, None] * Hk[None, :])
    cx = torch.round((qx / Wq)[:, None] * Wk[None, :])
    half = torch.div(ksz, 2, rounding_mode="floor")[None, :]
    fine = ((cy - ky[None, :]).abs() <= half) & ((cx - kx[None, :]).abs() <= half)
    fine |= (kv < sink)[None, :]
    pq, pk = (-Sq) % bq, (-Sk) % bk
    fine = F.pad(fine, (0, pk, 0, pq), value=False)
    return fine.view((Sq + pq) // bq, bq, (Sk + pk) // bk, bk).permute(0, 2, 1, 3).flatten(2).any(-1)


def block_mask_to_lists(mask: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """bool [..., nQ, nK] -> flex ``BlockMask`` lists: ``kv_num_blocks`` int32 [..., nQ] and
    ``kv_indices`` int32 [..., nQ, nK] (kept blocks first, ascending; unused tail zero): one compaction
    kernel (:func:`lvar_amd.sparse_attn_ops.mask_to_lists`); the mask must live on a HIP device."""
    from . import sparse_attn_ops as ops
    return ops.mask_to_lists(mask, 1)


def key_block_sums(cs: torch.Tensor, block_k: int = 64) -> torch.Tensor:
    """Sum of a colsum over blocks of ``block_k`` consecutive keys (ragged last block)."""
    Lk = cs.shape[-1]
    nb = (Lk + block_k - 1) // block_k
    return F.pad(cs, (0, nb * block_k - Lk)).unflatten(-1, (nb, block_k)).sum(-1)


def topk_block_lists(block_scores: torch.Tensor, keep_ratio: float, k_len: Optional[int] = None,
                     block_k: int = 64) -> Tuple[torch.Tensor, torch.Tensor]:
    """Best-scoring key blocks per row as ascending block lists.  The number kept follows the
    reference's token-count formula when ``k_len`` is given, ``block_k*round(keep_ratio*k_len/block_k)``
    tokens = that many blocks (models/sparvar/sparse_attn.py:1012), else ``round(keep_ratio*nK)``;
    at least one block is kept.  ``block_scores`` fp32 ``[B,H,nQ,nK]`` on a HIP device."""
    k = block_keep_count(keep_ratio, block_scores.shape[-1], k_len, block_k)
    from . import sparse_attn_ops as ops
    num, idx = ops.block_topk_lists(block_scores, k)          # HIP selection kernel; ties go to the smaller block
    return num, idx[..., :k].contiguous()


def block_keep_count(keep_ratio: float, n_blocks: int, k_len: Optional[int] = None, block_k: int = 64) -> int:
    """Key blocks kept per row by :func:`topk_block_lists`: the reference's token count
    ``block_k*round(keep_ratio*k_len/block_k)`` (models/sparvar/sparse_attn.py:1012) in blocks when ``k_len`` is
    given, else ``round(keep_ratio*n_blocks)``; at least one, at most all."""
    if k_len is not None:
        k = indices_count(keep_ratio, k_len, block_k) // block_k
    else:
        k = int(round(keep_ratio * n_blocks))
    return max(1, min(n_blocks, k))


def sink_window_base_mask(block_q: int = 128, block_k: int = 64, sink_scale: int = 7, window: int = 2,
                          scales: Sequence[int] = INFINITY_SCALES, device=None) -> torch.Tensor:
    """Score-independent part of the Infinity last-scale benchmark mask, bool [nQ, nK]: all key blocks
    of scales below ``sink_scale`` (keys < 521 for 7) and, in every later scale, +-``window`` key blocks
    around the query block's centre rescaled into that scale's grid."""
    offs = scale_offsets(scales)
    Hq = scales[-1]
    Sq, Sk = Hq * Hq, offs[-1]
    nQ, nK = (Sq + block_q - 1) // block_q, (Sk + block_k - 1) // block_k
    base = torch.zeros(nQ, nK, dtype=torch.bool, device=device)
    base[:, :(offs[sink_scale] + block_k - 1) // block_k] = True
    qc = torch.clamp(torch.arange(nQ, device=device) * block_q + block_q // 2, max=Sq - 1)
    qy, qx = qc // Hq, qc % Hq
    cols = torch.arange(nK, device=device)[None, :]
    for si in range(sink_scale, len(scales)):
        Hk = scales[si]
        ky = torch.clamp(qy * Hk // Hq, max=Hk - 1)
        kx = torch.clamp(qx * Hk // Hq, max=Hk - 1)
        j = (offs[si] + ky * Hk + kx) // block_k
        lo = torch.clamp(j - window, min=offs[si] // block_k)[:, None]
        hi = torch.clamp(j + window, max=(offs[si + 1] - 1) // block_k)[:, None]
        base |= (cols >= lo) & (cols <= hi)
    return base


def sink_window_topk_block_mask(block_scores: torch.Tensor, block_q: int = 128, block_k: int = 64, density: float = 0.25,
                                sink_scale: int = 7, window: int = 2, scales: Sequence[int] = INFINITY_SCALES) -> torch.Tensor:
    """Block mask of the Infinity last-scale benchmark configuration: :func:`sink_window_base_mask`,
    then the best-scoring remaining blocks by ``block_scores`` [B,H,nQ,nK] (colsum summed per query
    block and key block) up to ``round(density*nK)`` per row; ties go to the smaller block index.
    (The same selection runs on the GPU in ``sparse_attn_ops.block_topk_lists``.)"""
    base = sink_window_base_mask(block_q, block_k, sink_scale, window, scales, block_scores.device)
    nQ, nK = base.shape
    assert tuple(block_scores.shape[2:]) == (nQ, nK), (tuple(block_scores.shape), nQ, nK)
    target = int(round(density * nK))
    extra = (target - base.sum(-1)).clamp(min=0)                               # [nQ]
    score = block_scores.to(torch.float32).masked_fill(base, -float("inf"))
    rank = torch.argsort(torch.argsort(score, dim=-1, descending=True, stable=True), dim=-1, stable=True)
    return base | (rank < extra[None, None, :, None])


def video_window_base_mask(frames: int = 8, height: int = 64, width: int = 64, block: int = 128, frame_radius: int = 1,
                           spatial_radius: int = 1, device=None) -> torch.Tensor:
    """3D local-window block mask for video tokens laid out frame by frame (``frames x height x width``,
    row-major inside a frame), bool [nQ, nK] for ``block x block`` blocks: a key block is kept when it holds
    a token whose frame is within ``frame_radius`` frames and whose spatial block (``block`` consecutive
    tokens of a frame) is within ``spatial_radius`` of those of a token of the query block.  The frame length
    must be a multiple of ``block`` (every block then lies in one frame and is one spatial block)."""
    per_frame = height * width
    if per_frame % block:
        raise ValueError(f"tokens per frame ({per_frame}) must be a multiple of the block size ({block})")
    bpf = per_frame // block
    blk = torch.arange(frames * bpf, device=device)
    f, s = blk // bpf, blk % bpf
    return ((f[:, None] - f[None, :]).abs() <= frame_radius) & ((s[:, None] - s[None, :]).abs() <= spatial_radius)


def video_window_topk_block_lists(q: torch.Tensor, k: torch.Tensor, scale=None, density: float = 0.10, frames: int = 8,
                                  height: int = 64, width: int = 64, block: int = 128, query_stride: int = 4
                                  ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Block lists of the long-video configuration: :func:`video_window_base_mask` plus the best-scoring
    other key blocks per query block up to ``round(density * nK)`` blocks per row.  The scores are column
    sums of the softmax probabilities of every ``query_stride``-th query row, summed per key block (the
    colsum kernel and the block top-k kernel of the HIP library; ties go to the smaller block).  Returns
    ``(kv_num_blocks [B,H,nQ], kv_indices [B,H,nQ,nK], block_scores [B,H,nQ,nK])``."""
    from . import sparse_attn_ops as ops
    Lq, Lk = q.shape[2], k.shape[2]
    if Lq != frames * height * width or Lk != Lq:
        raise ValueError(f"expected Lq = Lk = {frames * height * width}, got {Lq}, {Lk}")
    if block % query_stride or (block // query_stride) % 32:
        raise ValueError("block / query_stride must be a multiple of 32 (the colsum group size)")
    nK = (Lk + block - 1) // block
    base = video_window_base_mask(frames, height, width, block, device=q.device)
    cs = ops.colsum(q[:, :, ::query_stride].contiguous(), k, scale, q_group_size=block // query_stride)
    score = key_block_sums(cs, block).contiguous()
    del cs
    num, idx = ops.block_topk_lists(score, int(round(density * nK)), base)
    return num, idx, score
