"""CPU restatement (torch, fp32/fp64 math) of the reference's sparse-attention hot path.

TEST INFRASTRUCTURE ONLY: the product package never imports this file.

Every function cites the reference lines it follows (paths relative to the
reference checkout).  Parity pinning of each function (what independent check a
plausible mistake would fail) is listed in ``tests/test_oracle.py``; all
functions here are pinned by closed forms, library routines or brute force, so
none is "parity unpinned" except for bf16 rounding details of the reference's
third-party Triton / ThunderKittens arithmetic, which only the reference's own
2e-2 ``allclose`` checks cover.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch
import torch.nn.functional as F

LOG2E = 1.4426950408889634

__all__ = [
    "LOG2E", "default_scale", "dense_attn", "dense_colsum_attn", "colsum_from_lse",
    "key_block_sums", "indices_count", "topk_index_list", "csp_attn_delta", "csp_attn",
    "block_sparse_attn", "block_mask_to_lists", "lists_to_block_mask",
    "map_inds_counts_across_scales", "local_window_indices", "crossscale_self_indices",
    "aggregate_group_indices", "upsample_ocache", "flex_block_mask", "infinity_cum",
    "INFINITY_SCALES", "config2_block_mask", "attn_flops_blocks",
    "topk_token_set", "append_local_run", "mask_to_lists", "window_key_scores",
    "video_window_block_mask", "base_plus_topk_block_mask", "expand_kv_heads",
]

# Infinity "1M" scale schedule, reference utils/dynamic_resolution.py:7 and
# models/sparvar/sparse_attn.py:893,909
INFINITY_SCALES = [1, 2, 4, 6, 8, 12, 16, 20, 24, 32, 40, 48, 64]


def infinity_cum(scales: Sequence[int] = INFINITY_SCALES) -> List[int]:
    """Prefix sums of tokens per scale (models/sparvar/sparse_attn.py:908-909)."""
    out = [0]
    for s in scales:
        out.append(out[-1] + s * s)
    return out


def default_scale(d: int, scale: Optional[float]) -> float:
    """``1/sqrt(d)`` when scale is None (kernels/sparse_attn/triton/attn_dense_colsum.py:247,
    kernels/sparse_attn/sparse_attn_ops.py:184)."""
    return 1.0 / math.sqrt(d) if scale is None else float(scale)


def _logits(q, k, scale, dtype):
    return torch.matmul(q.to(dtype), k.to(dtype).transpose(-1, -2)) * scale


def dense_attn(q, k, v, scale=None, dtype=torch.float32):
    """Dense softmax attention plus the base-2 pair (M, L).

    Follows kernels/sparse_attn/triton/attn_dense.py:87-183: ``M = max_n(qk*s*log2e)``,
    ``L = sum_n exp2(qk*s*log2e - M)``, ``o = softmax(qk*s) v``.
    Returns o [B,H,Lq,d], M [B,H,Lq,1], L [B,H,Lq,1] in ``dtype``.
    """
    s = default_scale(q.shape[-1], scale)
    t = _logits(q, k, s, dtype) * LOG2E
    M = t.max(dim=-1, keepdim=True).values
    e = torch.exp2(t - M)
    L = e.sum(dim=-1, keepdim=True)
    o = torch.matmul(e / L, v.to(dtype))
    return o, M, L


def dense_colsum_attn(q, k, v, scale=None, q_group_size=192, dtype=torch.float32):
    """``o`` and per-query-group column sums of the softmax probabilities.

    Follows naive_dense_colsum_attn (kernels/sparse_attn/sparse_attn_ops.py:179-200) and
    reference_blocksums (kernels/sparse_attn/triton/attn_dense_colsum.py:487-500):
    ``cs[b,h,g,n] = sum_{i in [g*G,(g+1)*G)} softmax(q k^T s)[b,h,i,n]``; rows beyond Lq add zero.
    Math is done in ``dtype`` (the reference runs it in the input dtype).
    Returns o, cs [B,H,ceil(Lq/G),Lk], (M, L).
    """
    B, H, Lq, d = q.shape
    Lk = k.shape[-2]
    o, M, L = dense_attn(q, k, v, scale, dtype)
    s = default_scale(d, scale)
    p = torch.exp2(_logits(q, k, s, dtype) * LOG2E - M) / L
    G = (Lq + q_group_size - 1) // q_group_size
    cs = torch.zeros(B, H, G, Lk, dtype=dtype)
    for g in range(G):
        cs[:, :, g] = p[:, :, g * q_group_size:min((g + 1) * q_group_size, Lq)].sum(dim=-2)
    return o, cs, (M, L)


def colsum_from_lse(q, k, M, L, scale=None, q_group_size=192, dtype=torch.float32):
    """Second pass of kernels/sparse_attn/triton/attn_dense_colsum.py:216-231 given (M, L):
    ``p = exp2(qk*s*log2e - M) / L`` column-reduced per group of ``q_group_size`` rows."""
    B, H, Lq, d = q.shape
    Lk = k.shape[-2]
    s = default_scale(d, scale)
    p = torch.exp2(_logits(q, k, s, dtype) * LOG2E - M.to(dtype)) / L.to(dtype)
    G = (Lq + q_group_size - 1) // q_group_size
    cs = torch.zeros(B, H, G, Lk, dtype=dtype)
    for g in range(G):
        cs[:, :, g] = p[:, :, g * q_group_size:min((g + 1) * q_group_size, Lq)].sum(dim=-2)
    return cs


def key_block_sums(cs, block_k=64):
    """Sum of colsum over blocks of ``block_k`` consecutive keys, ragged last block.
    Not in the reference (it ranks key tokens); defined by the benchmark configurations (per-64-key block sums of the colsum)."""
    Lk = cs.shape[-1]
    nb = (Lk + block_k - 1) // block_k
    pad = nb * block_k - Lk
    x = F.pad(cs, (0, pad))
    return x.view(*cs.shape[:-1], nb, block_k).sum(-1)


def indices_count(top_keys: float, Lk: int, multiple_of: int) -> int:
    """``m * round(top_keys*Lk/m)`` with Python's half-to-even ``round``
    (models/sparvar/sparse_attn.py:1012 and :913)."""
    return int(multiple_of * round((top_keys * Lk) / multiple_of))


def topk_index_list(bs, top_keys: float, multiple_of: int = 64, indices_pad_to: int = 1, bm: int = 192,
                    q_len: Optional[int] = None):
    """Full-step list build, models/sparvar/sparse_attn.py:1012-1036.

    ``bs`` [B,H,G,Lk] -> (inds int32 [B,H,G,Lk], counts int32 [B,H,G]).  The reference pads
    the list with uninitialised memory; here the padding is zero (columns >= count are never read).
    """
    B, H, G, Lk = bs.shape
    cnt = indices_count(top_keys, Lk, multiple_of)
    inds = torch.topk(bs, k=cnt, dim=-1).indices
    counts = torch.full((B, H, G), cnt, dtype=torch.int32)
    padding_amount = (Lk - cnt + indices_pad_to - 1) // indices_pad_to * indices_pad_to
    inds = torch.cat([inds.to(torch.int32), torch.zeros(B, H, G, padding_amount, dtype=torch.int32)], dim=-1)
    return inds[..., :Lk].contiguous(), counts


def csp_attn_delta(q, k, v, indices, counts, scale=None, bm=192, dtype=torch.float32):
    """Column-sparse attention over per-group key-token lists with MULTISET semantics.

    Follows kernels/sparse_attn/triton/attn_csp.py:30-100,140: query tile t (64 rows) uses
    group ``g = t // (bm/64)``; its keys are ``indices[b,h,g,:counts[b,h,g]]`` and duplicated
    indices are attended twice (the loop has no de-duplication).  ``count == 0`` yields a zero
    delta with (M, L) = (-inf, 1) (``l_i`` starts at 1.0, attn_csp.py:177).
    Returns delta [B,H,Lq,d], M, L.
    """
    B, H, Lq, d = q.shape
    s = default_scale(d, scale)
    out = torch.zeros(B, H, Lq, d, dtype=dtype)
    M = torch.full((B, H, Lq, 1), -float("inf"), dtype=dtype)
    L = torch.ones(B, H, Lq, 1, dtype=dtype)
    G = indices.shape[2]
    for b in range(B):
        for h in range(H):
            for g in range(G):
                lo, hi = g * bm, min((g + 1) * bm, Lq)
                if lo >= hi:
                    continue
                c = int(counts[b, h, g])
                if c == 0:
                    continue
                idx = indices[b, h, g, :c].long()
                kk = k[b, h].to(dtype)[idx]
                vv = v[b, h].to(dtype)[idx]
                t = (q[b, h, lo:hi].to(dtype) @ kk.T) * (s * LOG2E)
                m = t.max(dim=-1, keepdim=True).values
                e = torch.exp2(t - m)
                l = e.sum(dim=-1, keepdim=True)
                out[b, h, lo:hi] = (e / l) @ vv
                M[b, h, lo:hi] = m
                L[b, h, lo:hi] = l
    return out, M, L


def csp_attn(q, k, v, scale, indices, indices_counts, o, o_scale, bm=192, dtype=torch.float32):
    """``o + o_scale * delta`` (kernels/sparse_attn/sparse_attn_ops.py:273-292,
    epilogue kernels/sparse_attn/triton/attn_csp.py:209-211)."""
    delta, _, _ = csp_attn_delta(q, k, v, indices, indices_counts, scale, bm, dtype)
    return o.to(dtype) + float(o_scale) * delta


def block_sparse_attn(q, k, v, kv_num_blocks, kv_indices, block_q=128, block_k=64, scale=None, dtype=torch.float32):
    """Softmax attention restricted to a compacted per-query-block list of key blocks
    (flex ``BlockMask`` layout: kv_num_blocks [B,H,nQ], kv_indices [B,H,nQ,nKmax]; the
    reference consumes it through torch flex_attention, models/sparvar/basic_sparvar.py:55-72,187-194).
    Edge blocks are clipped to Lq / Lk.  A row with no block returns 0 with (M,L) = (-inf,1).
    """
    B, H, Lq, d = q.shape
    Lk = k.shape[-2]
    s = default_scale(d, scale)
    out = torch.zeros(B, H, Lq, d, dtype=dtype)
    M = torch.full((B, H, Lq, 1), -float("inf"), dtype=dtype)
    L = torch.ones(B, H, Lq, 1, dtype=dtype)
    nQ = (Lq + block_q - 1) // block_q
    for b in range(B):
        for h in range(H):
            for i in range(nQ):
                n = int(kv_num_blocks[b, h, i])
                if n == 0:
                    continue
                cols = []
                for j in kv_indices[b, h, i, :n].tolist():
                    cols.append(torch.arange(j * block_k, min((j + 1) * block_k, Lk)))
                idx = torch.cat(cols)
                if idx.numel() == 0:
                    continue
                lo, hi = i * block_q, min((i + 1) * block_q, Lq)
                t = (q[b, h, lo:hi].to(dtype) @ k[b, h].to(dtype)[idx].T) * (s * LOG2E)
                m = t.max(dim=-1, keepdim=True).values
                e = torch.exp2(t - m)
                l = e.sum(dim=-1, keepdim=True)
                out[b, h, lo:hi] = (e / l) @ v[b, h].to(dtype)[idx]
                M[b, h, lo:hi] = m
                L[b, h, lo:hi] = l
    return out, M, L


def block_mask_to_lists(mask):
    """bool [..., nQ, nK] -> (kv_num_blocks int32 [..., nQ], kv_indices int32 [..., nQ, nK]),
    ascending block order, unused tail = 0 (flex BlockMask convention,
    torch/nn/attention/flex_attention.py ``_dense_to_ordered``)."""
    m = mask.to(torch.int32)
    num = m.sum(-1).to(torch.int32)
    idx = torch.argsort(m, dim=-1, descending=True, stable=True).to(torch.int32)
    nK = mask.shape[-1]
    keep = torch.arange(nK).expand_as(idx) < num.unsqueeze(-1)
    return num, torch.where(keep, idx, torch.zeros_like(idx))


def lists_to_block_mask(num, idx, nK):
    mask = torch.zeros(*num.shape, nK, dtype=torch.bool)
    flat_m = mask.view(-1, nK)
    flat_n = num.reshape(-1)
    flat_i = idx.reshape(-1, idx.shape[-1])
    for r in range(flat_m.shape[0]):
        flat_m[r, flat_i[r, :int(flat_n[r])].long()] = True
    return mask


def map_inds_counts_across_scales(inds_S, counts_S, cur_q_len, cur_k_len, bm=192, indices_pad_to=1,
                                  add_sink=False, sink_len=0, sink_quota_frac=0.2):
    """Query-group remap between scales (models/sparvar/sparse_attn.py:366-469):
    ``gS = clamp(round((g+0.5)/Gk*Gs - 0.5), 0, Gs-1)`` with float32 arithmetic and round-half-to-even (torch.round).
    Without sink (:412-421): the first ``indices_count`` columns of the source row (cyclic ``repeat_interleave`` when
    the source is narrower), clamped to [0, Lk-1].
    With sink (:423-469): the first ``sink_quota = min(round(indices_count*frac), indices_count, sink_len)`` columns
    are the keys 0 .. sink_quota-1; the rest are the smallest entries >= ``sink_len`` of the WHOLE source row, in
    ascending order (entries below ``sink_len`` count as int32 max, so a row with too few large entries is filled up
    with that value; when the quota exceeds the row width every pick is repeated ``ceil(quota/Ks)`` times in place);
    then the clamp.  Pure-Python loops over rows."""
    B, H, Gs, Ks = inds_S.shape
    Gk = (cur_q_len + bm - 1) // bm
    raw = int(counts_S[0, 0, 0])
    cnt = max(indices_pad_to, (raw + indices_pad_to - 1) // indices_pad_to * indices_pad_to)
    out = torch.empty(B, H, Gk, cnt, dtype=torch.int32)
    sink = bool(add_sink) and sink_len > 0 and cnt > 0
    sink_quota = min(int(round(cnt * sink_quota_frac)), cnt, sink_len) if sink else 0
    big = int(np.iinfo(np.int32).max)
    for g in range(Gk):
        u = np.float32(np.float32(np.float32(g) + np.float32(0.5)) / np.float32(Gk)) * np.float32(Gs) - np.float32(0.5)
        gs = int(np.clip(np.rint(np.float32(u)), 0, Gs - 1))  # np.rint is half-to-even
        row = inds_S[:, :, gs]
        if not sink:
            if Ks >= cnt:
                out[:, :, g] = row[..., :cnt]
            else:
                rep = math.ceil(cnt / Ks)
                out[:, :, g] = row.repeat_interleave(rep, dim=-1)[..., :cnt]
            continue
        quota = cnt - sink_quota
        for b in range(B):
            for h in range(H):
                vals = sorted(int(x) if int(x) >= sink_len else big for x in row[b, h].tolist())
                if quota <= Ks:
                    pick = vals[:quota]
                else:
                    rep = math.ceil(quota / Ks)
                    pick = [x for x in vals for _ in range(rep)][:quota]
                full = list(range(sink_quota)) + pick
                out[b, h, g] = torch.tensor([min(x, big) for x in full], dtype=torch.int64).clamp(max=big).to(torch.int32)
    out.clamp_(0, max(0, cur_k_len - 1))
    counts = torch.full((B, H, Gk), cnt, dtype=torch.int32)
    return out, counts


def topk_token_set(scores, k):
    """Columns of the k largest entries of each row, ascending: the SET ``torch.topk(bs, k)`` selects
    in the full step (models/sparvar/sparse_attn.py:1016), with the one freedom torch leaves open
    (ties at the k-th value) fixed to "smaller column first", i.e. the first k entries of a stable
    descending sort.  ``scores`` [..., n] -> int32 [..., k]."""
    x = np.asarray(scores.detach().to(torch.float32).cpu().numpy())
    flat = x.reshape(-1, x.shape[-1])
    out = np.zeros((flat.shape[0], k), dtype=np.int32)
    for r in range(flat.shape[0]):
        order = np.argsort(-flat[r], kind="stable")      # descending by value, equal values by column
        out[r] = np.sort(order[:k])
    return torch.from_numpy(out.reshape(x.shape[:-1] + (k,)))


def append_local_run(inds, count, local_inds, local_count, k_len):
    """Sparse-step list: the first ``count`` remapped top-k keys followed by the scale's local run, zero
    padded to ``k_len`` columns (models/sparvar/sparse_attn.py:1096-1121).  inds [B,H,G,>=count],
    local_inds [G, local_count] -> (int32 [B,H,G,k_len], counts int32 [B,H,G])."""
    B, H, G, _ = inds.shape
    out = torch.zeros(B, H, G, k_len, dtype=torch.int32)
    for g in range(G):
        out[:, :, g, :count] = inds[:, :, g, :count].to(torch.int32)
        out[:, :, g, count:count + local_count] = local_inds[g, :local_count].to(torch.int32)
    return out, torch.full((B, H, G), count + local_count, dtype=torch.int32)


def mask_to_lists(mask, multiple_of=1):
    """Row-wise mask compaction with count padding, as the reference's mask_to_indices kernel
    (kernels/chipmunk/csrc/indexed_io/mask_to_indices.cu:21-97): ascending set columns, then the lowest
    unset columns until the count is a multiple of ``multiple_of`` (capped at the row length); the
    rest of the row is zero here (the reference leaves it untouched).  Pure-Python loops.
    bool [..., n] -> (counts int32 [...], indices int32 [..., n])."""
    m = np.asarray(mask.detach().cpu().numpy()).astype(bool)
    n = m.shape[-1]
    flat = m.reshape(-1, n)
    idx = np.zeros((flat.shape[0], n), dtype=np.int32)
    cnt = np.zeros((flat.shape[0],), dtype=np.int32)
    for r in range(flat.shape[0]):
        on = [j for j in range(n) if flat[r, j]]
        off = [j for j in range(n) if not flat[r, j]]
        padded = min(n, (len(on) + multiple_of - 1) // multiple_of * multiple_of)
        row = on + off[:padded - len(on)]
        idx[r, :len(row)] = row
        cnt[r] = len(row)
    return torch.from_numpy(cnt.reshape(m.shape[:-1])), torch.from_numpy(idx.reshape(m.shape))


def window_key_scores(q, k, window_keys, kernel_size=5, pooling="avgpool", dtype=torch.float32):
    """Masked, pooled key scores of ScaleKV's cache selection, models/scalekv/scale_kv.py:233-262: gather
    the window's queries (``local = clamp(window - (Lk - Lq), 0, Lq-1)``), logits against all keys divided
    by sqrt(d), ``-inf`` at the window's own keys, sum over the window queries, 1-D pool along the keys
    (padding ``kernel_size//2``, stride 1), ``-inf`` at the window keys again.  The reference does this
    in bf16 tensors; here in ``dtype``.  Returns [B,H,Lk]."""
    B, H, Lq, d = q.shape
    Lk = k.shape[2]
    local = torch.clamp(window_keys - (Lk - Lq), 0, Lq - 1)
    wq = torch.gather(q.to(dtype), 2, local.unsqueeze(-1).expand(-1, -1, -1, d))
    w = torch.matmul(wq, k.to(dtype).transpose(2, 3)) / math.sqrt(d)
    mask = torch.ones(B, H, 1, Lk, dtype=torch.bool)
    mask.scatter_(3, window_keys.unsqueeze(2), False)
    w = w.masked_fill(~mask, float("-inf"))
    s = w.sum(dim=2)
    if pooling == "avgpool":
        pooled = torch.nn.functional.avg_pool1d(s, kernel_size, padding=kernel_size // 2, stride=1)
    else:
        pooled = torch.nn.functional.max_pool1d(s, kernel_size, padding=kernel_size // 2, stride=1)
    pooled = pooled.clone()
    pooled.scatter_(2, window_keys, float("-inf"))
    return pooled


def local_window_indices(Hh, W, base, win):
    """Clamp-padded win x win window of absolute key indices for every query of an
    H x W grid (models/sparvar/sparse_attn.py:620-674, padding="clamp", dilation 1).
    Pure-Python loops (brute force).  Returns int64 [H*W, win*win]."""
    ry = (win - 1) // 2
    out = np.zeros((Hh * W, win * win), dtype=np.int64)
    for y in range(Hh):
        for x in range(W):
            c = 0
            for dy in range(-ry, win - ry):
                for dx in range(-ry, win - ry):
                    ny = min(max(y + dy, 0), Hh - 1)
                    nx = min(max(x + dx, 0), W - 1)
                    out[y * W + x, c] = ny * W + nx + base
                    c += 1
    return torch.from_numpy(out)


def crossscale_self_indices(scale_idx, win, scales=INFINITY_SCALES):
    """``build_crossscale_indices`` for the only spec the model uses, ``{0: (win, win)}``
    (models/sparvar/sparse_attn.py:678-768 as called at :925-927): the current scale's own
    window, then per-row sort + unique, right-padded with the row's last value."""
    cum = infinity_cum(scales)
    S = scales[scale_idx]
    raw = local_window_indices(S, S, cum[scale_idx], win)
    rows = [torch.unique(r) for r in raw]
    maxlen = max(int(r.numel()) for r in rows)
    out = torch.stack([torch.cat([r, r[-1:].repeat(maxlen - r.numel())]) for r in rows])
    return out, cum[scale_idx + 1]


def aggregate_group_indices(indices_abs, q_len, kv_len, bm=192, counts_multiple_of=None):
    """Per-group union -> count rounded up to a multiple -> ONE contiguous run per group,
    ``[tail-(L-1) .. tail]`` with ``tail = min(first_unique + L - 1, kv_len-1)``
    (models/sparvar/sparse_attn.py:778-857, in particular :845-855)."""
    idx = indices_abs.clamp(0, kv_len - 1)
    G = math.ceil(q_len / bm)
    firsts, cnts = [], []
    for g in range(G):
        u = torch.unique(idx[g * bm:min((g + 1) * bm, q_len)].reshape(-1))
        c = int(u.numel())
        if counts_multiple_of and counts_multiple_of > 1:
            c = (c + counts_multiple_of - 1) // counts_multiple_of * counts_multiple_of
        firsts.append(int(u[0]))
        cnts.append(c)
    Lrun = max(cnts)
    out = torch.empty(G, Lrun, dtype=torch.int64)
    for g in range(G):
        tail = min(firsts[g] + Lrun - 1, kv_len - 1)
        out[g] = torch.arange(tail - (Lrun - 1), tail + 1)
    return out, Lrun


def upsample_ocache(o_cache, L_src, L_tgt):
    """Bilinear, align_corners=False upsample of an O-cache laid out as an h x h token grid
    (models/sparvar/sparse_attn.py:324-362).  Written out as the closed-form half-pixel
    interpolation (fp64) so that library ``F.interpolate`` users can be checked against it."""
    B, H, _, Dh = o_cache.shape
    hs, ht = int(L_src ** 0.5), int(L_tgt ** 0.5)
    x = o_cache.to(torch.float64).view(B, H, hs, hs, Dh)
    sc = hs / ht

    def taps(n_out):
        i0, i1, w1 = [], [], []
        for t in range(n_out):
            src = max((t + 0.5) * sc - 0.5, 0.0)
            a = min(int(math.floor(src)), hs - 1)
            b = min(a + 1, hs - 1)
            i0.append(a); i1.append(b); w1.append(src - a)
        return torch.tensor(i0), torch.tensor(i1), torch.tensor(w1, dtype=torch.float64)

    a, b, w = taps(ht)
    rows = x[:, :, a] * (1 - w).view(1, 1, -1, 1, 1) + x[:, :, b] * w.view(1, 1, -1, 1, 1)
    out = rows[:, :, :, a] * (1 - w).view(1, 1, 1, -1, 1) + rows[:, :, :, b] * w.view(1, 1, 1, -1, 1)
    return out.reshape(B, H, ht * ht, Dh)


def flex_block_mask(q_scale_idx, kernel_schedule, attn_sink_scale, block_size=128, scales=INFINITY_SCALES,
                    block_k=None):
    """CSLA block mask (models/sparvar/basic_sparvar.py:74-185) by brute force over (q, kv):
    sink ``kv < cum[attn_sink_scale]`` OR a per-key-scale square window around the rescaled
    query position (``round(qy/Hq*Hk)`` computed in float32, half-to-even), negative kernel
    size => never attended; then ``any`` over block tiles.  ``scales``: side lengths or (h, w) pairs.
    Returns bool [nQ, nK]."""
    bq = block_size
    bk = block_size if block_k is None else block_k
    hw = [(s, s) if isinstance(s, int) else (s[0], s[1]) for s in scales]
    cum = [0]
    for h_, w_ in hw:
        cum.append(cum[-1] + h_ * w_)
    Hq, Wq = hw[q_scale_idx]
    Sq, Sk = Hq * Wq, cum[q_scale_idx + 1]
    sink = cum[attn_sink_scale] if attn_sink_scale > 0 else 0
    nQ, nK = (Sq + bq - 1) // bq, (Sk + bk - 1) // bk
    mask = np.zeros((nQ, nK), dtype=bool)
    for si in range(q_scale_idx + 1):
        Hk, Wk = hw[si]
        half = kernel_schedule[si] // 2  # python floor division: -1 // 2 == -1
        for kv in range(cum[si], cum[si + 1]):
            rel = kv - cum[si]
            ky, kx = rel // Wk, rel % Wk
            for qi in range(Sq):
                hit = kv < sink
                if not hit:
                    qy, qx = qi // Wq, qi % Wq
                    cy = np.rint(np.float32(np.float32(qy) / np.float32(Hq)) * np.float32(Hk))
                    cx = np.rint(np.float32(np.float32(qx) / np.float32(Wq)) * np.float32(Wk))
                    hit = abs(cy - ky) <= half and abs(cx - kx) <= half
                if hit:
                    mask[qi // bq, kv // bk] = True
    return torch.from_numpy(mask)


def config2_block_mask(colsum_blocks, block_q=128, block_k=64, density=0.25, sink_scale=7, window=2,
                       scales=INFINITY_SCALES):
    """Headline-benchmark mask for the last Infinity scale: key blocks of scales < ``sink_scale``
    (kv < cum[7] = 521) always kept, plus +-``window`` key blocks around the query block's
    rescaled position in every later scale, plus the top-ranked remainder by ``colsum_blocks``
    [B,H,nQ,nK] until ``round(density*nK)`` blocks per row.  Returns bool [B,H,nQ,nK]."""
    cum = infinity_cum(scales)
    Hq = scales[-1]
    Sq, Sk = Hq * Hq, cum[-1]
    nQ, nK = (Sq + block_q - 1) // block_q, (Sk + block_k - 1) // block_k
    B, H = colsum_blocks.shape[:2]
    base = np.zeros((nQ, nK), dtype=bool)
    base[:, :(cum[sink_scale] + block_k - 1) // block_k] = True
    for i in range(nQ):
        qc = min(i * block_q + block_q // 2, Sq - 1)
        qy, qx = qc // Hq, qc % Hq
        for si in range(sink_scale, len(scales)):
            Hk = scales[si]
            ky, kx = min(qy * Hk // Hq, Hk - 1), min(qx * Hk // Hq, Hk - 1)
            j = (cum[si] + ky * Hk + kx) // block_k
            lo_blk, hi_blk = cum[si] // block_k, (cum[si + 1] - 1) // block_k
            for jj in range(max(j - window, lo_blk), min(j + window, hi_blk) + 1):
                base[i, jj] = True
    target = int(round(density * nK))
    mask = torch.from_numpy(base).expand(B, H, nQ, nK).clone()
    score = colsum_blocks.clone().to(torch.float64)
    score[mask] = -float("inf")
    need = target - int(base.sum(-1).max())
    for i in range(nQ):
        extra = target - int(base[i].sum())
        if extra > 0:
            top = torch.topk(score[:, :, i], k=extra, dim=-1).indices
            mask[:, :, i].scatter_(-1, top, True)
    return mask


def attn_flops_blocks(kv_num_blocks, kv_indices, Lq, Lk, d, block_q, block_k):
    """``4*d*sum rows_i*cols_j`` over active blocks, edge blocks clipped."""
    B, H, nQ = kv_num_blocks.shape
    total = 0
    for b in range(B):
        for h in range(H):
            for i in range(nQ):
                rows = min(block_q, Lq - i * block_q)
                n = int(kv_num_blocks[b, h, i])
                js = kv_indices[b, h, i, :n].long()
                cols = torch.clamp(Lk - js * block_k, max=block_k).clamp(min=0).sum().item()
                total += rows * cols
    return 4 * d * total


def video_window_block_mask(frames=8, height=64, width=64, block=128, frame_radius=1, spatial_radius=1):
    """3D local-window block mask of the long-video benchmark configuration (no reference counterpart:
    the configuration is defined by the benchmark, tokens laid out frame by frame), by brute force over
    token pairs of every block pair: token t has frame ``t // (height*width)`` and spatial block
    ``(t % (height*width)) // block``; a block pair is kept if ANY of its token pairs is within
    ``frame_radius`` frames and ``spatial_radius`` spatial blocks.  bool [nQ, nK]."""
    per = height * width
    n = frames * per
    nb = (n + block - 1) // block
    tok = np.arange(n)
    fr, sb = tok // per, (tok % per) // block
    mask = np.zeros((nb, nb), dtype=bool)
    for i in range(nb):
        fi, si = fr[i * block:(i + 1) * block], sb[i * block:(i + 1) * block]
        for j in range(nb):
            fj, sj = fr[j * block:(j + 1) * block], sb[j * block:(j + 1) * block]
            # token pairs of the two blocks: distinct (frame, spatial block) combinations are enough
            pi = set(zip(fi.tolist(), si.tolist()))
            pj = set(zip(fj.tolist(), sj.tolist()))
            mask[i, j] = any(abs(a - c) <= frame_radius and abs(b - d_) <= spatial_radius for a, b in pi for c, d_ in pj)
    return torch.from_numpy(mask)


def base_plus_topk_block_mask(block_scores, base, target):
    """``base`` [nQ,nK] (always kept) plus, per row, the best-scoring other blocks until ``target`` blocks
    are kept; equal scores go to the smaller block index (the first entries of a stable descending sort).
    block_scores [B,H,nQ,nK] -> bool [B,H,nQ,nK]."""
    sc = np.asarray(block_scores.detach().to(torch.float32).cpu().numpy()).copy()
    bs = np.asarray(base.cpu().numpy()).astype(bool)
    B, H, nQ, nK = sc.shape
    out = np.broadcast_to(bs, sc.shape).copy()
    for i in range(nQ):
        extra = max(0, target - int(bs[i].sum()))
        if extra == 0:
            continue
        cand = np.where(~bs[i])[0]
        for b in range(B):
            for h in range(H):
                order = cand[np.argsort(-sc[b, h, i, cand], kind="stable")]
                out[b, h, i, order[:extra]] = True
    return torch.from_numpy(out)


def expand_kv_heads(k, qo_heads):
    """Grouped-query attention: K or V with ``kv_heads`` heads broadcast to ``qo_heads`` query heads, query head
    ``h`` reading K/V head ``h // (qo_heads // kv_heads)`` (kernels/sparse_attn/sparse_attn_ops.py:228-233:
    ``unsqueeze(2).expand(B, kv_h, hr, L, d).reshape(B, qo_h, L, d)``; kernels/chipmunk/csrc/attn/
    dense_colsum_attn.cu:106 ``kv_head_idx = blockIdx.y / hr``)."""
    B, kv_h, L, d = k.shape
    assert qo_heads % kv_h == 0, "qo_heads must be a multiple of kv_heads"
    hr = qo_heads // kv_h
    return k.unsqueeze(2).expand(B, kv_h, hr, L, d).reshape(B, qo_heads, L, d)
