"""Pins the CPU oracle (oracle/sparse_attn_oracle.py) against things it does not itself define:
library routines (SDPA, logsumexp, F.interpolate, torch.sort), brute-force pure-Python loops on tiny
inputs, closed-form special cases and the known answers written in the reference's sources
(models/sparvar/sparse_attn.py:909,913,934; the VAR-d16 benchmark case).  The reference ships no golden
vectors for this path, so these checks are what anchors parity."""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle


def rnd(*shape, seed=0, dtype=torch.float64):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=dtype)


def test_dense_attn_matches_sdpa_and_logsumexp():
    q, k, v = rnd(2, 3, 37, 16, seed=1), rnd(2, 3, 53, 16, seed=2), rnd(2, 3, 53, 16, seed=3)
    for scale in (None, 1.0, 0.3):
        o, M, L = oracle.dense_attn(q, k, v, scale, dtype=torch.float64)
        ref = F.scaled_dot_product_attention(q, k, v, scale=scale)
        assert torch.allclose(o, ref, atol=1e-12)
        s = oracle.default_scale(16, scale)
        lse = torch.logsumexp((q @ k.transpose(-1, -2)) * s, dim=-1, keepdim=True)
        assert torch.allclose(M * math.log(2) + torch.log(L), lse, atol=1e-12)
        # M is the row maximum of the base-2 logits (attn_dense.py:33-37 masks before the max)
        assert torch.allclose(M, ((q @ k.transpose(-1, -2)) * s * oracle.LOG2E).max(-1, keepdim=True).values)


def test_colsum_bruteforce_tiny():
    B, H, Lq, Lk, d, G = 1, 1, 40, 13, 4, 32
    q, k, v = rnd(B, H, Lq, d, seed=4), rnd(B, H, Lk, d, seed=5), rnd(B, H, Lk, d, seed=6)
    o, cs, _ = oracle.dense_colsum_attn(q, k, v, scale=0.7, q_group_size=G, dtype=torch.float64)
    exp_cs = [[0.0] * Lk for _ in range((Lq + G - 1) // G)]
    for i in range(Lq):
        logits = [0.7 * sum(float(q[0, 0, i, c]) * float(k[0, 0, n, c]) for c in range(d)) for n in range(Lk)]
        mx = max(logits)
        e = [math.exp(x - mx) for x in logits]
        z = sum(e)
        for n in range(Lk):
            exp_cs[i // G][n] += e[n] / z
        row = [sum(e[n] / z * float(v[0, 0, n, c]) for n in range(Lk)) for c in range(d)]
        assert torch.allclose(o[0, 0, i], torch.tensor(row, dtype=torch.float64), atol=1e-12)
    assert torch.allclose(cs[0, 0], torch.tensor(exp_cs, dtype=torch.float64), atol=1e-12)


def test_colsum_invariants_and_special_cases():
    B, H, Lq, Lk, d = 2, 2, 300, 77, 8
    q, k, v = rnd(B, H, Lq, d, seed=7), rnd(B, H, Lk, d, seed=8), rnd(B, H, Lk, d, seed=9)
    _, cs, (M, L) = oracle.dense_colsum_attn(q, k, v, dtype=torch.float64)
    assert cs.shape == (B, H, 2, Lk) and bool((cs >= 0).all())
    # each softmax row sums to one: the last group has 300 - 192 = 108 rows (rows >= Lq add zero)
    assert torch.allclose(cs.sum(-1), torch.tensor([192.0, 108.0], dtype=torch.float64).expand(B, H, 2))
    _, cs_all, _ = oracle.dense_colsum_attn(q, k, v, q_group_size=Lq, dtype=torch.float64)
    assert torch.allclose(cs.sum(2, keepdim=True), cs_all, atol=1e-12)
    # second pass given (M, L) reproduces the fused result
    assert torch.allclose(oracle.colsum_from_lse(q, k, M, L, dtype=torch.float64), cs, atol=1e-12)
    # q = 0 => uniform rows => cs = rows / Lk
    _, cs0, _ = oracle.dense_colsum_attn(torch.zeros_like(q), k, v, dtype=torch.float64)
    assert torch.allclose(cs0[:, :, 0], torch.full((B, H, Lk), 192.0 / Lk, dtype=torch.float64))
    # the reference's own PyTorch statement of the op (sparse_attn_ops.py:179-200), retyped from its
    # formula with library calls only
    attn = torch.softmax(q @ k.transpose(-2, -1) / math.sqrt(d), dim=-1)
    pad = F.pad(attn, (0, 0, 0, 2 * 192 - Lq)).view(B, H, 2, 192, Lk).sum(3)
    assert torch.allclose(cs, pad, atol=1e-12)


def test_key_block_sums_ragged():
    cs = torch.arange(680, dtype=torch.float64).view(1, 1, 1, 680)
    bs = oracle.key_block_sums(cs, 64)
    assert bs.shape[-1] == 11
    assert bs[0, 0, 0, 0] == sum(range(64)) and bs[0, 0, 0, 10] == sum(range(640, 680))


def test_indices_count_known_answers():
    # decision scale of Infinity-2B: Lk = 4121, top_keys = 0.2 (sparse-attn-config.yml:20)
    assert oracle.indices_count(0.2, 4121, 64) == 832
    assert oracle.indices_count(0.2, 4121, 112) == 784
    # VAR-d16 benchmark case: Lk = 680, keep 50 % => 320 tokens = 5 blocks of 64
    assert oracle.indices_count(0.5, 680, 64) == 320
    # half-to-even: 0.25*640/64 = 2.5 -> 2
    assert oracle.indices_count(0.25, 640, 64) == 128
    assert oracle.infinity_cum() == [0, 1, 5, 21, 57, 121, 265, 521, 921, 1497, 2521, 4121, 6425, 10521]


def test_topk_index_list_is_the_sorted_prefix():
    bs = rnd(1, 2, 3, 200, seed=10).abs()
    inds, counts = oracle.topk_index_list(bs, 0.3, multiple_of=16)
    cnt = 16 * round(0.3 * 200 / 16)
    assert inds.shape == (1, 2, 3, 200) and inds.dtype == torch.int32 and int(counts[0, 0, 0]) == cnt
    order = torch.sort(bs, dim=-1, descending=True, stable=True).indices[..., :cnt]
    assert torch.equal(inds[..., :cnt].long(), order)  # values are distinct, so the order is fixed


def _gather_attention_bruteforce(q, k, v, idx, scale):
    out = []
    for i in range(q.shape[0]):
        logits = [scale * float(q[i] @ k[j]) for j in idx]
        mx = max(logits)
        e = [math.exp(x - mx) for x in logits]
        z = sum(e)
        out.append(sum((e[t] / z) * v[j] for t, j in enumerate(idx)))
    return torch.stack(out)


def test_csp_attn_multiset_semantics():
    B, H, Lq, Lk, d, bm = 1, 2, 50, 30, 4, 32
    q, k, v = rnd(B, H, Lq, d, seed=11), rnd(B, H, Lk, d, seed=12), rnd(B, H, Lk, d, seed=13)
    G = 2
    inds = torch.zeros(B, H, G, Lk, dtype=torch.int32)
    counts = torch.zeros(B, H, G, dtype=torch.int32)
    lists = {(0, 0): [3, 3, 7, 29, 0], (0, 1): [5], (1, 0): list(range(30)), (1, 1): []}
    for (h, g), l in lists.items():
        inds[0, h, g, :len(l)] = torch.tensor(l, dtype=torch.int32)
        counts[0, h, g] = len(l)
    delta, M, L = oracle.csp_attn_delta(q, k, v, inds, counts, scale=0.5, bm=bm, dtype=torch.float64)
    for (h, g), l in lists.items():
        lo, hi = g * bm, min((g + 1) * bm, Lq)
        if not l:
            assert bool((delta[0, h, lo:hi] == 0).all()) and bool(torch.isinf(M[0, h, lo:hi]).all()) and bool((L[0, h, lo:hi] == 1).all())
            continue
        ref = _gather_attention_bruteforce(q[0, h, lo:hi], k[0, h], v[0, h], l, 0.5)
        assert torch.allclose(delta[0, h, lo:hi], ref, atol=1e-12)
    # full list == dense attention (attn_csp.py:313-338); o_scale epilogue (attn_csp.py:209-211)
    dense, _, _ = oracle.dense_attn(q[:, 1:2], k[:, 1:2], v[:, 1:2], 0.5, dtype=torch.float64)
    assert torch.allclose(delta[0, 1, :bm], dense[0, 0, :bm], atol=1e-12)
    o0 = rnd(B, H, Lq, d, seed=14)
    assert torch.allclose(oracle.csp_attn(q, k, v, 0.5, inds, counts, o0, -1, bm=bm, dtype=torch.float64), o0 - delta)


def test_csp_unique_list_equals_masked_softmax():
    """The reference's own oracle form (attn_csp.py:437-471): dense softmax, unselected logits -> -1e9."""
    B, H, Lq, Lk, d = 1, 1, 192, 64, 8
    q, k, v = rnd(B, H, Lq, d, seed=15), rnd(B, H, Lk, d, seed=16), rnd(B, H, Lk, d, seed=17)
    sel = torch.randperm(Lk, generator=torch.Generator().manual_seed(1))[:20]
    inds = torch.zeros(B, H, 1, Lk, dtype=torch.int32)
    inds[0, 0, 0, :20] = sel.to(torch.int32)
    counts = torch.full((B, H, 1), 20, dtype=torch.int32)
    delta, _, _ = oracle.csp_attn_delta(q, k, v, inds, counts, dtype=torch.float64)
    logits = (q @ k.transpose(-1, -2)) / math.sqrt(d)
    mask = torch.zeros(Lk, dtype=torch.bool)
    mask[sel] = True
    ref = torch.softmax(logits.masked_fill(~mask, -1e9), -1) @ v
    assert torch.allclose(delta, ref, atol=1e-12)


def test_block_sparse_equals_masked_dense():
    B, H, Lq, Lk, d, bq, bk = 1, 2, 200, 150, 8, 128, 64
    q, k, v = rnd(B, H, Lq, d, seed=18), rnd(B, H, Lk, d, seed=19), rnd(B, H, Lk, d, seed=20)
    mask = torch.tensor([[[1, 0, 1], [0, 1, 1]], [[0, 0, 1], [1, 1, 1]]], dtype=torch.bool).view(1, 2, 2, 3)
    num, idx = oracle.block_mask_to_lists(mask)
    assert num.tolist() == [[[2, 2], [1, 3]]] and idx[0, 0, 0, :2].tolist() == [0, 2]
    assert torch.equal(oracle.lists_to_block_mask(num, idx, 3), mask)
    o, M, L = oracle.block_sparse_attn(q, k, v, num, idx, bq, bk, dtype=torch.float64)
    fine = mask.repeat_interleave(bq, 2).repeat_interleave(bk, 3)[:, :, :Lq, :Lk]
    logits = (q @ k.transpose(-1, -2)) / math.sqrt(d)
    ref = torch.softmax(logits.masked_fill(~fine, -float("inf")), -1) @ v
    assert torch.allclose(o, ref, atol=1e-12)
    lse = torch.logsumexp(logits.masked_fill(~fine, -float("inf")), -1, keepdim=True)
    assert torch.allclose(M * math.log(2) + torch.log(L), lse, atol=1e-12)
    assert oracle.attn_flops_blocks(num, idx, Lq, Lk, d, bq, bk) == 4 * d * int(fine.sum())


def test_map_inds_counts_across_scales_bruteforce():
    # Gs = 9 (decision scale, 1600 rows), target scales 11 (2304 rows, G=12) and 12 (4096 rows, G=22)
    g = torch.Generator().manual_seed(3)
    inds_S = torch.randint(0, 4121, (2, 2, 9, 4121), generator=g, dtype=torch.int32)
    counts_S = torch.full((2, 2, 9), 832, dtype=torch.int32)
    for q_len, k_len in ((2304, 6425), (4096, 10521)):
        out, counts = oracle.map_inds_counts_across_scales(inds_S, counts_S, q_len, k_len)
        Gk = (q_len + 191) // 192
        assert out.shape == (2, 2, Gk, 832) and bool((counts == 832).all())
        for gk in range(Gk):
            gs = min(max(round((gk + 0.5) / Gk * 9 - 0.5), 0), 8)  # python round = half-to-even
            assert torch.equal(out[:, :, gk], inds_S[:, :, gs, :832])
    # narrower source than the padded count: cyclic repeat_interleave, then clamp to the key range
    small = torch.tensor([5, 9, 100], dtype=torch.int32).view(1, 1, 1, 3)
    out, counts = oracle.map_inds_counts_across_scales(small, torch.tensor([[[3]]]), 192, 50, indices_pad_to=4)
    assert out.tolist() == [[[[5, 5, 9, 9]]]] and int(counts[0, 0, 0]) == 4
    out, _ = oracle.map_inds_counts_across_scales(small, torch.tensor([[[3]]]), 192, 50)
    assert out.tolist() == [[[[5, 9, 49]]]]


def test_local_window_runs_known_answers():
    """Source comment models/sparvar/sparse_attn.py:934: windows (5, 7), counts_multiple_of 112
    -> scale 11: [12, 448], scale 12: [22, 672]."""
    for si, win, shape in ((11, 5, (12, 448)), (12, 7, (22, 672))):
        ia, kv = oracle.crossscale_self_indices(si, win)
        S = oracle.INFINITY_SCALES[si]
        assert ia.shape[0] == S * S and kv == oracle.infinity_cum()[si + 1]
        runs, L = oracle.aggregate_group_indices(ia, S * S, kv, 192, 112)
        assert tuple(runs.shape) == shape and L == shape[1]
        assert bool((runs[:, 1:] - runs[:, :-1] == 1).all())                  # contiguous runs
        assert int(runs.min()) >= oracle.infinity_cum()[si] and int(runs.max()) == kv - 1
    # Run starts worked out by hand (sparse_attn.py:845-855).  Scale 11 (48 x 48 grid at key 4121, Lk 6425), window 5,
    # 192-row groups = grid rows 4g..4g+3: the union of the clamped windows is the full rows max(4g-2, 0)..min(4g+5, 47),
    # i.e. first key 4121 + 48 * max(4g-2, 0) and 288 or 384 keys -> 448 after rounding up to a multiple of 112; the run
    # is [first, first + 447], pushed back to end at key 6424 for the last groups.
    # Scale 12 (64 x 64 grid at key 6425, Lk 10521), window 7, groups = grid rows 3g..3g+2 (the last group is row 63
    # alone): rows max(3g-3, 0)..min(3g+5, 63), at most 576 keys -> 672; first key 6425 + 64 * max(3g-3, 0).
    from lvar_amd import mask_build as mb
    hand = {(11, 5): {0: 4121, 1: 4217, 5: 4985, 10: 5945, 11: 5977},
            (12, 7): {0: 6425, 1: 6425, 2: 6617, 10: 8153, 20: 9849, 21: 9849}}
    for (si, win), starts in hand.items():
        ia, kv = oracle.crossscale_self_indices(si, win)
        S = oracle.INFINITY_SCALES[si]
        runs, L = oracle.aggregate_group_indices(ia, S * S, kv, 192, 112)
        runs_mb, L_mb = mb.local_group_runs(si, win, 192, 112)
        assert L_mb == L and torch.equal(runs_mb.cpu().to(torch.int64), runs)
        for g, first in starts.items():
            assert int(runs[g, 0]) == first and int(runs[g, -1]) == first + L - 1, (si, g)
            assert int(runs_mb[g, 0]) == first, (si, g)
    # interior query of an 8x8 grid, 3x3 window: the 9 neighbours, row-major
    w = oracle.local_window_indices(8, 8, 100, 3)
    assert w[9].tolist() == [100, 101, 102, 108, 109, 110, 116, 117, 118]
    assert w[0].tolist() == [100, 100, 101, 100, 100, 101, 108, 108, 109]     # clamp padding at the corner


def test_upsample_ocache_matches_interpolate():
    x = rnd(2, 3, 40 * 40, 8, seed=21)
    for tgt in (48, 64):
        got = oracle.upsample_ocache(x, 1600, tgt * tgt)
        ref = F.interpolate(x.view(2, 3, 40, 40, 8).permute(0, 1, 4, 2, 3).reshape(6, 8, 40, 40), size=(tgt, tgt),
                            mode="bilinear", align_corners=False)
        ref = ref.view(2, 3, 8, tgt, tgt).permute(0, 1, 3, 4, 2).reshape(2, 3, tgt * tgt, 8)
        assert torch.allclose(got, ref, atol=1e-10)


def test_flex_block_mask_properties():
    # scale index 8 (24x24 queries, 1497 keys) keeps the pure-Python brute force fast
    ks = [-1, -1, -1, -1, 1, 1, 3, 5, 7]
    m = oracle.flex_block_mask(8, ks, 3, 128)
    cum = oracle.infinity_cum()
    assert m.shape == ((576 + 127) // 128, (cum[9] + 127) // 128)
    assert bool(m[:, 0].all())                       # sink: keys < cum[3] = 21 are in block 0
    # hand check of one fine-grained entry: query (12, 12) of the 24x24 grid looks at the 16x16 scale
    # (index 6, kernel 3) around round(12/24*16) = 8: keys (7..9, 7..9); key (8, 8) = cum[6] + 8*16 + 8
    kv = cum[6] + 8 * 16 + 8
    assert bool(m[(12 * 24 + 12) // 128, kv // 128])
    # negative kernel size: a scale beyond the sink is never attended.  Scale 3 (keys 21..56) has
    # kernel -1; with 32-wide key blocks, block 1 (keys 32..63) holds scale 3 and the head of scale 4
    m32 = oracle.flex_block_mask(8, [-1] * 9, 3, 128, block_k=32)
    assert bool(m32[:, 0].all()) and not bool(m32[:, 1:].any())
    # mixed block shape (128 x 64) is the same predicate reduced over other tiles
    m2 = oracle.flex_block_mask(8, ks, 3, 128, block_k=64)
    pad = F.pad(m2, (0, m2.shape[1] % 2))
    assert torch.equal(pad.view(pad.shape[0], -1, 2).any(-1), m)


# Hand-computed fine-grained entries (block_size = block_k = 1) of the sink + window predicate
# (models/sparvar/basic_sparvar.py:113-151) on the schedule 2x2, 6x6, 4x4 with the 4x4 scale as queries:
# key offsets cum = [0, 4, 40, 56]; kernel sizes per KEY scale [1, 3, 5] (half = 0, 1, 2).
# Entry: (query (y, x), key scale, key (y, x), expected).
FLEX_FINE_SCALES, FLEX_FINE_KERNELS, FLEX_FINE_CUM = [2, 6, 4], [1, 3, 5], [0, 4, 40, 56]
FLEX_FINE_CASES = [
    # rounding tie 1/4*2 = 0.5 -> 0 (half-to-even; half-up would give 1)
    ((1, 0), 0, (0, 0), True), ((1, 0), 0, (1, 0), False),
    # rounding tie 3/4*2 = 1.5 -> 2: the centre falls off the 2x2 grid, nothing of that scale is attended
    ((3, 0), 0, (0, 0), False), ((3, 0), 0, (1, 0), False), ((3, 0), 0, (1, 1), False),
    # rounding tie 3/4*6 = 4.5 -> 4 (half-to-even; half-up would give 5): rows 3..5 of the 6x6 scale
    ((3, 0), 1, (3, 0), True), ((3, 0), 1, (5, 0), True),
    # window edge, key-scale kernel 3: distance 1 = half is kept, distance 2 = half + 1 is not
    # (the query scale's own kernel, 5, would keep distance 2)
    ((3, 0), 1, (2, 0), False), ((3, 0), 1, (4, 1), True), ((3, 0), 1, (4, 2), False),
    # rounding tie 1/4*6 = 1.5 -> 2 (both rules agree): rows 1..3
    ((1, 0), 1, (1, 0), True), ((1, 0), 1, (0, 0), False), ((1, 0), 1, (3, 0), True), ((1, 0), 1, (4, 0), False),
    # the query scale itself, kernel 5: distance 2 kept, distance 3 not
    ((0, 0), 2, (2, 2), True), ((0, 0), 2, (3, 0), False), ((0, 0), 2, (0, 3), False), ((3, 3), 2, (1, 1), True),
    ((3, 3), 2, (0, 3), False),
]


def flex_fine_entry(mask_fn, qyx, si, kyx, kernels=FLEX_FINE_KERNELS, sink=0):
    side_q, side_k = FLEX_FINE_SCALES[2], FLEX_FINE_SCALES[si]
    m = mask_fn(2, kernels, sink, 1, scales=FLEX_FINE_SCALES, block_k=1)
    assert tuple(m.shape) == (16, 56)
    return bool(m[qyx[0] * side_q + qyx[1], FLEX_FINE_CUM[si] + kyx[0] * side_k + kyx[1]])


def check_flex_fine_cases(mask_fn):
    for qyx, si, kyx, want in FLEX_FINE_CASES:
        assert flex_fine_entry(mask_fn, qyx, si, kyx) == want, (qyx, si, kyx, want)
    # sink: every key below cum[1] = 4 is attended by every query, also where the window misses
    assert flex_fine_entry(mask_fn, (3, 0), 0, (0, 0), sink=1) and flex_fine_entry(mask_fn, (3, 0), 0, (1, 1), sink=1)
    assert not flex_fine_entry(mask_fn, (3, 0), 1, (2, 0), sink=1)
    # negative kernel size: -1 // 2 = -1, not even the centre key is attended
    assert not flex_fine_entry(mask_fn, (1, 0), 1, (2, 0), kernels=[1, -1, 5])
    assert flex_fine_entry(mask_fn, (1, 0), 1, (2, 0), kernels=[1, 1, 5])
    # kernel 1 keeps the centre only
    assert not flex_fine_entry(mask_fn, (1, 0), 1, (1, 0), kernels=[1, 1, 5])


def test_flex_block_mask_hand_computed_fine_entries():
    check_flex_fine_cases(oracle.flex_block_mask)


def test_video_window_block_mask_hand_cases():
    """8 frames x 64 x 64 tokens, 128-token blocks: 32 blocks per frame, block = (frame, spatial block)."""
    m = oracle.video_window_block_mask()
    assert m.shape == (256, 256) and bool((m == m.T).all())
    assert bool(m[0, 0]) and bool(m[0, 1]) and not bool(m[0, 2])           # same frame: +-1 spatial block
    assert bool(m[0, 32]) and bool(m[0, 33]) and not bool(m[0, 34])        # next frame
    assert not bool(m[0, 64]) and not bool(m[0, 31])                       # two frames away; far end of the frame
    assert bool(m[40, 7]) and bool(m[40, 9]) and bool(m[40, 73]) and not bool(m[40, 104]) and not bool(m[40, 10])
    assert int(m[0].sum()) == 4 and int(m[40].sum()) == 9 and int(m[255].sum()) == 4 and int(m[31].sum()) == 4
    assert int(m[5].sum()) == 6 and int(m[32].sum()) == 6                  # frame edge / spatial edge
    # a layout whose blocks straddle frames: 2 frames x 2 x 3 tokens, 4-token blocks
    s = oracle.video_window_block_mask(2, 2, 3, 4, frame_radius=0, spatial_radius=0)
    # tokens 0..5 are frame 0 (spatial blocks 0,0,0,0,1,1), tokens 6..11 frame 1 (same pattern); the blocks
    # {0..3}, {4..7}, {8..11} hold the (frame, spatial block) pairs {(0,0)}, {(0,1),(1,0)}, {(1,0),(1,1)}
    assert s.tolist() == [[True, False, False], [False, True, True], [False, True, True]]


def test_config2_block_mask_density():
    scores = rnd(1, 2, 32, 165, seed=22).abs()
    mask = oracle.config2_block_mask(scores)
    assert mask.shape == (1, 2, 32, 165)
    target = round(0.25 * 165)
    assert bool((mask.sum(-1) == target).all())
    assert bool(mask[..., :9].all())                 # keys < 521 -> blocks 0..8 always kept
    # the score-independent part, and the score-selected remainder = best remaining blocks
    base = oracle.config2_block_mask(scores, density=0.0)
    assert bool((base[0, 0] == base[0, 1]).all()) and bool((mask | ~base).all())
    for h in range(2):
        for i in range(32):
            extra = (mask[0, h, i] & ~base[0, h, i]).nonzero().flatten()
            rest = scores[0, h, i].masked_fill(base[0, h, i], -1.0)
            best = torch.sort(rest, descending=True).indices[:extra.numel()]
            assert sorted(extra.tolist()) == sorted(best.tolist())


def test_topk_token_set_against_rank_definition_and_torch_topk():
    """The selected set is pinned by the rank definition (brute force) and, where all values are
    distinct, by torch.topk (library); ties go to the smaller column."""
    g = torch.Generator().manual_seed(11)
    x = torch.randn(3, 2, 57, generator=g)
    x[0, 0, 5] = x[0, 0, 40] = x[0, 0, 41] = x[0, 0].max() + 1.0       # ties above the cut
    x[1, 1, :] = torch.tensor([1.0, 2.0] * 28 + [1.0])                   # heavy ties through the cut
    for k in (0, 1, 7, 29, 57):
        got = oracle.topk_token_set(x, k)
        assert got.shape == (3, 2, k) and got.dtype == torch.int32
        for r in range(3):
            for c in range(2):
                row = x[r, c].tolist()
                exp = [j for j in range(57)
                       if sum(1 for t in range(57) if row[t] > row[j] or (row[t] == row[j] and t < j)) < k]
                assert got[r, c].tolist() == exp
        if k:
            ref = torch.topk(x[2], k, dim=-1).indices.sort(-1).values      # rows of x[2] have distinct values
            assert torch.equal(got[2].long(), ref)


def test_mask_to_lists_small_cases():
    m = torch.tensor([[0, 1, 0, 1, 1, 0, 0, 0], [0, 0, 0, 0, 0, 0, 0, 0], [1, 1, 1, 1, 1, 1, 1, 1]], dtype=torch.bool)
    cnt, idx = oracle.mask_to_lists(m, 1)
    assert cnt.tolist() == [3, 0, 8]
    assert idx.tolist() == [[1, 3, 4, 0, 0, 0, 0, 0], [0] * 8, list(range(8))]
    cnt, idx = oracle.mask_to_lists(m, 4)                                # pad with the lowest unset columns
    assert cnt.tolist() == [4, 0, 8]
    assert idx[0].tolist() == [1, 3, 4, 0, 0, 0, 0, 0]
    cnt, idx = oracle.mask_to_lists(m, 5)
    assert cnt.tolist() == [5, 0, 8] and idx[0].tolist() == [1, 3, 4, 0, 2, 0, 0, 0]
    # multiple_of = 1 on a block mask equals the flex BlockMask lists of block_mask_to_lists
    g = torch.Generator().manual_seed(3)
    bm = torch.rand(2, 3, 5, 19, generator=g) < 0.3
    num, bidx = oracle.block_mask_to_lists(bm)
    cnt, idx = oracle.mask_to_lists(bm, 1)
    assert torch.equal(cnt, num) and torch.equal(idx, bidx)


def test_append_local_run_layout():
    inds = torch.arange(2 * 1 * 3 * 10, dtype=torch.int32).reshape(2, 1, 3, 10)
    local = torch.tensor([[100, 101], [200, 201], [300, 301]])
    out, counts = oracle.append_local_run(inds, 4, local, 2, 9)
    assert out.shape == (2, 1, 3, 9) and counts.tolist() == [[[6] * 3]] * 2
    assert out[1, 0, 2].tolist() == [50, 51, 52, 53, 300, 301, 0, 0, 0]


def test_window_key_scores_bruteforce():
    """Pure-Python restatement of the masked, summed, pooled window logits on a tiny case."""
    B, H, Lq, Lk, d, ks = 1, 2, 6, 11, 4, 3
    q, k = rnd(B, H, Lq, d, seed=31), rnd(B, H, Lk, d, seed=32)
    win = torch.tensor([[[5, 7, 10], [6, 6, 9]]])                       # key positions; a repeat in head 1
    for pooling in ("avgpool", "maxpool"):
        got = oracle.window_key_scores(q, k, win, ks, pooling, dtype=torch.float64)
        for h in range(H):
            wk = win[0, h].tolist()
            raw = []
            for n in range(Lk):
                if n in wk:
                    raw.append(-math.inf)
                else:
                    raw.append(sum(sum(float(q[0, h, min(max(x - (Lk - Lq), 0), Lq - 1), c]) * float(k[0, h, n, c]) for c in range(d))
                                   for x in wk) / math.sqrt(d))
            for n in range(Lk):
                nb = [raw[m] if 0 <= m < Lk else (0.0 if pooling == "avgpool" else -math.inf) for m in range(n - 1, n + 2)]
                exp = -math.inf if n in wk else (sum(nb) / ks if pooling == "avgpool" else max(nb))
                g = float(got[0, h, n])
                assert (g == exp) if math.isinf(exp) else abs(g - exp) < 1e-9, (pooling, h, n, g, exp)


def test_expand_kv_heads_matches_repeat_interleave():
    k = rnd(2, 3, 5, 4, seed=1)
    e = oracle.expand_kv_heads(k, 12)
    assert e.shape == (2, 12, 5, 4) and torch.equal(e, k.repeat_interleave(4, dim=1))
    for h in range(12):
        assert torch.equal(e[:, h], k[:, h // 4])
    assert torch.equal(oracle.expand_kv_heads(k, 3), k)
