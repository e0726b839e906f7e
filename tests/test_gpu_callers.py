"""The caller-level mirrors (SparseFlexAttn, SparseDiffAttn, torch.ops.lvar.*) on the GPU against
compositions of oracle functions on the same seeded inputs."""
import math

import pytest
import torch

import oracle
from conftest import make_qkv

pytestmark = pytest.mark.gpu

SCALES9 = (1, 2, 4, 6, 8, 12, 16, 20, 24)   # Infinity's first nine scales: a small but real schedule


def close(a, b, atol=2e-2, rtol=1e-2):
    return bool(((a.float().cpu() - b).abs() <= atol + rtol * b.abs()).all())


def test_sparse_flex_attn_matches_oracle():
    from lvar_amd.sparse_flex_attn import SparseFlexAttn
    ks = [-1, -1, -1, -1, 1, 1, 3, 5, 7]
    mod = SparseFlexAttn([(s, s) for s in SCALES9], ks, q_scale_idx=8, attn_sink_scale=3, num_heads=2)
    mask = oracle.flex_block_mask(8, ks, 3, 128, scales=SCALES9)
    assert torch.equal(mod.block_level_mask.cpu(), mask)
    q, k, v = make_qkv(2, 2, 576, 1497, 128, seed=8, amp=0.5)
    num, idx = oracle.block_mask_to_lists(mask.expand(2, 2, *mask.shape))
    ref, _, _ = oracle.block_sparse_attn(q, k, v, num, idx, 128, 128, scale=1.0)
    # cosine-attention callers hand q, k in fp32 and v in bf16 (basic_sparvar.py:362-367)
    out = mod(q.float().cuda(), k.float().cuda(), v.cuda(), scale=1.0)
    assert out.dtype == torch.bfloat16 and close(out, ref)
    with pytest.raises(ValueError):
        mod(q[:, :, :100].cuda(), k.cuda(), v.cuda())
    # the other square block sizes flex takes as BLOCK_SIZE=int (basic_sparvar.py:55-72) and the kernel walks
    for bs in (64, 256):
        mod_b = SparseFlexAttn([(s, s) for s in SCALES9], ks, q_scale_idx=8, attn_sink_scale=3, block_size=bs, num_heads=2)
        mask_b = oracle.flex_block_mask(8, ks, 3, bs, scales=SCALES9)
        assert torch.equal(mod_b.block_level_mask.cpu(), mask_b)
        num_b, idx_b = oracle.block_mask_to_lists(mask_b.expand(2, 2, *mask_b.shape))
        ref_b, _, _ = oracle.block_sparse_attn(q, k, v, num_b, idx_b, bs, bs, scale=1.0)
        assert close(mod_b(q.float().cuda(), k.float().cuda(), v.cuda(), scale=1.0), ref_b), bs
    with pytest.raises(ValueError):
        SparseFlexAttn([(s, s) for s in SCALES9], ks, q_scale_idx=8, attn_sink_scale=3, block_size=96)


def test_torch_ops_list_building_schemas():
    """``torch.ops.chipmunk.mask_to_indices`` / ``topk_indices`` called as the reference's wrappers call them
    (kernels/sparse_attn/sparse_attn_ops.py:381-407; schemas of kernels/chipmunk/csrc/chipmunk.cu:66-68)."""
    import lvar_amd.torch_ops as tops
    tops.register_as("chipmunk")
    g = torch.Generator().manual_seed(31)
    mask = torch.rand(2, 3, 5, 300, generator=g) < 0.3
    mask[0, 0, 0] = False
    mask[0, 0, 1] = True
    for ns in (torch.ops.lvar, torch.ops.chipmunk):
        for mult, pad_to in ((1, 192), (64, 192), (7, 1)):
            indices, counts = ns.mask_to_indices(mask.cuda(), mult, pad_to)
            pad_n = (300 + pad_to - 1) // pad_to * pad_to
            assert indices.dtype == torch.int32 and tuple(indices.shape) == (2, 3, 5, pad_n) and tuple(counts.shape) == (2, 3, 5)
            c_ref, i_ref = oracle.mask_to_lists(mask, mult)
            assert torch.equal(counts.cpu(), c_ref) and torch.equal(indices[..., :300].cpu(), i_ref)
        with pytest.raises(Exception):
            ns.mask_to_indices(mask.cuda().to(torch.uint8), 1, 192)          # "mask must be bool type"
        with pytest.raises(Exception):
            ns.mask_to_indices(mask.cuda()[0], 1, 192)                        # "mask must be 4-dimensional"
    act = torch.randn(2, 4, 1000, generator=g)
    act[0, 0, 100:200] = 0.25                                                 # ties through the cut
    for ns in (torch.ops.lvar, torch.ops.chipmunk):
        for dtype in (torch.float32, torch.bfloat16):
            a = act.to(dtype)
            for sparsity, mult in ((0.8, 8), (0.75, 64), (0.0, 1), (0.5, 1)):
                indices = torch.full((2, 4, 1000), -1, dtype=torch.int32, device="cuda")
                counts = torch.zeros(2, 4, dtype=torch.int32, device="cuda")
                assert ns.topk_indices(a.cuda(), indices, counts, sparsity, mult, 0.0) is None
                keep = 1000 - int(1000 * sparsity)
                padded = min(1000, (keep + mult - 1) // mult * mult)
                assert bool((counts == padded).all())
                top = oracle.topk_token_set(a.float(), keep)                   # stable selection, ascending
                sel = torch.zeros(2, 4, 1000, dtype=torch.bool).scatter_(-1, top.long(), True)
                c_ref, i_ref = oracle.mask_to_lists(sel, mult)                 # + the lowest unselected columns as padding
                assert torch.equal(counts.cpu(), c_ref) and torch.equal(indices[..., :padded].cpu(), i_ref[..., :padded])
                assert bool((indices[..., padded:] == -1).all())                # left as the caller filled them
        indices = torch.zeros(2, 4, 1000, dtype=torch.int32, device="cuda")
        counts = torch.ones(2, 4, dtype=torch.int32, device="cuda")
        ns.topk_indices(act.cuda(), indices, counts, 1.0, 8, 0.0)               # quantile 1: no indices
        assert bool((indices == -1).all()) and bool((counts == 0).all())
        # random extras: the top set stays, every count is a multiple, lists are free of repeats
        indices.fill_(-1)
        ns.topk_indices(act.cuda(), indices, counts, 0.9, 16, 0.2)
        top = oracle.topk_token_set(act, 100)
        for b in range(2):
            for r in range(4):
                c = int(counts[b, r])
                row = indices[b, r, :c].cpu()
                assert c % 16 == 0 and c >= 112 and len(set(row.tolist())) == c and int(row.min()) >= 0 and int(row.max()) < 1000
                assert set(top[b, r].tolist()) <= set(row.tolist())
        with pytest.raises(Exception):
            ns.topk_indices(act.cuda(), indices, counts, 1.5, 8, 0.0)


def test_sparse_diff_attn_full_and_sparse_steps():
    from lvar_amd import sparse_attn_config as cfg
    from lvar_amd.sparse_diff_attn import SparseDiffAttn
    cfg.reset()
    cfg.GLOBAL_CONFIG["attn"]["top_keys"] = 0.25
    try:
        mod = SparseDiffAttn(scales=SCALES9, spsd_scale=6)
        cum = oracle.infinity_cum(SCALES9)
        B, H, d = 1, 2, 128
        g = torch.Generator().manual_seed(3)
        mk = lambda L: (torch.randn(B, H, L, d, generator=g) * 0.5).to(torch.bfloat16)
        # --- full step at the decision scale (16x16 queries, 521 keys) ---
        q, k, v = mk(256), mk(cum[7]), mk(cum[7])
        o = mod(q.cuda(), k.cuda(), v.cuda(), None, do_full_step=True, scale_ind=6)
        o_ref, cs_ref, _ = oracle.dense_colsum_attn(q, k, v)
        assert close(o, o_ref)
        cnt = oracle.indices_count(0.25, cum[7], 64)
        assert cnt == 128 and int(mod.counts[0, 0, 0]) == cnt and mod.indices.shape == (B, H, 2, cum[7])
        # the lists are the top-k of the HIP colsum; the oracle's top-k set agrees wherever the k-th
        # value is separated by more than the colsum tolerance
        sel = mod.indices[..., :cnt].cpu().long()
        picked = torch.gather(cs_ref, -1, sel)
        kth = torch.topk(cs_ref, cnt, dim=-1).values[..., -1:]
        assert bool((picked >= kth * (1 - 2e-3)).all())
        cache_ref = oracle.csp_attn(q, k, v, None, mod.indices.cpu(), mod.counts.cpu(), o.cpu(), -1)
        assert close(mod.out_cache, cache_ref)
        # --- sparse steps at the next two scales ---
        for si in (7, 8):
            S = SCALES9[si]
            inds_prev, counts_prev, cache_prev = mod.indices.cpu(), mod.counts.cpu(), mod.out_cache.cpu()
            q, k, v = mk(S * S), mk(cum[si + 1]), mk(cum[si + 1])
            out = mod(q.cuda(), k.cuda(), v.cuda(), None, scale_ind=si)
            mi, mc = oracle.map_inds_counts_across_scales(inds_prev, counts_prev, S * S, cum[si + 1])
            ia, kv = oracle.crossscale_self_indices(si, cfg.GLOBAL_CONFIG["attn"]["cs4a_ws"][-(9 - si)], SCALES9)
            runs, L = oracle.aggregate_group_indices(ia, S * S, kv, 192, 64)
            G = mi.shape[2]
            full = torch.zeros(B, H, G, cum[si + 1], dtype=torch.int32)
            full[..., :mi.shape[-1]] = mi
            full[..., mi.shape[-1]:mi.shape[-1] + L] = runs.to(torch.int32)
            counts = torch.full((B, H, G), mi.shape[-1] + L, dtype=torch.int32)
            up = oracle.upsample_ocache(cache_prev.float(), cache_prev.shape[-2], S * S).to(torch.bfloat16)
            ref = oracle.csp_attn(q, k, v, None, full, counts, up, 1)
            assert close(out, ref, atol=3e-2), si
            if si == 7:
                assert torch.equal(mod.indices.cpu()[..., :int(counts[0, 0, 0])], full[..., :int(counts[0, 0, 0])])
    finally:
        cfg.reset()


def test_torch_ops_chipmunk_schemas():
    """The ops under their default namespace and, after ``register_as("chipmunk")``, under the reference's, called
    exactly as the reference calls them (basic_sparvar.py:384; sparse_attn_ops.py:55,84,96,289)."""
    import lvar_amd.torch_ops as tops
    tops.register_as("chipmunk")
    tops.register_as("chipmunk")                                            # idempotent
    q, k, v = make_qkv(1, 2, 384, 500, 128, seed=12, amp=0.3)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    o_ref, M, L = oracle.dense_attn(q, k, v, scale=1.0)
    _, cs_ref, _ = oracle.dense_colsum_attn(q, k, v, scale=1.0)
    inds = torch.arange(500, dtype=torch.int32).flip(0).expand(1, 2, 2, 500).contiguous()
    counts = torch.full((1, 2, 2), 192, dtype=torch.int32)
    for ns in (torch.ops.lvar, torch.ops.chipmunk):
        o, lse = ns.dense_attn(qg, kg, vg)
        assert close(o, o_ref) and lse.shape == (1, 2, 384, 1)
        # the reference's constant: 1 / (2^M * L)  (dense_attn.cu:227-230)
        assert torch.allclose(lse.cpu(), 1.0 / (torch.exp2(M) * L), rtol=2e-3)
        o2, cs, l = ns.dense_colsum_attn(qg, kg, vg, lse)
        assert torch.equal(o2, o) and torch.allclose(cs.cpu(), cs_ref, rtol=2e-3, atol=1e-6) and torch.allclose(l, lse, rtol=1e-5)
        oc = o.clone()
        assert ns.csp_attn(qg, kg, vg, oc, inds.cuda(), counts.cuda(), -1) is None
        ref = oracle.csp_attn(q, k, v, 1.0, inds, counts, o.cpu(), -1)
        assert close(oc, ref) and not torch.equal(oc, o)
        with pytest.raises(Exception):
            ns.csp_attn(qg, kg, vg, oc, inds.cuda(), counts.cuda(), 2)
    # the native dense op takes strided inputs (copied) and refuses wrong dtypes
    qs = qg.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    o3, _ = torch.ops.chipmunk.dense_attn(qs, kg, vg)
    assert torch.equal(o3, o)
    with pytest.raises(Exception):
        torch.ops.chipmunk.dense_attn(qg.float(), kg, vg)
    # list checks of the in-place op: int64 lists are refused, lists sliced on the head or group axis are
    # read through their own strides (copied when they are not the packed ones)
    oc = o.clone()
    with pytest.raises(TypeError):
        torch.ops.lvar.csp_attn(qg, kg, vg, oc, inds.cuda().long(), counts.cuda(), 1)
    with pytest.raises(TypeError):
        torch.ops.lvar.csp_attn(qg, kg, vg, oc, inds.cuda(), counts.cuda().long(), 1)
    with pytest.raises(AssertionError):
        torch.ops.lvar.csp_attn(qg, kg, vg, oc, inds.cuda()[:, :, 0], counts.cuda(), 1)
    with pytest.raises(AssertionError):
        torch.ops.lvar.csp_attn(qg, kg, vg, oc, inds.cuda(), counts.cuda()[:, :1], 1)
    with pytest.raises(AssertionError):
        torch.ops.lvar.csp_attn(qg, kg, vg, oc, inds, counts.cuda(), 1)                      # list on another device
    g = torch.Generator().manual_seed(3)
    wide = torch.randint(0, 500, (1, 4, 3, 500), generator=g, dtype=torch.int32)
    wcnt = torch.randint(1, 500, (1, 4, 3), generator=g, dtype=torch.int32)
    sl_i, sl_c = wide[:, 1:3, :2], wcnt[:, 1:3, :2]                                       # head- and group-sliced views
    assert not sl_i.is_contiguous()
    oc = o.clone()
    torch.ops.lvar.csp_attn(qg, kg, vg, oc, wide.cuda()[:, 1:3, :2], wcnt.cuda()[:, 1:3, :2], 1)
    assert close(oc, oracle.csp_attn(q, k, v, 1.0, sl_i.contiguous(), sl_c.contiguous(), o.cpu(), 1))


def test_reference_shaped_callers_construct():
    """``SparseDiffAttn(layer_num, layer_counter, use_o_cache=True, spsd_scale=...)`` as basic_sparvar.py:255-259
    constructs it, with the counter advanced once per call; the kernel-level module under the names of
    kernels/sparse_attn/triton/__init__.py:1-5."""
    import lvar_amd.sattn_kernels as sattn_triton
    from lvar_amd import sparse_attn_config as cfg
    from lvar_amd.sparse_diff_attn import SparseDiffAttn

    class Counter:
        n = 0

        def increment(self):
            self.n += 1

    counter = Counter()
    mod = SparseDiffAttn(3, counter, use_o_cache=True, spsd_scale=10)
    assert mod.layer_num == 3 and mod.use_o_cache is True and sorted(mod.local_inds) == [11, 12]
    assert tuple(mod.local_inds[11][0].shape) == (12, 512) and tuple(mod.local_inds[12][0].shape) == (22, 704)   # windows 7, 9; counts in multiples of 64
    with pytest.raises(TypeError):
        SparseDiffAttn(3, True)
    q, k, v = make_qkv(1, 2, 1600, 4121, 128, seed=21, amp=0.5)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    o = mod(qg, kg, vg, None, do_full_step=True, scale_ind=10, layer_ind=3)
    assert counter.n == 1 and close(o[:, :1], oracle.dense_attn(q[:, :1], k[:, :1], v[:, :1])[0])
    cfg.reset()
    # kernel-level names
    o2, (M, L) = sattn_triton.dense_attn(qg, kg, vg, scale=None)
    o3, bs, (M3, L3) = sattn_triton.dense_colsum_attn(qg, kg, vg)
    assert torch.equal(o2, o3) and bs.shape == (1, 2, 9, 4121) and M.shape == (1, 2, 1600, 1)
    inds, counts = mod.indices, mod.counts
    delta, (Md, Ld) = sattn_triton.csp_attn(qg, kg, vg, inds, counts, scale=None)
    d_ref, _, _ = oracle.csp_attn_delta(q[:, :1], k[:, :1], v[:, :1], inds[:, :1].cpu(), counts[:, :1].cpu())
    assert close(delta[:, :1], d_ref)


@pytest.mark.gpu
def test_topk_token_lists_matches_oracle_set():
    """GPU radix select against the oracle's stable-sort selection: bit-exact index lists, with
    ties through the cut, k = 0, k = Lk, a ragged Lk, and the descending-by-value order option."""
    import oracle
    from lvar_amd import sparse_attn_ops as ops
    g = torch.Generator().manual_seed(5)
    for (shape, k) in (((2, 3, 4, 1000), 192), ((1, 2, 22, 10521), 2112), ((3, 777), 0), ((3, 777), 777), ((5, 130), 1),
                       ((2, 20000), 4000), ((2, 41000), 513)):   # > 48 KB of LDS; beyond the LDS-staged limit
        x = torch.rand(*shape, generator=g)
        if shape[-1] == 1000:
            x[0, 0, 0] = torch.tensor([1.0, 2.0] * 500)                   # half the row tied at the cut
            x[1, 2, 3] = 0.5                                              # constant row
            x[0, 1, 1, ::3] = -x[0, 1, 1, ::3]                            # negative values
        idx, cnt = ops.topk_token_lists(x.cuda(), k)
        assert idx.shape == shape and cnt.shape == shape[:-1] and bool((cnt == k).all())
        exp = oracle.topk_token_set(x, k)
        assert torch.equal(idx[..., :k].cpu(), exp), (shape, k)
        assert bool((idx[..., k:] == 0).all())
    # Rows whose values share most of their leading bits (what column sums look like): the digits of the radix
    # select start below the common prefix.  Values in one binade; in a range of a few ulps (ties on every level);
    # a row of two values one ulp apart; all-negative and sign-straddling narrow rows; -0.0 against +0.0.
    base = torch.full((8, 4121), 0.0181)
    x = base.clone()
    x[0] += torch.rand(4121, generator=g) * 1e-3
    x[1] = 0.0181 + torch.randint(0, 5, (4121,), generator=g).float() * 2.0 ** -29
    x[2, ::2] = torch.nextafter(torch.tensor(0.0181), torch.tensor(1.0))
    x[3] = -(0.0181 + torch.rand(4121, generator=g) * 1e-3)
    x[4] = (torch.rand(4121, generator=g) - 0.5) * 1e-6
    x[5] = torch.where(torch.rand(4121, generator=g) < 0.5, torch.tensor(-0.0), torch.tensor(0.0))
    x[6] = torch.softmax(torch.randn(192, 4121, generator=g), -1).sum(0)
    x[7, 100] = 5.0                                                     # one outlier above a constant row
    for k in (1, 832, 2060, 4121):
        idx, cnt = ops.topk_token_lists(x.cuda(), k)
        assert torch.equal(idx[..., :k].cpu(), oracle.topk_token_set(x, k)), k
    # row lengths on both sides of every keys-per-thread step of the kernel (512 keys per step up to 12288, then 14336
    # and 16384, beyond that the rows are re-read): ragged last chunks, a whole chunk of padding, ties through the cut
    for n in (1, 63, 64, 65, 511, 512, 513, 1024, 1025, 4607, 4608, 4609, 10240, 10752, 10753, 12288, 12289, 14336, 14337,
              16384, 16385):
        x = torch.rand(3, n, generator=g)
        x[1] = torch.randint(0, 7, (n,), generator=g).float()              # heavy ties
        x[2] = -x[2]
        for k in sorted({1, max(1, n // 5), n}):
            idx, cnt = ops.topk_token_lists(x.cuda(), k)
            assert torch.equal(idx[..., :k].cpu(), oracle.topk_token_set(x, k)), (n, k)
    x = torch.rand(2, 2, 3, 500, generator=g)
    idx, _ = ops.topk_token_lists(x.cuda(), 64, order="value")
    assert torch.equal(idx[..., :64].cpu().long(), torch.topk(x, 64, dim=-1).indices)   # distinct values: same order
    with pytest.raises(AssertionError):
        ops.topk_token_lists(x.cuda(), 501)


@pytest.mark.gpu
def test_list_kernels_seeded_sweep():
    """Seeded sweep of the two list builders against the oracle, bit-exact: row lengths around the chunk and
    keys-per-thread steps, value distributions with heavy ties / one binade / both signs, every k regime; masks of
    every density with count rounding."""
    import random
    import oracle
    from lvar_amd import sparse_attn_ops as ops
    rnd = random.Random(7)
    g = torch.Generator().manual_seed(7)
    for it in range(120):
        rows = rnd.randint(1, 4)
        n = rnd.choice([1, 2, 7, 63, 64, 65, 129, 511, 512, 513, 777, 2047, 2049, 4121, 6425, 10521, 13000, 16384, 17000])
        kind = rnd.random()
        x = torch.rand(rows, n, generator=g) ** rnd.choice([1, 4, 9])
        if kind < 0.2:
            x = (x * rnd.choice([3, 8, 50])).round()            # heavy ties
        elif kind < 0.3:
            x = 0.0181 + x * 1e-4                                 # one binade
        elif kind < 0.4:
            x = x - 0.5                                           # both signs
        k = rnd.choice([0, 1, max(1, n // 5), max(1, n // 2), n])
        idx, cnt = ops.topk_token_lists(x.cuda(), k)
        assert torch.equal(idx[..., :k].cpu(), oracle.topk_token_set(x, k)), (it, rows, n, k)
    for it in range(80):
        b, h, m = rnd.randint(1, 3), rnd.randint(1, 4), rnd.randint(1, 6)
        n = rnd.choice([1, 2, 5, 63, 64, 65, 100, 192, 300, 1000, 2049])
        dens = rnd.choice([0.0, 0.05, 0.3, 0.9, 1.0])
        mult = rnd.choice([1, 2, 7, 64, 192])
        mask = torch.rand(b, h, m, n, generator=g) < dens
        idx, cnt = ops.mask_to_indices(mask.cuda(), mult, rnd.choice([1, 8, 192]))
        c_ref, i_ref = oracle.mask_to_lists(mask, mult)
        assert torch.equal(cnt.cpu(), c_ref) and torch.equal(idx[..., :n].cpu(), i_ref), (it, b, h, m, n, dens, mult)


@pytest.mark.gpu
def test_remap_concat_lists_matches_oracle():
    import oracle
    from lvar_amd import sparse_attn_ops as ops
    g = torch.Generator().manual_seed(6)
    # decision scale 40x40 (Lq 1600, Gs 9) -> scales 48 (Gk 12) and 64 (Gk 22); Ks >= count and Ks < count
    for (Gs, Ks, count, q_len, k_len, L, pad) in ((9, 4121, 832, 2304, 6425, 448, 1), (9, 4121, 832, 4096, 10521, 672, 1),
                                                  (9, 100, 250, 4096, 10521, 0, 4), (1, 64, 64, 192, 300, 64, 1)):
        src = torch.randint(0, k_len + 50, (2, 3, Gs, Ks), generator=g, dtype=torch.int32)   # some beyond Lk: clamped
        Gk = (q_len + 191) // 192
        local = torch.randint(0, k_len, (Gk, L), generator=g) if L else None
        counts_S = torch.full((2, 3, Gs), count, dtype=torch.int32)
        e_idx, e_cnt = oracle.map_inds_counts_across_scales(src, counts_S, q_len, k_len, 192, pad)
        cnt = int(e_cnt[0, 0, 0])
        if L:
            e_idx, e_cnt = oracle.append_local_run(e_idx, cnt, local, L, k_len)
        out, counts = ops.remap_concat_lists(src.cuda(), count, q_len, k_len, local.cuda() if L else None, 192, pad)
        assert out.shape == (2, 3, Gk, k_len)
        assert torch.equal(counts.cpu(), e_cnt)
        assert torch.equal(out[..., :cnt + L].cpu(), e_idx[..., :cnt + L])
        assert bool((out[..., cnt + L:] == 0).all())


@pytest.mark.gpu
def test_mask_to_lists_matches_oracle():
    import oracle
    from lvar_amd import sparse_attn_ops as ops
    g = torch.Generator().manual_seed(7)
    for shape, p, mult in (((2, 2, 32, 165), 0.25, 1), ((3, 5, 700), 0.2, 64), ((4, 64), 0.0, 8), ((4, 65), 1.0, 8), ((2, 130), 0.97, 112)):
        m = torch.rand(*shape, generator=g) < p
        cnt, idx = ops.mask_to_lists(m.cuda(), mult)
        e_cnt, e_idx = oracle.mask_to_lists(m, mult)
        assert torch.equal(cnt.cpu(), e_cnt) and torch.equal(idx.cpu(), e_idx), (shape, p, mult)


@pytest.mark.gpu
def test_csp_attn_with_fused_ocache_upsample():
    """The sparse step with the O-cache resampled in the epilogue equals bilinear upsampling
    (library F.interpolate, align_corners=False, and the oracle's closed form) followed by the
    token-list attention; with empty lists it is the upsampling alone."""
    import torch.nn.functional as F
    import oracle
    from lvar_amd import sparse_attn_ops as ops
    g = torch.Generator().manual_seed(9)
    for (src, dst, d, Lk, cnt) in ((5, 8, 128, 200, 64), (16, 20, 64, 521, 128), (40, 48, 128, 1500, 192), (3, 16, 128, 300, 0)):
        B, H, Lq = 1, 2, dst * dst
        q = (torch.randn(B, H, Lq, d, generator=g) * 0.5).to(torch.bfloat16)
        k = (torch.randn(B, H, Lk, d, generator=g) * 0.5).to(torch.bfloat16)
        v = (torch.randn(B, H, Lk, d, generator=g) * 0.5).to(torch.bfloat16)
        cache = torch.randn(B, H, src * src, d, generator=g).to(torch.bfloat16)
        G = (Lq + 191) // 192
        idx = torch.zeros(B, H, G, Lk, dtype=torch.int32)
        for b in range(B):
            for h in range(H):
                for gg in range(G):
                    idx[b, h, gg, :cnt] = torch.randperm(Lk, generator=g)[:cnt].to(torch.int32)
        counts = torch.full((B, H, G), cnt, dtype=torch.int32)
        out = ops.csp_attn_upsampled(q.cuda(), k.cuda(), v.cuda(), None, idx.cuda(), counts.cuda(), cache.cuda(), 1)
        up = oracle.upsample_ocache(cache, src * src, dst * dst)
        lib = F.interpolate(cache.float().view(B * H, src, src, d).permute(0, 3, 1, 2), size=(dst, dst), mode="bilinear",
                            align_corners=False).permute(0, 2, 3, 1).reshape(B, H, Lq, d)
        assert torch.allclose(up.float(), lib, atol=1e-4)      # fp32 tap weights in the library routine
        ref = oracle.csp_attn(q, k, v, None, idx, counts, up, 1)
        assert close(out, ref), (src, dst, d)
        if cnt == 0:
            assert torch.allclose(out.float().cpu(), lib, atol=2e-2, rtol=1e-2)
    with pytest.raises(AssertionError):
        ops.csp_attn_upsampled(q.cuda(), k.cuda(), v.cuda(), None, idx.cuda(), counts.cuda(), cache[:, :, :8].cuda(), 1)


@pytest.mark.gpu
def test_ops_replay_correctly_from_a_hip_graph():
    """Every entry point only enqueues kernels on the caller's stream (no allocation, memset or
    synchronisation inside the library), so a decision-scale step can be captured once and replayed.
    Replays are interleaved with eager work and each one is compared with the eager result."""
    from lvar_amd import sparse_attn_ops as ops
    q, k, v = make_qkv(1, 2, 400, 921, 128, seed=21, amp=0.5)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()

    def step():
        o, cs, (M, L) = ops.dense_colsum_attn(qg, kg, vg)
        inds, counts = ops.topk_token_lists(cs, 192)
        cache = ops.csp_attn(qg, kg, vg, None, inds, counts, o, -1)
        _, bsum = ops.colsum(qg, kg, None, q_group_size=128, lse=(M, L), return_block_sums=True)
        num, idx = ops.block_topk_lists(bsum, 6)
        ob, _ = ops.block_sparse_attn(qg, kg, vg, num, idx, 128, 64)
        return o, cs, inds, cache, num, idx, ob

    eager = [t.clone() for t in step()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()                                                        # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for rep in range(3):
        qg.add_(0)                                                        # eager work between replays
        _ = ops.dense_attn(qg, kg, vg)
        torch.cuda.synchronize()
        for t in outs:
            t.zero_()                                                     # a replay must rewrite every output
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(outs, eager):
            assert torch.equal(a, b), rep


@pytest.mark.gpu
def test_window_key_scores_and_scalekv_selection():
    import oracle
    from lvar_amd import sparse_attn_ops as ops
    g = torch.Generator().manual_seed(15)
    for (B, H, Lq, Lk, d, W, ks, pooling) in ((1, 2, 400, 921, 128, 16, 5, "avgpool"), (2, 3, 64, 700, 64, 9, 7, "maxpool"),
                                              (1, 1, 300, 300, 128, 4, 1, "avgpool"), (1, 2, 1024, 2521, 128, 256, 5, "maxpool"),
                                              (1, 2, 200, 1300, 256, 24, 3, "avgpool")):
        q = (torch.randn(B, H, Lq, d, generator=g) * 0.5).to(torch.bfloat16)
        k = (torch.randn(B, H, Lk, d, generator=g) * 0.5).to(torch.bfloat16)
        win = torch.randint(Lk - Lq, Lk, (B, H, W), generator=g)
        if W >= 9:
            win[..., 1] = win[..., 0]                                     # a repeated window token
            win[..., 2] = Lk - 1                                          # the last key: pooling at the border
        got = ops.window_key_scores(q.cuda(), k.cuda(), win.cuda(), ks, pooling).cpu()
        ref = oracle.window_key_scores(q, k, win, ks, pooling)
        inf = torch.isinf(ref)
        assert torch.equal(torch.isinf(got), inf), (Lq, Lk, pooling)
        assert torch.allclose(got[~inf], ref[~inf], rtol=1e-3, atol=1e-3)
        keep = ops.scalekv_keep_indices(q.cuda(), k.cuda(), win.cuda(), W + 50, ks, pooling).cpu()
        assert keep.shape == (B, H, W + 50) and bool((keep[..., 1:] >= keep[..., :-1]).all())
        # the kept non-window keys are a top-50 set of the library's own scores
        sc = got.clone()
        for b in range(B):
            for h in range(H):
                rest = [x for x in keep[b, h].tolist() if x not in set(win[b, h].tolist())]
                if torch.isinf(sc[b, h]).sum() <= Lk - 50:
                    assert len(rest) == 50
                    thr = torch.topk(sc[b, h], 50).values[-1]
                    assert bool((sc[b, h, rest] >= thr).all())


def test_compiled_dense_binding_matches_ctypes_path():
    """dense_attn through the compiled torch binding (when built) and through the ctypes path: same bits;
    strided, misaligned or wrongly typed inputs fall through to the general path with its behaviour."""
    from lvar_amd import _lib, sparse_attn_ops as ops
    mod = _lib.torch_binding()
    if mod is None:
        pytest.skip("torch binding not built")
    q, k, v = make_qkv(2, 3, 200, 333, 128, seed=5, amp=0.5)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    for scale in (None, 0.07):
        fast = mod.fast_dense_attn(qg, kg, vg, scale)
        assert fast is not None
        o, M, L, _ = ops._dense_launch(qg, kg, vg, scale)
        assert torch.equal(fast[0], o) and torch.equal(fast[1], M) and torch.equal(fast[2], L)
        assert fast[1].shape == (2, 3, 200, 1) and fast[2].shape == (2, 3, 200, 1)
        o2, (M2, L2) = ops.dense_attn(qg, kg, vg, scale)
        assert torch.equal(o2, o) and torch.equal(M2, M) and torch.equal(L2, L)
    # not the plain case: strided views, fp16, mismatched shapes
    assert mod.fast_dense_attn(qg.transpose(1, 2), kg, vg, None) is None
    assert mod.fast_dense_attn(qg.half(), kg.half(), vg.half(), None) is None
    assert mod.fast_dense_attn(qg, kg, vg[:, :, :100], None) is None
    qs = qg.transpose(1, 2).contiguous().transpose(1, 2)          # [B,H,L,d] view of a [B,L,H,d] buffer
    o3, _ = ops.dense_attn(qs, kg, vg, None)
    o_ref, _, _, _ = ops._dense_launch(qg, kg, vg, None)
    assert torch.equal(o3, o_ref)
    with pytest.raises((TypeError, ValueError)):
        ops.dense_attn(qg.half(), kg.half(), vg.half())
    # a scale that is not a Python float (numpy scalar, 0-dim tensor) takes the same path with the same bits
    import numpy as np
    o_f, (M_f, _) = ops.dense_attn(qg, kg, vg, 0.07)
    for sc in (np.float32(0.07), torch.tensor(0.07), torch.tensor(0.07, device="cuda"), np.float64(0.07)):
        o_s, (M_s, _) = ops.dense_attn(qg, kg, vg, sc)
        assert (o_s.float() - o_f.float()).abs().max().item() < 1e-2 and (M_s - M_f).abs().max().item() < 1e-3
