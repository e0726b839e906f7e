"""Host-side list / mask construction (lvar_amd.mask_build, torch-vectorised) against the CPU
oracle's loop-based restatement of the reference arithmetic, and the configuration module."""
import os
import tempfile

import pytest
import torch

import oracle
from lvar_amd import mask_build as mb
from lvar_amd import sparse_attn_config as cfg


@pytest.fixture(autouse=True)
def _reset_config():
    cfg.reset()
    yield
    cfg.reset()


def test_kernel_config_and_yaml_merge():
    assert cfg.get_kernel_config_attn() == {"bm": 192, "counts_multiple_of": 64, "indices_pad_to": 1}
    with tempfile.NamedTemporaryFile("w", suffix=".yml", delete=False) as f:
        f.write("attn:\n  top_keys: 0.2\n  provider: cuda\n  cs4a_ws: [1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 7, 9]\n")
        path = f.name
    try:
        cfg.load_from_file(path)
    finally:
        os.unlink(path)
    assert cfg.GLOBAL_CONFIG["attn"]["top_keys"] == 0.2 and cfg.GLOBAL_CONFIG["attn"]["decision_scale"] == 10
    # the reference's provider names are accepted and keep their list granularity (sparse_attn_config.py:82-98)
    assert cfg.get_kernel_config_attn() == {"bm": 192, "counts_multiple_of": 112, "indices_pad_to": 4}
    assert mb.indices_count(0.2, 4121) == 784
    cfg.GLOBAL_CONFIG["attn"]["provider"] = "nope"
    with pytest.raises(ValueError):
        cfg.get_kernel_config_attn()


def test_list_builders_have_no_cpu_path():
    """The top-k list and the block-list compaction are HIP kernels: host tensors are refused, not served by torch
    (the GPU tests compare them with the oracle).  Argument errors are still reported before the device is looked at."""
    bs = torch.rand(2, 3, 4, 680, generator=torch.Generator().manual_seed(0))
    with pytest.raises(RuntimeError, match="no CPU path"):
        mb.topk_index_list(bs, 0.5)
    with pytest.raises(RuntimeError, match="no CPU path"):
        mb.block_mask_to_lists(bs > 0.5)
    with pytest.raises(ValueError):
        mb.topk_index_list(bs[..., :10], 7.0)


def test_map_inds_counts_matches_oracle():
    g = torch.Generator().manual_seed(1)
    inds_S = torch.randint(0, 4121, (2, 2, 9, 4121), generator=g, dtype=torch.int32)
    counts_S = torch.full((2, 2, 9), 832, dtype=torch.int32)
    for q_len, k_len, pad in ((2304, 6425, 1), (4096, 10521, 1), (4096, 10521, 4), (192, 100, 1)):
        a, ac = mb.map_inds_counts_across_scales(inds_S, counts_S, q_len, k_len, indices_pad_to=pad)
        b, bc = oracle.map_inds_counts_across_scales(inds_S, counts_S, q_len, k_len, indices_pad_to=pad)
        assert torch.equal(a, b) and torch.equal(ac, bc)
    small = torch.tensor([5, 9, 100], dtype=torch.int32).view(1, 1, 1, 3)
    a, _ = mb.map_inds_counts_across_scales(small, 3, 192, 50, indices_pad_to=4)
    b, _ = oracle.map_inds_counts_across_scales(small, torch.tensor([[[3]]]), 192, 50, indices_pad_to=4)
    assert torch.equal(a, b)


def test_map_inds_counts_with_sink_matches_oracle_and_hand_case():
    """The ``add_sink`` branch (models/sparvar/sparse_attn.py:423-469): torch mirror against the brute-force oracle on
    random lists, and one row worked out by hand."""
    g = torch.Generator().manual_seed(6)
    for (Ks, count, pad, sink_len, frac, q_len, k_len) in ((300, 100, 4, 21, 0.2, 2304, 6425), (40, 96, 1, 5, 0.5, 960, 30),
                                                             (64, 64, 64, 200, 0.2, 192, 4121), (50, 10, 1, 3, 1.0, 400, 77)):
        inds_S = torch.randint(0, 400, (2, 2, 9, Ks), generator=g, dtype=torch.int32)
        a, ac = mb.map_inds_counts_across_scales(inds_S, count, q_len, k_len, indices_pad_to=pad, add_sink=True,
                                                 sink_len=sink_len, sink_quota_frac=frac)
        b, bc = oracle.map_inds_counts_across_scales(inds_S, torch.tensor([[[count]]]), q_len, k_len, indices_pad_to=pad,
                                                     add_sink=True, sink_len=sink_len, sink_quota_frac=frac)
        assert torch.equal(a, b) and torch.equal(ac, bc) and a.dtype == torch.int32
    # one source group, count 6, sink_len 3, frac 0.5: sink quota min(round(3.0), 6, 3) = 3 -> keys 0, 1, 2; then the three
    # smallest entries >= 3 of the whole row [7, 1, 9, 3, 3, 50, 2, 8] -> 3, 3, 7; key 50 would be clamped to Lk - 1 = 9
    row = torch.tensor([7, 1, 9, 3, 3, 50, 2, 8], dtype=torch.int32).view(1, 1, 1, 8)
    for fn in (mb.map_inds_counts_across_scales, oracle.map_inds_counts_across_scales):
        out, cnt = fn(row, torch.tensor([[[6]]]), 192, 10, add_sink=True, sink_len=3, sink_quota_frac=0.5)
        assert out.tolist() == [[[[0, 1, 2, 3, 3, 7]]]] and int(cnt[0, 0, 0]) == 6
        out, _ = fn(row, torch.tensor([[[8]]]), 192, 10, add_sink=True, sink_len=3, sink_quota_frac=0.25)
        assert out.tolist() == [[[[0, 1, 3, 3, 7, 8, 9, 9]]]]           # sink quota 2; the six survivors 3, 3, 7, 8, 9, 50, the last clamped to Lk - 1
        # sink_len 0 or add_sink False: the plain path
        out, _ = fn(row, torch.tensor([[[4]]]), 192, 10, add_sink=True, sink_len=0)
        assert out.tolist() == [[[[7, 1, 9, 3]]]]


@pytest.mark.parametrize("si,win,m", [(11, 5, 112), (12, 7, 112), (11, 7, 64), (12, 9, 64), (10, 3, 64)])
def test_local_group_runs_matches_oracle(si, win, m):
    runs, L = mb.local_group_runs(si, win, 192, m)
    ia, kv = oracle.crossscale_self_indices(si, win)
    S = oracle.INFINITY_SCALES[si]
    ref, Lr = oracle.aggregate_group_indices(ia, S * S, kv, 192, m)
    assert L == Lr and torch.equal(runs, ref)


def test_append_local_run_layout():
    inds = torch.arange(2 * 1 * 3 * 128, dtype=torch.int32).view(2, 1, 3, 128) % 500
    local = torch.arange(3 * 64).view(3, 64) + 1000
    out, counts = mb.append_local_run(inds, 128, local, 64, k_len=2000)
    assert out.shape == (2, 1, 3, 2000) and bool((counts == 192).all())
    assert torch.equal(out[..., :128], inds) and torch.equal(out[0, 0, :, 128:192], local.to(torch.int32))
    assert bool((out[..., 192:] == 0).all())
    with pytest.raises(AssertionError):
        mb.append_local_run(inds, 100, local, 64, k_len=2000)      # 164 is not a multiple of 64


def test_upsample_ocache_matches_oracle():
    x = torch.randn(2, 2, 1600, 8, generator=torch.Generator().manual_seed(2))
    for tgt in (2304, 4096):
        assert torch.allclose(mb.upsample_ocache(x, 1600, tgt).double(), oracle.upsample_ocache(x, 1600, tgt), atol=1e-4)  # fp32 library vs fp64 closed form


def test_flex_block_mask_matches_oracle():
    ks = [-1, -1, -1, -1, 1, 1, 3, 5, 7]
    for bq, bk in ((128, 128), (128, 64), (64, 64)):
        a = mb.flex_block_mask(8, ks, 3, bq, block_k=bk)
        b = oracle.flex_block_mask(8, ks, 3, bq, block_k=bk)
        assert torch.equal(a, b)
    # the shipped CSLA configuration at the last scale: [32, 83] blocks of 128 (SparseFlexAttn, models/sparvar/basic_sparvar.py:55-72)
    m = mb.flex_block_mask(12, [-1, -1, -1, -1, -1, -1, -1, -1, 1, 1, 3, 5, 7], 5, 128)
    assert m.shape == (32, 83) and bool(m[:, 0].all())


def test_block_sums_and_keep_counts():
    cs = torch.rand(1, 2, 3, 680, generator=torch.Generator().manual_seed(4))
    assert torch.allclose(mb.key_block_sums(cs, 64), oracle.key_block_sums(cs, 64))
    assert mb.block_keep_count(0.5, 11, k_len=680) == 5       # 64*round(0.5*680/64)/64, VAR-d16 benchmark case
    assert mb.block_keep_count(0.5, 11) == 6                  # round(5.5), half-to-even
    assert mb.block_keep_count(0.0, 11) == 1 and mb.block_keep_count(3.0, 11) == 11


def test_sink_window_topk_mask_matches_oracle():
    scores = torch.rand(2, 2, 32, 165, generator=torch.Generator().manual_seed(5))
    for density, window in ((0.25, 2), (0.5, 1), (0.1, 2)):
        a = mb.sink_window_topk_block_mask(scores, density=density, window=window)
        b = oracle.config2_block_mask(scores, density=density, window=window)
        assert torch.equal(a, b)
    a = mb.sink_window_topk_block_mask(scores)
    assert bool((a.sum(-1) == 41).all())


def test_flex_block_mask_hand_computed_fine_entries():
    from test_oracle import check_flex_fine_cases
    check_flex_fine_cases(mb.flex_block_mask)


def test_video_window_base_mask_matches_oracle():
    assert torch.equal(mb.video_window_base_mask(), oracle.video_window_block_mask())
    for (f, h, w, blk, fr, sr) in ((3, 4, 8, 8, 1, 1), (4, 4, 4, 16, 1, 0), (2, 8, 8, 16, 0, 2), (5, 2, 8, 4, 2, 1)):
        assert torch.equal(mb.video_window_base_mask(f, h, w, blk, fr, sr), oracle.video_window_block_mask(f, h, w, blk, fr, sr))
    with pytest.raises(ValueError):
        mb.video_window_base_mask(2, 2, 3, 4)


def test_base_plus_topk_block_mask_equals_config2_selection():
    g = torch.Generator().manual_seed(3)
    scores = torch.rand(1, 2, 32, 165, generator=g)
    scores[0, 0, 4, 100:120] = 0.5                                  # ties through the cut go to the smaller block
    base = mb.sink_window_base_mask(128, 64)
    want = oracle.config2_block_mask(scores)
    got = oracle.base_plus_topk_block_mask(scores, base, round(0.25 * 165))
    assert torch.equal(got, want)
    assert torch.equal(mb.sink_window_topk_block_mask(scores), got)
