"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py): the CPU tests guard
the oracle against drift, the GPU tests check the HIP path against the committed expectations."""
import os

import numpy as np
import pytest
import torch

import oracle

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(GOLD, name), allow_pickle=False)


def bf16(a):
    return torch.from_numpy(a.astype(np.int16)).view(torch.bfloat16)


def t(a):
    return torch.from_numpy(np.asarray(a))


def close(a, b, atol, rtol):
    return bool(((a - b).abs() <= atol + rtol * b.abs()).all())


def test_oracle_reproduces_var_d16_fixture():
    z = load("var_d16_dense_colsum.npz")
    q, k, v = bf16(z["q"]), bf16(z["k"]), bf16(z["v"])
    assert q.shape == (1, 1, 256, 64) and k.shape == (1, 1, 680, 64)
    o, cs, (M, L) = oracle.dense_colsum_attn(q, k, v)          # fp32 math this time
    assert close(o, t(z["o"]), 1e-5, 1e-5) and close(cs, t(z["cs"]), 1e-6, 1e-4)
    assert close(M + torch.log2(L), t(z["lse2"]), 1e-4, 0)
    bs = oracle.key_block_sums(t(z["cs_all"]), 64)
    assert close(bs, t(z["block_sums"]), 1e-5, 1e-5) and bs.shape[-1] == 11
    # VAR-d16 benchmark case: keep 64*round(0.5*680/64)/64 = 5 of 11 key blocks; mask is exact given the colsum
    top = torch.topk(t(z["block_sums"]), k=oracle.indices_count(0.5, 680, 64) // 64, dim=-1).indices.sort(-1).values
    assert torch.equal(top.to(torch.int32), t(z["top5_blocks"]))


def test_oracle_reproduces_sparse_fixtures():
    z = load("csp_attn_d128.npz")
    q, k, v, o0 = bf16(z["q"]), bf16(z["k"]), bf16(z["v"]), bf16(z["o0"])
    inds, counts = t(z["inds"]), t(z["counts"])
    assert close(oracle.csp_attn(q, k, v, None, inds, counts, o0, -1), t(z["out_minus"]), 1e-5, 1e-5)
    assert close(oracle.csp_attn(q, k, v, None, inds, counts, o0, 1), t(z["out_plus"]), 1e-5, 1e-5)
    z = load("block_sparse_d128.npz")
    o, M, L = oracle.block_sparse_attn(bf16(z["q"]), bf16(z["k"]), bf16(z["v"]), t(z["num"]), t(z["idx"]), 128, 64)
    assert close(o, t(z["o"]), 1e-5, 1e-5) and close(M + torch.log2(L), t(z["lse2"]), 1e-4, 0)


def test_list_build_constants_fixture():
    from lvar_amd import mask_build as mb
    z = load("list_build_constants.npz")
    assert z["cum"].tolist() == mb.scale_offsets()
    r11, l11 = mb.local_group_runs(11, 7, 192, 112)
    r12, l12 = mb.local_group_runs(12, 9, 192, 112)
    assert torch.equal(r11, t(z["runs11"])) and torch.equal(r12, t(z["runs12"]))
    assert (l11, l12) == (z["runs11"].shape[1], z["runs12"].shape[1]) == (560, 784)
    m = mb.flex_block_mask(8, [-1, -1, -1, -1, 1, 1, 3, 5, 7], 3, 128)
    assert torch.equal(m, t(z["csla_scale8"]))


@pytest.mark.gpu
def test_hip_matches_var_d16_fixture():
    from lvar_amd import mask_build as mb
    from lvar_amd import sparse_attn_ops as ops
    z = load("var_d16_dense_colsum.npz")
    q, k, v = (bf16(z[n]).cuda() for n in "qkv")
    o, cs = ops.dense_colsum_attn_s(q, k, v)
    assert close(o.float().cpu(), t(z["o"]), 2e-2, 1e-2)
    assert close(cs.cpu(), t(z["cs"]), 1e-6, 1e-3)
    cs_all = ops.colsum(q, k, q_group_size=256)
    assert close(cs_all.cpu(), t(z["cs_all"]), 1e-6, 1e-3)
    bs = mb.key_block_sums(cs_all, 64)
    assert close(bs.cpu(), t(z["block_sums"]), 1e-5, 1e-3)
    # the mask derived from an identical colsum is bit-exact
    num, idx = mb.topk_block_lists(t(z["block_sums"]).cuda(), 0.5, k_len=680)
    assert int(num[0, 0, 0]) == 5 and torch.equal(idx.cpu(), t(z["top5_blocks"]))
    # and here the HIP colsum ranks the same blocks (block sums differ by far more than its error)
    num2, idx2 = mb.topk_block_lists(bs, 0.5, k_len=680)
    assert torch.equal(idx2.cpu(), t(z["top5_blocks"]))
    # block-sparse attention over those 5 blocks of 64 keys (one 128-row query block pair)
    nb = num2.expand(1, 1, 2).contiguous()
    ib = idx2.expand(1, 1, 2, 5).contiguous()
    ob, _ = ops.block_sparse_attn(q, k, v, nb, ib, 128, 64)
    ref, _, _ = oracle.block_sparse_attn(bf16(z["q"]), bf16(z["k"]), bf16(z["v"]), nb.cpu(), ib.cpu(), 128, 64)
    assert close(ob.float().cpu(), ref, 2e-2, 1e-2)


@pytest.mark.gpu
def test_hip_matches_sparse_fixtures():
    from lvar_amd import sparse_attn_ops as ops
    z = load("csp_attn_d128.npz")
    q, k, v, o0 = (bf16(z[n]).cuda() for n in ("q", "k", "v", "o0"))
    inds, counts = t(z["inds"]).cuda(), t(z["counts"]).cuda()
    assert close(ops.csp_attn(q, k, v, None, inds, counts, o0, -1).float().cpu(), t(z["out_minus"]), 2e-2, 1e-2)
    assert close(ops.csp_attn(q, k, v, None, inds, counts, o0, 1).float().cpu(), t(z["out_plus"]), 2e-2, 1e-2)
    z = load("block_sparse_d128.npz")
    o, (M, L) = ops.block_sparse_attn(bf16(z["q"]).cuda(), bf16(z["k"]).cuda(), bf16(z["v"]).cuda(),
                                      t(z["num"]).cuda(), t(z["idx"]).cuda(), 128, 64)
    assert close(o.float().cpu(), t(z["o"]), 2e-2, 1e-2)
    assert close((M + torch.log2(L)).cpu(), t(z["lse2"]), 1e-3, 0)


def test_oracle_and_host_mirrors_reproduce_list_kernel_fixture():
    from lvar_amd import mask_build as mb
    z = load("list_kernels.npz")
    assert torch.equal(oracle.topk_token_set(t(z["scores"]), 128), t(z["topk128"]))
    # the torch host arithmetic of lvar_amd.mask_build (remap + local-run append) gives the same lists
    assert mb.indices_count(128 / 700, t(z["scores"]).shape[-1], 64) == 128
    a, c = mb.map_inds_counts_across_scales(t(z["src"]), 192, 2304, 900)
    out, cnt = mb.append_local_run(a, 192, t(z["local"]), 64, 900, multiple_of=64)
    assert torch.equal(out, t(z["remap_concat"])) and torch.equal(cnt, t(z["remap_counts"]))
    mc, mi = oracle.mask_to_lists(t(z["mask"]), 64)
    assert torch.equal(mc, t(z["mask_counts"])) and torch.equal(mi, t(z["mask_idx"]))
    ws = oracle.window_key_scores(bf16(z["q"]), bf16(z["k"]), t(z["window"]), 5, "avgpool", dtype=torch.float64)
    ref = t(z["window_scores"])
    assert torch.equal(torch.isinf(ws), torch.isinf(ref)) and close(ws[~torch.isinf(ref)].float(), ref[~torch.isinf(ref)], 1e-5, 1e-5)


@pytest.mark.gpu
def test_hip_matches_list_kernel_fixture():
    from lvar_amd import sparse_attn_ops as ops
    z = load("list_kernels.npz")
    idx, cnt = ops.topk_token_lists(t(z["scores"]).cuda(), 128)
    assert torch.equal(idx[..., :128].cpu(), t(z["topk128"])) and bool((cnt == 128).all())
    from lvar_amd import mask_build as mb
    inds, counts = mb.topk_index_list(t(z["scores"]).unsqueeze(0).cuda(), 128 / 700, multiple_of=64, order="index")
    assert int(counts[0, 0, 0]) == 128 and torch.equal(inds[0, ..., :128].cpu(), t(z["topk128"]))
    out, counts = ops.remap_concat_lists(t(z["src"]).cuda(), 192, 2304, 900, t(z["local"]).cuda())
    assert torch.equal(out.cpu(), t(z["remap_concat"])) and torch.equal(counts.cpu(), t(z["remap_counts"]))
    mc, mi = ops.mask_to_lists(t(z["mask"]).cuda(), 64)
    assert torch.equal(mc.cpu(), t(z["mask_counts"])) and torch.equal(mi.cpu(), t(z["mask_idx"]))
    q, k, v, cache = (bf16(z[n]).cuda() for n in ("q", "k", "v", "cache"))
    up = ops.csp_attn_upsampled(q, k, v, None, t(z["uidx"]).cuda(), t(z["ucnt"]).cuda(), cache, 1)
    assert close(up.float().cpu(), t(z["upsampled_out"]), 2e-2, 1e-2)
    ws = ops.window_key_scores(q, k, t(z["window"]).cuda(), 5, "avgpool").cpu()
    ref = t(z["window_scores"])
    fin = ~torch.isinf(ref)
    assert torch.equal(torch.isinf(ws), ~fin) and close(ws[fin], ref[fin], 1e-3, 1e-3)
