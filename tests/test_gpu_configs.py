"""The benchmark configurations at their full sizes, beyond the headline one (which
``test_gpu_fullsize.py`` covers): the colsum kernel at Infinity-2B scale 48 and scale 64 with N(0,1)
inputs and block top-k at keep ratios 10 / 25 / 50 %, the Bernoulli density sweep, and the long-video
block-sparse configuration (B1 H24 Lq = Lk = 32768, 128x128 blocks, 3D window + colsum top-k at 10 %).
The CPU oracle is too slow for whole problems of this size, so each test checks size-independent
properties of the whole output and oracle parity on slices of the same launch."""
import pytest
import torch

import oracle
from conftest import make_qkv

pytestmark = pytest.mark.gpu

D = 128


def close(a, b, atol=2e-2, rtol=1e-2):
    return bool(((a.float().cpu() - b).abs() <= atol + rtol * b.abs()).all())


def oracle_rows(q, k, v, num, idx, b, h, blocks, bq, bk):
    """Oracle block-sparse attention of the query blocks ``blocks`` (a range) of one (batch, head)."""
    lo, hi = blocks.start * bq, min(blocks.stop * bq, q.shape[2])
    nb = num[b if num.shape[0] > 1 else 0, h if num.shape[1] > 1 else 0, blocks.start:blocks.stop][None, None]
    ib = idx[b if idx.shape[0] > 1 else 0, h if idx.shape[1] > 1 else 0, blocks.start:blocks.stop][None, None]
    return oracle.block_sparse_attn(q[b:b + 1, h:h + 1, lo:hi], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], nb, ib, bq, bk), (lo, hi)


# ---------------------------------------------------------------- colsum alone, scales 48 and 64

@pytest.mark.parametrize("Lq,Lk", [(2304, 6425), (4096, 10521)])
def test_colsum_config_block_sums_and_topk(Lq, Lk):
    """B2 H16 d128, N(0,1) inputs: fp32 colsum [B,H,G,Lk] (1e-3 relative against the oracle on two slices,
    every probability row sums to one), the per-64-key block sums from the same launch, the sum over the
    query groups = total colsum [B,H,Lk], and block top-k lists at keep 10 / 25 / 50 % bit-exact against
    the oracle selection on the same block sums."""
    from lvar_amd import sparse_attn_ops as ops
    B, H = 2, 16
    q, k, v = make_qkv(B, H, Lq, Lk, D, seed=Lq + 3 * Lk, amp=1.0)
    qg, kg = q.cuda(), k.cuda()
    cs, bs = ops.colsum(qg, kg, None, q_group_size=192, return_block_sums=True)
    G, nK = (Lq + 191) // 192, (Lk + 63) // 64
    assert cs.shape == (B, H, G, Lk) and bs.shape == (B, H, G, nK) and cs.dtype == torch.float32
    assert bool((cs >= 0).all())
    rows = torch.tensor([min(192, Lq - g * 192) for g in range(G)], dtype=torch.float32, device="cuda")
    assert torch.allclose(cs.sum(-1), rows.expand(B, H, G), rtol=1e-3)
    pad = torch.nn.functional.pad(cs, (0, 64 * nK - Lk))
    assert torch.allclose(pad.view(B, H, G, nK, 64).sum(-1), bs, rtol=1e-4, atol=1e-6)
    for (b, h) in ((0, 3), (1, 12)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        _, cs_ref, _ = oracle.dense_colsum_attn(q[sl], k[sl], v[sl])
        assert torch.allclose(cs[sl].cpu(), cs_ref, rtol=1e-3, atol=1e-6), (b, h)
        # total colsum over all queries [Lk] = sum over the group axis
        assert torch.allclose(cs[sl].sum(2).cpu(), cs_ref.sum(2), rtol=1e-3, atol=1e-6)
    # whole-sequence colsum in one group per 128 rows feeds the block selection
    _, bsum = ops.colsum(qg, kg, None, q_group_size=128, return_block_sums=True)
    bsum_cpu = bsum.cpu()
    for keep in (0.10, 0.25, 0.50):
        target = int(round(keep * nK))
        num, idx = ops.block_topk_lists(bsum, target)
        assert bool((num == target).all())
        ref = oracle.topk_token_set(bsum_cpu, target)                          # stable selection, ascending
        assert torch.equal(idx[..., :target].cpu(), ref), keep
        assert bool((idx[..., target:] == 0).all())


# ---------------------------------------------------------------- density sweep

@pytest.mark.parametrize("pct", [5, 10, 25, 50, 75])
def test_density_sweep_full_size(pct):
    """B1 H16 Lq4096 Lk10521, 128x64 blocks, Bernoulli(pct) block masks with at least one block per row."""
    from lvar_amd import mask_build as mb, sparse_attn_ops as ops
    B, H, Lq, Lk, bq, bk = 1, 16, 4096, 10521, 128, 64
    nQ, nK = Lq // bq, (Lk + bk - 1) // bk
    q, k, v = make_qkv(B, H, Lq, Lk, D, seed=77 + pct, amp=1.0)
    g = torch.Generator().manual_seed(7)
    mask = torch.rand(B, H, nQ, nK, generator=g) < pct / 100.0
    mask.scatter_(-1, torch.randint(0, nK, (B, H, nQ, 1), generator=g), True)
    num, idx = mb.block_mask_to_lists(mask.cuda())
    n_ref, i_ref = oracle.block_mask_to_lists(mask)
    assert torch.equal(num.cpu(), n_ref) and torch.equal(idx.cpu(), i_ref)
    assert int(num.min()) >= 1
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    o, (M, L) = ops.block_sparse_attn(qg, kg, vg, num, idx, bq, bk)
    assert bool(torch.isfinite(o.float()).all())
    # rows of P sum to one whatever the list
    o1, _ = ops.block_sparse_attn(qg, kg, torch.ones_like(vg), num, idx, bq, bk)
    assert (o1.float() - 1.0).abs().max().item() < 8e-3
    for (h, blocks) in ((2, range(0, 2)), (11, range(nQ - 2, nQ))):
        (o_ref, M_ref, L_ref), (lo, hi) = oracle_rows(q, k, v, n_ref, i_ref, 0, h, blocks, bq, bk)
        assert close(o[0:1, h:h + 1, lo:hi], o_ref), (pct, h)
        lse = M[0, h, lo:hi].cpu() + torch.log2(L[0, h, lo:hi].cpu())
        assert (lse - (M_ref[0, 0] + torch.log2(L_ref[0, 0]))).abs().max().item() < 1e-3


# ---------------------------------------------------------------- long video

def test_video_block_sparse_full_size():
    """B1 H24 d128 Lq = Lk = 32768 (8 frames x 64 x 64), 128x128 blocks: 3D window (+-1 frame, +-1 spatial
    block) plus colsum top-k blocks up to 10 % of the 256 key blocks per row."""
    from lvar_amd import mask_build as mb, sparse_attn_ops as ops
    B, H, L, bq = 1, 24, 32768, 128
    nQ = nK = L // bq
    q, k, v = make_qkv(B, H, L, L, D, seed=2468, amp=0.5)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    num, idx, score = mb.video_window_topk_block_lists(qg, kg, None, density=0.10)
    target = int(round(0.10 * nK))
    assert num.shape == (B, H, nQ) and idx.shape == (B, H, nQ, nK)
    assert bool((num == target).all())
    sel = idx[..., :target]
    assert bool((sel[..., 1:] > sel[..., :-1]).all()) and bool((idx[..., target:] == 0).all())
    # the window blocks are all present, and the whole selection equals the oracle's on the same scores
    base = oracle.video_window_block_mask()
    assert torch.equal(mb.video_window_base_mask(device="cuda").cpu(), base)
    got = oracle.lists_to_block_mask(num.cpu(), idx.cpu(), nK)
    assert bool((got | ~base).all())
    want = oracle.base_plus_topk_block_mask(score.cpu(), base, target)
    assert torch.equal(got, want)
    # the block scores are sums of colsum rows: every sampled query row adds probability one
    assert torch.allclose(score.sum(-1), torch.full((B, H, nQ), 32.0, device="cuda"), rtol=1e-3)

    o, (M, Lsum) = ops.block_sparse_attn(qg, kg, vg, num, idx, bq, 128)
    assert bool(torch.isfinite(o.float()).all())
    o1, _ = ops.block_sparse_attn(qg, kg, torch.ones_like(vg), num, idx, bq, 128)
    assert (o1.float() - 1.0).abs().max().item() < 8e-3
    n_cpu, i_cpu = num.cpu(), idx.cpu()
    for (h, blocks) in ((0, range(0, 2)), (13, range(100, 103)), (23, range(nQ - 1, nQ))):
        (o_ref, M_ref, L_ref), (lo, hi) = oracle_rows(q, k, v, n_cpu, i_cpu, 0, h, blocks, bq, 128)
        assert close(o[0:1, h:h + 1, lo:hi], o_ref), h
        lse = M[0, h, lo:hi].cpu() + torch.log2(Lsum[0, h, lo:hi].cpu())
        assert (lse - (M_ref[0, 0] + torch.log2(L_ref[0, 0]))).abs().max().item() < 1e-3
    # the complete list is dense attention, bit for bit, on one head
    full = torch.arange(nK, dtype=torch.int32, device="cuda").expand(1, 1, nQ, nK).contiguous()
    nfull = torch.full((1, 1, nQ), nK, dtype=torch.int32, device="cuda")
    o_full, (Mf, Lf) = ops.block_sparse_attn(qg[:, 5:6], kg[:, 5:6], vg[:, 5:6], nfull, full, bq, 128)
    o_dense, (Md, Ld) = ops.dense_attn(qg[:, 5:6], kg[:, 5:6], vg[:, 5:6])
    assert torch.equal(o_full, o_dense) and torch.equal(Mf, Md) and torch.equal(Lf, Ld)
    (o_ref, _, _), (lo, hi) = oracle_rows(q, k, v, nfull.cpu(), full.cpu(), 0, 5, range(17, 18), bq, 128)
    assert close(o_dense[0:1, 0:1, lo:hi], o_ref)
