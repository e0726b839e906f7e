"""Parity of the HIP kernels (through the C ABI) against the CPU oracle on seeded inputs.

Tolerances: attention output within 2e-2 abs / 1e-2 rel of the fp32 oracle (bf16 output),
colsum within 1e-3 relative, (M, L) compared through M + log2(L) (natural lse) to 1e-3 abs.
"""
import math

import pytest
import torch

import oracle
from conftest import make_qkv

pytestmark = pytest.mark.gpu

ATOL_O, RTOL_O = 2e-2, 1e-2


def dev(*ts):
    return [t.cuda() for t in ts]


def check_o(o_gpu, o_ref, what=""):
    o = o_gpu.float().cpu()
    err = (o - o_ref).abs()
    tol = ATOL_O + RTOL_O * o_ref.abs()
    assert bool((err <= tol).all()), f"{what}: max err {err.max().item():.4g}, worst excess {(err - tol).max().item():.4g}"


def check_lse(M_gpu, L_gpu, M_ref, L_ref):
    a = M_gpu.float().cpu() + torch.log2(L_gpu.float().cpu())
    b = M_ref + torch.log2(L_ref)
    fin = torch.isfinite(b)
    assert bool((torch.isfinite(a) == fin).all())
    assert (a[fin] - b[fin]).abs().max().item() < 1e-3


DENSE_SHAPES = [
    (2, 16, 256, 680, 64),    # VAR-d16 last scale (the CPU-runnable benchmark shape)
    (1, 2, 300, 1000, 128),   # ragged Lq and Lk
    (1, 3, 128, 64, 128),     # exactly one key tile
    (1, 2, 33, 25, 128),      # fewer keys than one tile, Lq not a multiple of 32
    (1, 1, 1, 1, 64),         # degenerate
    (1, 2, 1600, 4121, 128),  # Infinity decision scale, one batch x two heads
]


@pytest.mark.parametrize("B,H,Lq,Lk,d", DENSE_SHAPES)
def test_dense_attn(B, H, Lq, Lk, d):
    from lvar_amd import sparse_attn_ops as ops
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=Lq * 7 + Lk)
    o_ref, M_ref, L_ref = oracle.dense_attn(q, k, v)
    o, (M, L) = ops.dense_attn(*dev(q, k, v))
    torch.cuda.synchronize()
    assert o.shape == q.shape and M.shape == (B, H, Lq, 1) and L.shape == (B, H, Lq, 1)
    check_o(o, o_ref, "dense")
    check_lse(M, L, M_ref, L_ref)
    # M is the true row maximum of the base-2 logits
    assert (M.cpu() - M_ref).abs().max().item() < 1e-3


def test_dense_attn_scale_and_strides():
    from lvar_amd import sparse_attn_ops as ops
    q, k, v = make_qkv(2, 4, 200, 333, 128, seed=5, amp=0.5)
    # strided views: [B,L,H,d] storage permuted to [B,H,L,d] (what a fused qkv projection yields)
    qg = q.cuda().permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    kg = k.cuda().permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    vg = v.cuda().permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    assert not qg.is_contiguous()
    o, (M, L) = ops.dense_attn(qg, kg, vg, scale=1.0)
    o_ref, M_ref, L_ref = oracle.dense_attn(q, k, v, scale=1.0)
    check_o(o, o_ref, "dense strided scale=1")
    check_lse(M, L, M_ref, L_ref)


def test_dense_attn_large_logits_rescale():
    """Row maxima that keep growing along the key axis exercise the lazy accumulator rescale."""
    from lvar_amd import sparse_attn_ops as ops
    B, H, Lq, Lk, d = 1, 2, 128, 1024, 128
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=11)
    ramp = torch.linspace(0.2, 3.0, Lk).view(1, 1, Lk, 1)
    k = (k.float() * ramp).to(torch.bfloat16)
    o_ref, M_ref, L_ref = oracle.dense_attn(q, k, v, scale=1.0)
    o, (M, L) = ops.dense_attn(*dev(q, k, v), scale=1.0)
    check_o(o, o_ref, "dense growing max")
    check_lse(M, L, M_ref, L_ref)


COLSUM_SHAPES = [
    (1, 2, 33, 25, 128),      # one ragged tile, fewer keys than a block
    (1, 2, 4096, 300, 128),   # many stages: exercises the 4-deep LDS ring and its tail
    (1, 1, 160, 64, 64),      # odd number of 32-row tiles
    (2, 16, 256, 680, 64),
    (1, 4, 256, 1000, 64),    # the reference's enabled self-test shape (attn_dense_colsum.py:573)
    (1, 2, 300, 1000, 128),   # last group has 108 rows
    (1, 2, 1600, 4121, 128),
    (1, 1, 70, 30, 128),
]


@pytest.mark.parametrize("B,H,Lq,Lk,d", COLSUM_SHAPES)
def test_dense_colsum_attn(B, H, Lq, Lk, d):
    from lvar_amd import sparse_attn_ops as ops
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=Lq + 3 * Lk)
    o_ref, cs_ref, (M_ref, L_ref) = oracle.dense_colsum_attn(q, k, v)
    o, cs = ops.dense_colsum_attn_s(*dev(q, k, v))
    G = (Lq + 191) // 192
    assert cs.shape == (B, H, G, Lk) and cs.dtype == torch.float32
    check_o(o, o_ref, "colsum o")
    csc = cs.cpu()
    assert torch.allclose(csc, cs_ref, rtol=1e-3, atol=1e-6), (csc - cs_ref).abs().max()
    # every softmax row sums to one: sum_n cs[g, n] = rows in group g
    rows = torch.tensor([min(192, Lq - g * 192) for g in range(G)], dtype=torch.float32)
    assert torch.allclose(csc.sum(-1), rows.expand(B, H, G), rtol=1e-4)
    o2, cs2 = ops.dense_colsum_attn_q(*dev(q, k, v))
    assert torch.equal(cs2, cs) and torch.equal(o2, o)  # deterministic


def test_colsum_standalone_groups_and_zero_query():
    from lvar_amd import sparse_attn_ops as ops
    B, H, Lq, Lk, d = 1, 2, 256, 680, 64
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=3)
    qg, kg = dev(q, k)
    cs_all = ops.colsum(qg, kg, q_group_size=256).cpu()       # one group = total colsum [B,H,1,Lk]
    cs_192 = ops.colsum(qg, kg).cpu()
    cs_32 = ops.colsum(qg, kg, q_group_size=32).cpu()
    _, ref_all, _ = oracle.dense_colsum_attn(q, k, v, q_group_size=256)
    assert torch.allclose(cs_all, ref_all, rtol=1e-3, atol=1e-6)
    assert torch.allclose(cs_192.sum(2, keepdim=True), cs_all, rtol=1e-4, atol=1e-6)
    assert torch.allclose(cs_32.sum(2, keepdim=True), cs_all, rtol=1e-4, atol=1e-6)
    # fused per-64-key block sums (ragged last block: 680 = 10*64 + 40)
    cs2, bs2 = ops.colsum(qg, kg, return_block_sums=True)
    assert torch.equal(cs2.cpu(), cs_192) and bs2.shape == (B, H, 2, 11)
    assert torch.allclose(bs2.cpu(), oracle.key_block_sums(cs_192, 64), rtol=1e-5, atol=1e-6)
    # row statistics handed in from a previous dense pass give the same colsum
    _, (M, L) = ops.dense_attn(qg, kg, dev(v)[0])
    assert torch.allclose(ops.colsum(qg, kg, lse=(M, L)).cpu(), cs_192, rtol=1e-5, atol=1e-7)
    # q = 0  =>  uniform softmax  =>  cs = rows / Lk exactly representable up to rounding
    z = torch.zeros_like(qg)
    cs0 = ops.colsum(z, kg).cpu()
    assert torch.allclose(cs0[:, :, 0], torch.full((B, H, Lk), 192.0 / Lk), rtol=1e-5)
    assert torch.allclose(cs0[:, :, 1], torch.full((B, H, Lk), 64.0 / Lk), rtol=1e-5)


def _random_lists(B, H, G, Lk, count, seed, unique=True):
    g = torch.Generator().manual_seed(seed)
    inds = torch.zeros(B, H, G, Lk, dtype=torch.int32)
    for b in range(B):
        for h in range(H):
            for gg in range(G):
                if unique:
                    sel = torch.randperm(Lk, generator=g)[:count]
                else:
                    sel = torch.randint(0, Lk, (count,), generator=g)
                inds[b, h, gg, :count] = sel.to(torch.int32)
    counts = torch.full((B, H, G), count, dtype=torch.int32)
    return inds, counts


@pytest.mark.parametrize("B,H,Lq,Lk,d,count,unique", [
    (2, 4, 384, 1000, 128, 640, True),    # the reference self-test's 640 unique keys per group
    (1, 2, 300, 500, 128, 200, False),    # duplicates, ragged last group (108 rows), count % 64 != 0
    (1, 2, 256, 680, 64, 320, True),
    (1, 1, 192, 100, 128, 37, False),
])
def test_csp_attn(B, H, Lq, Lk, d, count, unique):
    from lvar_amd import sparse_attn_ops as ops
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=count)
    G = (Lq + 191) // 192
    inds, counts = _random_lists(B, H, G, Lk, count, seed=count + 1, unique=unique)
    o0 = (torch.randn(B, H, Lq, d, generator=torch.Generator().manual_seed(9)) * 0.5).to(torch.bfloat16)
    for o_scale in (1, -1):
        ref = oracle.csp_attn(q, k, v, None, inds, counts, o0, o_scale)
        out = ops.csp_attn(*dev(q, k, v), None, inds.cuda(), counts.cuda(), o0.cuda(), o_scale)
        assert out.shape == q.shape and out.dtype == torch.bfloat16
        check_o(out, ref, f"csp o_scale={o_scale}")
    delta, (M, L) = ops.csp_attn_delta(*dev(q, k, v), inds.cuda(), counts.cuda())
    dref, M_ref, L_ref = oracle.csp_attn_delta(q, k, v, inds, counts)
    check_o(delta, dref, "csp delta")
    check_lse(M, L, M_ref, L_ref)
    if unique:
        # the reference's own oracle form: dense softmax with unselected logits masked out
        mask = torch.zeros(B, H, G, Lk, dtype=torch.bool)
        mask.scatter_(-1, inds[..., :count].long(), True)
        rowmask = mask.repeat_interleave(192, dim=2)[:, :, :Lq]
        logits = (q.float() @ k.float().transpose(-1, -2)) / math.sqrt(d)
        logits = logits.masked_fill(~rowmask, -1e9)
        ref2 = torch.softmax(logits, -1) @ v.float()
        check_o(delta, ref2, "csp vs masked softmax")


def test_csp_attn_special_cases():
    from lvar_amd import sparse_attn_ops as ops
    B, H, Lq, Lk, d = 1, 2, 384, 300, 128
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=77)
    qg, kg, vg = dev(q, k, v)
    G = 2
    # full list == dense attention
    inds = torch.arange(Lk, dtype=torch.int32).expand(B, H, G, Lk).contiguous()
    counts = torch.full((B, H, G), Lk, dtype=torch.int32)
    delta, _ = ops.csp_attn_delta(qg, kg, vg, inds.cuda(), counts.cuda())
    o_dense, _ = ops.dense_attn(qg, kg, vg)
    assert (delta.float() - o_dense.float()).abs().max().item() < 2e-2
    # count == 0 leaves o unchanged and reports (M, L) = (-inf, 1)
    counts0 = torch.zeros(B, H, G, dtype=torch.int32)
    counts0[:, :, 1] = 64
    o0 = torch.randn(B, H, Lq, d).to(torch.bfloat16).cuda()
    out = ops.csp_attn(qg, kg, vg, None, inds.cuda(), counts0.cuda(), o0, 1)
    assert torch.equal(out[:, :, :192], o0[:, :, :192])
    assert not torch.equal(out[:, :, 192:], o0[:, :, 192:])
    _, (M, L) = ops.csp_attn_delta(qg, kg, vg, inds.cuda(), counts0.cuda())
    assert bool(torch.isinf(M[:, :, :192]).all()) and bool((L[:, :, :192] == 1).all())
    # -1 then +1 with the same list returns the original o up to bf16 rounding
    counts64 = torch.full((B, H, G), 128, dtype=torch.int32).cuda()
    a = ops.csp_attn(qg, kg, vg, None, inds.cuda(), counts64, o0, -1)
    bck = ops.csp_attn(qg, kg, vg, None, inds.cuda(), counts64, a, 1)
    assert (bck.float() - o0.float()).abs().max().item() < 4e-2
    # inputs are never written
    assert torch.equal(qg.cpu(), q) and torch.equal(kg.cpu(), k) and torch.equal(vg.cpu(), v)


def _random_block_lists(B, H, nQ, nK, density, seed):
    g = torch.Generator().manual_seed(seed)
    mask = torch.rand(B, H, nQ, nK, generator=g) < density
    force = torch.randint(0, nK, (B, H, nQ, 1), generator=g)
    mask.scatter_(-1, force, True)  # every query block keeps >= 1 block
    return mask


@pytest.mark.parametrize("B,H,Lq,Lk,d,bk,density", [
    (1, 2, 512, 1000, 128, 64, 0.25),
    (1, 2, 300, 1000, 128, 128, 0.3),   # ragged Lq; last 128-key block has 104 keys
    (2, 2, 256, 680, 64, 64, 0.5),      # config-1 shape, last block 40 keys
    (1, 1, 256, 1050, 128, 128, 1.0),   # last 128-block has only 26 keys: its second tile is empty
    (1, 2, 1024, 2521, 128, 64, 0.1),
])
def test_block_sparse_attn(B, H, Lq, Lk, d, bk, density):
    from lvar_amd import sparse_attn_ops as ops
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=Lk + bk)
    nQ, nK = (Lq + 127) // 128, (Lk + bk - 1) // bk
    mask = _random_block_lists(B, H, nQ, nK, density, seed=Lq)
    num, idx = oracle.block_mask_to_lists(mask)
    o_ref, M_ref, L_ref = oracle.block_sparse_attn(q, k, v, num, idx, 128, bk)
    o, (M, L) = ops.block_sparse_attn(*dev(q, k, v), num.cuda(), idx.cuda(), 128, bk)
    check_o(o, o_ref, "block sparse")
    check_lse(M, L, M_ref, L_ref)


@pytest.mark.parametrize("B,H,Lq,Lk,d,bq,bk,density", [
    (2, 3, 256, 680, 64, 64, 64, 0.5),     # the 64 x 64 blocks of the VAR-d16 benchmark case; last key block 40 keys
    (1, 2, 200, 300, 128, 64, 64, 0.4),    # two-wave workgroups at head_dim 128, ragged Lq (200 = 3 * 64 + 8)
    (1, 2, 150, 700, 128, 64, 128, 0.5),   # 64-row query blocks against 128-key blocks
    (1, 2, 600, 1000, 128, 256, 64, 0.3),  # 256-row query blocks: two workgroups share a list; last block 88 rows
    (1, 2, 384, 1100, 64, 384, 256, 0.6),  # 256-key blocks (four tiles per entry); last one has 76 keys
    (1, 1, 128, 900, 128, 128, 256, 1.0),  # every 256-key block; the last block's tail tiles are empty
])
def test_block_sparse_attn_block_shapes(B, H, Lq, Lk, d, bq, bk, density):
    """Block shapes other than 128 x {64, 128}: 64-row query blocks, query blocks that span several workgroups,
    256-key blocks; each against the oracle on a random list."""
    from lvar_amd import sparse_attn_ops as ops
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=Lq + Lk + bq + bk)
    nQ, nK = (Lq + bq - 1) // bq, (Lk + bk - 1) // bk
    mask = _random_block_lists(B, H, nQ, nK, density, seed=Lk + bq)
    num, idx = oracle.block_mask_to_lists(mask)
    o_ref, M_ref, L_ref = oracle.block_sparse_attn(q, k, v, num, idx, bq, bk)
    o, (M, L) = ops.block_sparse_attn(*dev(q, k, v), num.cuda(), idx.cuda(), bq, bk)
    check_o(o, o_ref, f"block sparse {bq}x{bk}")
    check_lse(M, L, M_ref, L_ref)


def test_var_d16_pipeline_64x64_blocks():
    """The CPU-runnable benchmark case end to end on the GPU (B2 H16 d64 Lq256 Lk680, N(0,1) inputs, scale 1/8):
    dense attention -> colsum over all 256 queries -> per-64-key block sums -> top 50 % = 5 of 11 key blocks per
    (batch, head) -> block-sparse attention with 64 x 64 blocks; every stage against the oracle, the block
    selection bit-exact on the same block sums."""
    from lvar_amd import mask_build as mb
    from lvar_amd import sparse_attn_ops as ops
    B, H, Lq, Lk, d = 2, 16, 256, 680, 64
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=2024)
    qg, kg, vg = dev(q, k, v)
    o_ref, cs_ref, (M_ref, L_ref) = oracle.dense_colsum_attn(q, k, v, q_group_size=256)
    o, (M, L) = ops.dense_attn(qg, kg, vg)
    cs, bs = ops.colsum(qg, kg, q_group_size=256, lse=(M, L), return_block_sums=True)
    check_o(o, o_ref, "dense")
    check_lse(M, L, M_ref, L_ref)
    assert cs.shape == (B, H, 1, Lk) and bs.shape == (B, H, 1, 11)
    assert ((cs.cpu() - cs_ref).abs() <= 1e-3 * cs_ref.abs() + 1e-6).all()
    assert ((bs.cpu() - oracle.key_block_sums(cs_ref, 64)).abs() <= 1e-3 * oracle.key_block_sums(cs_ref, 64)).all()
    # selection on the GPU block sums, GPU list build against torch.topk on the same values
    keep = oracle.indices_count(0.5, Lk, 64) // 64
    assert keep == 5
    nQ = Lq // 64
    scores = bs.expand(B, H, nQ, 11).contiguous()
    num, idx = ops.block_topk_lists(scores, keep)
    top = torch.topk(bs.cpu()[:, :, 0], k=keep, dim=-1).indices.sort(-1).values.to(torch.int32)
    assert bool((num == keep).all()) and torch.equal(idx.cpu()[..., :keep], top[:, :, None, :].expand(B, H, nQ, keep))
    o_bs_ref, M2_ref, L2_ref = oracle.block_sparse_attn(q, k, v, num.cpu(), idx.cpu(), 64, 64)
    o_bs, (M2, L2) = ops.block_sparse_attn(qg, kg, vg, num, idx, 64, 64)
    check_o(o_bs, o_bs_ref, "block sparse 64x64")
    check_lse(M2, L2, M2_ref, L2_ref)


def test_block_sparse_full_mask_equals_dense_and_broadcast():
    from lvar_amd import sparse_attn_ops as ops
    B, H, Lq, Lk, d = 2, 3, 256, 777, 128
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=21)
    qg, kg, vg = dev(q, k, v)
    nQ, nK = 2, (Lk + 63) // 64
    num = torch.full((1, 1, nQ), nK, dtype=torch.int32).cuda()            # broadcast over B and H
    idx = torch.arange(nK, dtype=torch.int32).expand(1, 1, nQ, nK).contiguous().cuda()
    o, (M, L) = ops.block_sparse_attn(qg, kg, vg, num, idx, 128, 64)
    od, (Md, Ld) = ops.dense_attn(qg, kg, vg)
    assert torch.equal(o, od) and torch.equal(M, Md) and torch.equal(L, Ld)
    # empty rows give zeros and (M, L) = (-inf, 1)
    num0 = num.clone()
    num0[..., 0] = 0
    o0, (M0, L0) = ops.block_sparse_attn(qg, kg, vg, num0, idx, 128, 64)
    assert bool((o0[:, :, :128] == 0).all()) and bool(torch.isinf(M0[:, :, :128]).all()) and bool((L0[:, :, :128] == 1).all())
    assert torch.equal(o0[:, :, 128:], od[:, :, 128:])


def test_block_topk_lists_bit_exact():
    """The GPU list build is a pure function of the scores: identical to the torch selection."""
    from lvar_amd import mask_build as mb
    from lvar_amd import sparse_attn_ops as ops
    g = torch.Generator().manual_seed(0)
    scores = torch.rand(2, 3, 32, 165, generator=g)
    scores[0, 0, 3, 20:60] = 0.5                       # ties: smaller block index wins
    base = mb.sink_window_base_mask()
    target = round(0.25 * 165)
    num, idx = ops.block_topk_lists(scores.cuda(), target, base)
    n_ref, i_ref = oracle.block_mask_to_lists(oracle.config2_block_mask(scores))
    assert torch.equal(num.cpu(), n_ref) and torch.equal(idx.cpu(), i_ref)
    assert bool((num == target).all())
    # no base mask, plain top-k; target larger than the row keeps everything; target 0 keeps nothing
    s2 = torch.rand(1, 2, 5, 70, generator=g)
    num, idx = ops.block_topk_lists(s2.cuda(), 7)
    n_ref, i_ref = oracle.block_mask_to_lists(oracle.base_plus_topk_block_mask(s2, torch.zeros(5, 70, dtype=torch.bool), 7))
    assert int(n_ref[0, 0, 0]) == 7 and torch.equal(num.cpu(), n_ref) and torch.equal(idx.cpu(), i_ref)
    n_mb, i_mb = mb.topk_block_lists(s2.cuda(), 0.1)          # the policy wrapper: round(0.1 * 70) = 7 blocks
    assert torch.equal(n_mb.cpu(), n_ref) and torch.equal(i_mb.cpu(), i_ref[..., :7]) and i_mb.dtype == torch.int32
    assert bool((idx.cpu()[..., 7:] == 0).all())
    num, idx = ops.block_topk_lists(s2.cuda(), 500)
    assert bool((num == 70).all()) and torch.equal(idx.cpu()[0, 0, 0], torch.arange(70, dtype=torch.int32))
    num, idx = ops.block_topk_lists(s2.cuda(), 0)
    assert bool((num == 0).all()) and bool((idx == 0).all())
    # base blocks are kept even when they exceed the target
    b2 = torch.zeros(5, 70, dtype=torch.bool)
    b2[:, :10] = True
    num, idx = ops.block_topk_lists(s2.cuda(), 4, b2)
    assert bool((num == 10).all()) and torch.equal(idx.cpu()[0, 1, 2, :10], torch.arange(10, dtype=torch.int32))


def test_errors():
    from lvar_amd import sparse_attn_ops as ops
    q, k, v = make_qkv(1, 1, 64, 64, 128, seed=1)
    qg, kg, vg = dev(q, k, v)
    with pytest.raises(TypeError):
        ops.dense_attn(qg.float(), kg.float(), vg.float())
    with pytest.raises(AssertionError):
        ops.dense_attn(qg, kg, vg[:, :, :32])
    with pytest.raises(AssertionError):
        ops.csp_attn(qg, kg, vg, None, torch.zeros(1, 1, 1, 63, dtype=torch.int32).cuda(),
                     torch.zeros(1, 1, 1, dtype=torch.int32).cuda(), qg, 1)
    with pytest.raises(RuntimeError):
        ops.dense_attn(q, k, v)  # CPU tensors: no fallback
    q48, k48, v48 = make_qkv(1, 1, 64, 64, 48, seed=1)
    with pytest.raises(AssertionError):
        ops.dense_attn(*dev(q48, k48, v48))      # head_dim 48: neither a kernel width nor padded to one


@pytest.mark.parametrize("H,Hkv", [(8, 2), (6, 1), (4, 4)])
def test_grouped_query_attention(H, Hkv):
    """Fewer K/V heads than query heads (dense_colsum_attn.cu:386-387; sparse_attn_ops.py:228-233): query head h
    reads K/V head h // (H // Hkv); dense attention, colsum (per query head) and the fused pair, through the operator
    API and the torch-library op."""
    import lvar_amd.torch_ops  # noqa: F401
    from lvar_amd import sparse_attn_ops as ops
    B, Lq, Lk, d = 2, 400, 777, 128
    q, _, _ = make_qkv(B, H, Lq, Lk, d, seed=H * 10 + Hkv, amp=0.7)
    _, k, v = make_qkv(B, Hkv, Lq, Lk, d, seed=H * 10 + Hkv + 1, amp=0.7)
    ke, ve = oracle.expand_kv_heads(k, H), oracle.expand_kv_heads(v, H)
    o_ref, cs_ref, (M_ref, L_ref) = oracle.dense_colsum_attn(q, ke, ve)[0], oracle.dense_colsum_attn(q, ke, ve)[1], oracle.dense_attn(q, ke, ve)[1:]
    qg, kg, vg = dev(q, k, v)
    o, (M, L) = ops.dense_attn(qg, kg, vg)
    check_o(o, o_ref, "gqa dense")
    check_lse(M, L, M_ref, L_ref)
    o2, cs, _ = ops.dense_colsum_attn(qg, kg, vg)
    assert torch.equal(o2, o) and cs.shape == (B, H, 3, Lk)
    assert torch.allclose(cs.cpu(), cs_ref, rtol=1e-3, atol=1e-6)
    assert torch.allclose(ops.colsum(qg, kg).cpu(), cs_ref, rtol=1e-3, atol=1e-6)
    o3, lse = torch.ops.lvar.dense_attn(qg, kg, vg)
    check_o(o3, oracle.dense_attn(q, ke, ve, scale=1.0)[0], "gqa torch op")
    if H != Hkv:
        with pytest.raises(AssertionError):
            ops.block_sparse_attn(qg, kg, vg, torch.ones(1, 1, 4, dtype=torch.int32).cuda(), torch.zeros(1, 1, 4, 13, dtype=torch.int32).cuda())
        with pytest.raises(AssertionError):
            ops.dense_attn(qg, kg[:, :0], vg[:, :0])


@pytest.mark.parametrize("d", [16, 32])
def test_small_head_dims_by_zero_padding(d):
    """head_dim 16 and 32 (attn_dense_colsum.py:246 takes them) run on the 64-wide kernels with zero columns."""
    from lvar_amd import mask_build as mb, sparse_attn_ops as ops
    B, H, Lq, Lk = 1, 3, 300, 450
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=d, amp=1.0)
    qg, kg, vg = dev(q, k, v)
    o_ref, M_ref, L_ref = oracle.dense_attn(q, k, v)
    o, (M, L) = ops.dense_attn(qg, kg, vg)
    assert o.shape == q.shape
    check_o(o, o_ref, f"d={d}")
    check_lse(M, L, M_ref, L_ref)
    o2, cs, _ = ops.dense_colsum_attn(qg, kg, vg)
    _, cs_ref, _ = oracle.dense_colsum_attn(q, k, v)
    assert torch.equal(o2, o) and torch.allclose(cs.cpu(), cs_ref, rtol=1e-3, atol=1e-6)
    inds, counts = mb.topk_index_list(cs, 0.3)
    out = ops.csp_attn(qg, kg, vg, 0.3, inds, counts, o, -1)
    check_o(out, oracle.csp_attn(q, k, v, 0.3, inds.cpu(), counts.cpu(), o.cpu(), -1), "csp small d")
    mask = torch.rand(B, H, 3, (Lk + 63) // 64, generator=torch.Generator().manual_seed(d)) < 0.5
    num, idx = oracle.block_mask_to_lists(mask)
    ob, _ = ops.block_sparse_attn(qg, kg, vg, num.cuda(), idx.cuda(), 128, 64)
    check_o(ob, oracle.block_sparse_attn(q, k, v, num, idx, 128, 64)[0], "block small d")
    with pytest.raises(AssertionError):
        ops.dense_attn(*dev(*make_qkv(1, 1, 8, 8, 512, seed=1)))


def test_head_dim_256():
    """head_dim 256, the top of the range the reference's Triton kernels take (attn_dense_colsum.py:246): every
    operator of the path, ragged sizes, against the oracle."""
    from lvar_amd import mask_build as mb, sparse_attn_ops as ops
    d = 256
    for (B, H, Lq, Lk) in [(1, 2, 300, 1000), (2, 3, 33, 25), (1, 1, 1, 1), (1, 2, 520, 2100)]:
        q, k, v = make_qkv(B, H, Lq, Lk, d, seed=Lq + Lk)
        o_ref, M_ref, L_ref = oracle.dense_attn(q, k, v)
        o, (M, L) = ops.dense_attn(*dev(q, k, v))
        check_o(o, o_ref, f"dense d=256 {Lq}x{Lk}")
        check_lse(M, L, M_ref, L_ref)
    B, H, Lq, Lk = 1, 2, 520, 2100
    qg, kg, vg = dev(q, k, v)
    # colsum next to the dense pass
    o2, cs, _ = ops.dense_colsum_attn(qg, kg, vg)
    _, cs_ref, _ = oracle.dense_colsum_attn(q, k, v)
    assert torch.equal(o2, o) and torch.allclose(cs.cpu(), cs_ref, rtol=1e-3, atol=1e-6)
    # token lists: 192-row groups (two 3-wave workgroups per group), cache delta
    inds, counts = mb.topk_index_list(cs, 0.3)
    out = ops.csp_attn(qg, kg, vg, 0.3, inds, counts, o, -1)
    check_o(out, oracle.csp_attn(q, k, v, 0.3, inds.cpu(), counts.cpu(), o.cpu(), -1), "csp d=256")
    # block lists: 128-row and 64-row query blocks, 64- and 128-key blocks
    for bq, bk in [(128, 64), (64, 64), (128, 128)]:
        nq, nk = (Lq + bq - 1) // bq, (Lk + bk - 1) // bk
        mask = torch.rand(B, H, nq, nk, generator=torch.Generator().manual_seed(bq + bk)) < 0.4
        mask[0, 0, 1] = False    # an empty list
        num, idx = oracle.block_mask_to_lists(mask)
        ob, _ = ops.block_sparse_attn(qg, kg, vg, num.cuda(), idx.cuda(), bq, bk)
        check_o(ob, oracle.block_sparse_attn(q, k, v, num, idx, bq, bk)[0], f"block d=256 {bq}x{bk}")
    # grouped-query attention
    kq, vq = k[:, :1].contiguous(), v[:, :1].contiguous()
    og, _ = ops.dense_attn(qg, kq.cuda(), vq.cuda())
    check_o(og, oracle.dense_attn(q, kq.expand(-1, H, -1, -1), vq.expand(-1, H, -1, -1))[0], "gqa d=256")


@pytest.mark.parametrize("d", [64, 128, 256])
def test_memory_behind_the_last_key_never_reaches_the_result(d):
    """K and V are views whose storage continues with NaN rows behind the last key (and NaN heads around them): a
    ragged last tile, the unused sub-tiles of a 256-key block and the two-tile prefetch must not let them into ``o``
    (a masked probability is an exact zero, and 0 * NaN would still be NaN)."""
    from lvar_amd import mask_build as mb, sparse_attn_ops as ops
    B, H, Lq, Lk, pad = 1, 3, 200, 333, 400
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=5)

    def poisoned(t):
        big = torch.full((B, H, Lk + pad, d), float("nan"), dtype=torch.bfloat16, device="cuda")
        big[:, :, :Lk] = t.cuda()
        return big[:, :, :Lk]

    qg, kg, vg = q.cuda(), poisoned(k), poisoned(v)
    assert not kg.is_contiguous()
    o_ref, M_ref, L_ref = oracle.dense_attn(q, k, v)
    o, (M, L) = ops.dense_attn(qg, kg, vg)
    check_o(o, o_ref, "dense")
    check_lse(M, L, M_ref, L_ref)
    o2, cs, _ = ops.dense_colsum_attn(qg, kg, vg)
    _, cs_ref, _ = oracle.dense_colsum_attn(q, k, v)
    check_o(o2, o_ref, "dense + colsum")
    assert torch.allclose(cs.cpu(), cs_ref, rtol=1e-3, atol=1e-6)
    for bq, bk in [(128, 64), (64, 64), (128, 128), (128, 256), (64, 256)]:
        nq, nk = (Lq + bq - 1) // bq, (Lk + bk - 1) // bk
        mask = torch.rand(B, H, nq, nk, generator=torch.Generator().manual_seed(bq + bk)) < 0.5
        mask[..., -1] = True     # the ragged last key block is always attended
        num, idx = oracle.block_mask_to_lists(mask)
        ob, _ = ops.block_sparse_attn(qg, kg, vg, num.cuda(), idx.cuda(), bq, bk)
        check_o(ob, oracle.block_sparse_attn(q, k, v, num, idx, bq, bk)[0], f"block {bq}x{bk}")
    inds, counts = mb.topk_index_list(cs, 0.3)
    out = ops.csp_attn(qg, kg, vg, None, inds, counts, o, -1)
    check_o(out, oracle.csp_attn(q, k, v, None, inds.cpu(), counts.cpu(), o.cpu(), -1), "token lists")
