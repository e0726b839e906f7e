"""Full-size checks at the headline shape (Infinity-2B 1024^2 last scale: B2 H16 d128 Lq4096 Lk10521),
where the CPU oracle is too slow for the whole problem: size-independent properties of the whole
output plus oracle parity on a few (batch, head) slices and query ranges of the same launch."""
import math

import pytest
import torch

import oracle
from conftest import make_qkv

pytestmark = pytest.mark.gpu

B, H, LQ, LK, D = 2, 16, 4096, 10521, 128
SLICES = ((0, 0), (1, 7), (1, 15))


def close(a, b, atol=2e-2, rtol=1e-2):
    return bool(((a.float().cpu() - b).abs() <= atol + rtol * b.abs()).all())


@pytest.fixture(scope="module")
def data():
    from lvar_amd import sparse_attn_ops as ops
    q, k, v = make_qkv(B, H, LQ, LK, D, seed=1234, amp=0.5)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    o, (M, L) = ops.dense_attn(qg, kg, vg)
    return dict(q=q, k=k, v=v, qg=qg, kg=kg, vg=vg, o=o, M=M, L=L)


def test_dense_slices_and_unit_value_rows(data):
    from lvar_amd import sparse_attn_ops as ops
    for (b, h) in SLICES:
        sl = (slice(b, b + 1), slice(h, h + 1))
        o_ref, M_ref, L_ref = oracle.dense_attn(data["q"][sl], data["k"][sl], data["v"][sl])
        assert close(data["o"][sl], o_ref), (b, h)
        lse = data["M"][sl].cpu() + torch.log2(data["L"][sl].cpu())
        assert (lse - (M_ref + torch.log2(L_ref))).abs().max().item() < 1e-3
    # softmax rows sum to one: with v = 1 the output is 1 up to the bf16 rounding of P and of o
    ones = torch.ones_like(data["vg"])
    o1, _ = ops.dense_attn(data["qg"], data["kg"], ones)
    assert (o1.float() - 1.0).abs().max().item() < 8e-3


def test_colsum_invariants_and_slices(data):
    from lvar_amd import sparse_attn_ops as ops
    cs, bs = ops.colsum(data["qg"], data["kg"], None, q_group_size=192, lse=(data["M"], data["L"]), return_block_sums=True)
    G = (LQ + 191) // 192
    assert cs.shape == (B, H, G, LK) and bool((cs >= 0).all())
    rows = torch.tensor([min(192, LQ - g * 192) for g in range(G)], dtype=torch.float32, device="cuda")
    assert torch.allclose(cs.sum(-1), rows.expand(B, H, G), rtol=1e-3)             # every probability row sums to 1
    assert torch.allclose(bs.sum(-1), rows.expand(B, H, G), rtol=1e-3)
    pad = torch.nn.functional.pad(cs, (0, 64 * bs.shape[-1] - LK))
    assert torch.allclose(pad.view(B, H, G, -1, 64).sum(-1), bs, rtol=1e-4, atol=1e-6)   # block sums = sums of the columns
    cs2 = ops.colsum(data["qg"], data["kg"], None, q_group_size=192)                   # self-contained two-pass form
    assert torch.allclose(cs2, cs, rtol=1e-3, atol=1e-7)
    for (b, h) in SLICES[:2]:
        sl = (slice(b, b + 1), slice(h, h + 1))
        _, cs_ref, _ = oracle.dense_colsum_attn(data["q"][sl], data["k"][sl], data["v"][sl])
        assert torch.allclose(cs[sl].cpu(), cs_ref, rtol=1e-3, atol=1e-6), (b, h)


def test_block_sparse_headline_mask(data):
    from lvar_amd import mask_build as mb, sparse_attn_ops as ops
    _, bsum = ops.colsum(data["qg"], data["kg"], None, q_group_size=128, lse=(data["M"], data["L"]), return_block_sums=True)
    base = mb.sink_window_base_mask(128, 64, device="cuda")
    num, idx = ops.block_topk_lists(bsum, int(round(0.25 * bsum.shape[-1])), base)
    assert bool((num == 41).all())
    srt = idx[..., :41]
    assert bool((srt[..., 1:] > srt[..., :-1]).all()) and bool((idx[..., 41:] == 0).all())     # ascending, zero tail
    # bit-exact against the torch selection on the same scores (ties to the smaller block index)
    n_ref, i_ref = oracle.block_mask_to_lists(oracle.config2_block_mask(bsum.cpu()))
    assert torch.equal(num.cpu(), n_ref) and torch.equal(idx.cpu(), i_ref)
    o, (M, L) = ops.block_sparse_attn(data["qg"], data["kg"], data["vg"], num, idx, 128, 64)
    for (b, h) in SLICES[:2]:
        sl = (slice(b, b + 1), slice(h, h + 1))
        o_ref, _, _ = oracle.block_sparse_attn(data["q"][sl], data["k"][sl], data["v"][sl], n_ref[sl], i_ref[sl], 128, 64)
        assert close(o[sl], o_ref), (b, h)
    # the full list is the dense computation, instruction for instruction
    nK = (LK + 63) // 64
    full = torch.arange(nK, dtype=torch.int32, device="cuda").expand(1, 1, LQ // 128, nK).contiguous()
    nfull = torch.full((1, 1, LQ // 128), nK, dtype=torch.int32, device="cuda")
    o_full, (Mf, Lf) = ops.block_sparse_attn(data["qg"], data["kg"], data["vg"], nfull, full, 128, 64)
    assert torch.equal(o_full, data["o"]) and torch.equal(Mf, data["M"]) and torch.equal(Lf, data["L"])


def test_token_lists_full_size(data):
    from lvar_amd import mask_build as mb, sparse_attn_ops as ops
    cs = ops.colsum(data["qg"], data["kg"], None, lse=(data["M"], data["L"]))
    cnt = mb.indices_count(0.2, LK, 64)
    assert cnt == 2112
    inds, counts = ops.topk_token_lists(cs, cnt)
    assert bool((counts == cnt).all())
    sel = inds[..., :cnt].long()
    assert bool((sel[..., 1:] > sel[..., :-1]).all())                                       # ascending, no repeats
    picked = cs.gather(-1, sel)
    rest = cs.scatter(-1, sel, float("-inf"))
    assert bool((picked.min(-1).values >= rest.max(-1).values).all())                        # a top-k set
    assert torch.equal(sel, torch.topk(cs, cnt, dim=-1).indices.sort(-1).values)             # distinct values: the top-k set
    zero = torch.zeros_like(data["qg"])
    delta = ops.csp_attn(data["qg"], data["kg"], data["vg"], None, inds, counts, zero, 1)
    for (b, h) in SLICES[:1]:
        sl = (slice(b, b + 1), slice(h, h + 1))
        ref = oracle.csp_attn(data["q"][sl], data["k"][sl], data["v"][sl], None, inds[sl].cpu(), counts[sl].cpu(),
                              torch.zeros_like(data["q"][sl]), 1)
        assert close(delta[sl], ref)
    # O_cache = O_dense - delta, then + delta gives O_dense back up to two bf16 roundings
    cache = ops.csp_attn(data["qg"], data["kg"], data["vg"], None, inds, counts, data["o"], -1)
    back = ops.csp_attn(data["qg"], data["kg"], data["vg"], None, inds, counts, cache, 1)
    assert (back.float() - data["o"].float()).abs().max().item() < 2e-2
    # the complete key list (10521 keys, not a multiple of 64) is dense attention
    G = inds.shape[2]
    allk = torch.arange(LK, dtype=torch.int32, device="cuda").expand(1, 2, G, LK).contiguous()
    call = torch.full((1, 2, G), LK, dtype=torch.int32, device="cuda")
    o_all = ops.csp_attn(data["qg"][:1, :2], data["kg"][:1, :2], data["vg"][:1, :2], None, allk, call, zero[:1, :2], 1)
    assert (o_all.float() - data["o"][:1, :2].float()).abs().max().item() < 1e-2
