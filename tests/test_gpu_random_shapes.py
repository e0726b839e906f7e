"""Seeded random-shape sweep of every attention entry point against the CPU oracle: ragged lengths,
both head dims, strided inputs, random block and token lists (duplicates, empty lists, counts that
are not multiples of 64)."""
import pytest
import torch

import oracle
from conftest import make_qkv

pytestmark = pytest.mark.gpu


def close(a, b, atol=2e-2, rtol=1e-2):
    return bool(((a.float().cpu() - b).abs() <= atol + rtol * b.abs()).all())


def lse_close(M, L, M_ref, L_ref):
    a = M.float().cpu() + torch.log2(L.float().cpu())
    b = M_ref + torch.log2(L_ref)
    fin = torch.isfinite(b)
    return bool((torch.isfinite(a) == fin).all()) and (not fin.any() or (a[fin] - b[fin]).abs().max().item() < 1e-3)


def strided(t, mode):
    """Same values, different storage: contiguous, [B,L,H,d] storage, or a slice of a padded row."""
    g = t.cuda()
    if mode == 1:
        return g.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    if mode == 2:
        pad = torch.zeros(*g.shape[:-1], g.shape[-1] + 8, dtype=g.dtype, device=g.device)
        pad[..., :g.shape[-1]] = g
        return pad[..., :g.shape[-1]]
    return g


@pytest.mark.parametrize("seed", range(12))
def test_dense_and_colsum_random(seed):
    from lvar_amd import sparse_attn_ops as ops
    g = torch.Generator().manual_seed(1000 + seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    B, H, d = r(1, 2), r(1, 3), (64, 128)[r(0, 1)]
    Lq, Lk = r(1, 700), r(1, 900)
    scale = (None, 1.0, 0.05)[r(0, 2)]
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=seed, amp=(0.3, 1.0)[r(0, 1)])
    mode = r(0, 2)
    qg, kg, vg = strided(q, mode), strided(k, mode), strided(v, mode)
    o, (M, L) = ops.dense_attn(qg, kg, vg, scale)
    o_ref, M_ref, L_ref = oracle.dense_attn(q, k, v, scale)
    assert close(o, o_ref) and lse_close(M, L, M_ref, L_ref), (B, H, Lq, Lk, d, scale, mode)
    grp = (32, 64, 128, 192)[r(0, 3)]
    cs = ops.colsum(qg, kg, scale, q_group_size=grp)
    _, cs_ref, _ = oracle.dense_colsum_attn(q, k, v, scale, q_group_size=grp)
    assert torch.allclose(cs.cpu(), cs_ref, rtol=2e-3, atol=1e-6), (B, H, Lq, Lk, d, grp)


@pytest.mark.parametrize("seed", range(12))
def test_block_sparse_random(seed):
    from lvar_amd import sparse_attn_ops as ops
    g = torch.Generator().manual_seed(2000 + seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    B, H, d = r(1, 2), r(1, 3), (64, 128)[r(0, 1)]
    Lq, Lk, bk = r(1, 600), r(1, 1500), (64, 128)[r(0, 1)]
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=seed, amp=0.5)
    nQ, nK = (Lq + 127) // 128, (Lk + bk - 1) // bk
    mask = torch.rand(B, H, nQ, nK, generator=g) < (0.1, 0.5, 1.0)[r(0, 2)]
    if r(0, 1):
        mask[:, :, 0] = False                                            # an empty row of blocks
    num, idx = oracle.block_mask_to_lists(mask)
    o, (M, L) = ops.block_sparse_attn(q.cuda(), k.cuda(), v.cuda(), num.cuda(), idx.cuda(), 128, bk)
    o_ref, M_ref, L_ref = oracle.block_sparse_attn(q, k, v, num, idx, 128, bk)
    assert close(o, o_ref) and lse_close(M, L, M_ref, L_ref), (B, H, Lq, Lk, d, bk)


@pytest.mark.parametrize("seed", range(12))
def test_token_lists_random(seed):
    from lvar_amd import sparse_attn_ops as ops
    g = torch.Generator().manual_seed(3000 + seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    B, H, d = r(1, 2), r(1, 2), (64, 128)[r(0, 1)]
    Lq, Lk = r(1, 800), r(1, 1200)
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=seed, amp=0.5)
    G = (Lq + 191) // 192
    idx = torch.randint(0, Lk, (B, H, G, Lk), generator=g, dtype=torch.int32)        # duplicates allowed
    counts = torch.randint(0, Lk + 1, (B, H, G), generator=g, dtype=torch.int32)
    if r(0, 1):
        counts[:, :, 0] = 0
    o0 = (torch.randn(B, H, Lq, d, generator=g) * 0.5).to(torch.bfloat16)
    sgn = (1, -1)[r(0, 1)]
    out = ops.csp_attn(q.cuda(), k.cuda(), v.cuda(), None, idx.cuda(), counts.cuda(), o0.cuda(), sgn)
    ref = oracle.csp_attn(q, k, v, None, idx, counts, o0, sgn)
    assert close(out, ref), (B, H, Lq, Lk, d, sgn)
    delta, (M, L) = ops.csp_attn_delta(q.cuda(), k.cuda(), v.cuda(), idx.cuda(), counts.cuda())
    d_ref, M_ref, L_ref = oracle.csp_attn_delta(q, k, v, idx, counts)
    assert close(delta, d_ref) and lse_close(M, L, M_ref, L_ref)


@pytest.mark.parametrize("seed", range(6))
def test_head_dim_256_random(seed):
    """The three attention forms and the colsum at head_dim 256 on random ragged shapes, strided storage included."""
    from lvar_amd import sparse_attn_ops as ops
    g = torch.Generator().manual_seed(4000 + seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    B, H, d = r(1, 2), r(1, 2), 256
    Lq, Lk = r(1, 500), r(1, 900)
    scale = (None, 0.05)[r(0, 1)]
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=seed, amp=(0.3, 0.7)[r(0, 1)])
    mode = r(0, 2)
    qg, kg, vg = strided(q, mode), strided(k, mode), strided(v, mode)
    o, (M, L) = ops.dense_attn(qg, kg, vg, scale)
    o_ref, M_ref, L_ref = oracle.dense_attn(q, k, v, scale)
    assert close(o, o_ref) and lse_close(M, L, M_ref, L_ref), (B, H, Lq, Lk, scale, mode)
    grp = (32, 64, 128, 192)[r(0, 3)]
    cs = ops.colsum(qg, kg, scale, q_group_size=grp)
    _, cs_ref, _ = oracle.dense_colsum_attn(q, k, v, scale, q_group_size=grp)
    assert torch.allclose(cs.cpu(), cs_ref, rtol=2e-3, atol=1e-6), (B, H, Lq, Lk, grp)
    bq, bk = (64, 128, 256)[r(0, 2)], (64, 128, 256)[r(0, 2)]
    mask = torch.rand(B, H, (Lq + bq - 1) // bq, (Lk + bk - 1) // bk, generator=g) < (0.2, 0.6)[r(0, 1)]
    num, idx = oracle.block_mask_to_lists(mask)
    ob, (Mb, Lb) = ops.block_sparse_attn(qg, kg, vg, num.cuda(), idx.cuda(), bq, bk, scale)
    ob_ref, Mb_ref, Lb_ref = oracle.block_sparse_attn(q, k, v, num, idx, bq, bk, scale)
    assert close(ob, ob_ref) and lse_close(Mb, Lb, Mb_ref, Lb_ref), (B, H, Lq, Lk, bq, bk)
    G = (Lq + 191) // 192
    tidx = torch.randint(0, Lk, (B, H, G, Lk), generator=g, dtype=torch.int32)
    tcnt = torch.randint(0, Lk + 1, (B, H, G), generator=g, dtype=torch.int32)
    o0 = (torch.randn(B, H, Lq, d, generator=g) * 0.5).to(torch.bfloat16)
    out = ops.csp_attn(qg, kg, vg, scale, tidx.cuda(), tcnt.cuda(), o0.cuda(), -1)
    assert close(out, oracle.csp_attn(q, k, v, scale, tidx, tcnt, o0, -1)), (B, H, Lq, Lk, "csp")


def test_token_lists_slice_matches_full_launch():
    """A (batch, head) slice launched alone must reproduce a launch of 512 groups (two workgroups per CU on
    a 256-CU part) bit for bit: the result of a group does not depend on how many others share the launch,
    the XCD remap of the workgroup index or the order the groups run in; both match the oracle."""
    from lvar_amd import sparse_attn_ops as ops
    B, H, Lq, Lk, d = 2, 16, 3072, 333, 64
    g = torch.Generator().manual_seed(77)
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=77, amp=0.5)
    G = (Lq + 191) // 192
    assert B * H * G >= 512
    idx = torch.randint(0, Lk, (B, H, G, Lk), generator=g, dtype=torch.int32)
    counts = torch.randint(1, Lk + 1, (B, H, G), generator=g, dtype=torch.int32)
    o0 = (torch.randn(B, H, Lq, d, generator=g) * 0.5).to(torch.bfloat16)
    qg, kg, vg, ig, cg, og = q.cuda(), k.cuda(), v.cuda(), idx.cuda(), counts.cuda(), o0.cuda()
    big = ops.csp_attn(qg, kg, vg, None, ig, cg, og, 1)
    for (b, h) in ((0, 0), (1, 9)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        small = ops.csp_attn(qg[sl].contiguous(), kg[sl].contiguous(), vg[sl].contiguous(), None,
                             ig[sl].contiguous(), cg[sl].contiguous(), og[sl].contiguous(), 1)
        assert torch.equal(small, big[sl]), (b, h)
        ref = oracle.csp_attn(q[sl], k[sl], v[sl], None, idx[sl], counts[sl], o0[sl], 1)
        assert close(big[sl], ref), (b, h)


def _csp_abi(q, k, v, idx, cnt, o0, group_rows, o_scale):
    """lvar_csp_attn_fwd through ctypes with an explicit query-group size."""
    from lvar_amd import _lib
    from lvar_amd import sparse_attn_ops as ops
    B, H, Lq, d = q.shape
    out = torch.empty_like(q)
    st = _lib.load().lvar_csp_attn_fwd(ops._view(q), ops._view(k), ops._view(v), ops._view(o0), ops._view(out), None, None,
                                      idx.data_ptr(), cnt.data_ptr(), idx.shape[2], idx.stride(2), group_rows,
                                      B, H, Lq, k.shape[2], d, float(o_scale), 1.0 / d ** 0.5,
                                      torch.cuda.current_stream().cuda_stream)
    return st, out


@pytest.mark.parametrize("d", [64, 128, 256])
def test_token_lists_every_workgroup_shape(d):
    """Query groups of 192 rows run as 8-wave workgroups (six computing waves + two fetch waves; at head_dim 256 as
    two 3-wave workgroups), other multiples
    of 96 / 64 rows as 3- / 2-wave workgroups that fetch for themselves.  Each variant against the oracle at its
    own group size, and, with every 192-row list repeated for its 96- / 64-row parts, bit for bit against each
    other: the arithmetic of a query row does not depend on the workgroup shape."""
    from lvar_amd import _lib
    g = torch.Generator().manual_seed(11 + d)
    B, H, Lq, Lk = 1, 3, 500, 700
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=11, amp=0.5)
    o0 = (torch.randn(B, H, Lq, d, generator=g) * 0.5).to(torch.bfloat16)
    G = (Lq + 191) // 192
    idx = torch.randint(0, Lk, (B, H, G, Lk), generator=g, dtype=torch.int32)
    cnt = torch.randint(0, Lk + 1, (B, H, G), generator=g, dtype=torch.int32)
    cnt[0, 1, 0] = 0
    qg, kg, vg, og = q.cuda(), k.cuda(), v.cuda(), o0.cuda()
    outs = {}
    for rows in (192, 96, 64):
        rep = 192 // rows
        idx_r = idx.repeat_interleave(rep, dim=2).contiguous()
        cnt_r = cnt.repeat_interleave(rep, dim=2).contiguous()
        st, out = _csp_abi(qg, kg, vg, idx_r.cuda(), cnt_r.cuda(), og, rows, -1)
        assert st == 0, (rows, st)
        ref = oracle.csp_attn(q, k, v, None, idx_r, cnt_r, o0, -1, bm=rows)
        assert close(out, ref), rows
        outs[rows] = out
    assert torch.equal(outs[192], outs[96]) and torch.equal(outs[192], outs[64])
    # independent lists per 64-row group
    G64 = (Lq + 63) // 64
    idx64 = torch.randint(0, Lk, (B, H, G64, Lk), generator=g, dtype=torch.int32)
    cnt64 = torch.randint(0, Lk + 1, (B, H, G64), generator=g, dtype=torch.int32)
    st, out = _csp_abi(qg, kg, vg, idx64.cuda(), cnt64.cuda(), og, 64, 1)
    assert st == 0 and close(out, oracle.csp_attn(q, k, v, None, idx64, cnt64, o0, 1, bm=64))
    # group sizes that no workgroup shape divides are refused, not mis-run
    lib = _lib.load()
    for rows in (32, 160, 224):
        Gr = (Lq + rows - 1) // rows
        st, _ = _csp_abi(qg, kg, vg, torch.zeros(B, H, Gr, Lk, dtype=torch.int32).cuda(),
                         torch.zeros(B, H, Gr, dtype=torch.int32).cuda(), og, rows, 1)
        assert st == -2 and b"group" in lib.lvar_status_string(st)
