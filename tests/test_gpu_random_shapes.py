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


def test_token_lists_fetch_waves_match_six_wave_groups(tmp_path):
    """A 192-row group runs with six computing waves plus two fetch waves by default and with six waves that do
    both under LVAR_CSP_WAVES=6 (read once per process, hence the child processes): same arithmetic per row,
    so the outputs must agree bit for bit."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = (
        "import sys, torch\n"
        f"sys.path.insert(0, {root!r}); sys.path.insert(0, {os.path.join(root, 'tests')!r})\n"
        "from conftest import make_qkv\n"
        "from lvar_amd import sparse_attn_ops as ops\n"
        "g = torch.Generator().manual_seed(11)\n"
        "B, H, Lq, Lk, d = 1, 3, 500, 700, 128\n"
        "q, k, v = make_qkv(B, H, Lq, Lk, d, seed=11, amp=0.5)\n"
        "G = (Lq + 191) // 192\n"
        "idx = torch.randint(0, Lk, (B, H, G, Lk), generator=g, dtype=torch.int32)\n"
        "cnt = torch.randint(0, Lk + 1, (B, H, G), generator=g, dtype=torch.int32)\n"
        "o0 = (torch.randn(B, H, Lq, d, generator=g) * 0.5).to(torch.bfloat16)\n"
        "out = ops.csp_attn(q.cuda(), k.cuda(), v.cuda(), None, idx.cuda(), cnt.cuda(), o0.cuda(), -1)\n"
        "torch.save(out.cpu(), sys.argv[1])\n")
    outs = []
    for waves in ("8", "6"):
        path = str(tmp_path / f"o{waves}.pt")
        env = dict(os.environ, LVAR_CSP_WAVES=waves)
        subprocess.run([sys.executable, "-c", code, path], check=True, env=env, timeout=100)
        outs.append(torch.load(path, weights_only=True))
    assert torch.equal(outs[0], outs[1])
