"""Balanced launches (``*_ws_fwd`` entry points with a partial-result workspace): every attention family, at
shapes whose plain grid fills the chip unevenly, against the CPU oracle and against the plain launch of the same
call; pieces of a cut query tile are added up in launch order, so two runs agree bit for bit, and the arrival
counters at the head of the workspace are zero again after every launch."""
import pytest
import torch

import oracle
from conftest import make_qkv

pytestmark = pytest.mark.gpu


def close(a, b, atol=2e-2, rtol=1e-2):
    return bool(((a.float().cpu() - b).abs() <= atol + rtol * b.abs()).all())


def lse_close(M, L, M_ref, L_ref, tol=1e-3):
    a = M.float().cpu() + torch.log2(L.float().cpu())
    b = M_ref + torch.log2(L_ref)
    fin = torch.isfinite(b)
    return bool((torch.isfinite(a) == fin).all()) and (not fin.any() or (a[fin] - b[fin]).abs().max().item() < tol)


@pytest.fixture()
def ops():
    from lvar_amd import sparse_attn_ops as o
    o._set_balanced_launch(True)
    yield o
    o._set_balanced_launch(False)        # the default


def plan(ops, kind, q, k, group_rows=192, block_k=64, list_len=0):
    """Workgroups the balanced launch of this call would use (0 = plain launch)."""
    from lvar_amd import _lib
    B, H, Lq, d = q.shape
    ws = ops._workspace(q, ops._stream(q))
    return _lib.load().lvar_attn_balanced_workgroups(kind, group_rows, block_k, B, H, Lq, k.shape[2], list_len, d, ws)


def counters_zero(ops, q):
    ws = ops._workspaces[(q.device.index, ops._stream(q))][1]
    return not bool(ws[:4096].any())


def both(ops, fn):
    """fn() with the balanced launch on (twice) and off."""
    ops._set_balanced_launch(True)
    a1 = fn()
    a2 = fn()
    ops._set_balanced_launch(False)
    b = fn()
    ops._set_balanced_launch(True)
    return a1, a2, b


def same(x, y):
    if isinstance(x, torch.Tensor):
        return torch.equal(x, y)
    return all(same(a, b) for a, b in zip(x, y))


@pytest.mark.parametrize("B,H,Lq,Lk,d", [
    (2, 16, 576, 1497, 128),    # Infinity scale 24: 160 query tiles
    (2, 16, 400, 961, 128),     # about scale 20, ragged Lq and Lk
    (2, 16, 1024, 2521, 128),   # scale 32: 256 query tiles
    (1, 3, 300, 5000, 64),      # few tiles, long lists: every tile is cut many times
    (1, 1, 100, 40000, 128),    # one query tile shared by the whole chip
])
def test_dense_balanced(ops, B, H, Lq, Lk, d):
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=Lq + Lk, amp=0.7)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    assert plan(ops, 0, qg, kg) > 0
    (o1, M1, L1, _), r2, (o0, M0, L0, _) = both(ops, lambda: ops._dense_launch(qg, kg, vg, None))
    assert same((o1, M1, L1), r2[:3])                                 # deterministic
    assert counters_zero(ops, qg)
    o_ref, M_ref, L_ref = oracle.dense_attn(q, k, v)
    assert close(o1, o_ref) and lse_close(M1, L1, M_ref, L_ref)
    assert (M1.cpu() - M_ref).abs().max().item() < 1e-3
    # against the plain launch: same maxima, sums and outputs up to the order of fp32 additions
    assert torch.equal(M1, M0) and torch.allclose(L1, L0, rtol=1e-5)
    assert (o1.float() - o0.float()).abs().max().item() <= 1e-2 * max(1.0, float(o0.float().abs().max()))


def test_dense_balanced_growing_maxima(ops):
    """Row maxima that grow along the key axis: the pieces of a tile carry different reference maxima."""
    B, H, Lq, Lk, d = 1, 2, 256, 8192, 128
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=5)
    k = (k.float() * torch.linspace(0.2, 3.0, Lk).view(1, 1, Lk, 1)).to(torch.bfloat16)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    assert plan(ops, 0, qg, kg) > 0
    o, M, L, _ = ops._dense_launch(qg, kg, vg, None)
    o_ref, M_ref, L_ref = oracle.dense_attn(q, k, v)
    assert close(o, o_ref) and lse_close(M, L, M_ref, L_ref)


@pytest.mark.parametrize("bk", [64, 128])
@pytest.mark.parametrize("seed", range(4))
def test_block_lists_balanced(ops, bk, seed):
    """Ragged Bernoulli block lists (some rows empty, some full) over enough query tiles to take the balanced path."""
    g = torch.Generator().manual_seed(100 + seed)
    B, H, d = 2, 8, (64, 128)[seed % 2]
    Lq, Lk = 128 * 20 + (57 if seed % 2 else 0), 3000 + 517 * seed
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=seed, amp=0.6)
    nQ, nK = (Lq + 127) // 128, (Lk + bk - 1) // bk
    dens = torch.rand(B, H, nQ, 1, generator=g) ** 2                     # row densities from ~0 to 1
    mask = torch.rand(B, H, nQ, nK, generator=g) < dens
    mask[:, :, 3] = False
    mask[:, :, 5] = True
    num, idx = oracle.block_mask_to_lists(mask)
    qg, kg, vg, ng, ig = q.cuda(), k.cuda(), v.cuda(), num.cuda(), idx.cuda()
    assert plan(ops, 1, qg, kg, block_k=bk, list_len=nK) > 0
    (o1, (M1, L1)), r2, (o0, (M0, L0)) = both(ops, lambda: ops.block_sparse_attn(qg, kg, vg, ng, ig, 128, bk))
    assert same((o1, M1, L1), (r2[0], r2[1][0], r2[1][1]))
    assert counters_zero(ops, qg)
    o_ref, M_ref, L_ref = oracle.block_sparse_attn(q, k, v, num, idx, 128, bk)
    assert close(o1, o_ref) and lse_close(M1, L1, M_ref, L_ref)
    assert torch.equal(M1, M0) and torch.allclose(L1, L0, rtol=1e-5)
    assert bool((o1[:, :, 3 * 128:4 * 128] == 0).all())                  # the empty row of blocks


def test_block_lists_balanced_density_sweep_shape(ops):
    """The density-sweep configuration at 5 %: B1 H16 Lq4096 Lk10521, 512 query tiles with 1..20 blocks each."""
    from lvar_amd import mask_build as mb
    B, H, Lq, Lk = 1, 16, 4096, 10521
    q, k, v = make_qkv(B, H, Lq, Lk, 128, seed=82, amp=1.0)
    g = torch.Generator().manual_seed(7)
    mask = torch.rand(B, H, 32, 165, generator=g) < 0.05
    mask.scatter_(-1, torch.randint(0, 165, (B, H, 32, 1), generator=g), True)
    num, idx = mb.block_mask_to_lists(mask.cuda())
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    assert plan(ops, 1, qg, kg, list_len=165) > 0
    (o1, (M1, L1)), r2, (o0, (M0, L0)) = both(ops, lambda: ops.block_sparse_attn(qg, kg, vg, num, idx, 128, 64))
    assert torch.equal(o1, r2[0]) and counters_zero(ops, qg)
    assert torch.equal(M1, M0) and torch.allclose(L1, L0, rtol=1e-5)
    assert (o1.float() - o0.float()).abs().max().item() < 2e-2
    for h in (0, 9):
        ref, _, _ = oracle.block_sparse_attn(q[:, h:h + 1], k[:, h:h + 1], v[:, h:h + 1], num[:, h:h + 1].cpu(), idx[:, h:h + 1].cpu(), 128, 64)
        assert close(o1[:, h:h + 1], ref), h


@pytest.mark.parametrize("rows,d", [(192, 128), (192, 64), (96, 128), (64, 64)])
def test_token_lists_balanced(ops, rows, d):
    """Token lists (duplicates, ragged counts, an empty group) for every workgroup shape; the operator-level
    calls use 192-row groups, the others go through the C ABI."""
    from lvar_amd import _lib
    g = torch.Generator().manual_seed(rows + d)
    B, H, Lq, Lk = 2, 8, 1600, 2600
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=3, amp=0.5)
    G = (Lq + rows - 1) // rows
    idx = torch.randint(0, Lk, (B, H, G, Lk), generator=g, dtype=torch.int32)
    cnt = torch.randint(0, Lk + 1, (B, H, G), generator=g, dtype=torch.int32)
    cnt[0, 1, 0] = 0
    cnt[1, 2, 1] = Lk
    o0 = (torch.randn(B, H, Lq, d, generator=g) * 0.5).to(torch.bfloat16)
    qg, kg, vg, ig, cg, og = q.cuda(), k.cuda(), v.cuda(), idx.cuda(), cnt.cuda(), o0.cuda()
    assert plan(ops, 2, qg, kg, group_rows=rows, list_len=Lk) > 0

    def run():
        out = torch.empty_like(qg)
        M = torch.empty(B, H, Lq, 1, dtype=torch.float32, device="cuda")
        L = torch.empty_like(M)
        stream = ops._stream(qg)
        st = _lib.load().lvar_csp_attn_ws_fwd(ops._view(qg), ops._view(kg), ops._view(vg), ops._view(og), ops._view(out),
                                             M.data_ptr(), L.data_ptr(), ig.data_ptr(), cg.data_ptr(), G, Lk, rows,
                                             B, H, Lq, Lk, d, -1.0, 1.0 / d ** 0.5, ops._workspace(qg, stream), stream)
        assert st == 0
        return out, M, L
    (o1, M1, L1), r2, (op, Mp, Lp) = both(ops, run)
    assert same((o1, M1, L1), r2) and counters_zero(ops, qg)
    ref = oracle.csp_attn(q, k, v, None, idx, cnt, o0, -1, bm=rows)
    _, M_ref, L_ref = oracle.csp_attn_delta(q, k, v, idx, cnt, bm=rows)
    assert close(o1, ref) and lse_close(M1, L1, M_ref, L_ref)
    assert torch.equal(M1, Mp) and torch.allclose(L1, Lp, rtol=1e-5)
    assert (o1.float() - op.float()).abs().max().item() < 2e-2


def test_token_lists_balanced_with_fused_upsample(ops):
    """Sparse step of the CS4A caller at Infinity scale 40 sizes: 9 groups x 32 (batch, head) on a 256-CU part."""
    B, H, d, src, dst, Lk = 2, 16, 128, 32, 40, 4121
    Lq = dst * dst
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=40, amp=0.5)
    g = torch.Generator().manual_seed(40)
    G = (Lq + 191) // 192
    idx = torch.randint(0, Lk, (B, H, G, Lk), generator=g, dtype=torch.int32)
    cnt = torch.full((B, H, G), 1344, dtype=torch.int32)
    cache = (torch.randn(B, H, src * src, d, generator=g) * 0.5).to(torch.bfloat16)
    qg, kg, vg, ig, cg, chg = q.cuda(), k.cuda(), v.cuda(), idx.cuda(), cnt.cuda(), cache.cuda()
    assert plan(ops, 2, qg, kg, list_len=Lk) > 0
    o1, o2, o0 = both(ops, lambda: ops.csp_attn_upsampled(qg, kg, vg, None, ig, cg, chg, 1))
    assert torch.equal(o1, o2) and counters_zero(ops, qg)
    assert (o1.float() - o0.float()).abs().max().item() < 2e-2
    up = oracle.upsample_ocache(cache[:1, :2].float(), src * src, Lq)
    ref = oracle.csp_attn(q[:1, :2], k[:1, :2], v[:1, :2], None, idx[:1, :2], cnt[:1, :2], up, 1)
    assert close(o1[:1, :2], ref, atol=3e-2)


def test_dense_attn_operator_goes_through_the_workspace(ops):
    """With the hook on, ``dense_attn`` leaves its compiled host path (which takes no workspace) and runs the balanced
    grid: the partial-result slots behind the counters are written, the counters are zero again afterwards."""
    B, H, Lq, Lk, d = 1, 3, 300, 5000, 64
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=17, amp=0.7)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    ops.dense_attn(qg, kg, vg)                                        # allocates the workspace of this stream
    assert plan(ops, 0, qg, kg) > 0
    ws = ops._workspaces[(qg.device.index, ops._stream(qg))][1]
    ws.zero_()
    o, (M, L) = ops.dense_attn(qg, kg, vg)
    assert bool(ws[4096:].any()) and counters_zero(ops, qg)
    o_ref, M_ref, L_ref = oracle.dense_attn(q, k, v)
    assert close(o, o_ref) and lse_close(M, L, M_ref, L_ref)
    # stale arrival counters (a launch cut short, a workspace used before) are cleared by the launch itself
    ws[:4096] = 0x5a
    o2, (M2, L2) = ops.dense_attn(qg, kg, vg)
    assert torch.equal(o2, o) and torch.equal(M2, M) and torch.equal(L2, L)
    ops._set_balanced_launch(False)
    ws.zero_()
    ops.dense_attn(qg, kg, vg)
    assert not bool(ws.any())                                         # off: the workspace is not touched
    ops._set_balanced_launch(True)


def test_piece_exchange_gives_the_same_bits_launch_after_launch(ops):
    """The pieces of a cut query tile travel between compute-unit groups through device-coherent stores and loads
    ordered by the arrival counter alone; a stale read would be a silent wrong answer.  Many-piece launches (a dense
    one whose every tile is cut eight times, a token-list one with ragged lists) repeated a few hundred times must
    reproduce the first result bit for bit; the loop stops at the first launch that does not."""
    from lvar_amd import _lib
    q, k, v = make_qkv(1, 3, 300, 5000, 64, seed=23, amp=0.7)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    assert plan(ops, 0, qg, kg) > 0
    first = ops._dense_launch(qg, kg, vg, None)[:3]
    assert close(first[0], oracle.dense_attn(q, k, v)[0])
    for rep in range(300):
        again = ops._dense_launch(qg, kg, vg, None)[:3]
        assert same(again, first), f"dense launch {rep} differs from the first"
    g = torch.Generator().manual_seed(29)
    B, H, Lq, Lk, d, rows = 2, 8, 1600, 2600, 128, 192
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=4, amp=0.5)
    G = (Lq + rows - 1) // rows
    idx = torch.randint(0, Lk, (B, H, G, Lk), generator=g, dtype=torch.int32).cuda()
    cnt = torch.randint(0, Lk + 1, (B, H, G), generator=g, dtype=torch.int32).cuda()
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    o0 = torch.zeros_like(qg)
    assert plan(ops, 2, qg, kg, group_rows=rows, list_len=Lk) > 0
    first = ops.csp_attn(qg, kg, vg, None, idx, cnt, o0, 1)
    for rep in range(200):
        assert torch.equal(ops.csp_attn(qg, kg, vg, None, idx, cnt, o0, 1), first), f"token-list launch {rep} differs from the first"
    assert counters_zero(ops, qg)


def test_small_workspace_and_plain_fallback(ops):
    """A workspace that holds one slot pair per CU halves the workgroups; one too small for that, a null
    workspace, or too little work for a share per workgroup give the plain launch, bit for bit."""
    from lvar_amd import _lib
    lib = _lib.load()
    B, H, Lq, Lk, d = 2, 16, 576, 1497, 128
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=1, amp=0.7)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    full = int(lib.lvar_attn_workspace_bytes(d))
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    slot = (d * 32 * 4 + 3 * 64 * 4) * 4

    def need(P):      # arrival counters, item table for 1024 query tiles + P shares (256-byte granules), 2 * P slots
        return 4096 + ((8 + 8 * (1024 + P)) * 4 + 255) // 256 * 256 + 2 * P * slot
    ops._set_balanced_launch(False)
    o_plain, M_plain, L_plain, _ = ops._dense_launch(qg, kg, vg, None)
    ops._set_balanced_launch(True)
    o_ref, _, _ = oracle.dense_attn(q, k, v)
    assert full >= need(2 * cus)
    for nbytes, want in ((full, 2 * cus), (need(2 * cus), 2 * cus), (need(cus), cus), (need(cus) - 256, 0), (4096, 0)):
        buf = torch.full((nbytes,), 0x33 if want else 0, dtype=torch.uint8, device="cuda")   # contents need no preparation
        ws = _lib.LvarWorkspace(buf.data_ptr(), nbytes, 0, 0)
        assert lib.lvar_attn_balanced_workgroups(0, 0, 0, B, H, Lq, Lk, 0, d, ws) == want
        o = torch.empty_like(qg)
        M = torch.empty(B, H, Lq, 1, dtype=torch.float32, device="cuda")
        L = torch.empty_like(M)
        st = lib.lvar_dense_attn_ws_fwd(ops._view(qg), ops._view(kg), ops._view(vg), ops._view(o), M.data_ptr(), L.data_ptr(), None,
                                        B, H, H, Lq, Lk, d, 1.0 / d ** 0.5, ws, ops._stream(qg))
        assert st == 0 and close(o, o_ref)
        if want == 0:
            assert torch.equal(o, o_plain) and torch.equal(M, M_plain) and torch.equal(L, L_plain)
        assert not bool(buf[:4 * B * H * ((Lq + 127) // 128)].any())      # the arrival counters of this launch's query tiles
    # tiny problem: no share of work per workgroup -> plain
    qs, ks = qg[:, :, :64], kg[:, :, :100]
    assert plan(ops, 0, qs.contiguous(), ks.contiguous()) == 0
    # a misaligned workspace is refused
    buf = torch.zeros(full + 256, dtype=torch.uint8, device="cuda")
    ws = _lib.LvarWorkspace(buf.data_ptr() + 16, full, 0, 0)
    o = torch.empty_like(qg)
    assert lib.lvar_dense_attn_ws_fwd(ops._view(qg), ops._view(kg), ops._view(vg), ops._view(o), None, None, None,
                                      B, H, H, Lq, Lk, d, 1.0 / d ** 0.5, ws, ops._stream(qg)) == -1


def test_balanced_share_and_piece_knobs(ops):
    """Any choice of the two tuning values gives the same attention up to fp32 summation order."""
    B, H, Lq, Lk, d = 1, 4, 700, 3000, 128
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=9, amp=0.7)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    o_ref, M_ref, L_ref = oracle.dense_attn(q, k, v)
    try:
        for share, piece in ((1, 1), (2, 1), (8, 4), (16, 16), (64, 3)):
            ops._set_balanced_launch(True, share, piece)
            o, M, L, _ = ops._dense_launch(qg, kg, vg, None)
            assert close(o, o_ref) and lse_close(M, L, M_ref, L_ref), (share, piece)
            assert counters_zero(ops, qg)
    finally:
        ops._set_balanced_launch(True, 0, 0)


def test_head_dim_256_takes_the_plain_launch(ops):
    """head_dim 256 has no balanced launch: the planning query says 0, the size query returns the 4 KiB minimum and
    the workspace entry point gives the plain launch's result bit for bit."""
    from lvar_amd import _lib
    lib = _lib.load()
    B, H, Lq, Lk, d = 1, 4, 576, 1497, 256
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=2, amp=0.7)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    assert int(lib.lvar_attn_workspace_bytes(d)) == 4096
    assert plan(ops, 0, qg, kg) == 0
    a1, a2, b = both(ops, lambda: ops.dense_attn(qg, kg, vg))
    assert same(a1, b) and same(a2, b)
    assert close(b[0], oracle.dense_attn(q, k, v)[0])
