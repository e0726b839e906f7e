"""``lvar_block_sparse_attn_static_fwd``: block-sparse attention whose partial-result workspace is a buffer inside
the library (no allocation, no workspace argument), against ``lvar_block_sparse_attn_ws_fwd`` with a caller-owned
workspace of the same size: bit for bit, on two calls in a row, the second with a smaller input; and against the
CPU oracle.  Both go through the C ABI."""
import pytest
import torch

import oracle
from conftest import make_qkv

pytestmark = pytest.mark.gpu

STATIC_BYTES = 34 << 20
MAX_TILES = 1024


def _call(fn_name, q, k, v, num, idx, bk, ws=None):
    from lvar_amd import _lib
    from lvar_amd import sparse_attn_ops as ops
    lib = _lib.load()
    B, H, Lq, d = q.shape
    o = torch.empty_like(q)
    M = torch.empty(B, H, Lq, 1, dtype=torch.float32, device=q.device)
    L = torch.empty_like(M)
    args = [ops._view(q), ops._view(k), ops._view(v), ops._view(o), M.data_ptr(), L.data_ptr(),
            num.data_ptr(), num.stride(0), num.stride(1), idx.data_ptr(), idx.stride(0), idx.stride(1), idx.stride(2), idx.shape[3],
            128, bk, B, H, Lq, k.shape[2], d, 1.0 / d ** 0.5]
    if ws is not None:
        args.append(ws)
    st = getattr(lib, fn_name)(*args, ops._stream(q))
    return st, o, M, L


def _case(B, H, Lq, Lk, d, bk, seed):
    g = torch.Generator().manual_seed(seed)
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=seed, amp=0.6)
    nQ, nK = (Lq + 127) // 128, (Lk + bk - 1) // bk
    dens = torch.rand(B, H, nQ, 1, generator=g) ** 2
    mask = torch.rand(B, H, nQ, nK, generator=g) < dens
    mask[:, :, 0] = True                                   # a full row: cut into pieces for sure
    if nQ > 2:
        mask[:, :, 2] = False                              # an empty row
    num, idx = oracle.block_mask_to_lists(mask)
    return q, k, v, num, idx


def test_static_scratch_matches_workspace_entry_point():
    from lvar_amd import _lib
    lib = _lib.load()
    buf = torch.zeros(STATIC_BYTES, dtype=torch.uint8, device="cuda")
    ws = _lib.LvarWorkspace(buf.data_ptr(), STATIC_BYTES, 0, 0)
    # two calls in a row on the library's buffer, the second with a smaller input (and another block shape)
    for (B, H, Lq, Lk, d, bk, seed) in ((2, 8, 2560 + 57, 5000, 128, 64, 1), (1, 3, 700, 2100, 64, 128, 2)):
        q, k, v, num, idx = _case(B, H, Lq, Lk, d, bk, seed)
        qg, kg, vg, ng, ig = q.cuda(), k.cuda(), v.cuda(), num.cuda(), idx.cuda()
        planned = lib.lvar_attn_balanced_workgroups(1, 0, bk, B, H, Lq, Lk, idx.shape[3], d, ws)
        assert planned > 0, "the case must take the balanced launch, or the scratch buffer is not exercised"
        st_ws, o_ws, M_ws, L_ws = _call("lvar_block_sparse_attn_ws_fwd", qg, kg, vg, ng, ig, bk, ws)
        st, o, M, L = _call("lvar_block_sparse_attn_static_fwd", qg, kg, vg, ng, ig, bk)
        torch.cuda.synchronize()
        assert st_ws == 0 and st == 0
        assert torch.equal(o, o_ws) and torch.equal(M, M_ws) and torch.equal(L, L_ws)
        o_ref, M_ref, L_ref = oracle.block_sparse_attn(q, k, v, num, idx, 128, bk)
        assert bool(((o.float().cpu() - o_ref).abs() <= 2e-2 + 1e-2 * o_ref.abs()).all())
        fin = torch.isfinite(M_ref)
        lse = (M.cpu() + torch.log2(L.cpu()))[fin]
        assert (lse - (M_ref + torch.log2(L_ref))[fin]).abs().max().item() < 1e-3
        # the same call again gives the same bits (the buffer's leftovers do not matter)
        st2, o2, M2, L2 = _call("lvar_block_sparse_attn_static_fwd", qg, kg, vg, ng, ig, bk)
        assert st2 == 0 and torch.equal(o2, o) and torch.equal(M2, M) and torch.equal(L2, L)


def test_static_scratch_limits():
    """More query tiles than the buffer's tables hold, or a head dimension beyond its slots, are refused."""
    from lvar_amd import _lib
    lib = _lib.load()
    q, k, v, num, idx = _case(1, 2, 256, 512, 128, 64, 3)
    qg, kg, vg, ng, ig = q.cuda(), k.cuda(), v.cuda(), num.cuda(), idx.cuda()
    st, _, _, _ = _call("lvar_block_sparse_attn_static_fwd", qg, kg, vg, ng, ig, 64)
    assert st == 0
    from lvar_amd import sparse_attn_ops as ops
    big_B = MAX_TILES // (2 * 2) + 1                        # B * H * ceil(Lq / 128) = 1028 > 1024
    fake_q = torch.empty(1, 2, 256, 128, dtype=torch.bfloat16, device="cuda")
    o = torch.empty_like(fake_q)
    M = torch.empty(1, 2, 256, 1, dtype=torch.float32, device="cuda")
    st = lib.lvar_block_sparse_attn_static_fwd(ops._view(fake_q), ops._view(kg), ops._view(vg), ops._view(o), M.data_ptr(), M.data_ptr(),
                                               ng.data_ptr(), 0, 0, ig.data_ptr(), 0, 0, ig.stride(2), ig.shape[3],
                                               128, 64, big_B, 2, 256, 512, 128, 0.1, ops._stream(fake_q))
    assert st == -4 and b"static scratch" in lib.lvar_status_string(st)
    # arguments are checked before the scratch is looked at: the same refusals as the workspace entry point
    for (bq, scale, want) in ((96, 0.1, -2), (128, -1.0, -1)):
        st = lib.lvar_block_sparse_attn_static_fwd(ops._view(qg), ops._view(kg), ops._view(vg), ops._view(torch.empty_like(qg)), M.data_ptr(), M.data_ptr(),
                                                   ng.data_ptr(), 0, 0, ig.data_ptr(), 0, 0, ig.stride(2), ig.shape[3],
                                                   bq, 64, 1, 2, 256, 512, 128, scale, ops._stream(qg))
        assert st == want
