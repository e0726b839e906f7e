#!/usr/bin/env python3
"""Writes the golden fixtures in this directory from the CPU oracle (fp64 math on bf16-rounded inputs).

    python tests/golden/make_fixtures.py

The reference ships no stored vectors for this path (its self-tests draw inputs from a CUDA generator
at run time), so these fixtures are authored here: inputs are seeded on the CPU, the expected outputs
come from the oracle after it has been pinned by tests/test_oracle.py.  Each .npz holds the bf16
inputs as uint16 bit patterns plus float32 expectations.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle  # noqa: E402


def bits(t):
    return t.view(torch.int16).numpy().astype(np.uint16)


def qkv(B, H, Lq, Lk, d, seed, amp=1.0):
    g = torch.Generator().manual_seed(seed)
    mk = lambda L: (torch.randn(B, H, L, d, generator=g) * amp).to(torch.bfloat16)
    return mk(Lq), mk(Lk), mk(Lk)


def f32(t):
    return t.to(torch.float32).numpy()


def main():
    # 1. VAR-d16 last scale (the CPU-runnable benchmark case), one batch x two heads: dense + colsum + block sums + top-5 blocks
    q, k, v = qkv(1, 1, 256, 680, 64, seed=101)
    o, cs, (M, L) = oracle.dense_colsum_attn(q, k, v, dtype=torch.float64)
    _, cs_all, _ = oracle.dense_colsum_attn(q, k, v, q_group_size=256, dtype=torch.float64)
    bs = oracle.key_block_sums(cs_all, 64)
    top = torch.topk(bs, k=5, dim=-1).indices.sort(-1).values
    np.savez_compressed(os.path.join(HERE, "var_d16_dense_colsum.npz"), q=bits(q), k=bits(k), v=bits(v), o=f32(o), cs=f32(cs),
                        lse2=f32(M + torch.log2(L)), cs_all=f32(cs_all), block_sums=f32(bs), top5_blocks=top.numpy().astype(np.int32))

    # 2. column-sparse attention with duplicated indices and a ragged count, d = 128
    q, k, v = qkv(1, 2, 200, 128, 128, seed=102, amp=0.5)
    g = torch.Generator().manual_seed(5)
    inds = torch.zeros(1, 2, 2, 128, dtype=torch.int32)
    counts = torch.tensor([[[100, 37], [64, 0]]], dtype=torch.int32)
    for h in range(2):
        for gg in range(2):
            c = int(counts[0, h, gg])
            inds[0, h, gg, :c] = torch.randint(0, 128, (c,), generator=g, dtype=torch.int32)
    o0 = (torch.randn(1, 2, 200, 128, generator=g) * 0.5).to(torch.bfloat16)
    out_m = oracle.csp_attn(q, k, v, None, inds, counts, o0, -1, dtype=torch.float64)
    out_p = oracle.csp_attn(q, k, v, None, inds, counts, o0, 1, dtype=torch.float64)
    np.savez_compressed(os.path.join(HERE, "csp_attn_d128.npz"), q=bits(q), k=bits(k), v=bits(v), o0=bits(o0), inds=inds.numpy(),
                        counts=counts.numpy(), out_minus=f32(out_m), out_plus=f32(out_p))

    # 3. block-sparse attention, 128x64 blocks, ragged Lq and Lk
    q, k, v = qkv(1, 1, 200, 300, 128, seed=103)
    mask = torch.rand(1, 1, 2, 5, generator=g) < 0.4
    mask[..., 4] = True
    num, idx = oracle.block_mask_to_lists(mask)
    o, M, L = oracle.block_sparse_attn(q, k, v, num, idx, 128, 64, dtype=torch.float64)
    np.savez_compressed(os.path.join(HERE, "block_sparse_d128.npz"), q=bits(q), k=bits(k), v=bits(v), num=num.numpy(), idx=idx.numpy(),
                        o=f32(o), lse2=f32(M + torch.log2(L)))

    # 4. integer-only fixtures: list build constants of the reference configuration
    runs11, l11 = oracle.aggregate_group_indices(*oracle.crossscale_self_indices(11, 7)[:1], 2304, 6425, 192, 112)
    runs12, l12 = oracle.aggregate_group_indices(*oracle.crossscale_self_indices(12, 9)[:1], 4096, 10521, 192, 112)
    csla = oracle.flex_block_mask(8, [-1, -1, -1, -1, 1, 1, 3, 5, 7], 3, 128)
    np.savez_compressed(os.path.join(HERE, "list_build_constants.npz"), runs11=runs11.numpy(), runs12=runs12.numpy(),
                        csla_scale8=csla.numpy(), cum=np.array(oracle.infinity_cum(), dtype=np.int64))
    # 5. list kernels of the sparse step: token top-k set (with ties through the cut), group remap + local run,
    #    mask compaction with count padding, O-cache upsample + column-sparse attention, window-query key scores
    sc = torch.rand(2, 3, 700, generator=g)
    sc[0, 0, ::2] = 0.5
    topk = oracle.topk_token_set(sc, 128)
    src = torch.randint(0, 1000, (1, 2, 9, 300), generator=g, dtype=torch.int32)
    local = torch.randint(0, 900, (12, 64), generator=g)
    rm, rc = oracle.map_inds_counts_across_scales(src, torch.full((1, 2, 9), 192, dtype=torch.int32), 2304, 900)
    rl, rlc = oracle.append_local_run(rm, 192, local, 64, 900)
    msk = torch.rand(3, 4, 165, generator=g) < 0.2
    mc, mi = oracle.mask_to_lists(msk, 64)
    q, k, v = qkv(1, 2, 64, 200, 128, seed=105, amp=0.5)
    cache = torch.randn(1, 2, 25, 128, generator=g).to(torch.bfloat16)
    uidx = torch.zeros(1, 2, 1, 200, dtype=torch.int32)
    for h in range(2):
        uidx[0, h, 0, :64] = torch.randperm(200, generator=g)[:64].to(torch.int32)
    ucnt = torch.full((1, 2, 1), 64, dtype=torch.int32)
    up = oracle.csp_attn(q, k, v, None, uidx, ucnt, oracle.upsample_ocache(cache, 25, 64), 1, dtype=torch.float64)
    win = torch.randint(136, 200, (1, 2, 9), generator=g)
    ws = oracle.window_key_scores(q, k, win, 5, "avgpool", dtype=torch.float64)
    np.savez_compressed(os.path.join(HERE, "list_kernels.npz"), scores=f32(sc), topk128=topk.numpy(), src=src.numpy(), local=local.numpy(),
                        remap_concat=rl.numpy(), remap_counts=rlc.numpy(), mask=msk.numpy(), mask_counts=mc.numpy(), mask_idx=mi.numpy(),
                        q=bits(q), k=bits(k), v=bits(v), cache=bits(cache), uidx=uidx.numpy(), ucnt=ucnt.numpy(), upsampled_out=f32(up),
                        window=win.numpy(), window_scores=f32(ws))

    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)) // 1024, "KiB")


if __name__ == "__main__":
    main()
