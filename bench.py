#!/usr/bin/env python3
"""Benchmark of the sparse-attention hot path on one MI355X.

A "step" is one block-sparse flash-attention forward over the Infinity-2B 1024x1024 last-scale
self-attention batch (B=2 cond+uncond, H=16, d=128, Lq=4096, Lk=10521, bf16, 128x64 blocks at 25 %
density: keys of scales <= 16 always kept, +-2 key blocks around the query position in every later
scale, remainder chosen by colsum top-k).  Inputs are synthetic, seeded, resident in HBM before the
timed region.  The headline value is effective TFLOP/s over ACTIVE blocks (4*d*rows*cols per active
block, softmax flops not counted).

Prints ONE JSON line.  ``--workload`` selects the other single-GPU configurations for profiling.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X published dense bf16 MFMA peak
PEAK_HBM_GBS = 8000.0

# HBM bytes per launch are measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a copy kernel of known
# size, and recorded in the summary under profiles/ that covers the workload, as the line
#   traffic_bytes_per_launch: <bytes>
# next to the SHA-256 of the kernel source the measurement was taken with:
#   kernel_source_sha256: <file under lvar_amd/csrc> <hex digest>
# The bench line carries the figure only while that source file is unchanged.
PROFILE_OF_WORKLOAD = {
    "block_sparse_25": "attn_fwd_block_sparse_infinity2b_1024_last_scale_25pct.txt",
    "dense": "attn_fwd_dense_infinity2b_1024_last_scale.txt",
    "colsum": "colsum_infinity2b_1024_last_scale.txt",
    "csp": "attn_fwd_token_list_infinity2b_1024_last_scale_top20pct.txt",
}


def measured_traffic(workload):
    """(bytes per launch or None, where it comes from / why it is missing)."""
    import hashlib
    import re
    name = PROFILE_OF_WORKLOAD.get(workload)
    if name is None:
        return None, "no counter profile for this workload"
    path = os.path.join(ROOT, "profiles", name)
    try:
        text = open(path).read()
    except OSError:
        return None, f"profiles/{name} is missing"
    m = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", text, re.M)
    h = re.search(r"^kernel_source_sha256:\s*(\S+)\s+([0-9a-f]{64})", text, re.M)
    if not m or not h:
        return None, f"profiles/{name} records no traffic figure"
    try:
        digest = hashlib.sha256(open(os.path.join(ROOT, "lvar_amd", "csrc", h.group(1)), "rb").read()).hexdigest()
    except OSError:
        return None, f"lvar_amd/csrc/{h.group(1)} is missing"
    if digest != h.group(2):
        return None, f"lvar_amd/csrc/{h.group(1)} has changed since profiles/{name} was taken"
    return float(m.group(1)), f"profiles/{name}"


def make_qkv(B, H, Lq, Lk, d, seed, amp):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, H, Lq, d, generator=g) * amp).to(torch.bfloat16)
    k = (torch.randn(B, H, Lk, d, generator=g) * amp).to(torch.bfloat16)
    v = (torch.randn(B, H, Lk, d, generator=g) * amp).to(torch.bfloat16)
    return q, k, v


def block_flops(num, idx, Lq, Lk, d, bq, bk, B, H):
    """4*d*sum(rows_i*cols_j) over active blocks, edge blocks clipped; lists may broadcast over B/H."""
    nQ = num.shape[-1]
    rows = torch.clamp(Lq - torch.arange(nQ, device=num.device) * bq, max=bq).double()
    cols = torch.clamp(Lk - idx.long() * bk, min=0, max=bk).double()
    valid = torch.arange(idx.shape[-1], device=num.device) < num.unsqueeze(-1)
    per_row = (cols * valid).sum(-1) * rows
    mult = (B // num.shape[0]) * (H // num.shape[1])
    return 4.0 * d * float(per_row.sum().item()) * mult


SETTLE_MS = 150.0   # untimed load before the warm-up steps; set from --settle-ms


def device_summary():
    """Name, CU count and maximum engine clock of the GPU as `rocminfo` reports them, and the bf16 MFMA
    rate they imply (4096 flop per clock per CU: four SIMDs, one 32x32x16 MFMA = 32768 flop in 32 cycles
    each).  The roofline peak stays the published figure; this line shows what the part in hand can do."""
    import re
    import subprocess
    pr = torch.cuda.get_device_properties(0)
    out = {"name": pr.name, "arch": pr.gcnArchName, "cus": pr.multi_processor_count, "hbm_gib": round(pr.total_memory / 2 ** 30, 1)}
    try:
        txt = subprocess.run(["/opt/rocm/bin/rocminfo"], capture_output=True, text=True, timeout=30).stdout
        for agent in txt.split("*******")[1:]:
            if re.search(r"Name:\s+gfx950", agent):
                mhz = int(re.search(r"Max Clock Freq\. \(MHz\):\s+(\d+)", agent).group(1))
                cus = int(re.search(r"Compute Unit:\s+(\d+)", agent).group(1))
                out.update({"cus": cus, "max_clock_mhz": mhz, "bf16_mfma_tflops_from_cus_and_clock": round(cus * 4096 * mhz / 1e6, 1)})
                break
    except Exception as e:                      # the summary is informative only
        out["rocminfo_error"] = repr(e)[:80]
    return out


def sustained_mfma_rate():
    """bf16 MFMA TFLOP/s of a register-resident loop (``lvar_amd/csrc/mfma_probe.hip``: every wave cycles through 8 A and
    8 B fragments it holds in registers, 8 waves per CU) on random N(0,1)*0.5 operand bits and on all-zero bits, timed
    on this box after the same settle period as the workload.  The clock under a matrix load follows the switching
    activity of the operands, so the random-operand figure is the rate a bf16 MFMA kernel on this box can approach;
    the published peak assumes the maximum clock.  None when the probe library is not built."""
    import ctypes
    path = os.path.join(ROOT, "lvar_amd", "liblvar_bench_probe.so")
    if not os.path.exists(path):
        return None
    lib = ctypes.CDLL(path)
    lib.lvar_probe_mfma.restype = ctypes.c_int
    lib.lvar_probe_mfma.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    blocks, iters = 2 * torch.cuda.get_device_properties(0).multi_processor_count, 2048
    dst = torch.empty(blocks * 256, dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    flops = blocks * 4.0 * iters * 16 * 32768
    out = {"kernel": "mfma_probe_kernel: %d workgroups x 4 waves x %d x 16 MFMA 32x32x16" % (blocks, iters)}
    g = torch.Generator().manual_seed(5)
    for name, src in (("random_operands_tflops", (torch.randn(16 * 256 * 8, generator=g) * 0.5).to(torch.bfloat16).cuda()),
                      ("zero_operands_tflops", torch.zeros(16 * 256 * 8, dtype=torch.bfloat16, device="cuda"))):
        def fn():
            st = lib.lvar_probe_mfma(src.data_ptr(), dst.data_ptr(), blocks, iters, stream)
            assert st == 0, st
        ms, _ = time_launches(fn, 30, 5)
        out[name] = round(flops / ms / 1e9, 1)
    return out


def settle_clocks(fn, ms):
    """Keep the GPU busy with the workload for ``ms`` milliseconds.  After an idle period the part
    needs ~20 ms of load before its clocks settle (the first ~100 launches of the headline kernel
    take 200 us, every later one 170 us); timing a short burst right after idle measures that ramp."""
    if ms <= 0:
        return
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()


def time_launches(fn, steps, warmup):
    """Average duration of ``steps`` back-to-back launches measured with HIP events recorded on the
    stream the kernels are enqueued on (torch's current stream), plus host wall time."""
    settle_clocks(fn, SETTLE_MS)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return e0.elapsed_time(e1) / steps, wall * 1e3 / steps


def time_graph_replay(fn, calls, steps, warmup):
    """Per-call duration of ``fn`` when ``calls`` consecutive calls are captured into one HIP graph and the
    graph is replayed (what a caller sees that captures its layer loop): no host work per call."""
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for _ in range(calls):
            fn()
    ms, _ = time_launches(graph.replay, steps, warmup)
    return ms / calls


def per_launch_stats(fn, n=50):
    """Median and minimum duration of single launches (one event pair per launch, same stream)."""
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    t = sorted(a.elapsed_time(b) for a, b in evs)
    return {"median_ms": round(t[len(t) // 2], 5), "min_ms": round(t[0], 5), "launches": n}


def cpu_baseline_block_sparse(q, k, v, num, idx, bq, bk, budget_s=20.0):
    """Oracle (torch fp32 on the host cores) on a bounded sample of the same workload: whole
    (batch, head) slices until ~budget_s of CPU time is spent.  Returns TFLOP/s and a description."""
    import oracle
    torch.set_num_threads(os.cpu_count() or 1)
    B, H, Lq, d = q.shape
    Lk = k.shape[2]
    done, flops, t_used = 0, 0.0, 0.0
    while t_used <= budget_s:          # cycle over the (batch, head) slices until the time budget is spent
        b, h = divmod(done % (B * H), H)
        nb = num[b:b + 1, h:h + 1] if num.shape[0] > 1 else num[:, h:h + 1] if num.shape[1] > 1 else num
        ib = idx[b:b + 1, h:h + 1] if idx.shape[0] > 1 else idx[:, h:h + 1] if idx.shape[1] > 1 else idx
        t0 = time.perf_counter()
        oracle.block_sparse_attn(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], nb, ib, bq, bk)
        t_used += time.perf_counter() - t0
        flops += block_flops(nb, ib, Lq, Lk, d, bq, bk, 1, 1)
        done += 1
    return flops / t_used / 1e12, (f"{done} (batch,head) slices (the workload has {B * H}; cycled) of the same inputs and "
                                   f"block lists, {t_used:.1f} s of host time")


def cpu_baseline_dense(q, k, v, budget_s=20.0, colsum=False):
    import oracle
    torch.set_num_threads(os.cpu_count() or 1)
    B, H, Lq, d = q.shape
    Lk = k.shape[2]
    done, t_used = 0, 0.0
    while t_used <= budget_s:          # cycle over the (batch, head) slices until the time budget is spent
        b, h = divmod(done % (B * H), H)
        t0 = time.perf_counter()
        if colsum:
            oracle.dense_colsum_attn(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1])
        else:
            oracle.dense_attn(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1])
        t_used += time.perf_counter() - t0
        done += 1
    return done, t_used


def run_infinity_schedule(args, dev):
    """Attention time of one Infinity-2B 1024^2 image (13 scales x 32 layers, B=2 for classifier-free
    guidance, H16 d128): every layer dense, against the SparVAR schedule of the reference's shipped
    configuration (models/sparvar/sparse-attn-config.yml:15-34): scales 0-9 dense; scales 10-12:
    layers 0-10 column-sparse (full step at scale 10, sparse steps with the upsampled O-cache at 11 and
    12), layers 11-31 sink + local-window block masks.  One layer of every distinct shape is timed and
    multiplied by its layer count."""
    from lvar_amd import mask_build as mb
    from lvar_amd import sparse_attn_config as cfg
    from lvar_amd import sparse_attn_ops as ops
    from lvar_amd.sparse_diff_attn import SparseDiffAttn
    from lvar_amd.sparse_flex_attn import SparseFlexAttn
    scales = list(mb.INFINITY_SCALES)
    offs = mb.scale_offsets(scales)
    B, H, d, n_layers, bound = 2, 16, 128, 32, 10
    win = [-1, -1, -1, -1, -1, -1, -1, -1, 1, 1, 3, 5, 7]
    cfg.reset()
    cfg.GLOBAL_CONFIG["attn"]["top_keys"] = 0.2                        # the shipped value (sparse-attn-config.yml:19)
    steps, warm = max(5, args.steps // 5), max(3, args.warmup // 4)
    g = torch.Generator().manual_seed(99)
    mk = lambda L: (torch.randn(B, H, L, d, generator=g) * 0.5).to(torch.bfloat16).to(dev)
    dense_ms, sparse_ms, graph_saving_ms, rows = 0.0, 0.0, 0.0, []
    diff = SparseDiffAttn(scales=scales, spsd_scale=10)
    for si, S in enumerate(scales):
        Lq, Lk = S * S, offs[si + 1]
        q, k, v = mk(Lq), mk(Lk), mk(Lk)
        t_dense, _ = time_launches(lambda: ops.dense_attn(q, k, v, None), steps, warm)
        dense_ms += n_layers * t_dense
        if si < 10:
            sparse_ms += n_layers * t_dense
            t_graph = time_graph_replay(lambda: ops.dense_attn(q, k, v, None), n_layers, max(3, steps // 4), 2)
            graph_saving_ms += n_layers * max(0.0, t_dense - t_graph)
            rows.append({"scale": S, "Lq": Lq, "Lk": Lk, "dense_us": round(t_dense * 1e3, 1), "dense_graph_replay_us": round(t_graph * 1e3, 1)})
            continue
        flex = SparseFlexAttn([(s, s) for s in scales], win, q_scale_idx=si, attn_sink_scale=5, num_heads=H, device=dev)
        t_flex, _ = time_launches(lambda: flex(q, k, v, None), steps, warm)
        if si == 10:
            t_cs4a, _ = time_launches(lambda: diff(q, k, v, None, do_full_step=True, scale_ind=si), steps, warm)
        else:
            saved = (diff.indices, diff.counts, diff.count_host)

            def sparse_step():
                diff.indices, diff.counts, diff.count_host = saved      # every timed call starts from the same cached lists
                return diff(q, k, v, None, scale_ind=si)
            t_cs4a, _ = time_launches(sparse_step, steps, warm)
            diff.indices, diff.counts, diff.count_host = saved
            diff(q, k, v, None, scale_ind=si)                             # leaves the lists of this scale for the next one
        sparse_ms += (bound + 1) * t_cs4a + (n_layers - bound - 1) * t_flex
        rows.append({"scale": S, "Lq": Lq, "Lk": Lk, "dense_us": round(t_dense * 1e3, 1), "cs4a_layer_us": round(t_cs4a * 1e3, 1),
                     "csla_layer_us": round(t_flex * 1e3, 1), "csla_block_density": round(flex.density, 4)})
    print(json.dumps({
        "metric": "self-attention time per Infinity-2B 1024^2 image (all scales, 32 layers), SparVAR schedule", "value": round(sparse_ms, 3),
        "unit": "ms", "n_gpus": 1, "steps": steps, "warmup": warm, "ms_per_step": round(sparse_ms, 3), "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic (seeded N(0,1)*0.5, random-init, no checkpoint)",
        "config": {"workload": "infinity2b_schedule", "B": B, "H": H, "head_dim": d, "layers": n_layers, "scales": scales,
                   "decision_scale": 10, "top_keys": cfg.GLOBAL_CONFIG["attn"]["top_keys"], "bound_layer": bound, "attn_sink": 5, "win_size": win},
        "all_dense_ms": round(dense_ms, 3), "speedup_vs_all_dense": round(dense_ms / sparse_ms, 3),
        "with_dense_scales_replayed_from_hip_graph_ms": round(sparse_ms - graph_saving_ms, 3), "per_scale": rows,
        "device": torch.cuda.get_device_name(0)}))
    cfg.reset()


def run_hbm_workload(args, dev, wl):
    """The HBM-bound helper kernels at the headline shape, priced against 8 TB/s: token top-k
    (``topk_tokens``), group remap + local-run append (``remap_lists``), window-query key scores
    (``window_scores``).  Algorithmic bytes: inputs read once + outputs written once."""
    import oracle
    from lvar_amd import _lib
    from lvar_amd import mask_build as mb
    from lvar_amd import sparse_attn_ops as ops
    B, H, Lq, Lk, d, G = 2, 16, 4096, 10521, 128, 22
    g = torch.Generator().manual_seed(4321)
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    cpu = None
    if wl == "topk_tokens":
        cnt = mb.indices_count(0.2, Lk, 64)
        cs_cpu = torch.rand(B, H, G, Lk, generator=g) ** 4                                  # heavy-tailed like column sums
        cs = cs_cpu.to(dev)
        idx = torch.zeros(B, H, G, Lk, dtype=torch.int32, device=dev)
        cn = torch.empty(B, H, G, dtype=torch.int32, device=dev)
        fn = lambda: lib.lvar_topk_token_lists(cs.data_ptr(), Lk, idx.data_ptr(), Lk, cn.data_ptr(), B * H * G, Lk, cnt, 0, stream)
        nbytes = B * H * G * (Lk * 4 + cnt * 4 + 4)
        kernel, unit_desc = f"topk_token_lists_kernel<{(Lk + 511) // 512},512>", f"{B * H * G} rows x {Lk} fp32 scores, k = {cnt}"
        fn()
        assert torch.equal(idx[..., :cnt].cpu(), oracle.topk_token_set(cs_cpu, cnt)), "top-k differs from the oracle"
        if not args.no_cpu_baseline:
            t0 = time.perf_counter()
            rows = 0
            while time.perf_counter() - t0 < args.cpu_budget_s:
                oracle.topk_token_set(cs_cpu[0, rows % H], cnt)
                rows += G
            t = time.perf_counter() - t0
            cpu = {"value": round(rows * (Lk * 4 + cnt * 4 + 4) / t / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                   "sample": f"{rows} rows of the same scores (numpy stable argsort per row), {t:.1f} s of host time"}
    elif wl == "remap_lists":
        Gs, Ks, cnt, L = 9, 4121, 832, 704
        src = torch.randint(0, Ks, (B, H, Gs, Ks), generator=g, dtype=torch.int32).to(dev)
        loc = torch.randint(0, Lk, (G, L), generator=g).to(dev)
        out = torch.zeros(B, H, G, Lk, dtype=torch.int32, device=dev)
        cn = torch.empty(B, H, G, dtype=torch.int32, device=dev)
        fn = lambda: lib.lvar_remap_concat_lists(src.data_ptr(), Ks, Ks, loc.data_ptr(), L, L, out.data_ptr(), Lk, cn.data_ptr(),
                                                 B * H, Gs, G, cnt, Lk, 0, stream)
        nbytes = B * H * G * ((cnt + L) * 4 + cnt * 4 + L * 8 + 4)
        kernel, unit_desc = "remap_concat_lists_kernel", f"{B * H * G} output rows: {cnt} remapped + {L} local keys"
        if not args.no_cpu_baseline:
            src_c, loc_c, cs_c = src.cpu(), loc.cpu(), torch.full((B, H, Gs), cnt, dtype=torch.int32)
            t0, reps = time.perf_counter(), 0
            while time.perf_counter() - t0 < args.cpu_budget_s:
                a, _ = oracle.map_inds_counts_across_scales(src_c, cs_c, Lq, Lk)
                oracle.append_local_run(a, cnt, loc_c, L, Lk)
                reps += 1
            t = time.perf_counter() - t0
            cpu = {"value": round(reps * nbytes / t / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                   "sample": f"{reps} passes over the same lists, {t:.1f} s of host time"}
    elif wl == "window_scores":
        W = 256
        q = (torch.randn(B, H, Lq, d, generator=g) * 0.5).to(torch.bfloat16).to(dev)
        k = (torch.randn(B, H, Lk, d, generator=g) * 0.5).to(torch.bfloat16).to(dev)
        win = torch.randint(Lk - Lq, Lk, (B, H, W), generator=g).to(dev)
        fn = lambda: ops.window_key_scores(q, k, win, 5, "avgpool")
        nbytes = B * H * (Lk * d * 2 + Lk * 4 + W * (d * 2 + 8))
        kernel, unit_desc = "window_scores_kernel<128>", f"{B * H} (batch,head) x {Lk} keys, {W} window queries, avg pool 5"
        if not args.no_cpu_baseline:
            torch.set_num_threads(os.cpu_count() or 1)
            qc, kc, wc = q.cpu(), k.cpu(), win.cpu()
            t0, reps = time.perf_counter(), 0
            while time.perf_counter() - t0 < args.cpu_budget_s:
                oracle.window_key_scores(qc, kc, wc, 5, "avgpool")
                reps += 1
            t = time.perf_counter() - t0
            cpu = {"value": round(reps * nbytes / t / 1e9, 4), "unit": "GB/s", "cores": os.cpu_count(), "kind": "port",
                   "sample": f"{reps} passes over the same inputs (gather + [W x Lk] matmul + pool), {t:.1f} s of host time"}
    else:
        raise SystemExit(f"unknown workload {wl}")
    ms, wall_ms = time_launches(fn, args.steps, args.warmup)
    gbs = nbytes / ms / 1e6
    print(json.dumps({
        "metric": f"{wl} effective GB/s", "value": round(gbs, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32/i32" if wl != "window_scores" else "bf16", "data": "synthetic (seeded)",
        "config": {"workload": wl, "shape": unit_desc},
        "roofline": {"bound": "hbm", "kernel": kernel, "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": None, "bytes_per_launch": nbytes,
                     "host_wall_ms_per_step": round(wall_ms, 5)},
        "cpu_baseline": cpu, "device": torch.cuda.get_device_name(0)}))


def setup_workload(wl, args, dev, want_cpu, want_parts):
    """Inputs, launch closure, algorithmic flops and description of one attention / colsum workload.  ``want_cpu``:
    also time the oracle on the host cores; ``want_parts``: also time the workload's component kernels."""
    from lvar_amd import mask_build as mb
    from lvar_amd import sparse_attn_ops as ops
    dense_ms = None
    num = idx = None
    d = 128
    aux = {}
    cpu = None

    if wl in ("block_sparse_25", "dense", "colsum", "csp") or wl.startswith("density_"):
        B, H, Lq, Lk = (1 if wl.startswith("density_") else 2), 16, 4096, 10521
        amp = 1.0 if (wl.startswith("density_") or wl == "colsum") else 0.5
    elif wl == "colsum_scale48":
        B, H, Lq, Lk, amp = 2, 16, 2304, 6425, 1.0
    elif wl == "full_step":
        B, H, Lq, Lk, amp = 2, 16, 1600, 4121, 0.5
    elif wl == "video_10":
        B, H, Lq, Lk, amp = 1, 24, 32768, 32768, 0.5
    else:
        raise SystemExit(f"unknown workload {wl}")
    if args.amp is not None:
        amp = args.amp
    q, k, v = make_qkv(B, H, Lq, Lk, d, seed=1234, amp=amp)
    qg, kg, vg = q.to(dev), k.to(dev), v.to(dev)
    scale = 1.0 / math.sqrt(d)
    dense_flops = 4.0 * B * H * Lq * Lk * d
    config = {"workload": wl, "B": B, "H": H, "head_dim": d, "Lq": Lq, "Lk": Lk}

    if wl == "block_sparse_25" or wl.startswith("density_") or wl == "video_10":
        bq, bk = 128, (128 if wl == "video_10" else 64)
        nQ, nK = (Lq + bq - 1) // bq, (Lk + bk - 1) // bk
        if wl == "block_sparse_25":
            cs, bsum = ops.colsum(qg, kg, scale, q_group_size=bq, return_block_sums=True)   # [B,H,nQ,Lk], [B,H,nQ,nK]
            mask = mb.sink_window_topk_block_mask(bsum, bq, bk, density=0.25)
            del cs
            config.update({"block": [bq, bk], "mask": "sink(scales<=16)+window(+-2 blocks/scale)+colsum top-k", "density": 0.25})
        elif wl == "video_10":
            # 3D local window over a latent grid of 8 frames x 64 x 64 tokens (+-1 frame, +-1 spatial
            # block of 128 tokens) plus colsum top-k blocks (scores from every 4th query row) up to 10 % density
            num, idx, _ = mb.video_window_topk_block_lists(qg, kg, scale, density=0.10)
            mask = None
            config.update({"block": [bq, bk], "mask": "3D window (+-1 frame, +-1 spatial block) + colsum top-k blocks up to 10 %"})
        else:
            pct = float(wl.split("_")[1])
            g = torch.Generator().manual_seed(7)
            mask = torch.rand(B, H, nQ, nK, generator=g) < pct / 100.0
            mask.scatter_(-1, torch.randint(0, nK, (B, H, nQ, 1), generator=g), True)
            mask = mask.to(dev)
            config.update({"block": [bq, bk], "mask": f"Bernoulli({pct}%) blocks, >=1 per row"})
        if mask is not None:
            num, idx = mb.block_mask_to_lists(mask)
        flops = block_flops(num, idx, Lq, Lk, d, bq, bk, B, H)
        config["active_block_fraction"] = round(float(num.float().mean().item()) / nK, 4)
        fn = lambda: ops.block_sparse_attn(qg, kg, vg, num, idx, bq, bk, scale)
        kernel = "attn_fwd_kernel<128,4,MODE_BLOCK>"
        if want_cpu:
            val, sample = cpu_baseline_block_sparse(q, k, v, num.cpu(), idx.cpu(), bq, bk, args.cpu_budget_s)
            cpu = {"value": round(val, 5), "unit": "TFLOP/s", "cores": os.cpu_count(), "kind": "port", "sample": sample}
    elif wl == "dense":
        flops = dense_flops
        fn = lambda: ops.dense_attn(qg, kg, vg, scale)
        kernel = "attn_fwd_kernel<128,4,MODE_BLOCK> (identity list)"
        if want_cpu:
            done, t = cpu_baseline_dense(q, k, v, args.cpu_budget_s)
            cpu = {"value": round(dense_flops / (B * H) * done / t / 1e12, 5), "unit": "TFLOP/s", "cores": os.cpu_count(),
                   "kind": "port", "sample": f"{done} (batch,head) slices (the workload has {B * H}; cycled), {t:.1f} s of host time"}
    elif wl in ("colsum", "colsum_scale48"):
        lse2 = ops._lse_only(qg, kg, scale)
        flops = 2.0 * B * H * Lq * Lk * d      # column sweep with the row statistics supplied
        fn = lambda: ops._colsum_given_lse(qg, kg, lse2, scale, 192)
        kernel = "colsum_kernel<128>"
        config["form"] = "one-pass given (M,L): 2*B*H*Lq*Lk*d flops"
        if want_cpu:
            done, t = cpu_baseline_dense(q, k, v, args.cpu_budget_s, colsum=True)
            cpu = {"value": round(1.5 * dense_flops / (B * H) * done / t / 1e12, 5), "unit": "TFLOP/s", "cores": os.cpu_count(),
                   "kind": "port", "sample": f"{done} (batch,head) slices (the workload has {B * H}; cycled) of dense attention + colsum (6*Lq*Lk*d flops each), {t:.1f} s of host time"}
    elif wl == "full_step":
        # decision-scale step of the CS4A caller (models/sparvar/sparse_attn.py:1006-1049): dense attention + colsum +
        # top-k key lists + O_cache = O - delta over the selected keys; effective rate over the dense flops
        from lvar_amd import sparse_attn_config as cfgmod
        from lvar_amd.sparse_diff_attn import SparseDiffAttn
        cfgmod.reset()
        cfgmod.GLOBAL_CONFIG["attn"]["top_keys"] = 0.2
        mod = SparseDiffAttn(0, None, spsd_scale=10)
        flops = dense_flops
        fn = lambda: mod(qg, kg, vg, scale, do_full_step=True, scale_ind=10)
        kernel = "attn_fwd_kernel<128,4,MODE_BLOCK> + colsum_kernel<128> + topk_token_lists_kernel + attn_fwd_kernel<128,8,MODE_GATHER>"
        dense_ms, _ = time_launches(lambda: ops.dense_attn(qg, kg, vg, scale), 20, 5)
        lse2 = ops._lse_only(qg, kg, scale)
        o_d, _, _, _ = ops._dense_launch(qg, kg, vg, scale)
        cs = ops._colsum_given_lse(qg, kg, lse2, scale, 192)
        i_d, c_d = mb.topk_index_list(cs, 0.2, order="index")
        parts = {"dense_attn_us": dense_ms * 1e3}
        if want_parts:
            parts.update({
                "colsum_us": time_launches(lambda: ops._colsum_given_lse(qg, kg, lse2, scale, 192), 20, 5)[0] * 1e3,
                "topk_lists_us": time_launches(lambda: mb.topk_index_list(cs, 0.2, order="index"), 20, 5)[0] * 1e3,
                "ocache_csp_us": time_launches(lambda: ops.csp_attn(qg, kg, vg, scale, i_d, c_d, o_d, -1), 20, 5)[0] * 1e3})
        aux = {k_: round(v_, 1) for k_, v_ in parts.items()}
        config.update({"top_keys": 0.2, "decision_scale": 10, "count": int(c_d[0, 0, 0])})
    elif wl == "csp":
        G = (Lq + 191) // 192
        cs = ops.colsum(qg, kg, scale)
        inds, counts = mb.topk_index_list(cs, 0.2, order="index")     # GPU radix select, ascending key order
        cnt = int(counts[0, 0, 0])
        if want_parts:
            topk_ms, _ = time_launches(lambda: ops.topk_token_lists(cs, cnt), 10, 3)
            torch_ms, _ = time_launches(lambda: torch.topk(cs, cnt, dim=-1), 5, 2)
            ref_set = torch.topk(cs, cnt, dim=-1).indices.sort(-1).values
            assert torch.equal(inds[..., :cnt].long(), ref_set), "GPU top-k set differs from torch.topk"
            aux = {"topk_token_lists_us": round(topk_ms * 1e3, 1), "torch_topk_us": round(torch_ms * 1e3, 1)}
        del cs
        rows = torch.tensor([min(192, Lq - g * 192) for g in range(G)], dtype=torch.float64)
        flops = 4.0 * d * B * H * float(rows.sum()) * cnt
        o0 = torch.zeros_like(qg)
        fn = lambda: ops.csp_attn(qg, kg, vg, scale, inds, counts, o0, 1)
        kernel = "attn_fwd_kernel<128,6,MODE_GATHER>"
        config.update({"top_keys": 0.2, "count": cnt})

    return {"fn": fn, "flops": flops, "kernel": kernel, "config": config, "cpu": cpu, "aux": aux, "amp": amp, "dense_ms": dense_ms,
            "q": qg, "k": kg, "v": vg, "scale": scale, "num": num, "idx": idx, "dense_flops": dense_flops}


def headline_companions(w, ms):
    """The numbers the metric names beside the block-sparse rate: colsum and the GPU mask build against the dense
    attention they replace, in the form that reuses the row statistics of a dense pass (given ``lse2``) and in the
    self-contained two-pass form (statistics sweep + column sweep)."""
    from lvar_amd import mask_build as mb
    from lvar_amd import sparse_attn_ops as ops
    qg, kg, vg, scale, num, idx = w["q"], w["k"], w["v"], w["scale"], w["num"], w["idx"]
    dense_ms, _ = time_launches(lambda: ops.dense_attn(qg, kg, vg, scale), 10, 3)
    lse2 = ops._lse_only(qg, kg, scale)
    cs_ms, _ = time_launches(lambda: ops._colsum_given_lse(qg, kg, lse2, scale, 128), 10, 3)
    lse_ms, _ = time_launches(lambda: ops._lse_only(qg, kg, scale), 10, 3)
    base = mb.sink_window_base_mask(128, 64, device=qg.device)
    target = int(round(0.25 * base.shape[1]))

    def build():
        _, bs = ops._colsum_given_lse(qg, kg, lse2, scale, 128, want_block_sums=True)
        return ops.block_topk_lists(bs, target, base)

    def build_two_pass():
        _, bs = ops.colsum(qg, kg, scale, q_group_size=128, return_block_sums=True)
        return ops.block_topk_lists(bs, target, base)
    n2, i2 = build()
    assert torch.equal(n2, num) and torch.equal(i2, idx), "GPU list build differs from the torch selection"
    n3, i3 = build_two_pass()
    assert torch.equal(n3, num) and torch.equal(i3, idx), "two-pass GPU list build differs from the torch selection"
    build_ms, _ = time_launches(build, 5, 2)
    build2_ms, _ = time_launches(build_two_pass, 5, 2)
    return {"dense_attn_ms": round(dense_ms, 4), "dense_attn_tflops": round(w["dense_flops"] / dense_ms / 1e9, 1),
            "colsum_given_lse_us": round(cs_ms * 1e3, 1), "lse_pass_us": round(lse_ms * 1e3, 1),
            "colsum_plus_mask_build_ms": round(build_ms, 4),
            "colsum_plus_mask_build_two_pass_ms": round(build2_ms, 4),
            "colsum_plus_mask_build_over_dense": round(build_ms / dense_ms, 3),
            "colsum_plus_mask_build_two_pass_over_dense": round(build2_ms / dense_ms, 3),
            "speedup_vs_dense": round(dense_ms / ms, 3)}


def colsum_config(args, dev, Lq, Lk):
    """BASELINE configuration 3: the colsum kernel alone at one scale (B2 H16 d128, N(0,1) inputs, 192-row groups),
    its per-64-key block sums and the block top-k lists at keep ratios 10 / 25 / 50 %; given the row statistics of a
    dense pass, and self-contained (statistics sweep + column sweep)."""
    from lvar_amd import sparse_attn_ops as ops
    B, H, d = 2, 16, 128
    q, k, _ = make_qkv(B, H, Lq, Lk, d, seed=1234, amp=1.0)
    qg, kg = q.to(dev), k.to(dev)
    scale = 1.0 / math.sqrt(d)
    lse2 = ops._lse_only(qg, kg, scale)
    flops = 2.0 * B * H * Lq * Lk * d
    st, wu = max(5, args.steps // 3), max(3, args.warmup // 4)
    cs_ms, _ = time_launches(lambda: ops._colsum_given_lse(qg, kg, lse2, scale, 192, want_block_sums=True), st, wu)
    two_ms, _ = time_launches(lambda: ops.colsum(qg, kg, scale, q_group_size=192, return_block_sums=True), st, wu)
    _, bs = ops._colsum_given_lse(qg, kg, lse2, scale, 192, want_block_sums=True)
    out = {"Lq": Lq, "Lk": Lk, "colsum_given_lse_us": round(cs_ms * 1e3, 1), "tflops": round(flops / cs_ms / 1e9, 1),
           "frac": round(flops / cs_ms / 1e9 / PEAK_BF16_TFLOPS, 4),
           "colsum_two_pass_us": round(two_ms * 1e3, 1), "two_pass_tflops": round(2 * flops / two_ms / 1e9, 1),
           "two_pass_frac": round(2 * flops / two_ms / 1e9 / PEAK_BF16_TFLOPS, 4)}
    nK = bs.shape[-1]
    for keep in (10, 25, 50):
        target = int(round(keep / 100.0 * nK))
        t_ms, _ = time_launches(lambda: ops.block_topk_lists(bs, target), st, wu)
        out[f"block_topk_{keep}pct_us"] = round(t_ms * 1e3, 1)
    return out


def other_configs(args, dev):
    """The benchmark configurations beside the headline one, each timed in this run with fewer steps: density sweep
    against dense attention on the same shape (configuration 4), long-video block-sparse attention (5), colsum alone
    at scales 48 and 64 (3), and the two steps of the column-sparse caller (token-list attention at the last scale,
    the full decision-scale step)."""
    st, wu = max(5, args.steps // 3), max(3, args.warmup // 4)
    out = {"steps": st, "warmup": wu}

    def one(wl, parts=False):
        w = setup_workload(wl, args, dev, want_cpu=False, want_parts=parts)
        ms, _ = time_launches(w["fn"], st, wu)
        tf = w["flops"] / ms / 1e9
        r = {"us": round(ms * 1e3, 1), "tflops": round(tf, 1), "frac": round(tf / PEAK_BF16_TFLOPS, 4)}
        if "active_block_fraction" in w["config"]:
            r["active_block_fraction"] = w["config"]["active_block_fraction"]
        return r, w, ms
    sweep = {}
    for pct in (5, 10, 25, 50, 75, 100):
        r, w, ms = one(f"density_{pct}")
        if pct == 100:
            from lvar_amd import sparse_attn_ops as ops
            d_ms, _ = time_launches(lambda: ops.dense_attn(w["q"], w["k"], w["v"], w["scale"]), st, wu)
            sweep["dense_same_shape"] = {"us": round(d_ms * 1e3, 1), "tflops": round(w["dense_flops"] / d_ms / 1e9, 1)}
        sweep[str(pct)] = r
        del w
    for pct in (5, 10, 25, 50, 75, 100):
        sweep[str(pct)]["vs_dense_tflops"] = round(sweep[str(pct)]["tflops"] / sweep["dense_same_shape"]["tflops"], 3)
    out["density_sweep_B1"] = sweep
    torch.cuda.empty_cache()
    out["video_10"], w, _ = one("video_10")
    del w
    torch.cuda.empty_cache()
    out["colsum_scale48"] = colsum_config(args, dev, 2304, 6425)
    out["colsum_scale64"] = colsum_config(args, dev, 4096, 10521)
    out["csp_top20pct_last_scale"], w, _ = one("csp")
    del w
    r, w, ms = one("full_step", parts=True)
    r.update(w["aux"])
    r["full_step_over_dense"] = round(ms / w["dense_ms"], 3)
    r.pop("tflops"), r.pop("frac")
    out["full_step_decision_scale"] = r
    del w
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="block_sparse_25",
                    help="block_sparse_25 (headline) | dense | colsum | colsum_scale48 | csp | full_step | density_<pct> | video_10 | infinity2b_schedule | topk_tokens | remap_lists | window_scores | copy_1gib")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-aux", action="store_true", help="skip the companion dense/colsum/mask-build timings")
    ap.add_argument("--cpu-budget-s", type=float, default=12.0)
    ap.add_argument("--settle-ms", type=float, default=150.0,
                    help="untimed load run before the warm-up steps so that the clocks have settled (0 = off)")
    ap.add_argument("--amp", type=float, default=None, help="override the input amplitude (0 = all-zero inputs, for power experiments)")
    args = ap.parse_args()
    global SETTLE_MS
    SETTLE_MS = args.settle_ms
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the hot path on ONE GPU; --gpus N with N > 1 is not supported "
              "(the path shards over (batch, head) with no exchange step: give every GPU its own heads).", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU fallback)", file=sys.stderr)
        sys.exit(1)

    from lvar_amd import mask_build as mb
    from lvar_amd import sparse_attn_ops as ops

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    wl = args.workload
    if wl in ("topk_tokens", "remap_lists", "window_scores"):
        run_hbm_workload(args, dev, wl)
        return
    if wl == "infinity2b_schedule":
        run_infinity_schedule(args, dev)
        return
    if wl == "copy_1gib":
        # plain device copy of known size: calibrates the FETCH_SIZE / WRITE_SIZE counters
        x = torch.empty(1 << 28, dtype=torch.float32, device=dev)
        y = torch.empty_like(x)
        ms, _ = time_launches(lambda: y.copy_(x), args.steps, args.warmup)
        print(json.dumps({"metric": "device copy bandwidth", "value": round(2 * x.numel() * 4 / ms / 1e6, 1), "unit": "GB/s",
                          "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 5),
                          "config": {"workload": wl, "bytes_read": x.numel() * 4, "bytes_written": x.numel() * 4}}))
        return
    w = setup_workload(wl, args, dev, want_cpu=not args.no_cpu_baseline, want_parts=not args.no_aux)
    fn, flops, aux, cpu, kernel, config, amp = w["fn"], w["flops"], w["aux"], w["cpu"], w["kernel"], w["config"], w["amp"]
    ms, wall_ms = time_launches(fn, args.steps, args.warmup)
    tflops = flops / (ms * 1e-3) / 1e12
    single = per_launch_stats(fn)
    if wl == "full_step":
        aux["full_step_us"] = round(ms * 1e3, 1)
        aux["full_step_over_dense"] = round(ms / w["dense_ms"], 3)
    probe = None if args.no_aux else sustained_mfma_rate()
    if wl == "block_sparse_25" and not args.no_aux:
        # the numbers the metric names beside the block-sparse rate, then the other benchmark configurations
        aux.update(headline_companions(w, ms))
        del w, fn
        torch.cuda.empty_cache()
        aux["configs"] = other_configs(args, dev)

    traffic, traffic_src = measured_traffic(wl)
    dev_sum = device_summary()
    # CU count x 4096 flop per clock x maximum engine clock, as the device reports them at run time; `peak` and
    # `frac` stay the published 2.5 PFLOP/s
    peak_rt = dev_sum.get("bf16_mfma_tflops_from_cus_and_clock")
    out = {
        "metric": ("block-sparse attn effective TFLOP/s (% bf16 MFMA peak); colsum us @Infinity-2B 1024^2"
                   if wl == "block_sparse_25" else f"{wl} effective TFLOP/s"),
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic (seeded N(0,1)*%.1f, random-init, no checkpoint)" % amp,
        "config": config,
        "roofline": {"bound": "mfma", "kernel": kernel, "achieved": round(tflops, 2), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / PEAK_BF16_TFLOPS, 4), "traffic": traffic, "traffic_source": traffic_src,
                     "peak_runtime": peak_rt, "frac_runtime": (round(tflops / peak_rt, 4) if peak_rt else None),
                     "flops_per_launch": flops, "host_wall_ms_per_step": round(wall_ms, 5),
                     "single_launch": single, "cache_state": "warm: back-to-back launches on the same inputs, no L2 flush",
                     "settle_ms": SETTLE_MS, "sustained_mfma": probe,
                     "frac_of_sustained_random": (round(tflops / probe["random_operands_tflops"], 4) if probe else None)},
        "cpu_baseline": cpu,
        "device": torch.cuda.get_device_name(0), "device_summary": dev_sum,
    }
    if aux:
        out["aux"] = aux
    print(json.dumps(out))


if __name__ == "__main__":
    main()
