// Colsum kernel for gfx950: cs[b,h,g,n] = sum over the query rows i of group g of
// exp2(q_i.k_n*scale*log2e - lse2_i), with lse2 = M + log2(L) the base-2 log-sum-exp of row i.
//
// Key-stationary decomposition: a wave keeps one 64-key block (the B operand, K^T) in registers
// for the whole sweep over Lq; the workgroup (4 waves = 256 keys) streams 64-row Q stages and their
// lse2 through a 4-deep LDS ring filled by global->LDS DMA three stages ahead.  In the 32x32
// accumulator a lane owns ONE key column and 16 query rows, so the reduction over queries is an
// in-register add, one exchange with lane^32 at each group boundary and a single plain store per
// (group, key): no atomics, no partial buffers, and a summation order fixed by the shapes alone.
// The per-64-key block sums fall out of the same registers (one wave = one key block).
//
// Inner loop, software-pipelined by hand: while the matrix cores compute S(u) = Q_tile(u) K^T for
// 32-row tile u (16 MFMA for d = 128), the vector ALU turns S(u-1) into probabilities and adds them
// to the column accumulators.
#include <type_traits>
#include "common.h"
#include "launch.h"

namespace lvar {

template <int D>
__global__ __launch_bounds__(256, (D <= 128 ? 2 : 1)) void colsum_kernel(const ColsumParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int KS = D / 16;
  constexpr int ROWB = D * 2, CPR = ROWB / 16;
  constexpr int RPI = 1024 / ROWB, NI = 64 / RPI, SLOTS = NI / 4;
  constexpr int SWD = ROWB >= 256 ? 1 : 256 / ROWB;   // chunk swizzle of row t: (t / SWD) & SWM, 16 rows per period
  constexpr int SWM = ROWB >= 256 ? 15 : CPR - 1;
  constexpr int QTILE = 64 * ROWB;         // one 64-row Q stage
  constexpr int NSTAGE = 4, NLSE = 8;      // ring depths
  constexpr int LSE_OFF = NSTAGE * QTILE;  // lse2 ring: NLSE x 64 floats
  extern __shared__ __attribute__((aligned(1024))) char smem[];  // NSTAGE * QTILE + NLSE * 256 bytes

  const int per_xcd = gridDim.x >> 3;
  const int w = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (w >= p.total_wg) return;
  // workgroup = (batch*head, key tile of 256 keys, range of query groups): the query axis is cut at group
  // boundaries when the plain grid would fill the chip unevenly; every range writes its own groups of cs
  const int per_bh = p.nkt * p.q_splits;
  const int bh = w / per_bh, rem = w - bh * per_bh;
  const int kt = rem / p.q_splits, sp = rem - kt * p.q_splits;
  const int b = bh / p.H, h = bh - b * p.H;
  const int qoff = __builtin_amdgcn_readfirstlane(sp * p.split_rows);   // first query row of this range (a multiple of 64 and of group_rows)
  const int Lq_l = min(p.Lq, qoff + p.split_rows) - qoff;   // rows of this range
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int hh = lane >> 5, r = lane & 31;
  const int kblk = kt * 4 + wave;  // 64-key block owned by this wave
  const int n0 = kblk * 64;
  const float c = p.c;

  // stationary K^T fragments: lane holds key column n0 + nt*32 + r, d = ks*16 + 8*hh .. +7
  const bf16_t* kbase = p.k + b * p.k_sb + (h / p.kv_group) * p.k_sh;   // grouped-query attention: shared key heads
  bf16x8 kf[2][KS];
#pragma unroll
  for (int nt = 0; nt < 2; nt++) {
    const int krow = min(n0 + nt * 32 + r, p.Lk - 1);
    const bf16_t* kp = kbase + (int64_t)krow * p.k_sr + hh * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) kf[nt][ks] = *(const bf16x8*)(kp + ks * 16);
  }

  auto make_rsrc = [](const void* base) -> i32x4 {
    const uint64_t a = (uint64_t)base;
    i32x4 rs = {__builtin_amdgcn_readfirstlane((int)(uint32_t)a),
                __builtin_amdgcn_readfirstlane((int)(uint32_t)((a >> 32) & 0xffffu)), 0x7fffffff, 0x00020000};
    return rs;
  };
  const i32x4 qrsrc = make_rsrc(p.q + b * p.q_sb + h * p.q_sh);
  const i32x4 lrsrc = make_rsrc(p.lse2 + ((int64_t)b * p.H + h) * p.Lq);
  const int q_srb = (int)p.q_sr * 2;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(LVAR_LDS char*)smem;
  const int lrow = lane / CPR, lcs = lane % CPR;

  // global->LDS fill of stage s (Q rows s*64 .. +63, clamped to Lq-1, chunk-swizzled; lse2 by wave 0)
  // lane offset of a Q fill: row within the first instruction(s) of this wave, swizzled chunk.  The swizzle
  // repeats every 16 rows and instruction i = wave + 4 * slot covers rows i * RPI ..: slots a whole period apart
  // share the lane offset (PER = 1: all of them; head_dim 256 has two rows per instruction and PER = 2).
  constexpr int PER = (4 * RPI >= 16) ? 1 : 16 / (4 * RPI);
  static_assert((PER * 4 * RPI) % 16 == 0 && SLOTS % PER == 0, "slots PER apart must be whole swizzle periods apart");
  int fill_voff[PER];
#pragma unroll
  for (int ph = 0; ph < PER; ph++) {
    const int trow = (wave + 4 * ph) * RPI + lrow;
    fill_voff[ph] = trow * q_srb + ((lcs ^ ((trow / SWD) & SWM)) << 4);
  }
  auto issue_stage = [&](int s) {
    const uint32_t dst = lds0 + (s & (NSTAGE - 1)) * QTILE;
    if (s * 64 + 64 <= Lq_l) {
      // all 64 rows exist: constant lane offset, stage and slot move the scalar offset
#pragma unroll
      for (int sl = 0; sl < SLOTS; sl++) {
        const int i = wave + sl * 4;
        const int soff = (qoff + s * 64 + (sl / PER) * PER * 4 * RPI) * q_srb;
        const uint32_t m0v = dst + i * 1024;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" : : "s"(m0v), "v"(fill_voff[sl % PER]), "s"(qrsrc), "s"(soff) : "memory");
      }
    } else {
#pragma unroll
      for (int sl = 0; sl < SLOTS; sl++) {
        const int i = wave + sl * 4;
        const int trow = i * RPI + lrow;
        const int grow = min(qoff + s * 64 + trow, p.Lq - 1);
        const int voff = grow * q_srb + ((lcs ^ ((trow / SWD) & SWM)) << 4);
        const uint32_t m0v = dst + i * 1024;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" : : "s"(m0v), "v"(voff), "s"(qrsrc) : "memory");
      }
    }
    if (wave == 0) {
      const int voff = min(qoff + s * 64 + lane, p.Lq - 1) * 4;
      const uint32_t m0v = lds0 + LSE_OFF + (s & (NLSE - 1)) * 256;
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds" : : "s"(m0v), "v"(voff), "s"(lrsrc) : "memory");
    }
  };
  // wait until at most `younger` later stages of this wave's fills are still in flight
  // (s_waitcnt immediate: vmcnt is split into bits 3:0 and 15:14; expcnt and lgkmcnt stay at "don't wait")
  constexpr auto vm = [](int n) constexpr { return 0x0f70 | (n & 15) | (((n >> 4) & 3) << 14); };
  auto wait_fills = [&](int younger) {
    if (younger >= 2) {
      if (wave == 0) __builtin_amdgcn_s_waitcnt(vm(2 * (SLOTS + 1))); else __builtin_amdgcn_s_waitcnt(vm(2 * SLOTS));
    } else if (younger == 1) {
      if (wave == 0) __builtin_amdgcn_s_waitcnt(vm(SLOTS + 1)); else __builtin_amdgcn_s_waitcnt(vm(SLOTS));
    } else {
      __builtin_amdgcn_s_waitcnt(0x0f70);
    }
  };

  float* csp = p.cs + ((int64_t)b * p.H + h) * p.G * (int64_t)p.Lk;
  float* bsp = p.bs ? p.bs + ((int64_t)b * p.H + h) * p.G * (int64_t)p.nkb : nullptr;
  // store the finished column sums of group g and reset the accumulators
  auto flush = [&](int g, float (&acc)[2]) {
    float blk = 0.f;
#pragma unroll
    for (int nt = 0; nt < 2; nt++) {
      const float tot = xhalf_sum(acc[nt]);
      const int key = n0 + nt * 32 + r;
      const bool ok = key < p.Lk;
      if (hh == 0 && ok) csp[(int64_t)g * p.Lk + key] = tot;
      blk += ok ? tot : 0.f;
      acc[nt] = 0.f;
    }
    if (bsp) {
      blk = group_sum<32>(blk);
      if (lane == 0 && n0 < p.Lk) bsp[(int64_t)g * p.nkb + kblk] = blk;
    }
  };

  const int S = (Lq_l + 63) >> 6;          // stages of this range
  const int U = (Lq_l + 31) >> 5;          // 32-row tiles
  const int kbase_l = r * ROWB + ((hh ^ ((r / SWD) & SWM)) << 4);
  float acc[2] = {0.f, 0.f};

  // probabilities of tile u from its logits: p = exp2(s*c - lse2[row]); rows >= Lq add nothing
  auto exp_acc = [&](int u, const f32x16& s0, const f32x16& s1) {
    const char* ll = smem + LSE_OFF + ((u >> 1) & (NLSE - 1)) * 256 + ((u & 1) * 32 + 4 * hh) * 4;
    f32x4 lse[4];
#pragma unroll
    for (int j = 0; j < 4; j++) lse[j] = *(const f32x4*)(ll + j * 32);
    const bool ragged = (u * 32 + 32 > Lq_l);
    const int lim = Lq_l - u * 32 - 4 * hh;
    float pa = 0.f, pb = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) {
      float x0 = fast_exp2(fmaf(s0[i], c, -lse[i >> 2][i & 3]));
      float x1 = fast_exp2(fmaf(s1[i], c, -lse[i >> 2][i & 3]));
      if (ragged) {
        const bool ok = (8 * (i >> 2) + (i & 3)) < lim;
        x0 = ok ? x0 : 0.f;
        x1 = ok ? x1 : 0.f;
      }
      pa += x0;
      pb += x1;
    }
    acc[0] += pa;
    acc[1] += pb;
    const int qend = u * 32 + 32;
    if (qend % p.group_rows == 0 || qend >= Lq_l) flush((qoff + u * 32) / p.group_rows, acc);
  };

  // prologue: up to three stages in flight
  issue_stage(0);
  if (S > 1) issue_stage(1);
  if (S > 2) issue_stage(2);
  __builtin_amdgcn_s_waitcnt(0x0f70);
  __syncthreads();

  // One pipelined step: S(u) -> (n0, n1) on the matrix cores, probabilities of tile u-1 from (c0, c1)
  // on the vector ALU, interleaved by hand (sched_barrier(0) pins each group).
  auto step = [&](int u, f32x16& n0a, f32x16& n1a, const f32x16& c0, const f32x16& c1, bool have_prev) {
    const char* qb = smem + ((u >> 1) & (NSTAGE - 1)) * QTILE + (u & 1) * 32 * ROWB;
    constexpr int AHEAD = 3;
    bf16x8 frag[KS];
    const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};   // constant addend of the first MFMA
#pragma unroll
    for (int j = 0; j < AHEAD && j < KS; j++) frag[j] = *(const bf16x8*)(qb + (kbase_l ^ (j << 5)));
    if (have_prev) {
      const int up = u - 1;
      const char* ll = smem + LSE_OFF + ((up >> 1) & (NLSE - 1)) * 256 + ((up & 1) * 32 + 4 * hh) * 4;
      f32x4 lse[4];
#pragma unroll
      for (int j = 0; j < 4; j++) lse[j] = *(const f32x4*)(ll + j * 32);
      float pa = 0.f, pb = 0.f;
      // probabilities of tile u-1 as a three-stage pipeline over the MFMA steps (scale | exp2 | add), 16 / KS
      // accumulator indices of both key tiles per step, so that no vector instruction waits for the last one
      constexpr int EPS = 16 / KS;
      float xs0[16], xs1[16];
      auto st_scale = [&](int g) {
#pragma unroll
        for (int e = 0; e < EPS; e++) {
          const int i = g * EPS + e;
          xs0[i] = fmaf(c0[i], c, -lse[i >> 2][i & 3]);
          xs1[i] = fmaf(c1[i], c, -lse[i >> 2][i & 3]);
        }
      };
      auto st_exp = [&](int g) {
#pragma unroll
        for (int e = 0; e < EPS; e++) {
          const int i = g * EPS + e;
          xs0[i] = fast_exp2(xs0[i]);
          xs1[i] = fast_exp2(xs1[i]);
        }
      };
      auto st_add = [&](int g) {
#pragma unroll
        for (int e = 0; e < EPS; e++) {
          const int i = g * EPS + e;
          pa += xs0[i];
          pb += xs1[i];
        }
      };
      st_scale(0);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        if (ks + AHEAD < KS) frag[ks + AHEAD] = *(const bf16x8*)(qb + (kbase_l ^ ((ks + AHEAD) << 5)));
        n0a = mfma32(frag[ks], kf[0][ks], ks == 0 ? zero : n0a);
        n1a = mfma32(frag[ks], kf[1][ks], ks == 0 ? zero : n1a);
        if (ks >= 1) st_add(ks - 1);
        st_exp(ks);
        if (ks + 1 < KS) st_scale(ks + 1);
        __builtin_amdgcn_sched_barrier(0);
      }
      st_add(KS - 1);
      acc[0] += pa;
      acc[1] += pb;
      const int qend = up * 32 + 32;
      if (qend % p.group_rows == 0) flush((qoff + up * 32) / p.group_rows, acc);
    } else {
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        if (ks + AHEAD < KS) frag[ks + AHEAD] = *(const bf16x8*)(qb + (kbase_l ^ ((ks + AHEAD) << 5)));
        n0a = mfma32(frag[ks], kf[0][ks], ks == 0 ? zero : n0a);
        n1a = mfma32(frag[ks], kf[1][ks], ks == 0 ? zero : n1a);
      }
    }
  };

  // Tiles 0 .. U-2 go through the pipelined step (their successor exists); every tile whose rows are
  // all valid is consumed inside the next step, the last tile (possibly ragged) by exp_acc below.
  f32x16 sa0, sa1, sb0, sb1;
  for (int s = 0; s < S; s++) {
    if (s + 3 < S) issue_stage(s + 3);
    const int u0 = 2 * s;
    step(u0, sa0, sa1, sb0, sb1, u0 > 0);
    if (u0 + 1 < U) step(u0 + 1, sb0, sb1, sa0, sa1, true);
    wait_fills(min(s + 3, S - 1) - (s + 1));
    __syncthreads();
  }
  // last tile U-1: in (sb) if U is even, else in (sa)
  if (U & 1) exp_acc(U - 1, sa0, sa1); else exp_acc(U - 1, sb0, sb1);
#endif  // __HIP_DEVICE_COMPILE__
}

template <int D>
static int launch_cs(const ColsumParams& p0, hipStream_t stream) {
  ColsumParams p = p0;
  if (p.kv_group < 1) p.kv_group = 1;
  p.nkb = (p.Lk + 63) / 64;
  p.nkt = (p.Lk + 255) / 256;
  // Ranges of query groups per key tile.  Workgroups are handed to the resident slots (two per compute unit) as slots
  // fall free, so a launch takes about its total work spread over the slots plus a part of the longest workgroup, during
  // which the chip drains.  More, shorter ranges shorten that tail and pay the fixed cost of a workgroup more often.
  // In 64-row stages, fitted to launches of 0.06 .. 0.37 ms on 256 compute units:
  //   cost = workgroups x (stages of a range + 1.5) / slots  +  0.4 x (stages of the longest range + 1.5)
  const int unit = (p.group_rows % 64 == 0) ? p.group_rows : (p.group_rows % 32 == 0 ? 2 * p.group_rows : 0);   // lcm(group_rows, 64)
  p.q_splits = 1;
  p.split_rows = ((p.Lq + 63) / 64) * 64 + (unit > 0 ? unit : 64);   // one range covers everything
  const int base_wg = p.B * p.H * p.nkt, slots = 2 * device_cus();
  if (unit > 0 && slots > 0 && base_wg < 4 * slots) {   // longer launches: the tail is small whatever the cut
    const int units_total = (p.Lq + unit - 1) / unit;
    double best = -1.0;
    for (int s = 1; s <= 8 && s <= units_total; s++) {
      const int rows = ((units_total + s - 1) / s) * unit;          // rows per range
      const int n = (p.Lq + rows - 1) / rows;                       // ranges that hold rows
      const int st_long = (std::min(rows, p.Lq) + 63) / 64, st_last = (p.Lq - (n - 1) * rows + 63) / 64;
      const double work = (double)base_wg * ((n - 1) * (st_long + 1.5) + (st_last + 1.5)) / slots;
      const double cost = work + 0.4 * (st_long + 1.5);
      if (best < 0.0 || cost < best) { best = cost; p.q_splits = n; p.split_rows = rows; }
    }
  }
  p.total_wg = base_wg * p.q_splits;
  const int grid = ((p.total_wg + 7) / 8) * 8;
  constexpr int SMEM = 4 * 64 * D * 2 + 8 * 256;
  static std::atomic<uint64_t> lds_ready{0};
  if (!ensure_lds_limit((const void*)colsum_kernel<D>, SMEM, lds_ready)) return LVAR_ELAUNCH;
  hipLaunchKernelGGL((colsum_kernel<D>), dim3(grid), dim3(256), SMEM, stream, p);
  return hipGetLastError() == hipSuccess ? LVAR_OK : LVAR_ELAUNCH;
}

int launch_colsum(const ColsumParams& p, int head_dim, hipStream_t s) {
  if (head_dim == 128) return launch_cs<128>(p, s);
  if (head_dim == 64) return launch_cs<64>(p, s);
  if (head_dim == 256) return launch_cs<256>(p, s);
  return LVAR_EUNSUPPORTED;
}

}  // namespace lvar
