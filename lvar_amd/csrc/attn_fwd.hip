// Flash-attention forward for gfx950 over a list of 64-key tiles: dense, block-list
// (flex BlockMask layout) and token-list (column-sparse, gathered keys) variants.
//
// Work decomposition
//   workgroup  = NWAVES waves, 32 query rows per wave, all waves share one K/V tile in LDS
//   wave       = S^T[64 keys x 32 queries] = K_tile . Q^T with 32x32x16 bf16 MFMA (K rows are
//                the A operand read from LDS, Q^T is the B operand held in registers), so a
//                lane owns ONE query column: the softmax row max / sum are in-register
//                reductions plus one exchange with lane^32.
//                O^T[d x 32 queries] += V^T . P^T: the S^T accumulators, packed to bf16, are
//                already in B-operand layout; V^T comes from a row-major V tile through
//                transposing LDS reads (ds_read_b64_tr_b16).
//   pipeline   = K/V tile t+1 is fetched global->registers while tile t is computed, then
//                stored to the other LDS stage; one barrier per tile.
// Softmax runs in the exp2 domain with a lazily updated reference maximum: accumulators are
// rescaled only when some row maximum grows by more than RESCALE_TAU, which is exact
// because numerator and denominator share the same reference.
#include "common.h"
#include "launch.h"

namespace lvar {

static constexpr float RESCALE_TAU = 8.0f;
static constexpr float NEG_BIG = -1.0e30f;

template <int D, int NWAVES, int MODE, bool ACCUM, bool LSE_ONLY>
__global__ __launch_bounds__(NWAVES * 64, (NWAVES <= 4 ? 2 : 1)) void attn_fwd_kernel(const AttnParams p) {
  constexpr int NT = NWAVES * 64, WGROWS = NWAVES * 32;
  constexpr int KS = D / 16, MTD = D / 32, CPR = D / 8;
  constexpr int KSTR = D * 2 + 16, VSTR = D * 2 + 64;
  constexpr int CHUNKS = 64 * CPR, CPT = (CHUNKS + NT - 1) / NT;
  constexpr bool EXACT = (CHUNKS % NT) == 0;
  constexpr int STAGE = 64 * (KSTR + VSTR);
  constexpr int OSTR = D * 2 + 16;  // epilogue transpose buffer row stride (bytes)
  static_assert(NWAVES * 32 * OSTR <= 2 * STAGE, "epilogue buffer must fit in the K/V stages");
  extern __shared__ __attribute__((aligned(16))) char smem[];

  // Consecutive workgroup ids are dealt round-robin to the 8 XCDs; remap so that each XCD
  // walks a contiguous range of (batch, head, q-tile) and K/V of one head stay in its L2.
  const int per_xcd = gridDim.x >> 3;
  const int w = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (w >= p.total_wg) return;
  const int bh = w / p.nqt, qt = w - bh * p.nqt;
  const int b = bh / p.H, h = bh - b * p.H;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int hh = lane >> 5, r = lane & 31;
  const int q0 = qt * WGROWS;
  const int g = q0 / p.group_rows;

  const int32_t* list = nullptr;
  int T, count = 0;
  if (MODE == MODE_DENSE) {
    T = (p.Lk + 63) >> 6;
  } else {
    count = max(0, min(p.cnt[b * p.cnt_sb + h * p.cnt_sh + g], p.list_len));
    list = p.list + b * p.list_sb + h * p.list_sh + (int64_t)g * p.list_sg;
    T = (MODE == MODE_BLOCK) ? (count << p.sub_shift) : ((count + 63) >> 6);
  }

  const bf16_t* kbase = p.k + b * p.k_sb + h * p.k_sh;
  const bf16_t* vbase = p.v + b * p.v_sb + h * p.v_sh;

  // per-thread chunk coordinates inside a tile
  int crow[CPT], ccol[CPT];
#pragma unroll
  for (int i = 0; i < CPT; i++) {
    int c = tid + i * NT;
    crow[i] = c / CPR;
    ccol[i] = c - crow[i] * CPR;
  }

  auto fetch_rows = [&](int t, int (&rows)[CPT], int& nvalid) {
    if (MODE == MODE_DENSE) {
      int base = t << 6;
      nvalid = min(64, p.Lk - base);
#pragma unroll
      for (int i = 0; i < CPT; i++) rows[i] = min(base + crow[i], p.Lk - 1);
    } else if (MODE == MODE_BLOCK) {
      int blk = list[t >> p.sub_shift];
      int base = ((blk << p.sub_shift) + (t & ((1 << p.sub_shift) - 1))) << 6;
      nvalid = max(0, min(64, p.Lk - base));
#pragma unroll
      for (int i = 0; i < CPT; i++) rows[i] = max(0, min(base + crow[i], p.Lk - 1));
    } else {
      int base = t << 6;
      nvalid = min(64, count - base);
#pragma unroll
      for (int i = 0; i < CPT; i++) {
        int pos = base + crow[i];
        int idx = (pos < count && (EXACT || crow[i] < 64)) ? list[pos] : 0;
        rows[i] = max(0, min(idx, p.Lk - 1));
      }
    }
  };

  u32x4 kreg[CPT], vreg[CPT];
  auto load_tile = [&](const int (&rows)[CPT]) {
#pragma unroll
    for (int i = 0; i < CPT; i++) {
      if (EXACT || tid + i * NT < CHUNKS) {
        kreg[i] = *(const u32x4*)(kbase + (int64_t)rows[i] * p.k_sr + ccol[i] * 8);
        if (!LSE_ONLY) vreg[i] = *(const u32x4*)(vbase + (int64_t)rows[i] * p.v_sr + ccol[i] * 8);
      }
    }
  };
  auto store_tile = [&](int stage) {
    char* ks = smem + stage * STAGE;
    char* vs = ks + 64 * KSTR;
#pragma unroll
    for (int i = 0; i < CPT; i++) {
      if (EXACT || tid + i * NT < CHUNKS) {
        *(u32x4*)(ks + crow[i] * KSTR + ccol[i] * 16) = kreg[i];
        if (!LSE_ONLY) *(u32x4*)(vs + crow[i] * VSTR + ccol[i] * 16) = vreg[i];
      }
    }
  };

  // accumulators and softmax state (one query column per lane pair l, l^32)
  f32x16 oacc[MTD];
#pragma unroll
  for (int m = 0; m < MTD; m++)
#pragma unroll
    for (int i = 0; i < 16; i++) oacc[m][i] = 0.f;
  float m_ref = NEG_BIG, m_true = -INFINITY, lsum = 0.f;
  const float c = p.c;

  if (T > 0) {
    // Q^T fragments stay in registers for the whole key loop
    const int qrow = min(q0 + wave * 32 + r, p.Lq - 1);
    const bf16_t* qp = p.q + b * p.q_sb + h * p.q_sh + (int64_t)qrow * p.q_sr + hh * 8;
    bf16x8 qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = *(const bf16x8*)(qp + ks * 16);

    int rows_next[CPT], nv_cur, nv_next = 0;
    {
      int rows0[CPT];
      fetch_rows(0, rows0, nv_cur);
      load_tile(rows0);
      if (T > 1) fetch_rows(1, rows_next, nv_next);
      store_tile(0);
    }
    __syncthreads();

    for (int t = 0; t < T; t++) {
      const int stage = t & 1;
      if (t + 1 < T) load_tile(rows_next);
      int nv_next2 = 0;
      if (t + 2 < T) fetch_rows(t + 2, rows_next, nv_next2);

      // ---- S^T = K_tile . Q^T ----
      f32x16 s0, s1;
#pragma unroll
      for (int i = 0; i < 16; i++) { s0[i] = 0.f; s1[i] = 0.f; }
      const char* kl = smem + stage * STAGE + r * KSTR + hh * 16;
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        bf16x8 a0 = *(const bf16x8*)(kl + ks * 32);
        bf16x8 a1 = *(const bf16x8*)(kl + 32 * KSTR + ks * 32);
        s0 = mfma32(a0, qf[ks], s0);
        s1 = mfma32(a1, qf[ks], s1);
      }
      if (nv_cur < 64) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
          int kr = 8 * (i >> 2) + 4 * hh + (i & 3);
          if (kr >= nv_cur) s0[i] = -INFINITY;
          if (kr + 32 >= nv_cur) s1[i] = -INFINITY;
        }
      }
      // ---- online softmax (base 2) ----
      float mx = fmaxf(s0[0], s1[0]);
#pragma unroll
      for (int i = 1; i < 16; i++) mx = fmaxf(mx, fmaxf(s0[i], s1[i]));
      mx = xhalf_max(mx);
      const float mt = mx * c;
      m_true = fmaxf(m_true, mt);
      if (__builtin_amdgcn_ballot_w64(mt > m_ref + RESCALE_TAU) != 0) {
        const float m_new = fmaxf(m_ref, mt);
        const float alpha = fast_exp2(m_ref - m_new);
        lsum *= alpha;
        if (!LSE_ONLY) {
#pragma unroll
          for (int m = 0; m < MTD; m++)
#pragma unroll
            for (int i = 0; i < 16; i++) oacc[m][i] *= alpha;
        }
        m_ref = m_new;
      }
      const float negm = -m_ref;
#pragma unroll
      for (int i = 0; i < 16; i++) {
        s0[i] = fast_exp2(fmaf(s0[i], c, negm));
        s1[i] = fast_exp2(fmaf(s1[i], c, negm));
        lsum += s0[i] + s1[i];
      }
      if (!LSE_ONLY) {
        // ---- O^T += V^T . P^T ----
        bf16x8 pb[4];
        pb[0] = pack8(s0[0], s0[1], s0[2], s0[3], s0[4], s0[5], s0[6], s0[7]);
        pb[1] = pack8(s0[8], s0[9], s0[10], s0[11], s0[12], s0[13], s0[14], s0[15]);
        pb[2] = pack8(s1[0], s1[1], s1[2], s1[3], s1[4], s1[5], s1[6], s1[7]);
        pb[3] = pack8(s1[8], s1[9], s1[10], s1[11], s1[12], s1[13], s1[14], s1[15]);
        const char* vl = smem + stage * STAGE + 64 * KSTR + (((lane & 15) >> 2) + 4 * hh) * VSTR +
                         ((lane >> 4) & 1) * 32 + (lane & 3) * 8;
#pragma unroll
        for (int kb = 0; kb < 4; kb++) {
#pragma unroll
          for (int m = 0; m < MTD; m++) {
            bf16x4 lo = lds_read_tr(vl + (kb * 16) * VSTR + m * 64);
            bf16x4 hi = lds_read_tr(vl + (kb * 16 + 8) * VSTR + m * 64);
            bf16x8 a = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            oacc[m] = mfma32(a, pb[kb], oacc[m]);
          }
        }
      }
      if (t + 1 < T) store_tile(stage ^ 1);
      nv_cur = nv_next;
      nv_next = nv_next2;
      __syncthreads();
    }
  }

  // ---- epilogue ----
  const float ltot = xhalf_sum(lsum);
  const bool empty = !(ltot > 0.f);
  const float inv = empty ? 0.f : 1.0f / ltot;
  const int qrow_w = q0 + wave * 32 + r;
  if (hh == 0 && qrow_w < p.Lq) {
    const int64_t off = ((int64_t)b * p.H + h) * p.Lq + qrow_w;
    if (p.M) p.M[off] = empty ? -INFINITY : m_true;
    if (p.L) p.L[off] = empty ? 1.0f : ltot * fast_exp2(m_ref - m_true);
  }
  if (LSE_ONLY) return;

  const float osc = ACCUM ? p.o_scale * inv : inv;
  char* ob = smem + wave * (32 * OSTR);
  const bf16_t* oap = nullptr;
  if (ACCUM && p.o_accum)
    oap = p.o_accum + b * p.oa_sb + h * p.oa_sh + (int64_t)min(qrow_w, p.Lq - 1) * p.oa_sr;
#pragma unroll
  for (int m = 0; m < MTD; m++) {
#pragma unroll
    for (int a = 0; a < 4; a++) {
      const int dcol = m * 32 + 8 * a + 4 * hh;
      float x0 = oacc[m][4 * a + 0] * osc, x1 = oacc[m][4 * a + 1] * osc;
      float x2 = oacc[m][4 * a + 2] * osc, x3 = oacc[m][4 * a + 3] * osc;
      if (ACCUM && oap) {
        u32x2 acc = *(const u32x2*)(oap + dcol);
        x0 += bf16_lo(acc[0]); x1 += bf16_hi(acc[0]);
        x2 += bf16_lo(acc[1]); x3 += bf16_hi(acc[1]);
      }
      u32x2 pk = {pack_bf16(x0, x1), pack_bf16(x2, x3)};
      *(u32x2*)(ob + r * OSTR + dcol * 2) = pk;
    }
  }
  // each wave re-reads only its own 32 rows: a wave-local fence is enough
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
  __builtin_amdgcn_wave_barrier();
  bf16_t* op = p.o + b * p.o_sb + h * p.o_sh;
#pragma unroll
  for (int i = 0; i < (32 * CPR) / 64; i++) {
    const int cidx = lane + i * 64;
    const int orow = cidx / CPR, ocol = cidx - orow * CPR;
    const int grow = q0 + wave * 32 + orow;
    if (grow < p.Lq) {
      u32x4 val = *(const u32x4*)(ob + orow * OSTR + ocol * 16);
      *(u32x4*)(op + (int64_t)grow * p.o_sr + ocol * 8) = val;
    }
  }
}

template <int D, int NWAVES, int MODE, bool ACCUM, bool LSE_ONLY>
static int launch_one(const AttnParams& p0, hipStream_t stream) {
  AttnParams p = p0;
  constexpr int WGROWS = NWAVES * 32;
  constexpr int STAGE = 64 * ((D * 2 + 16) + (D * 2 + 64));
  if (p.group_rows % WGROWS != 0 && MODE != MODE_DENSE) return LVAR_EINVAL;
  if (MODE == MODE_DENSE) p.group_rows = WGROWS;
  p.nqt = (p.Lq + WGROWS - 1) / WGROWS;
  p.total_wg = p.B * p.H * p.nqt;
  const int grid = ((p.total_wg + 7) / 8) * 8;
  auto kern = attn_fwd_kernel<D, NWAVES, MODE, ACCUM, LSE_ONLY>;
  static bool attr_set = false;
  const int smem = 2 * STAGE;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem) != hipSuccess)
      return LVAR_ELAUNCH;
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(NWAVES * 64), smem, stream, p);
  return hipGetLastError() == hipSuccess ? LVAR_OK : LVAR_ELAUNCH;
}

template <int D>
static int launch_d(const AttnParams& p, int mode, bool accum, bool lse_only, int nwaves, hipStream_t s) {
  if (mode == MODE_DENSE) {
    return lse_only ? launch_one<D, 4, MODE_DENSE, false, true>(p, s) : launch_one<D, 4, MODE_DENSE, false, false>(p, s);
  } else if (mode == MODE_BLOCK) {
    return launch_one<D, 4, MODE_BLOCK, false, false>(p, s);
  } else {
    if (nwaves == 6) return launch_one<D, 6, MODE_GATHER, true, false>(p, s);
    if (nwaves == 3) return launch_one<D, 3, MODE_GATHER, true, false>(p, s);
    if (nwaves == 2) return launch_one<D, 2, MODE_GATHER, true, false>(p, s);
    return LVAR_EUNSUPPORTED;
  }
}

int launch_attn(const AttnParams& p, int head_dim, int mode, bool accum, bool lse_only, int nwaves, hipStream_t s) {
  if (head_dim == 128) return launch_d<128>(p, mode, accum, lse_only, nwaves, s);
  if (head_dim == 64) return launch_d<64>(p, mode, accum, lse_only, nwaves, s);
  return LVAR_EUNSUPPORTED;
}

}  // namespace lvar
