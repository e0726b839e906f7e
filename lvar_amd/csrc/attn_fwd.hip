// Flash-attention forward for gfx950 over a list of 64-key tiles: dense, block-list
// (flex BlockMask layout) and token-list (column-sparse, gathered keys) variants.
//
// Work decomposition
//   workgroup  = NWAVES waves, 32 query rows per wave, all waves share the K/V tiles in LDS
//                (token lists with 192-row groups: 8 waves = 6 computing waves + 2 waves that only fetch, see NPROD)
//   wave       = S^T[64 keys x 32 queries] = K_tile . Q^T with 32x32x16 bf16 MFMA (K rows are
//                the A operand read from LDS, Q^T is the B operand held in registers), so a
//                lane owns ONE query column: the softmax row max / sum are in-register
//                reductions plus one exchange with lane^32.
//                O^T[d x 32 queries] += V^T . P^T: the S^T accumulators, packed to bf16, are
//                already in B-operand layout; V^T comes from the row-major V tile through
//                transposing LDS reads (ds_read_b64_tr_b16).
//   data path  = K/V rows go global -> LDS directly (buffer_load ... lds, 16 B per lane, no
//                register staging).  An instruction fills 1 KiB of consecutive LDS, so rows are
//                unpadded; bank conflicts are avoided by an XOR swizzle of the 16-byte chunk index
//                applied on the global side (each lane fetches the chunk that belongs in its slot).
//   pipeline   = iteration t issues the loads of K(t+2) and V(t+1); the matrix cores run
//                S(t+1) = K(t+1) Q^T and then O += P(t) V(t) while the vector ALU computes
//                P(t) = exp2(S(t)) and then the row maximum of S(t+1).  K and V are double-buffered,
//                one barrier per tile.
// Softmax runs in the exp2 domain with a lazily updated reference maximum: accumulators are
// rescaled only when some row maximum grows by more than RESCALE_TAU, which is exact
// because numerator and denominator share the same reference.
#include <type_traits>
#include "common.h"
#include "launch.h"
#include "sk_partition.h"

namespace lvar {

constexpr int READ_AHEAD = 4;    // operand fragments requested from LDS this many MFMAs before their use
constexpr int EXP_IN_QK = 24;    // of the 32 exp2 per lane and tile, how many run next to the QK MFMAs

// First S element of softmax slot g: EA elements spread over the NQK steps of the QK phase, the other
// 32 - EA over the first HB steps of the PV phase; slots before 0 and after the last one are empty.
template <int NQK, int HB, int EA>
struct ExpSlots {
  static constexpr int lo(int g) {
    return g <= 0 ? 0 : g < NQK ? g * EA / NQK : g < NQK + HB ? EA + (g - NQK) * (32 - EA) / (HB ? HB : 1) : 32;
  }
};

// f(integral_constant<int, i>) for i = LO .. HI-1, unrolled at compile time
template <int LO, int HI, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (LO < HI) {
    f(std::integral_constant<int, LO>{});
    static_for<LO + 1, HI>(f);
  }
}
static constexpr float RESCALE_TAU = 8.0f;
static constexpr float NEG_BIG = -1.0e30f;

template <int D>
struct Swz {
  static constexpr int ROWB = D * 2;      // bytes per K/V row
  static constexpr int CPR = ROWB / 16;   // 16-byte chunks per row
  // chunk-index XOR of the K tile: makes ds_read_b128 of 16 consecutive rows conflict-free
  // (rows of 256 bytes or more: the row index itself, 16 rows per period)
  __device__ static __forceinline__ int fk(int row) {
    if constexpr (ROWB >= 256) return row & 15; else return (row / (256 / ROWB)) & (CPR - 1);
  }
  // chunk-index XOR of the V tile: moves the 64-byte segment read by the transposing loads of
  // 4 consecutive rows onto 4 different bank groups
  __device__ static __forceinline__ int fv(int row) { return (D >= 128) ? ((row & 3) << 2) : (((row >> 1) & 1) << 2); }
};

// Context of a balanced launch (see sk_partition.h); unused by the plain launch.
#if defined(__HIP_DEVICE_COMPILE__)
struct SkCtx {
  int slot0;        // workspace slot of piece 0 of this item's query tile
  int pieces;       // pieces of the tile (1 = whole)
  int kp;           // which piece this item is
  int tile_units;   // units of the whole tile
};

// One query tile w (or, in a balanced launch, the units [u0, u1) of its tile list; `whole` = all of them).
template <int D, int NWAVES, int MODE, bool ACCUM, bool LSE_ONLY, bool SK>
__device__ __forceinline__ void attn_item(const AttnParams& p, char* smem, const int w, const int u0, const int u1,
                                          const bool whole, const SkCtx& sk) {
  // Token lists with 8 waves: waves 0..5 compute (one 192-row group), waves 6 and 7 only fetch -- they read
  // the list, form the gather addresses and issue every K/V fill.  One 6-wave group fills 6 of the 8 wave
  // slots of a CU; the two fetch waves take the idle ones and the compute waves lose ~10 % of their
  // instructions.  Everywhere else all waves do both.
  constexpr int NPROD = (MODE == MODE_GATHER && NWAVES == 8) ? 2 : 0;
  constexpr int NCOMP = NWAVES - NPROD;     // computing waves, 32 query rows each
  constexpr int FW = NPROD ? NPROD : NWAVES;  // waves that issue the fills
  constexpr int WGROWS = NCOMP * 32;
  constexpr int KS = D / 16, MTD = D / 32;
  constexpr int ROWB = Swz<D>::ROWB, CPR = Swz<D>::CPR;
  constexpr int RPI = 1024 / ROWB;          // rows filled by one 64-lane x 16 B load
  constexpr int NI = 64 / RPI;              // loads per 64-row tile
  constexpr int SLOTS = (NI + FW - 1) / FW;
  constexpr int TILE = 64 * ROWB;
  // block lists: the rows of a tile are consecutive, so a fill's lane offset can be a constant (see issue_slot)
  constexpr bool CONST_OFF = MODE == MODE_BLOCK && ((FW * RPI) % 16 == 0 || 16 % (FW * RPI) == 0) && NI % FW == 0;
  constexpr int CONST_PER = (FW * RPI) >= 16 ? 1 : 16 / (FW * RPI);
  constexpr int OSTR = D * 2 + 16;  // epilogue transpose buffer row stride (bytes)
  static_assert(NCOMP * 32 * OSTR <= 4 * TILE, "epilogue buffer must fit in the K/V buffers");
  // LDS map: K buffers at 0 and TILE, V buffers at 2*TILE and 3*TILE

  const int bh = w / p.nqt, qt = w - bh * p.nqt;
  const int b = bh / p.H, h = bh - b * p.H;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int hh = lane >> 5, r = lane & 31;
  const int fwave = NPROD ? wave - NCOMP : wave;   // index among the filling waves (negative: this wave does not fill)
  const int q0 = qt * WGROWS;
  const int g = q0 / p.group_rows;

  // Key-tile list of this query group.  Dense attention is the block-list variant with a null
  // list pointer, read as the identity list of ceil(Lk/64) 64-key blocks.
  const bool identity = (MODE == MODE_BLOCK) && p.list == nullptr;
  const int32_t* list = nullptr;
  int T, count;
  int tile0 = 0;   // identity list of a balanced launch: first tile of this piece
  int avail = 0;   // entries of the list row from `list` on (token lists)
  // first four entries of a block list, read together with the count (not after it): one memory
  // round trip less before the first tile can be fetched; entries beyond the count are never used
  int head[4] = {0, 0, 0, 0};
  if (identity) {
    count = (p.Lk + 63) >> 6;
    if (SK) { tile0 = u0; count = max(0, min(u1, count) - u0); }
    T = count;
  } else {
    list = p.list + b * p.list_sb + h * p.list_sh + (int64_t)g * p.list_sg;
    const int first = SK ? (MODE == MODE_BLOCK ? u0 : (u0 << 6)) : 0;   // first list entry of this piece
    if (MODE == MODE_BLOCK) {
#pragma unroll
      for (int i = 0; i < 4; i++)
        if (first + i < p.list_len) head[i] = list[first + i];
    }
    count = max(0, min(p.cnt[b * p.cnt_sb + h * p.cnt_sh + g], p.list_len));
    avail = p.list_len - first;
    if (SK) {
      const int last = (MODE == MODE_BLOCK) ? u1 : (u1 << 6);
      count = max(0, min(count, last) - first);
      list += first;
    }
    T = (MODE == MODE_BLOCK) ? (count << p.sub_shift) : ((count + 63) >> 6);
  }
  const int sub_shift = identity ? 0 : p.sub_shift;

  // accumulators and softmax state (one query column per lane pair l, l^32)
  f32x16 oacc[MTD];
#pragma unroll
  for (int m = 0; m < MTD; m++)
#pragma unroll
    for (int i = 0; i < 16; i++) oacc[m][i] = 0.f;
  float m_ref = NEG_BIG, m_true = -INFINITY, lsum = 0.f;
  const float c = p.c;

  if (T > 0) do {
    // raw buffer descriptors of this (batch, head) slice of K and V: base, stride 0, bound = the bytes of
    // the slice (below 2^31, checked on the host), so a fill beyond the last key row reads zeros
    auto make_rsrc = [](const void* base, int bytes) -> i32x4 {
      const uint64_t a = (uint64_t)base;
      i32x4 rs = {__builtin_amdgcn_readfirstlane((int)(uint32_t)a),
                  __builtin_amdgcn_readfirstlane((int)(uint32_t)((a >> 32) & 0xffffu)),
                  __builtin_amdgcn_readfirstlane(bytes), 0x00020000};
      return rs;
    };
    const int k_srb = (int)p.k_sr * 2, v_srb = (int)p.v_sr * 2;  // row strides in bytes
    const int hkv = h / p.kv_group;   // grouped-query attention: kv_group query heads share a K/V head
    const i32x4 krsrc = make_rsrc(p.k + b * p.k_sb + hkv * p.k_sh, (p.Lk - 1) * k_srb + ROWB);
    const i32x4 vrsrc = make_rsrc(p.v + b * p.v_sb + hkv * p.v_sh, (p.Lk - 1) * v_srb + ROWB);
    const uint32_t lds0 = (uint32_t)(uintptr_t)(LVAR_LDS char*)smem;

    // per-lane role in a tile load: row (within the RPI rows of one instruction) and chunk slot
    const int lrow = lane / CPR, lcs = lane % CPR;

    // Tile addressing is a two-step pipeline so that no list load is consumed in the iteration
    // that issued it: prefetch_raw(t) issues the list reads of tile t, finish_rows(t) turns them
    // (one iteration later) into a tile descriptor: for token lists the NR = SLOTS rows this lane
    // fetches, otherwise (NR = 1) the wave-uniform first row of the tile; plus nvalid = number of
    // leading tile rows that take part in the softmax.
    constexpr int NR = (MODE == MODE_GATHER) ? SLOTS : 1;
    auto prefetch_raw = [&](int t, int (&raw)[NR]) {
      if (MODE == MODE_BLOCK) {
        raw[0] = identity ? t + tile0 : list[t >> sub_shift];
      } else {
        // bounded by the row of the list, not by the count: entries behind the count are never used (they are
        // clamped and masked), and the read then does not have to wait for the count to arrive
#pragma unroll
        for (int s = 0; s < SLOTS; s++) {
          const int trow = (fwave + s * FW) * RPI + lrow;
          const int pos = (t << 6) + trow;
          raw[s] = (pos < avail && trow < 64) ? list[pos] : 0;
        }
      }
    };
    auto finish_rows = [&](int t, const int (&raw)[NR], int (&rows)[NR], int& nvalid) {
      if (MODE == MODE_BLOCK) {
        // a block index outside the key range (a caller's mistake) is clamped before it is scaled
        const int blk = max(0, min(__builtin_amdgcn_readfirstlane(raw[0]), (p.Lk - 1) >> (6 + sub_shift)));
        rows[0] = ((blk << sub_shift) + (t & ((1 << sub_shift) - 1))) << 6;
        nvalid = max(0, min(64, p.Lk - rows[0]));
      } else {
        nvalid = min(64, count - (t << 6));
#pragma unroll
        for (int s = 0; s < NR; s++) rows[s] = max(0, min(raw[s], p.Lk - 1));   // clamped once, used by the K and the V fill
      }
    };
    // Issue the global->LDS loads of one tile (K or V) into the LDS buffer at byte address `dst`.
    // Written as inline assembly so that the compiler does not serialise later LDS reads of the
    // OTHER buffers behind these fills; completion is awaited with vmcnt(0) before the barrier.
    // issue_slot: the s-th of the SLOTS fill instructions this wave contributes to a tile; issue: all of them.
    auto issue_slot = [&](const i32x4& rsrc, int srb, bool is_v, const int (&rows)[NR], uint32_t dst, int s) {
      const int i = fwave + s * FW;
      if (!((NI % FW == 0) || i < NI)) return;
      const uint32_t m0v = dst + i * 1024;
      // Block lists, tile fully inside K/V: the rows of a tile are consecutive, so the per-lane byte
      // offset (row within the first instruction, swizzled chunk: the swizzle does not depend on the
      // slot) is a constant and tile and slot only move a scalar offset.
      // The buffer descriptor ends with the last key row, so the rows of a ragged last tile that lie beyond it read
      // as zeros (they are masked in the softmax); the first row is never negative (finish_rows clamps the block).
      // (The swizzle has a period of 16 rows: slots whose rows are a whole period apart share the lane offset.  When
      // the FW * RPI rows that the filling waves cover per slot are fewer than 16, CONST_PER such offsets alternate.)
      if constexpr (CONST_OFF) {
        const int row0 = __builtin_amdgcn_readfirstlane(rows[0]);  // wave-uniform for block lists
        const int trow0 = (fwave + (s % CONST_PER) * FW) * RPI + lrow;
        const int voff = trow0 * srb + ((lcs ^ (is_v ? Swz<D>::fv(trow0) : Swz<D>::fk(trow0))) << 4);
        const int soff = (row0 + (s / CONST_PER) * CONST_PER * FW * RPI) * srb;
        asm volatile(
            "s_mov_b32 m0, %0\n\t"
            "s_nop 0\n\t"
            "buffer_load_dwordx4 %1, %2, %3 offen lds"
            :
            : "s"(m0v), "v"(voff), "s"(rsrc), "s"(soff)
            : "memory");
        return;
      }
      const int trow = i * RPI + lrow;
      const int chunk = lcs ^ (is_v ? Swz<D>::fv(trow) : Swz<D>::fk(trow));
      int voff;
      if (MODE == MODE_GATHER) {
        // token rows and row strides are below 2^24 (checked on the host): one full-rate 24-bit multiply-add
        voff = (int)(((unsigned)rows[s < NR ? s : 0] & 0xffffffu) * ((unsigned)srb & 0xffffffu) + (unsigned)(chunk * 16));
      } else {
        const int grow = max(0, min(rows[0] + trow, p.Lk - 1));
        voff = grow * srb + chunk * 16;
      }
      asm volatile(
          "s_mov_b32 m0, %0\n\t"
          "s_nop 0\n\t"
          "buffer_load_dwordx4 %1, %2, 0 offen lds"
          :
          : "s"(m0v), "v"(voff), "s"(rsrc)
          : "memory");  // m0 is scratch here: nothing else in this kernel keeps a value in it
    };
    auto issue = [&](const i32x4& rsrc, int srb, bool is_v, const int (&rows)[NR], uint32_t dst) {
#pragma unroll
      for (int s = 0; s < SLOTS; s++) issue_slot(rsrc, srb, is_v, rows, dst, s);
    };

    // valid keys of tile t of a token list (only the last tile can be ragged)
    auto nvalid_gather = [&](int t) { return max(0, min(64, count - (t << 6))); };

    if (NPROD && wave >= NCOMP) {
      // ---- fetch waves: the fill schedule of the loop below and nothing else; one barrier per tile ----
      int rows_v[NR], rows_k[NR], rows_n[NR], raw[NR], rows0[NR];
      int nv_unused;
#pragma unroll
      for (int s = 0; s < NR; s++) { rows_v[s] = 0; rows_k[s] = 0; rows_n[s] = 0; raw[s] = 0; }
      // the list entries of the first four tiles are requested together (one memory round trip, not one per tile)
      int raw0[NR], raw1[NR], raw2[NR];
      prefetch_raw(0, raw0);
      prefetch_raw(1, raw1);
      prefetch_raw(2, raw2);
      prefetch_raw(3, raw);
      finish_rows(0, raw0, rows0, nv_unused);
      finish_rows(1, raw1, rows_v, nv_unused);
      finish_rows(2, raw2, rows_k, nv_unused);
      issue(krsrc, k_srb, false, rows0, lds0);
      issue(vrsrc, v_srb, true, rows0, lds0 + 2 * TILE);
      if (T > 1) issue(krsrc, k_srb, false, rows_v, lds0 + TILE);
      __builtin_amdgcn_s_waitcnt(0x0f70);
      __syncthreads();
      __syncthreads();   // the computing waves have read K(0): its buffer may be refilled
      for (int t = 0; t + 1 < T; t++) {
        const int par = t & 1;
        issue(vrsrc, v_srb, true, rows_v, lds0 + (3 - par) * TILE);
        if (t + 2 < T) issue(krsrc, k_srb, false, rows_k, lds0 + par * TILE);
        if (t + 3 < T) finish_rows(t + 3, raw, rows_n, nv_unused);
        if (t + 4 < T) prefetch_raw(t + 4, raw);
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
#pragma unroll
        for (int s = 0; s < NR; s++) { rows_v[s] = rows_k[s]; rows_k[s] = rows_n[s]; }
      }
      __syncthreads();   // the one after the last tile
      if (SK) break;     // a balanced launch has more barriers to meet below
      return;
    }

    // Q^T fragments stay in registers for the whole key loop
    const int qrow = min(q0 + wave * 32 + r, p.Lq - 1);
    const bf16_t* qp = p.q + b * p.q_sb + h * p.q_sh + (int64_t)qrow * p.q_sr + hh * 8;
    bf16x8 qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = *(const bf16x8*)(qp + ks * 16);

    // per-lane LDS read offsets (swizzled); K: row r (+32), chunk 2*ks+hh; V: see lds_read_tr
    const int kbase_l = r * ROWB + ((hh ^ Swz<D>::fk(r)) << 4);
    const int sq = (lane & 15) >> 2, sm = lane & 3;
    const int vbase_l = (4 * hh + sq) * ROWB + (((Swz<D>::fv(sq)) | (((lane >> 4) & 1) << 1) | (sm >> 1)) << 4) + (sm & 1) * 8;

    // S^T tile = K_tile . Q^T (16 MFMA for d = 128)
    auto qk_tile = [&](const char* kbuf, f32x16& s0, f32x16& s1) {
#pragma unroll
      for (int i = 0; i < 16; i++) { s0[i] = 0.f; s1[i] = 0.f; }
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        const char* a = kbuf + (kbase_l ^ (ks << 5));
        bf16x8 a0 = *(const bf16x8*)(a);
        bf16x8 a1 = *(const bf16x8*)(a + 32 * ROWB);
        s0 = mfma32(a0, qf[ks], s0);
        s1 = mfma32(a1, qf[ks], s1);
      }
    };
    // keys beyond nvalid do not take part (only the last tile of a list can be ragged)
    auto mask_tile = [&](f32x16& s0, f32x16& s1, int nvalid) {
      // accumulator i of this lane is tile row 8*(i/4) + 4*hh + (i%4): compare against a per-lane
      // limit so that the per-element constants stay immediates
      const int lim = nvalid - 4 * hh;
#pragma unroll
      for (int i = 0; i < 16; i++) {
        const int kc = 8 * (i >> 2) + (i & 3);
        s0[i] = (kc < lim) ? s0[i] : -INFINITY;
        s1[i] = (kc + 32 < lim) ? s1[i] : -INFINITY;
      }
    };
    // row maximum of the raw logits of one tile (both lane halves)
    auto max_tile = [&](const f32x16& s0, const f32x16& s1) -> float {
      float ma = fmaxf(s0[0], s1[0]), mb = fmaxf(s0[1], s1[1]);
#pragma unroll
      for (int i = 2; i < 16; i += 2) {
        ma = fmaxf(fmaxf(ma, s0[i]), s1[i]);
        mb = fmaxf(fmaxf(mb, s0[i + 1]), s1[i + 1]);
      }
      return xhalf_max(fmaxf(ma, mb));
    };
    // lazy reference-maximum update for a tile whose raw row maximum is mx
    auto rescale_check = [&](float mx) {
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
    };
    // P = exp2(S*c - m_ref), row-sum partials, bf16 pack into the B-operand layout of the PV MFMA
    auto exp_tile = [&](f32x16& s0, f32x16& s1, bf16x8 (&pb)[4]) {
      const float negm = -m_ref;
      float la = 0.f, lb = 0.f;
#pragma unroll
      for (int i = 0; i < 16; i++) {
        s0[i] = fast_exp2(fmaf(s0[i], c, negm));
        s1[i] = fast_exp2(fmaf(s1[i], c, negm));
        la += s0[i];
        lb += s1[i];
      }
      lsum += la + lb;
      pb[0] = pack8(s0[0], s0[1], s0[2], s0[3], s0[4], s0[5], s0[6], s0[7]);
      pb[1] = pack8(s0[8], s0[9], s0[10], s0[11], s0[12], s0[13], s0[14], s0[15]);
      pb[2] = pack8(s1[0], s1[1], s1[2], s1[3], s1[4], s1[5], s1[6], s1[7]);
      pb[3] = pack8(s1[8], s1[9], s1[10], s1[11], s1[12], s1[13], s1[14], s1[15]);
    };
    // O^T += V^T . P^T (16 MFMA for d = 128)
    auto pv_tile = [&](const bf16x8 (&pb)[4], const char* vbuf) {
#pragma unroll
      for (int kb = 0; kb < 4; kb++) {
#pragma unroll
        for (int m = 0; m < MTD; m++) {
          const char* a = vbuf + (vbase_l ^ (m << 6)) + kb * 16 * ROWB;
          bf16x4 lo = lds_read_tr(a);
          bf16x4 hi = lds_read_tr(a + 8 * ROWB);
          bf16x8 av = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
          oacc[m] = mfma32(av, pb[kb], oacc[m]);
        }
      }
    };

    // ---- prologue: tiles 0 and 1 in flight, S(0) computed ----
    // rows_v: rows of tile t+1 (its V is fetched next), rows_k: rows of tile t+2 (its K is next),
    // rows_n: rows of tile t+3, raw: list reads of tile t+4
    int rows_v[NR], rows_k[NR], rows_n[NR], raw[NR];
#pragma unroll
    for (int s = 0; s < NR; s++) { rows_v[s] = 0; rows_k[s] = 0; rows_n[s] = 0; raw[s] = 0; }
    int nv0, nv1 = 64, nv2 = 64, nv3 = 64;
    if (NPROD) {
      nv0 = nvalid_gather(0); nv1 = nvalid_gather(1); nv2 = nvalid_gather(2);
    } else {
      int rows0[NR];
      // tiles 0..3: block lists use the entries read next to the count
      auto first_raw = [&](int t, int (&raw)[NR]) {
        if (MODE == MODE_BLOCK && !identity) {
          const int e = t >> sub_shift;
          raw[0] = (e == 0) ? head[0] : (e == 1) ? head[1] : (e == 2) ? head[2] : head[3];
        } else {
          prefetch_raw(t, raw);
        }
      };
      if constexpr (MODE == MODE_GATHER) {
        // the list entries of the first four tiles are requested together (one memory round trip, not one per tile)
        int raw0[NR], raw1[NR], raw2[NR];
        prefetch_raw(0, raw0);
        prefetch_raw(1, raw1);
        prefetch_raw(2, raw2);
        prefetch_raw(3, raw);
        finish_rows(0, raw0, rows0, nv0);
        finish_rows(1, raw1, rows_v, nv1);
        finish_rows(2, raw2, rows_k, nv2);
        nv1 = max(nv1, 0); nv2 = max(nv2, 0);
      } else {
        first_raw(0, raw);
        finish_rows(0, raw, rows0, nv0);
        if (T > 1) { first_raw(1, raw); finish_rows(1, raw, rows_v, nv1); }
        if (T > 2) { first_raw(2, raw); finish_rows(2, raw, rows_k, nv2); }
        if (T > 3) first_raw(3, raw);
      }
      issue(krsrc, k_srb, false, rows0, lds0);
      if (!LSE_ONLY) issue(vrsrc, v_srb, true, rows0, lds0 + 2 * TILE);
      if (T > 1) issue(krsrc, k_srb, false, rows_v, lds0 + TILE);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's LDS fills have landed
    __syncthreads();
    f32x16 sa0, sa1, sb0, sb1;
    qk_tile(smem, sa0, sa1);
    // K(2) is fetched into the buffer of K(0) at the top of the first iteration: every wave must have read
    // K(0) before any wave issues that fill
    __syncthreads();
    if (nv0 < 64) mask_tile(sa0, sa1, nv0);
    rescale_check(max_tile(sa0, sa1));

    // Pipelined iteration for a tile t that has a successor; PAR = t & 1 picks the buffers:
    //   K(t+1) is in K buffer (1-PAR), K(t+2) goes to K buffer PAR,
    //   V(t) is in V buffer PAR, V(t+1) goes to V buffer (1-PAR).
    // Between the two barriers the body is one straight-line block: the matrix cores run
    // S(t+1) = K(t+1) Q^T and then O += P(t) V(t) while the vector ALU turns S(t) into P(t) and
    // then reduces the row maximum of S(t+1); the reference-maximum update (a rare branch)
    // sits after the barrier.
    auto body = [&](int t, auto par, auto masked, f32x16& c0, f32x16& c1, f32x16& n0, f32x16& n1) {
      constexpr int PAR = decltype(par)::value;
      constexpr bool MASKED = decltype(masked)::value;
      // The fills of V(t+1) and K(t+2) are not issued in one burst up front (a wave spends tens of cycles on each and
      // the matrix cores would sit idle meanwhile) but one by one between the QK MFMAs, where their issue runs in the
      // shadow of the MFMA before.  NFILL instructions, one every FSTRIDE steps; if there are more than steps, up front.
      constexpr int NQK_ = 2 * KS;
      constexpr int NFILL = NPROD ? 0 : (LSE_ONLY ? SLOTS : 2 * SLOTS);
      constexpr int FSTRIDE = (CONST_OFF && NFILL > 0 && NFILL <= NQK_) ? NQK_ / NFILL : 0;
      const bool fill_k = t + 2 < T;
      auto fill_step = [&](auto jc) {
        constexpr int j = decltype(jc)::value;
        if constexpr (FSTRIDE > 0) {
          if constexpr (j % FSTRIDE == 0 && j / FSTRIDE < NFILL) {
            constexpr int f = j / FSTRIDE;
            if constexpr (!LSE_ONLY && f < SLOTS) issue_slot(vrsrc, v_srb, true, rows_v, lds0 + (3 - PAR) * TILE, f);
            else if (fill_k) issue_slot(krsrc, k_srb, false, rows_k, lds0 + PAR * TILE, LSE_ONLY ? f : f - SLOTS);
          }
        }
      };
      if (NPROD) {
        nv3 = nvalid_gather(t + 3);
      } else {
        if constexpr (FSTRIDE == 0) {
          if (!LSE_ONLY) issue(vrsrc, v_srb, true, rows_v, lds0 + (3 - PAR) * TILE);
          if (fill_k) issue(krsrc, k_srb, false, rows_k, lds0 + PAR * TILE);
        }
        if (t + 3 < T) finish_rows(t + 3, raw, rows_n, nv3);
        if (t + 4 < T) prefetch_raw(t + 4, raw);
      }
      // The block below is software-pipelined by hand; sched_barrier(0) after every step stops the
      // compiler from regrouping it.  Phase A: QK MFMA j | K-fragment read j+4 | softmax slot j of
      // S(t).  Phase B: PV MFMA j | the two transposing V reads of MFMA j+4 | the last softmax slots
      // of S(t) (first half) or a slice of the row-maximum reduction of S(t+1) (second half).
      constexpr int NQK = 2 * KS, NPV = LSE_ONLY ? 0 : 4 * MTD, AHEAD = READ_AHEAD;
      const char* kbuf = smem + (1 - PAR) * TILE;
      const char* vbuf = smem + (2 + PAR) * TILE;
      auto kread = [&](int j) -> bf16x8 {
        return *(const bf16x8*)(kbuf + (kbase_l ^ ((j >> 1) << 5)) + (j & 1) * 32 * ROWB);
      };
      auto vread = [&](int j) -> bf16x8 {
        const int kb = j / MTD, m = j % MTD;
        const char* a = vbuf + (vbase_l ^ (m << 6)) + kb * 16 * ROWB;
        bf16x4 lo = lds_read_tr(a);
        bf16x4 hi = lds_read_tr(a + 8 * ROWB);
        return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      };
      bf16x8 frag[NQK > NPV ? NQK : NPV];
      uint32_t pw[16];
      const float negm = -m_ref;
      float la = 0.f, lb = 0.f;
      // The softmax of S(t) runs as a three-stage pipeline over the MFMA steps so that no vector instruction
      // waits for the one before it: step g scales the elements of slot g, takes exp2 of slot g-1 and
      // adds / packs slot g-2.  Slots: EA elements over the QK steps, the rest over the first half of the
      // PV steps (quarter kb of P is complete before PV step kb * MTD needs it); the row maximum of
      // S(t+1) goes next to the second half of the PV steps.
      auto st_scale = [&](auto ec) {
        constexpr int e = decltype(ec)::value;
        if constexpr (e < 16) c0[e] = fmaf(c0[e], c, negm); else c1[e - 16] = fmaf(c1[e - 16], c, negm);
      };
      auto st_exp = [&](auto ec) {
        constexpr int e = decltype(ec)::value;
        if constexpr (e < 16) c0[e] = fast_exp2(c0[e]); else c1[e - 16] = fast_exp2(c1[e - 16]);
      };
      auto st_sum = [&](auto ec) {
        constexpr int e = decltype(ec)::value;
        float r;
        if constexpr (e < 16) r = c0[e]; else r = c1[e - 16];
        if constexpr (e & 1) {
          lb += r;
          float prev;
          if constexpr (e < 16) prev = c0[e - 1]; else prev = c1[e - 17];
          pw[e >> 1] = pack_bf16(prev, r);
        } else {
          la += r;
        }
      };
      using Sch = ExpSlots<2 * KS, (LSE_ONLY ? 0 : 4 * MTD) / 2, LSE_ONLY ? 32 : EXP_IN_QK>;
      auto softmax_step = [&](auto gc) {
        constexpr int g = decltype(gc)::value;
        static_for<Sch::lo(g - 2), Sch::lo(g - 1)>(st_sum);
        static_for<Sch::lo(g - 1), Sch::lo(g)>(st_exp);
        static_for<Sch::lo(g), Sch::lo(g + 1)>(st_scale);
      };
      constexpr int HB = NPV / 2;
#pragma unroll
      for (int j = 0; j < AHEAD; j++) frag[j] = kread(j);
      __builtin_amdgcn_sched_barrier(0);
      static_for<0, NQK>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        if constexpr (j + AHEAD < NQK) frag[j + AHEAD] = kread(j + AHEAD);
        // the first MFMA of each accumulator takes the constant 0 as its addend (no register clearing)
        if constexpr (j == 0) n0 = mfma32(frag[j], qf[0], f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0});
        else if constexpr (j == 1) n1 = mfma32(frag[j], qf[0], f32x16{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0});
        else if constexpr (j & 1) n1 = mfma32(frag[j], qf[j >> 1], n1);
        else n0 = mfma32(frag[j], qf[j >> 1], n0);
        fill_step(jc);
        softmax_step(jc);
        __builtin_amdgcn_sched_barrier(0);
      });
      float ma = -INFINITY, mb = -INFINITY;
      if (!LSE_ONLY) {
        bf16x8 pb[4];
#pragma unroll
        for (int j = 0; j < AHEAD; j++) frag[j] = vread(j);
        __builtin_amdgcn_sched_barrier(0);
        if (MASKED) mask_tile(n0, n1, nv1);
        static_for<0, NPV>([&](auto jc) {
          constexpr int j = decltype(jc)::value;
          if constexpr (j + AHEAD < NPV) frag[j + AHEAD] = vread(j + AHEAD);
          if constexpr (j % MTD == 0) {
            constexpr int kb = j / MTD;
            u32x4 u = {pw[4 * kb], pw[4 * kb + 1], pw[4 * kb + 2], pw[4 * kb + 3]};
            pb[kb] = __builtin_bit_cast(bf16x8, u);
          }
          oacc[j % MTD] = mfma32(frag[j], pb[j / MTD], oacc[j % MTD]);
          softmax_step(std::integral_constant<int, NQK + j>{});
          if constexpr (j >= HB) {
            constexpr int e0 = (j - HB) * 16 / (NPV - HB), e1 = (j - HB + 1) * 16 / (NPV - HB);
#pragma unroll
            for (int e = e0; e < e1; e++) ma = fmaxf(fmaxf(ma, n0[e]), n1[e]);
          }
          __builtin_amdgcn_sched_barrier(0);
        });
      } else {
        softmax_step(std::integral_constant<int, NQK>{});
        softmax_step(std::integral_constant<int, NQK + 1>{});
        if (MASKED) mask_tile(n0, n1, nv1);
#pragma unroll
        for (int e = 0; e < 16; e++) ma = fmaxf(fmaxf(ma, n0[e]), n1[e]);
      }
      lsum += la + lb;
      const float mx = xhalf_max(fmaxf(ma, mb));
      __builtin_amdgcn_s_waitcnt(0x0f70);
      __syncthreads();
      rescale_check(mx);
      nv0 = nv1; nv1 = nv2; nv2 = nv3;
      if (!NPROD) {
#pragma unroll
        for (int s = 0; s < NR; s++) { rows_v[s] = rows_k[s]; rows_k[s] = rows_n[s]; }
      }
    };
    auto step = [&](int t, auto par, f32x16& c0, f32x16& c1, f32x16& n0, f32x16& n1) {
      if (nv1 < 64) body(t, par, std::true_type{}, c0, c1, n0, n1);
      else body(t, par, std::false_type{}, c0, c1, n0, n1);
    };
    // last tile of the list: no successor to prefetch or to multiply
    auto last = [&](auto par, f32x16& c0, f32x16& c1) {
      constexpr int PAR = decltype(par)::value;
      bf16x8 pb[4];
      exp_tile(c0, c1, pb);
      if (!LSE_ONLY) pv_tile(pb, smem + (2 + PAR) * TILE);
      __syncthreads();
    };

    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    int t = 0;
    for (; t + 2 < T; t += 2) {
      step(t, P0{}, sa0, sa1, sb0, sb1);
      step(t + 1, P1{}, sb0, sb1, sa0, sa1);
    }
    if (t + 1 < T) {
      step(t, P0{}, sa0, sa1, sb0, sb1);
      last(P1{}, sb0, sb1);
    } else {
      last(P0{}, sa0, sa1);
    }
  } while (false);

  if constexpr (SK) {
    if (!whole) {
      // ---- a piece of a query tile: park the unnormalised state in the piece's workspace slot; the workgroup
      // whose piece completes the tile adds all pieces up, in list order, and runs the epilogue ----
      constexpr int SLOT_FLOATS = D * 32 * NCOMP + 3 * 64 * NCOMP;
      const bool computes = !(NPROD && wave >= NCOMP);
      // The pieces travel between XCDs, whose L2 caches do not see each other's lines.  Rather than writing back
      // and invalidating whole caches around the exchange (what device-scope fences do), every workspace access is
      // itself device-coherent: relaxed device-scope atomic stores and loads write through / read past the L2.  The
      // stores are awaited before the arrival counter is bumped, the loads are issued after its value came back.
      auto put2 = [](float* dst, float a, float b) {
        const uint64_t v = (uint64_t)__builtin_bit_cast(uint32_t, a) | ((uint64_t)__builtin_bit_cast(uint32_t, b) << 32);
        __hip_atomic_store((uint64_t*)dst, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      };
      auto get2 = [](const float* src, float& a, float& b) {
        const uint64_t v = __hip_atomic_load((const uint64_t*)src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        a = __builtin_bit_cast(float, (uint32_t)v);
        b = __builtin_bit_cast(float, (uint32_t)(v >> 32));
      };
      auto put1 = [](float* dst, float a) {
        __hip_atomic_store((uint32_t*)dst, __builtin_bit_cast(uint32_t, a), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      };
      auto get1 = [](const float* src) -> float {
        return __builtin_bit_cast(float, __hip_atomic_load((const uint32_t*)src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
      };
      // slot layout: accumulator pair (m, i/2) of wave and lane at ((m*8 + i/2)*NCOMP + wave)*128 + lane*2; then
      // three statistics per lane
      if (computes) {
        float* slot = p.sk_slots + (int64_t)(sk.slot0 + sk.kp) * SLOT_FLOATS;
#pragma unroll
        for (int m = 0; m < MTD; m++)
#pragma unroll
          for (int a = 0; a < 8; a++) put2(slot + ((m * 8 + a) * NCOMP + wave) * 128 + lane * 2, oacc[m][2 * a], oacc[m][2 * a + 1]);
        float* st = slot + D * 32 * NCOMP + wave * 64 + lane;
        put1(st, m_ref);
        put1(st + 64 * NCOMP, lsum);
        put1(st + 128 * NCOMP, m_true);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   // compiler ordering only
      __builtin_amdgcn_s_waitcnt(0x0f70);                        // vmcnt(0): this wave's stores have been written through
      __syncthreads();
      volatile int* flag = (volatile int*)smem;   // the K/V buffers are idle from here on
      if (tid == 0) {
        const int n = u1 - u0;
        const int old = __hip_atomic_fetch_add(p.sk_counters + w, n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        flag[0] = (old + n == sk.tile_units) ? 1 : 0;
      }
      __syncthreads();
      const bool finisher = flag[0] != 0;
      __syncthreads();   // everyone has read the flag before the epilogue reuses the buffer
      if (!finisher) return;
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");   // compiler ordering only
      if (tid == 0) __hip_atomic_store(p.sk_counters + w, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next launch
      if (computes) {
        // pass 1: common reference maximum (independent loads, one round trip); pass 2: the pieces in list order,
        // this workgroup's own included, every one read back from its slot: the same arithmetic whoever finishes
        const float* st0 = p.sk_slots + (int64_t)sk.slot0 * SLOT_FLOATS + D * 32 * NCOMP + wave * 64 + lane;
        float m_star = NEG_BIG;
        m_true = -INFINITY;
#pragma unroll
        for (int kp = 0; kp < SK_MAX_PIECES; kp++)
          if (kp < sk.pieces) {
            m_star = fmaxf(m_star, get1(st0 + (int64_t)kp * SLOT_FLOATS));
            m_true = fmaxf(m_true, get1(st0 + (int64_t)kp * SLOT_FLOATS + 128 * NCOMP));
          }
#pragma unroll
        for (int m = 0; m < MTD; m++)
#pragma unroll
          for (int i = 0; i < 16; i++) oacc[m][i] = 0.f;
        lsum = 0.f;
        for (int kp = 0; kp < sk.pieces; kp++) {
          const float* slot = p.sk_slots + (int64_t)(sk.slot0 + kp) * SLOT_FLOATS;
          const float* st = slot + D * 32 * NCOMP + wave * 64 + lane;
          const float alpha = fast_exp2(get1(st) - m_star);
          lsum = fmaf(get1(st + 64 * NCOMP), alpha, lsum);
#pragma unroll
          for (int m = 0; m < MTD; m++)
#pragma unroll
            for (int a = 0; a < 8; a++) {
              float x, y;
              get2(slot + ((m * 8 + a) * NCOMP + wave) * 128 + lane * 2, x, y);
              oacc[m][2 * a] = fmaf(x, alpha, oacc[m][2 * a]);
              oacc[m][2 * a + 1] = fmaf(y, alpha, oacc[m][2 * a + 1]);
            }
        }
        m_ref = m_star;
      }
    }
  }

  // ---- epilogue ----
  if (NPROD && wave >= NCOMP) return;   // fetch waves own no query rows (only reached with an empty list)
  const float ltot = xhalf_sum(lsum);
  const bool empty = !(ltot > 0.f);
  const float inv = empty ? 0.f : 1.0f / ltot;
  const int qrow_w = q0 + wave * 32 + r;
  if (hh == 0 && qrow_w < p.Lq) {
    const int64_t off = ((int64_t)b * p.H + h) * p.Lq + qrow_w;
    if (p.M) p.M[off] = empty ? -INFINITY : m_true;
    if (p.L) p.L[off] = empty ? 1.0f : ltot * fast_exp2(m_ref - m_true);
    if (p.LSE2) p.LSE2[off] = empty ? -INFINITY : m_ref + __builtin_amdgcn_logf(ltot);
    if (p.RCP) p.RCP[off] = empty ? INFINITY : fast_exp2(-m_ref) * inv;
  }
  if (LSE_ONLY) return;

  const float osc = ACCUM ? p.o_scale * inv : inv;
  if constexpr (ACCUM) {
    if (p.o_accum) {
      // o = o_accum (or its bilinear upsample) + o_scale * O / l, formed in fp32 and rounded once.  The accumulators
      // go through LDS as fp32, half of the head dimension at a time (the K/V buffers hold 32 rows x D/2 floats per
      // wave), so that a lane ends up with 8 consecutive columns of one row: the o_accum rows (four taps of the
      // coarser grid when upsampling: half-pixel centres, edge clamp, src = max(0, (dst + 0.5) * src_side / dst_side
      // - 0.5), the align_corners = False rule) are then read with 16-byte loads that 8 neighbouring lanes share a
      // row of, and o is stored the same way.
      constexpr int HD = D / 2, FSTR = HD * 4 + 16, CPRH = HD / 8, ITER = (32 * CPRH) / 64;
      static_assert(NCOMP * 32 * FSTR <= 4 * TILE, "fp32 epilogue buffer must fit in the K/V buffers");
      char* fb = smem + wave * (32 * FSTR);
      const bf16_t* abase = p.o_accum + b * p.oa_sb + h * p.oa_sh;
      bf16_t* op = p.o + b * p.o_sb + h * p.o_sh;
#pragma unroll
      for (int pass = 0; pass < 2; pass++) {
#pragma unroll
        for (int mm = 0; mm < MTD / 2; mm++) {
          const int m = pass * (MTD / 2) + mm;
#pragma unroll
          for (int a = 0; a < 4; a++) {
            const f32x4 x = {oacc[m][4 * a + 0] * osc, oacc[m][4 * a + 1] * osc, oacc[m][4 * a + 2] * osc, oacc[m][4 * a + 3] * osc};
            *(f32x4*)(fb + r * FSTR + (mm * 32 + 8 * a + 4 * hh) * 4) = x;
          }
        }
        // each wave re-reads only its own 32 rows: a wave-local fence is enough
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int i = 0; i < ITER; i++) {
          const int cidx = lane + i * 64;
          const int orow = cidx / CPRH, oc = cidx - orow * CPRH;
          const int grow = q0 + wave * 32 + orow;
          if (grow < p.Lq) {
            const f32x4 xa = *(const f32x4*)(fb + orow * FSTR + oc * 32), xb = *(const f32x4*)(fb + orow * FSTR + oc * 32 + 16);
            float x[8] = {xa[0], xa[1], xa[2], xa[3], xb[0], xb[1], xb[2], xb[3]};
            const int col = pass * HD + oc * 8;
            if (p.up_src > 0) {
              const int y = grow / p.up_dst, xq = grow - y * p.up_dst;
              const float sc = (float)p.up_src / (float)p.up_dst;
              const float sy = fmaxf(sc * ((float)y + 0.5f) - 0.5f, 0.f), sx = fmaxf(sc * ((float)xq + 0.5f) - 0.5f, 0.f);
              const int y0 = min((int)sy, p.up_src - 1), x0 = min((int)sx, p.up_src - 1);
              const int y1 = min(y0 + 1, p.up_src - 1), x1 = min(x0 + 1, p.up_src - 1);
              const float wy1 = sy - (float)y0, wx1 = sx - (float)x0, wy0 = 1.f - wy1, wx0 = 1.f - wx1;
              const u32x4 t00 = *(const u32x4*)(abase + (int64_t)(y0 * p.up_src + x0) * p.oa_sr + col);
              const u32x4 t01 = *(const u32x4*)(abase + (int64_t)(y0 * p.up_src + x1) * p.oa_sr + col);
              const u32x4 t10 = *(const u32x4*)(abase + (int64_t)(y1 * p.up_src + x0) * p.oa_sr + col);
              const u32x4 t11 = *(const u32x4*)(abase + (int64_t)(y1 * p.up_src + x1) * p.oa_sr + col);
#pragma unroll
              for (int e = 0; e < 4; e++) {
                x[2 * e] += wy0 * (wx0 * bf16_lo(t00[e]) + wx1 * bf16_lo(t01[e])) + wy1 * (wx0 * bf16_lo(t10[e]) + wx1 * bf16_lo(t11[e]));
                x[2 * e + 1] += wy0 * (wx0 * bf16_hi(t00[e]) + wx1 * bf16_hi(t01[e])) + wy1 * (wx0 * bf16_hi(t10[e]) + wx1 * bf16_hi(t11[e]));
              }
            } else {
              const u32x4 t = *(const u32x4*)(abase + (int64_t)grow * p.oa_sr + col);
#pragma unroll
              for (int e = 0; e < 4; e++) { x[2 * e] += bf16_lo(t[e]); x[2 * e + 1] += bf16_hi(t[e]); }
            }
            const u32x4 val = {pack_bf16(x[0], x[1]), pack_bf16(x[2], x[3]), pack_bf16(x[4], x[5]), pack_bf16(x[6], x[7])};
            *(u32x4*)(op + (int64_t)grow * p.o_sr + col) = val;
          }
        }
        __builtin_amdgcn_wave_barrier();   // the buffer is rewritten by the next pass
      }
      return;
    }
  }
  char* ob = smem + wave * (32 * OSTR);
#pragma unroll
  for (int m = 0; m < MTD; m++) {
#pragma unroll
    for (int a = 0; a < 4; a++) {
      const int dcol = m * 32 + 8 * a + 4 * hh;
      float x0 = oacc[m][4 * a + 0] * osc, x1 = oacc[m][4 * a + 1] * osc;
      float x2 = oacc[m][4 * a + 2] * osc, x3 = oacc[m][4 * a + 3] * osc;
      u32x2 pk = {pack_bf16(x0, x1), pack_bf16(x2, x3)};
      *(u32x2*)(ob + r * OSTR + dcol * 2) = pk;
    }
  }
  // each wave re-reads only its own 32 rows: a wave-local fence is enough
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
  __builtin_amdgcn_wave_barrier();
  bf16_t* op = p.o + b * p.o_sb + h * p.o_sh;
  constexpr int OCPR = D / 8;
#pragma unroll
  for (int i = 0; i < (32 * OCPR) / 64; i++) {
    const int cidx = lane + i * 64;
    const int orow = cidx / OCPR, ocol = cidx - orow * OCPR;
    const int grow = q0 + wave * 32 + orow;
    if (grow < p.Lq) {
      u32x4 val = *(const u32x4*)(ob + orow * OSTR + ocol * 16);
      *(u32x4*)(op + (int64_t)grow * p.o_sr + ocol * 8) = val;
    }
  }
}
#endif  // __HIP_DEVICE_COMPILE__

template <int D, int NWAVES, int MODE, bool ACCUM, bool LSE_ONLY>
__global__ __launch_bounds__(NWAVES * 64, ((NWAVES <= 4 && D <= 128) ? 2 : 1)) void attn_fwd_kernel(const AttnParams p) {
  // The body is compiled for the device only: the host pass just needs the launch stub, and it
  // silently drops the stub when the body uses the LDS-DMA builtins.
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  // Consecutive workgroup ids are dealt round-robin to the 8 XCDs; remap so that each XCD
  // walks a contiguous range of (batch, head, q-tile) and K/V of one head stay in its L2.
  const int per_xcd = gridDim.x >> 3;
  const int w = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (w >= p.total_wg) return;
  attn_item<D, NWAVES, MODE, ACCUM, LSE_ONLY, false>(p, smem, w, 0, 0, true, SkCtx{});
#endif
}

// Balanced launch: every workgroup runs one item of the partition described in sk_partition.h, which it reads from
// the item table built by plan_kernel, or, for dense attention (all lists equally long, sk_uniform_n pieces per
// tile), computes from its index.
template <int D, int NWAVES, int MODE, bool ACCUM>
__global__ __launch_bounds__(NWAVES * 64, (NWAVES <= 4 ? 2 : 1)) void attn_fwd_balanced_kernel(const AttnParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int N = p.total_wg;
  const bool uniform = p.sk_uniform_n > 0;
  const int items = uniform ? N * p.sk_uniform_n : min(max(p.sk_plan[1], 0), (int)gridDim.x);
  // consecutive items go to the same XCD (workgroup ids are dealt round-robin to the 8 XCDs): the K/V of a head
  // stay in its L2 and the pieces of a query tile meet there
  const int per_xcd = (items + 7) >> 3;
  const int slot_in_xcd = blockIdx.x >> 3;
  const int k = (blockIdx.x & 7) * per_xcd + slot_in_xcd;
  if (slot_in_xcd >= per_xcd || k >= items) return;
  SkCtx sk;
  int w, u0, u1;
  if (uniform) {
    const int n = p.sk_uniform_n, T = (p.Lk + 63) >> 6;
    w = k / n;
    sk.kp = k - w * n;
    sk.pieces = n;
    sk.slot0 = w * n;
    sk.tile_units = T;
    sk_piece(T, n, sk.kp, u0, u1);
  } else {
    const int* it = p.sk_plan + SK_PLAN_HEADER + SK_PLAN_ITEM * k;
    w = max(0, min(it[0], N - 1));
    u0 = it[1];
    u1 = it[2];
    sk.slot0 = it[3];
    sk.pieces = it[4];
    sk.kp = it[5];
    sk.tile_units = it[6];
    // a damaged table must not send a store outside the workspace
    if (sk.pieces < 1 || sk.pieces > SK_MAX_PIECES || sk.kp < 0 || sk.kp >= sk.pieces || (sk.pieces > 1 && (sk.slot0 < 0 || sk.slot0 + sk.pieces > 2 * p.sk_wgs))) return;
  }
  attn_item<D, NWAVES, MODE, ACCUM, false, true>(p, smem, w, u0, u1, sk.pieces == 1, sk);
#endif
}

// words [0, n) of a device buffer := 0 (a kernel, not hipMemsetAsync: callers may be capturing a HIP graph)
__global__ void zero_words_kernel(uint32_t* dst, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = 0u;
}

// Item table of a balanced launch over tile lists, from the list lengths: one workgroup.  Also clears the arrival
// counters of the launch's query tiles, so that a launch does not depend on what the last one left in the workspace.
template <int WGROWS, int MODE>
__global__ __launch_bounds__(256) void plan_kernel(const AttnParams p, int* plan) {
  __shared__ int units[SK_MAX_QTILES];    // units of tile u
  __shared__ int ipfx[SK_MAX_QTILES + 1]; // items before tile u
  __shared__ int spfx[SK_MAX_QTILES + 1]; // slots before tile u
  __shared__ int total[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int N = p.total_wg;
  for (int u = tid; u < N; u += 256) {
    const int bh = u / p.nqt, qt = u - bh * p.nqt;
    const int b = bh / p.H, h = bh - b * p.H;
    const int g = (qt * WGROWS) / p.group_rows;
    const int cnt = max(0, min(p.cnt[b * p.cnt_sb + h * p.cnt_sh + g], p.list_len));
    units[u] = (MODE == MODE_BLOCK) ? cnt : ((cnt + 63) >> 6);
    p.sk_counters[u] = 0;
  }
  __syncthreads();
  if (wave == 0) {
    // every lane owns a run of consecutive tiles; U first, then the two prefix tables
    const int per = (N + 63) >> 6, first = lane * per;
    int sum = 0;
    for (int j = 0; j < per; j++)
      if (first + j < N) sum += max(units[first + j], 1);
    int U = sum;
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) U += __shfl_xor(U, d, 64);
    int S = sk_share(U, p.sk_wgs, p.sk_min_share);
    const bool cut = sk_worth_cutting(U, S, N, p.sk_wgs);
    int it = 0, sl = 0;
    for (int j = 0; j < per; j++)
      if (first + j < N) {
        const int n = cut ? sk_pieces(units[first + j], S, p.sk_min_piece) : 1;
        it += n;
        sl += n > 1 ? n : 0;
      }
    int it_incl = it, sl_incl = sl;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const int a = __shfl_up(it_incl, d, 64), c = __shfl_up(sl_incl, d, 64);
      if (lane >= d) { it_incl += a; sl_incl += c; }
    }
    int irun = it_incl - it, srun = sl_incl - sl;
    for (int j = 0; j < per; j++)
      if (first + j < N) {
        const int n = cut ? sk_pieces(units[first + j], S, p.sk_min_piece) : 1;
        ipfx[first + j] = irun;
        spfx[first + j] = srun;
        irun += n;
        srun += n > 1 ? n : 0;
      }
    if (lane == 63) { total[0] = it_incl; total[1] = sl_incl; total[2] = S; total[3] = cut ? 1 : 0; }
  }
  __syncthreads();
  const int S = total[2];
  const bool cut = total[3] != 0;
  // the pieces-per-share bound keeps both totals inside the launch (N + sk_wgs items) and the workspace (2 * sk_wgs
  // slots); if a list-length table breaks it after all, every tile stays whole
  const bool fits = total[0] <= N + p.sk_wgs && total[1] <= 2 * p.sk_wgs;
  if (tid == 0) {
    plan[0] = SK_PLAN_MAGIC;
    plan[1] = fits ? total[0] : N;
    plan[2] = N;
    plan[3] = S;
    plan[4] = fits ? total[1] : 0;
    plan[5] = plan[6] = plan[7] = 0;
  }
  for (int u = tid; u < N; u += 256) {
    const int T = units[u];
    const int n = (cut && fits) ? sk_pieces(T, S, p.sk_min_piece) : 1;
    const int base = fits ? ipfx[u] : u;
    for (int kp = 0; kp < n; kp++) {
      int u0, u1;
      sk_piece(T, n, kp, u0, u1);
      int* it = plan + SK_PLAN_HEADER + SK_PLAN_ITEM * (base + kp);
      it[0] = u; it[1] = u0; it[2] = u1; it[3] = n > 1 ? spfx[u] : -1;
      it[4] = n; it[5] = kp; it[6] = T; it[7] = 0;
    }
  }
}

template <int D, int NWAVES, int MODE, bool ACCUM, bool LSE_ONLY>
static int launch_one(const AttnParams& p0, hipStream_t stream) {
  AttnParams p = p0;
  if (p.kv_group < 1) p.kv_group = 1;
  constexpr int WGROWS = ((MODE == MODE_GATHER && NWAVES == 8) ? 6 : NWAVES) * 32;   // two of eight token-list waves only fetch
  constexpr int SMEM = 4 * 64 * D * 2;
  if (MODE == MODE_BLOCK && p.list == nullptr) p.group_rows = WGROWS;  // dense: any row grouping
  if (p.group_rows % WGROWS != 0) return LVAR_EINVAL;
  p.nqt = (p.Lq + WGROWS - 1) / WGROWS;
  p.total_wg = p.B * p.H * p.nqt;
  if constexpr (!LSE_ONLY) {
    const bool dense = (MODE == MODE_BLOCK && p.list == nullptr);
    const int64_t per_tile = (MODE == MODE_BLOCK) ? (p.list ? p.list_len : (p.Lk + 63) / 64) : (p.list_len + 63) / 64;
    const int sub = (MODE == MODE_BLOCK && p.list) ? p.sub_shift : 0;
    // (64-row query blocks always take the plain launch)
    p.sk_wgs = (p.sk_ws && NWAVES != 2 && D <= 128) ? sk_plan(p.total_wg, NWAVES, sk_slot_floats(D, MODE, NWAVES), per_tile, sub, p.sk_ws_bytes,
                                 p.sk_min_share, p.sk_min_piece) : 0;
    p.sk_uniform_n = 0;
    if (p.sk_wgs > 0 && dense) {
      // all lists have (Lk + 63) / 64 entries: the pieces per tile follow from the sizes alone
      p.sk_uniform_n = sk_dense_pieces(p.total_wg, (int)per_tile, p.sk_wgs, p.sk_min_share, p.sk_min_piece);
      if (p.sk_uniform_n == 0) p.sk_wgs = 0;   // whole tiles: the plain launch
    }
    if constexpr (NWAVES != 2 && D <= 128) if (p.sk_wgs > 0) {
      p.sk_counters = (int*)p.sk_ws;
      p.sk_slots = (float*)((char*)p.sk_ws + SK_COUNTER_BYTES + sk_plan_bytes(p.sk_wgs));
      int grid_sk;
      if (p.sk_uniform_n > 0 || p.sk_plan) {
        // no table kernel ahead of this launch: the arrival counters are cleared by a fill of their own
        hipLaunchKernelGGL(zero_words_kernel, dim3((p.total_wg + 255) / 256), dim3(256), 0, stream, (uint32_t*)p.sk_counters, p.total_wg);
        if (hipGetLastError() != hipSuccess) return LVAR_ELAUNCH;
      }
      if (p.sk_uniform_n > 0) {
        grid_sk = ((p.total_wg * p.sk_uniform_n + 7) / 8) * 8;
      } else {
        if (!p.sk_plan) {
          // no table from the caller: build it now, in the workspace
          int* plan = (int*)((char*)p.sk_ws + SK_COUNTER_BYTES);
          hipLaunchKernelGGL((plan_kernel<WGROWS, MODE>), dim3(1), dim3(256), 0, stream, p, plan);
          if (hipGetLastError() != hipSuccess) return LVAR_ELAUNCH;
          p.sk_plan = plan;
        }
        grid_sk = ((p.total_wg + p.sk_wgs + 7) / 8) * 8;   // at most one item per query tile plus one per share
      }
      auto kern = attn_fwd_balanced_kernel<D, NWAVES, MODE, ACCUM>;
      static std::atomic<uint64_t> lds_ready_sk{0};
      if (!ensure_lds_limit((const void*)kern, SMEM, lds_ready_sk)) return LVAR_ELAUNCH;
      hipLaunchKernelGGL(kern, dim3(grid_sk), dim3(NWAVES * 64), SMEM, stream, p);
      return hipGetLastError() == hipSuccess ? LVAR_OK : LVAR_ELAUNCH;
    }
  }
  const int grid = ((p.total_wg + 7) / 8) * 8;
  auto kern = attn_fwd_kernel<D, NWAVES, MODE, ACCUM, LSE_ONLY>;
  static std::atomic<uint64_t> lds_ready{0};
  if (!ensure_lds_limit((const void*)kern, SMEM, lds_ready)) return LVAR_ELAUNCH;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(NWAVES * 64), SMEM, stream, p);
  return hipGetLastError() == hipSuccess ? LVAR_OK : LVAR_ELAUNCH;
}

template <int D>
static int launch_d(const AttnParams& p, int mode, bool accum, bool lse_only, int nwaves, hipStream_t s) {
  if (mode == MODE_BLOCK) {
    if (nwaves == 2 && !lse_only) return launch_one<D, 2, MODE_BLOCK, false, false>(p, s);   // 64-row query blocks
    if (nwaves != 4) return LVAR_EUNSUPPORTED;
    return lse_only ? launch_one<D, 4, MODE_BLOCK, false, true>(p, s) : launch_one<D, 4, MODE_BLOCK, false, false>(p, s);
  } else if (mode == MODE_GATHER) {
    // (head_dim 256: a wave needs more than 256 registers, so one wave per SIMD: 192-row groups run as two 3-wave workgroups)
    if constexpr (D > 128) { if (nwaves == 8) nwaves = 3; }
    else if (nwaves == 8) return launch_one<D, 8, MODE_GATHER, true, false>(p, s);
    if (nwaves == 3) return launch_one<D, 3, MODE_GATHER, true, false>(p, s);
    if (nwaves == 2) return launch_one<D, 2, MODE_GATHER, true, false>(p, s);
  }
  return LVAR_EUNSUPPORTED;
}

int launch_attn(const AttnParams& p, int head_dim, int mode, bool accum, bool lse_only, int nwaves, hipStream_t s) {
  if (head_dim == 128) return launch_d<128>(p, mode, accum, lse_only, nwaves, s);
  if (head_dim == 64) return launch_d<64>(p, mode, accum, lse_only, nwaves, s);
  if (head_dim == 256) return launch_d<256>(p, mode, accum, lse_only, nwaves, s);
  return LVAR_EUNSUPPORTED;
}

int device_cus() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  const int slot = dev & 63;
  int n = cached[slot].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
    cached[slot].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Workgroups of the balanced launch, or 0 for the plain launch.  Balanced when the plain grid would leave the chip
// unevenly filled, i.e. fewer than four rounds of workgroups: one workgroup per resident slot (two per CU for the
// 4-wave kernels), or one per CU if the workspace only holds that many slot pairs.  `per_tile` is an upper bound
// of the list entries of a query tile; min_share / min_piece come in as 64-key tiles (0 = default) and go out
// as list entries (a list entry of a 128-key block list is two tiles: sub = 1).
int sk_plan(int total_wg, int nwaves, int slot_floats, int64_t per_tile, int sub, int64_t ws_bytes, int& min_share, int& min_piece) {
  const int cus = device_cus();
  const int slots = cus * (nwaves <= 4 ? 2 : 1);
  if (cus < 8 || cus % 8 != 0 || total_wg > SK_MAX_QTILES || total_wg >= 4 * slots || ws_bytes <= SK_COUNTER_BYTES) return 0;
  if (per_tile * total_wg >= (1ll << 30)) return 0;   // unit counts stay well inside 32 bits
  auto fits = [&](int P) { return SK_COUNTER_BYTES + sk_plan_bytes(P) + 2 * (int64_t)P * slot_floats * 4 <= ws_bytes; };
  const int P = fits(slots) ? slots : (fits(cus) ? cus : 0);
  const int share = min_share > 0 ? min_share : 8, piece = min_piece > 0 ? min_piece : 4;
  min_piece = (piece >> sub) > 0 ? (piece >> sub) : 1;
  min_share = (share >> sub) > min_piece ? (share >> sub) : min_piece;   // shares no smaller than pieces
  // With fewer query tiles than slots the plain launch already runs them all at once, and cutting only pays if
  // it makes the longest walk shorter: lists of at least one and a half shares (were every list full; the kernel
  // looks at the real lists and leaves the tiles whole if they are shorter).
  if (P == 0) return 0;
  if (total_wg < slots && 2 * per_tile < 3 * (int64_t)min_share) return 0;
  return P;
}

// Pieces per query tile of a balanced dense launch (every list has T tiles) on sk_wgs shares, or 0 when the tiles
// stay whole or the pieces would not fit the launch's slots: then the launch is the plain one.
int sk_dense_pieces(int total_wg, int T, int sk_wgs, int min_share, int min_piece) {
  if (sk_wgs <= 0 || total_wg <= 0 || T <= 0) return 0;
  const int U = total_wg * T;
  const int S = sk_share(U, sk_wgs, min_share);
  const int n = sk_worth_cutting(U, S, total_wg, sk_wgs) ? sk_pieces(T, S, min_piece) : 1;
  return (n > 1 && (int64_t)n * total_wg <= 2 * (int64_t)sk_wgs) ? n : 0;
}

// bytes of the item-table area of a workspace for P shares (256-byte granules)
int64_t sk_plan_bytes(int P) {
  const int64_t b = (int64_t)(SK_PLAN_HEADER + SK_PLAN_ITEM * (SK_MAX_QTILES + P)) * 4;
  return (b + 255) / 256 * 256;
}

// floats of one workspace slot of a balanced launch: the accumulators and three statistics of every lane
int sk_slot_floats(int head_dim, int mode, int nwaves) {
  const int ncomp = (mode == MODE_GATHER && nwaves == 8) ? 6 : nwaves;
  return head_dim * 32 * ncomp + 3 * 64 * ncomp;
}

}  // namespace lvar
