// Colsum kernel for gfx950: cs[b,h,g,n] = sum over the query rows i of group g of
// exp2(q_i.k_n*scale*log2e - lse2_i), lse2 = M + log2(L).
//
// Key-stationary decomposition: a wave keeps NTK*32 keys (the B operand, K^T) in registers for
// the whole sweep over Lq, the workgroup streams 64-row Q stages (+ their lse2) through LDS as
// the A operand.  In the 32x32 accumulator a lane owns ONE key column and 16 query rows, so the
// reduction over queries is an in-register add, one exchange with lane^32 at each group
// boundary, and a single plain store per (group, key): no atomics, no partial buffers, and a
// summation order that depends only on the shapes.
#include "common.h"
#include "launch.h"

namespace lvar {

template <int D, int NTK>
__global__ __launch_bounds__(256, 2) void colsum_kernel(const ColsumParams p) {
  constexpr int KS = D / 16, CPR = D / 8;
  constexpr int QSTR = D * 2 + 16;
  constexpr int QROWS = 64;
  constexpr int CPT = (QROWS * CPR) / 256;
  constexpr int STAGE = QROWS * QSTR + QROWS * 4;
  __shared__ __attribute__((aligned(16))) char smem[2 * STAGE];

  const int per_xcd = gridDim.x >> 3;
  const int w = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
  if (w >= p.total_wg) return;
  const int bh = w / p.nkt, kt = w - bh * p.nkt;
  const int b = bh / p.H, h = bh - b * p.H;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int hh = lane >> 5, r = lane & 31;
  const int n0 = (kt * 4 + wave) * (NTK * 32);

  // stationary K^T fragments
  const bf16_t* kbase = p.k + b * p.k_sb + h * p.k_sh;
  bf16x8 kf[NTK][KS];
#pragma unroll
  for (int nt = 0; nt < NTK; nt++) {
    const int krow = min(n0 + nt * 32 + r, p.Lk - 1);
    const bf16_t* kp = kbase + (int64_t)krow * p.k_sr + hh * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) kf[nt][ks] = *(const bf16x8*)(kp + ks * 16);
  }

  const bf16_t* qbase = p.q + b * p.q_sb + h * p.q_sh;
  const float* Mp = p.M + ((int64_t)b * p.H + h) * p.Lq;
  const float* Lp = p.L + ((int64_t)b * p.H + h) * p.Lq;
  float* csp = p.cs + ((int64_t)b * p.H + h) * p.G * (int64_t)p.Lk;

  int crow[CPT], ccol[CPT];
#pragma unroll
  for (int i = 0; i < CPT; i++) {
    int c = tid + i * 256;
    crow[i] = c / CPR;
    ccol[i] = c - crow[i] * CPR;
  }
  u32x4 qreg[CPT];
  float lsereg = 0.f;
  auto load_stage = [&](int s) {
    const int base = s * QROWS;
#pragma unroll
    for (int i = 0; i < CPT; i++) {
      const int row = min(base + crow[i], p.Lq - 1);
      qreg[i] = *(const u32x4*)(qbase + (int64_t)row * p.q_sr + ccol[i] * 8);
    }
    if (tid < QROWS) {
      const int row = base + tid;
      lsereg = (row < p.Lq) ? Mp[row] + __builtin_amdgcn_logf(Lp[row]) : INFINITY;
    }
  };
  auto store_stage = [&](int st) {
    char* qs = smem + st * STAGE;
#pragma unroll
    for (int i = 0; i < CPT; i++) *(u32x4*)(qs + crow[i] * QSTR + ccol[i] * 16) = qreg[i];
    if (tid < QROWS) *(float*)(qs + QROWS * QSTR + tid * 4) = lsereg;
  };

  const int S = (p.Lq + QROWS - 1) / QROWS;
  const float c = p.c;
  float acc[NTK];
#pragma unroll
  for (int nt = 0; nt < NTK; nt++) acc[nt] = 0.f;

  load_stage(0);
  store_stage(0);
  __syncthreads();

  for (int s = 0; s < S; s++) {
    const int st = s & 1;
    if (s + 1 < S) load_stage(s + 1);
    const char* qs = smem + st * STAGE;
#pragma unroll
    for (int qt = 0; qt < 2; qt++) {
      const int qrow0 = s * QROWS + qt * 32;
      if (qrow0 < p.Lq) {
        bf16x8 a[KS];
        const char* ql = qs + (qt * 32 + r) * QSTR + hh * 16;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) a[ks] = *(const bf16x8*)(ql + ks * 32);
        f32x4 lse[4];
        const char* ll = qs + QROWS * QSTR + (qt * 32 + 4 * hh) * 4;
#pragma unroll
        for (int j = 0; j < 4; j++) lse[j] = *(const f32x4*)(ll + j * 32);
#pragma unroll
        for (int nt = 0; nt < NTK; nt++) {
          f32x16 sacc;
#pragma unroll
          for (int i = 0; i < 16; i++) sacc[i] = 0.f;
#pragma unroll
          for (int ks = 0; ks < KS; ks++) sacc = mfma32(a[ks], kf[nt][ks], sacc);
          float part = 0.f;
#pragma unroll
          for (int i = 0; i < 16; i++) part += fast_exp2(fmaf(sacc[i], c, -lse[i >> 2][i & 3]));
          acc[nt] += part;
        }
        const int qend = qrow0 + 32;
        if (qend % p.group_rows == 0 || qend >= p.Lq) {
          const int g = qrow0 / p.group_rows;
#pragma unroll
          for (int nt = 0; nt < NTK; nt++) {
            const float tot = xhalf_sum(acc[nt]);
            const int key = n0 + nt * 32 + r;
            if (hh == 0 && key < p.Lk) csp[(int64_t)g * p.Lk + key] = tot;
            acc[nt] = 0.f;
          }
        }
      }
    }
    if (s + 1 < S) store_stage(st ^ 1);
    __syncthreads();
  }
}

template <int D, int NTK>
static int launch_cs(const ColsumParams& p0, hipStream_t stream) {
  ColsumParams p = p0;
  p.nkt = (p.Lk + 4 * NTK * 32 - 1) / (4 * NTK * 32);
  p.total_wg = p.B * p.H * p.nkt;
  const int grid = ((p.total_wg + 7) / 8) * 8;
  hipLaunchKernelGGL((colsum_kernel<D, NTK>), dim3(grid), dim3(256), 0, stream, p);
  return hipGetLastError() == hipSuccess ? LVAR_OK : LVAR_ELAUNCH;
}

int launch_colsum(const ColsumParams& p, int head_dim, hipStream_t s) {
  if (head_dim == 128) return launch_cs<128, 2>(p, s);
  if (head_dim == 64) return launch_cs<64, 2>(p, s);
  return LVAR_EUNSUPPORTED;
}

}  // namespace lvar
