// Measurement aid for bench.py, not part of the attention library: the bf16 MFMA rate this GPU sustains on a
// register-resident loop, with operands the caller provides (random or all-zero bits).  The published peak assumes
// the maximum engine clock; under a matrix load the clock follows the switching activity of the operands, so the
// sustained rate on random data is the ceiling any bf16 MFMA kernel on this box can approach.
#include "common.h"

using namespace lvar;

namespace {

// Every wave holds 8 A and 8 B fragments (read once from `src`, 16 B per lane and fragment) and runs
// iters x 16 MFMA 32x32x16 over four accumulators; the operand pair changes with every instruction.
__global__ __launch_bounds__(256, 2) void mfma_probe_kernel(const bf16_t* src, float* dst, int iters) {
  const int tid = threadIdx.x;
  bf16x8 a[8], b[8];
#pragma unroll
  for (int j = 0; j < 8; j++) {
    a[j] = *(const bf16x8*)(src + ((2 * j) * 256 + tid) * 8);
    b[j] = *(const bf16x8*)(src + ((2 * j + 1) * 256 + tid) * 8);
  }
  f32x16 acc[4];
#pragma unroll
  for (int m = 0; m < 4; m++)
#pragma unroll
    for (int i = 0; i < 16; i++) acc[m][i] = 0.f;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int j = 0; j < 16; j++) acc[j & 3] = mfma32(a[j & 7], b[(j * 3 + (j >> 3)) & 7], acc[j & 3]);
  }
  float s = 0.f;
#pragma unroll
  for (int m = 0; m < 4; m++)
#pragma unroll
    for (int i = 0; i < 16; i++) s += acc[m][i];
  dst[blockIdx.x * 256 + tid] = s;
}

}  // namespace

// src: 16 * 256 * 8 bf16 (64 KiB) of operand bits; dst: blocks * 256 floats.  Launches blocks x 256 threads;
// flops = blocks * 4 waves * iters * 16 * 32768.  Returns 0, or -1 for bad arguments, -3 if the launch failed.
extern "C" int lvar_probe_mfma(const void* src, void* dst, int blocks, int iters, void* stream) {
  if (!src || !dst || blocks <= 0 || iters <= 0) return -1;
  hipLaunchKernelGGL(mfma_probe_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)src, (float*)dst, iters);
  return hipGetLastError() == hipSuccess ? 0 : -3;
}
