// Shared device helpers for the gfx950 sparse-attention kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

namespace lvar {

typedef __bf16 bf16_t;
typedef bf16_t bf16x8 __attribute__((ext_vector_type(8)));
typedef bf16_t bf16x4 __attribute__((ext_vector_type(4)));
typedef bf16_t bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

#define LVAR_LDS __attribute__((address_space(3)))

// One 32x32x16 bf16 MFMA: D(32x32 f32) += A(32x16) * B(16x32).
// Lane l holds A row (l%32) and B column (l%32), both with k = 8*(l/32) .. +7.
// Accumulator register i of lane l is D[8*(i/4) + 4*(l/32) + (i%4)][l%32].
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Exchange between lane l and lane l^32 (one VALU op, no LDS traffic).
__device__ __forceinline__ float xhalf(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), false, false);
  // lower half receives (own, upper's); upper half receives (lower's, own)
  int other = (threadIdx.x & 32) ? r[0] : r[1];
  return __builtin_bit_cast(float, other);
}
__device__ __forceinline__ float xhalf_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), false, false);
  return __builtin_fmaxf(__builtin_bit_cast(float, (int)r[0]), __builtin_bit_cast(float, (int)r[1]));
}
__device__ __forceinline__ float xhalf_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), false, false);
  return __builtin_bit_cast(float, (int)r[0]) + __builtin_bit_cast(float, (int)r[1]);
}

// Sum over aligned groups of LANES lanes (8, 16 or 32), every lane of a group receiving the total: butterfly steps as
// data-parallel-primitive moves (swap inside pairs, swap of pairs inside quads, mirror inside 8, mirror inside 16), which
// pair the same partial sums as exchanges with lane^1, ^2, ^4, ^8 and so give the same bits, without the round trips
// through the LDS crossbar that a shuffle costs.
template <int LANES>
__device__ __forceinline__ float group_sum(float x) {
  static_assert(LANES == 8 || LANES == 16 || LANES == 32, "group size");
  auto mv = [](float v, auto ctrl) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), decltype(ctrl)::value, 0xf, 0xf, true));
  };
  x += mv(x, std::integral_constant<int, 0xB1>{});    // quad_perm [1,0,3,2]
  x += mv(x, std::integral_constant<int, 0x4E>{});    // quad_perm [2,3,0,1]
  x += mv(x, std::integral_constant<int, 0x141>{});   // row_half_mirror
  if constexpr (LANES >= 16) x += mv(x, std::integral_constant<int, 0x140>{});   // row_mirror
  if constexpr (LANES >= 32) x += __shfl_xor(x, 16, 64);
  return x;
}

__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  f32x2 f = {a, b};
  bf16x2 h = __builtin_convertvector(f, bf16x2);
  return __builtin_bit_cast(uint32_t, h);
}

__device__ __forceinline__ bf16x8 pack8(float a0, float a1, float a2, float a3, float a4, float a5, float a6, float a7) {
  u32x4 u = {pack_bf16(a0, a1), pack_bf16(a2, a3), pack_bf16(a4, a5), pack_bf16(a6, a7)};
  return __builtin_bit_cast(bf16x8, u);
}

__device__ __forceinline__ float bf16_lo(uint32_t u) { return __builtin_bit_cast(float, u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __builtin_bit_cast(float, u & 0xffff0000u); }

// Order-preserving map float -> uint32 (larger float <=> larger key); -0.0 and +0.0 get the same key (adding +0.0
// turns -0.0 into +0.0 and changes nothing else), so that they tie as they do in a comparison of the values.
__device__ __forceinline__ uint32_t sort_key(float x) {
  const uint32_t u = __builtin_bit_cast(uint32_t, x + 0.0f);
  return u ^ ((u >> 31) ? 0xffffffffu : 0x80000000u);
}

// Key of a real entry in the selection kernels: never 0, which is kept for entries that do not compete (padding
// columns, always-on blocks).  Only a NaN with every bit set maps to 0; it is lifted to 1.
__device__ __forceinline__ uint32_t real_key(float x) {
  const uint32_t k = sort_key(x);
  return k > 1u ? k : 1u;
}

// Transposing LDS read: the 16 lanes of a group each point at 4 consecutive bf16 of a row;
// lane i of the group receives element (i%4) of the rows addressed by lanes (i/4), (i/4)+4,
// (i/4)+8, (i/4)+12.  With lane s addressing row (s/4), columns 4*(s%4)..+3 of a 4x16 block,
// lane i ends up with column i of rows 0..3.
__device__ __forceinline__ bf16x4 lds_read_tr(const char* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4bf16((LVAR_LDS bf16x4*)(p));
}

}  // namespace lvar
