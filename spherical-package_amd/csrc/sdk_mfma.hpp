// MFMA helpers for gfx950: accumulator type, bf16 packing, register layouts.
//
// v_mfma_f32_32x32x2_f32 (wave64, lane l):
//   A operand: A[i = l % 32][k = l / 32]          B operand: B[k = l / 32][j = l % 32]
// v_mfma_f32_32x32x16_bf16: each lane supplies 8 bf16 per operand,
//   A[i = l % 32][k = 8 * (l / 32) + 0..7]         B[k = 8 * (l / 32) + 0..7][j = l % 32]
// D (both): 16 registers v, D[i = 8*(v/4) + 4*(l/32) + v%4][j = l % 32].
#pragma once
#include <hip/hip_runtime.h>

namespace sdk {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// Two floats -> two bf16 (round to nearest even) in one 32-bit word, `lo` in the low half.
__device__ __forceinline__ unsigned pack_bf16x2(float lo, float hi) {
  unsigned a = __float_as_uint(lo), b = __float_as_uint(hi);
  a += 0x7fffu + ((a >> 16) & 1u);
  b += 0x7fffu + ((b >> 16) & 1u);
  return (a >> 16) | (b & 0xffff0000u);
}

union Bf16Frag {
  bf16x8 v;
  unsigned u[4];
};

__device__ __forceinline__ Bf16Frag pack_bf16x8(const float (&f)[8]) {
  Bf16Frag r;
#pragma unroll
  for (int i = 0; i < 4; ++i) r.u[i] = pack_bf16x2(f[2 * i], f[2 * i + 1]);
  return r;
}

__device__ __forceinline__ floatx16 mfma_bf16(const Bf16Frag& a, const Bf16Frag& b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c, 0, 0, 0);
}

}  // namespace sdk
