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

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// Two floats -> two bf16 (round to nearest even) in one 32-bit word, `lo` in the low half:
// the packed conversion instruction of gfx950 (v_cvt_pk_bf16_f32) instead of five integer
// operations per pair.
__device__ __forceinline__ unsigned pack_bf16x2(float lo, float hi) {
  const f32x2 v = {lo, hi};
  const bf16x2 r = __builtin_convertvector(v, bf16x2);
  return __builtin_bit_cast(unsigned, r);
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

// Eight floats as three bf16 fragments whose sum is the float exactly: hi = the top 8 mantissa
// bits (truncated), mid = the top 8 bits of the remainder, lo = the rest.  Each remainder is
// exact in fp32 (it has at most 16, then 8, significant bits), so a product of two floats is
// the sum of nine piece products, each exact in the matrix unit's fp32 accumulator.
struct Bf16Split {
  Bf16Frag hi, mid, lo;
};

__device__ __forceinline__ Bf16Split split_bf16x8(const float (&f)[8]) {
  unsigned h[8], m[8], l[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    h[i] = __float_as_uint(f[i]) & 0xffff0000u;
    const float r = f[i] - __uint_as_float(h[i]);
    m[i] = __float_as_uint(r) & 0xffff0000u;
    const float r2 = r - __uint_as_float(m[i]);
    l[i] = __float_as_uint(r2) & 0xffff0000u;
  }
  Bf16Split s;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    s.hi.u[i] = (h[2 * i] >> 16) | h[2 * i + 1];
    s.mid.u[i] = (m[2 * i] >> 16) | m[2 * i + 1];
    s.lo.u[i] = (l[2 * i] >> 16) | l[2 * i + 1];
  }
  return s;
}

__device__ __forceinline__ floatx16 mfma_bf16(const Bf16Frag& a, const Bf16Frag& b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.v, b.v, c, 0, 0, 0);
}

// c += a * b from the six largest of the nine piece products (smallest first); the three left
// out (mid*lo, lo*mid, lo*lo) are below 2^-23 of the product.
__device__ __forceinline__ floatx16 mfma_split(const Bf16Split& a, const Bf16Split& b, floatx16 c) {
  c = mfma_bf16(a.lo, b.hi, c);
  c = mfma_bf16(a.hi, b.lo, c);
  c = mfma_bf16(a.mid, b.mid, c);
  c = mfma_bf16(a.mid, b.hi, c);
  c = mfma_bf16(a.hi, b.mid, c);
  return mfma_bf16(a.hi, b.hi, c);
}

// Matrix arithmetic of a fused kernel: fp32 MFMA, operands rounded to bf16, or fp32 operands
// split into bf16 pieces (fp32 accuracy on the bf16 matrix unit).
constexpr int kMmF32 = 0, kMmBf16 = 1, kMmSplit = 2;

}  // namespace sdk
