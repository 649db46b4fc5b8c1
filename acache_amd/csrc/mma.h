// Matrix-core helpers shared by the attention and importance kernels (gfx950, wave64).
//
// v_mfma_f32_16x16x32_{bf16,f16}: lane l of the A operand holds row l % 16, k = 8 * (l / 16) .. + 8; the B
// operand is laid out the same way over columns; element i of the result is row 4 * (l / 16) + i, column l % 16.
#pragma once
#include "common.h"

namespace acache {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

template <int DTYPE> struct Mma;
template <> struct Mma<ACACHE_BF16> {
  __device__ static __forceinline__ f32x4 run(const vec16 &a, const vec16 &b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
  // round-to-nearest-even pair conversion: one v_cvt_pk_bf16_f32 on gfx950
  __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
  }
};
template <> struct Mma<ACACHE_F16> {
  __device__ static __forceinline__ f32x4 run(const vec16 &a, const vec16 &b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
  __device__ static __forceinline__ uint32_t pack2(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, f16x2));
  }
};

// Rotate the (lo, hi) 16-byte chunk pair of one row: elements d0..d0+7 and
// d0+half..d0+half+7, half = head_dim / 2.  sign = +1: x*cos + rot_half(x)*sin (key side);
// sign = -1: x*cos - rot_half(x)*sin (query side).  Rounded once to DTYPE.
template <int DTYPE>
__device__ __forceinline__ void rotate_pair_half(vec16 &lo, vec16 &hi, const float *cos_row,
                                                 const float *sin_row, int d0, int half, float sign) {
  // products and sum rounded separately, exactly like the stand-alone relocation
  // kernel, so key-side attention and attention over a materialised copy see
  // bit-identical keys
#pragma clang fp contract(off)
  using E = Elem<DTYPE>;
  float a[8], b[8], ya[8], yb[8];
  E::unpack(lo, a);
  E::unpack(hi, b);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float cl = cos_row[d0 + j], sl = sign * sin_row[d0 + j];
    const float ch = cos_row[d0 + half + j], sh = sign * sin_row[d0 + half + j];
    ya[j] = a[j] * cl + (-b[j]) * sl;
    yb[j] = b[j] * ch + a[j] * sh;
  }
  lo = E::pack(ya);
  hi = E::pack(yb);
}

// The same rotation with the hardware pair conversions for the final rounding (round to nearest even, the
// result of Elem<DTYPE>::pack for every finite value; NaN payloads may differ) and the sign folded into the
// sine once: a third of the instructions, for the in-loop key-side rotation of the attention kernel.
template <int DTYPE>
__device__ __forceinline__ void rotate_pair_half_fast(vec16 &lo, vec16 &hi, const float *cos_row,
                                                      const float *sin_row, int d0, int half, float sign) {
#pragma clang fp contract(off)
  using E = Elem<DTYPE>;
  using M = Mma<DTYPE>;
  float a[8], b[8], ya[8], yb[8];
  E::unpack(lo, a);
  E::unpack(hi, b);
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float cl = cos_row[d0 + j], sl = sign * sin_row[d0 + j];
    const float ch = cos_row[d0 + half + j], sh = sign * sin_row[d0 + half + j];
    ya[j] = a[j] * cl + (-b[j]) * sl;
    yb[j] = b[j] * ch + a[j] * sh;
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    lo.w[j] = M::pack2(ya[2 * j], ya[2 * j + 1]);
    hi.w[j] = M::pack2(yb[2 * j], yb[2 * j + 1]);
  }
}

template <int DTYPE, int D>
__device__ __forceinline__ void rotate_pair(vec16 &lo, vec16 &hi, const float *cos_row,
                                            const float *sin_row, int d0, float sign) {
  rotate_pair_half<DTYPE>(lo, hi, cos_row, sin_row, d0, D / 2, sign);
}

}  // namespace acache
