// v_mfma_f32_16x16x32_bf16 wrapper and the bf16 hi/lo split that carries FP32 data through it.
// Operand layout: lane (r = lane % 16, kb = lane / 16) holds eight contraction elements of row r (A)
// or column r (B); the 16x16 FP32 result tile has lane (r, kb) holding rows 4 kb .. 4 kb + 3 of
// column r.  Any assignment of contraction elements to (kb, element) works as long as A and B agree.
#pragma once

#include "common.h"

namespace pla {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x8_t __attribute__((ext_vector_type(8)));
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned u32x8_t __attribute__((ext_vector_type(8)));

__device__ __forceinline__ f32x4_t mfma16(bf16x8_t a, bf16x8_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// hi = bf16(x), lo = bf16(x - hi) for two accumulator quads (eight contraction elements).
struct HiLo { bf16x8_t hi, lo; };
__device__ __forceinline__ HiLo split8(f32x4_t a, f32x4_t b) {
  const f32x8_t x = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
  HiLo r;
  r.hi = __builtin_convertvector(x, bf16x8_t);
  // widen the packed pairs back with one shift or mask each
  const u32x4_t w = __builtin_bit_cast(u32x4_t, r.hi);
  const u32x8_t wide = {w[0] << 16, w[0] & 0xffff0000u, w[1] << 16, w[1] & 0xffff0000u,
                        w[2] << 16, w[2] & 0xffff0000u, w[3] << 16, w[3] & 0xffff0000u};
  const f32x8_t back = __builtin_bit_cast(f32x8_t, wide);
  r.lo = __builtin_convertvector(x - back, bf16x8_t);
  return r;
}
__device__ __forceinline__ bf16x8_t round8(f32x4_t a, f32x4_t b) {
  const f32x8_t x = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
  return __builtin_convertvector(x, bf16x8_t);
}

// The same instruction shape with fp16 operands (v_mfma_f32_16x16x32_f16, same rate).  Operands travel as
// eight 16-bit lanes in a bf16x8_t container (loads, LDS reads and transposing reads do not care what the
// bits mean); half8 rounds two accumulator quads to fp16 (round to nearest even, 11 significant bits).
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
__device__ __forceinline__ f32x4_t mfma16h(bf16x8_t a, bf16x8_t b, f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}
__device__ __forceinline__ bf16x8_t half8(f32x4_t a, f32x4_t b) {
  const f32x8_t x = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
  return __builtin_bit_cast(bf16x8_t, __builtin_convertvector(x, f16x8_t));
}

}  // namespace pla
