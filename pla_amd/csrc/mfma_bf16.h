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
// Saturating roundings: a magnitude beyond the fp16 range becomes the largest finite fp16 (65504), never an
// infinity, so that out-of-range operands degrade the result instead of turning it into NaN.
//   half8_sat   round to nearest even after a clamp to +-65504 (one v_med3_f32 per element)
//   half8_rtz   round toward zero (v_cvt_pkrtz_f16_f32 saturates by itself); the error is one-sided, up to one
//               unit in the last place, which is fine where many roundings average (the state slices) or where
//               a low part follows
//   half8_pair  hi = nearest after the clamp, lo = the rest rounded toward zero: x to about 22 bits, hi + lo
//               saturating at 2 x 65504.  (hi is rounded to nearest so that values in fp16's subnormal range,
//               where lo underflows to zero, keep an unbiased error.)
typedef __fp16 fp16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ bf16x8_t half8_sat(f32x4_t a, f32x4_t b) {
  auto c = [](float v) { return __builtin_amdgcn_fmed3f(v, -65504.f, 65504.f); };
  return half8(f32x4_t{c(a.x), c(a.y), c(a.z), c(a.w)}, f32x4_t{c(b.x), c(b.y), c(b.z), c(b.w)});
}
__device__ __forceinline__ bf16x8_t half8_rtz(f32x4_t a, f32x4_t b) {
  const u32x4_t w = {__builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(a.x, a.y)),
                     __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(a.z, a.w)),
                     __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(b.x, b.y)),
                     __builtin_bit_cast(unsigned, __builtin_amdgcn_cvt_pkrtz(b.z, b.w))};
  return __builtin_bit_cast(bf16x8_t, w);
}
struct HalfPair { bf16x8_t hi, lo; };
__device__ __forceinline__ HalfPair half8_pair(f32x4_t a, f32x4_t b) {
  HalfPair r;
  r.hi = half8_sat(a, b);
  const f32x8_t back = __builtin_convertvector(__builtin_bit_cast(f16x8_t, r.hi), f32x8_t);
  r.lo = half8_rtz(f32x4_t{a.x - back[0], a.y - back[1], a.z - back[2], a.w - back[3]},
                   f32x4_t{b.x - back[4], b.y - back[5], b.z - back[6], b.w - back[7]});
  return r;
}
// Two floats rounded toward zero to fp16 and packed, `x` in the low half (saturating, exact for values fp16 holds).
__device__ __forceinline__ uint32_t pack2_rtz(float x, float y) {
  return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(x, y));
}
// Two floats as a packed (hi, lo) fp16 pair each: hi to nearest after a clamp, the rest toward zero in `lo`.
__device__ __forceinline__ void pack2_pair(float x, float y, uint32_t& hi, uint32_t& lo) {
  const f32x2_t c = {__builtin_amdgcn_fmed3f(x, -65504.f, 65504.f), __builtin_amdgcn_fmed3f(y, -65504.f, 65504.f)};
  const f16x2_t h = __builtin_convertvector(c, f16x2_t);
  hi = __builtin_bit_cast(uint32_t, h);
  lo = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(x - (float)h[0], y - (float)h[1]));
}

}  // namespace pla
