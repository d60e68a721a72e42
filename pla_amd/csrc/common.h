// Shared host/device helpers for the gfx950 gated delta-rule kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <cstdarg>
#include <cstdio>

#include "../../include/pla_gfx950.h"

namespace pla {

// ---- error reporting (host) -------------------------------------------------
char* error_buffer();   // thread-local, 512 bytes
inline int fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return 1;
}
inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail("%s: %s", what, hipGetErrorString(e));
  return 0;
}
#define PLA_REQUIRE(cond, ...) \
  do { if (!(cond)) return ::pla::fail(__VA_ARGS__); } while (0)

// ---- 16-bit activation types -------------------------------------------------
struct bf16_t { uint16_t bits; };
struct f16_t  { uint16_t bits; };

__device__ __forceinline__ float to_float(bf16_t x) {
  return __builtin_bit_cast(float, (uint32_t)x.bits << 16);
}
__device__ __forceinline__ float to_float(f16_t x) {
  return (float)__builtin_bit_cast(_Float16, x.bits);
}
template <typename T> __device__ __forceinline__ T from_float(float f);
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float f) {
  return bf16_t{__builtin_bit_cast(uint16_t, (__bf16)f)};   // v_cvt_pk_bf16_f32, round to nearest even
}
template <> __device__ __forceinline__ f16_t from_float<f16_t>(float f) {
  return f16_t{__builtin_bit_cast(uint16_t, (_Float16)f)};
}

// Low / high half of a packed pair of 16-bit activations.
template <typename T> __device__ __forceinline__ float lo16(uint32_t w) { return to_float(T{(uint16_t)(w & 0xffffu)}); }
template <typename T> __device__ __forceinline__ float hi16(uint32_t w) { return to_float(T{(uint16_t)(w >> 16)}); }
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
// Two floats rounded (nearest even) and packed, `a` in the low half.
template <typename T> __device__ __forceinline__ uint32_t pack2(float a, float b);
template <> __device__ __forceinline__ uint32_t pack2<bf16_t>(float a, float b) {
  const f32x2_t v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));   // one v_cvt_pk_bf16_f32
}
template <> __device__ __forceinline__ uint32_t pack2<f16_t>(float a, float b) {
  const f32x2_t v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
}

// ---- DPP cross-lane sums -----------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float x) {
  return __builtin_bit_cast(float,
      __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}
// Sum over each aligned group of 16 lanes; every lane of the group gets the total.
__device__ __forceinline__ float row16_allreduce(float x) {
  x += dpp_mov<0xB1>(x);    // quad_perm [1,0,3,2]
  x += dpp_mov<0x4E>(x);    // quad_perm [2,3,0,1]
  x += dpp_mov<0x141>(x);   // row_half_mirror
  x += dpp_mov<0x140>(x);   // row_mirror
  return x;
}
// Cross-row exchanges use the gfx950 lane-swap instructions through inline asm
// (inline asm keeps both results of the swap in plain scalar registers).  The s_nop pairs cover the VALU -> lane-swap
// and lane-swap -> VALU wait states that the hazard recogniser cannot see
// inside an asm statement.
struct LanePair { float lo, hi; };
// lo: the value held by lanes 0-31 (replicated to all lanes), hi: by lanes 32-63.
__device__ __forceinline__ LanePair swap_halves(float x) {
  float a = x, b = x;
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return LanePair{a, b};
}
// lo: the value of the even DPP row of each row pair, hi: of the odd DPP row.
__device__ __forceinline__ LanePair swap_rows16(float x) {
  float a = x, b = x;
  asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return LanePair{a, b};
}

// Sum over each aligned group of 32 lanes (one state row); every lane gets the total.
__device__ __forceinline__ float row32_allreduce(float x) {
  const LanePair r = swap_rows16(row16_allreduce(x));
  return r.lo + r.hi;
}

// Sum over the whole 64-lane wavefront; every lane gets the total.
__device__ __forceinline__ float wave64_allreduce(float x) {
  const LanePair r = swap_halves(row32_allreduce(x));
  return r.lo + r.hi;
}

__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }     // v_rcp_f32, 1 ulp
__device__ __forceinline__ float fast_rsqrt(float x) { return __builtin_amdgcn_rsqf(x); }  // v_rsq_f32, 1 ulp
__device__ __forceinline__ float fast_sigmoid(float x) { return fast_rcp(1.0f + __expf(-x)); }

}  // namespace pla
