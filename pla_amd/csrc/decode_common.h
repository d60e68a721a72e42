// Device helpers shared by the k-last decode kernels: typed loads of activations, streaming access to
// 128x128 FP32 state tiles, the per-row delta-rule step and the gate.
#pragma once

#include "common.h"

namespace pla {

// ---- branch-free loads of inputs whose element type is a run-time property -------------
// Every load below is issued unconditionally (addresses are selected, not branches), so
// the compiler never has to close a basic block - and drain the memory counter - between
// the small activation loads and the sixteen state-tile loads that follow them.

// One scalar stored as float32 (wide) or as a 16-bit float: two 16-bit loads.
struct RawScalar { uint32_t lo, hi; };
__device__ __forceinline__ RawScalar fetch_scalar(const void* p, bool wide, int64_t i) {
  const char* b = reinterpret_cast<const char*>(p) + i * (wide ? 4 : 2);
  RawScalar r;
  r.lo = *reinterpret_cast<const uint16_t*>(b);
  r.hi = *reinterpret_cast<const uint16_t*>(b + (wide ? 2 : 0));
  return r;
}
__device__ __forceinline__ float decode_scalar(RawScalar r, int dtype) {
  const float wide = __builtin_bit_cast(float, r.lo | (r.hi << 16));
  const float b16 = to_float(bf16_t{(uint16_t)r.lo});
  const float h16 = to_float(f16_t{(uint16_t)r.lo});
  return dtype == PLA_F32 ? wide : (dtype == PLA_BF16 ? b16 : h16);
}
template <typename act_t>
__device__ __forceinline__ float decode_scalar_act(RawScalar r, bool wide) {
  const float w = __builtin_bit_cast(float, r.lo | (r.hi << 16));
  const float n = to_float(act_t{(uint16_t)r.lo});
  return wide ? w : n;
}

// The lane's four K channels [4c, 4c+4) of a 128-wide row stored as float32 (wide, 16 bytes)
// or as 16-bit activations (8 bytes): two 8-byte loads (the second is a duplicate when narrow).
struct RawK4 { uint2 a, b; };
__device__ __forceinline__ RawK4 fetch_k4(const void* row, bool wide, int c) {
  const char* p = reinterpret_cast<const char*>(row) + c * (wide ? 16 : 8);
  RawK4 r;
  r.a = *reinterpret_cast<const uint2*>(p);
  r.b = *reinterpret_cast<const uint2*>(p + (wide ? 8 : 0));
  return r;
}
template <typename act_t>
__device__ __forceinline__ void decode_k4(const RawK4& r, bool wide, float (&x)[4]) {
  x[0] = wide ? __builtin_bit_cast(float, r.a.x) : lo16<act_t>(r.a.x);
  x[1] = wide ? __builtin_bit_cast(float, r.a.y) : hi16<act_t>(r.a.x);
  x[2] = wide ? __builtin_bit_cast(float, r.b.x) : lo16<act_t>(r.a.y);
  x[3] = wide ? __builtin_bit_cast(float, r.b.y) : hi16<act_t>(r.a.y);
}
// Plain typed variants for inputs whose type is fixed.
template <typename act_t>
__device__ __forceinline__ void load_k4(const act_t* row, int c, float (&x)[4]) {
  const uint2 w = *reinterpret_cast<const uint2*>(row + 4 * c);
  x[0] = lo16<act_t>(w.x); x[1] = hi16<act_t>(w.x); x[2] = lo16<act_t>(w.y); x[3] = hi16<act_t>(w.y);
}
__device__ __forceinline__ void load_k4(const float* row, int c, float (&x)[4]) {
  const float4 w = *reinterpret_cast<const float4*>(row + 4 * c);
  x[0] = w.x; x[1] = w.y; x[2] = w.z; x[3] = w.w;
}

// Per-row scalars of the wave's RPW consecutive rows.  A lane of half `half`
// (lanes 0-31: 0, lanes 32-63: 1) owns rows rowbase + 2j + half, so it reads the
// RPW contiguous activations once (raw words) and later keeps element 2j + half.
template <int RPW>
__device__ __forceinline__ void load_row_words(const void* p, uint32_t (&w)[RPW / 2]) {
  static_assert(RPW == 8 || RPW == 16 || RPW == 32, "rows per wave");
#pragma unroll
  for (int i = 0; i < RPW / 8; ++i) {
    const uint4 q = reinterpret_cast<const uint4*>(p)[i];
    w[4 * i] = q.x; w[4 * i + 1] = q.y; w[4 * i + 2] = q.z; w[4 * i + 3] = q.w;
  }
}
template <typename act_t, int RPW>
__device__ __forceinline__ void row_scalars(const uint32_t (&w)[RPW / 2], int half, float (&x)[RPW / 2]) {
  const int sh = 16 * half;
#pragma unroll
  for (int j = 0; j < RPW / 2; ++j) x[j] = to_float(act_t{(uint16_t)(w[j] >> sh)});
}

// Lane 0 receives the odd rows' values from lane 32 and writes the wave's RPW
// outputs as one contiguous run.
template <typename act_t, int RPW>
__device__ __forceinline__ void store_row_scalars(act_t* p, int lane, const float (&x)[RPW / 2]) {
  uint32_t w[RPW / 2];
#pragma unroll
  for (int j = 0; j < RPW / 2; ++j) {
    const LanePair both = swap_halves(x[j]);   // even row from lanes 0-31, odd row from lanes 32-63
    w[j] = pack2<act_t>(both.lo, both.hi);
  }
  if (lane == 0) {
#pragma unroll
    for (int i = 0; i < RPW / 8; ++i)
      reinterpret_cast<uint4*>(p)[i] = make_uint4(w[4 * i], w[4 * i + 1], w[4 * i + 2], w[4 * i + 3]);
  }
}

// State tiles are streamed exactly once per call, so they are moved with raw
// buffer instructions carrying streaming cache hints: loads are non-temporal,
// stores non-temporal with agent-scope write-through.  On MI355X this raises
// the mixed read+write rate from ~5.0 TB/s (plain global accesses) to ~5.6 TB/s.
// The descriptor covers exactly one 64 KiB tile, so stray offsets cannot touch
// neighbouring slots.
typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef float v4f_t __attribute__((ext_vector_type(4)));
constexpr int kLoadPolicy = 2;        // nt
constexpr int kStorePolicy = 2 | 16;  // nt | sc1

// state_t is float or bf16_t (pools stored in bf16: the recurrence still runs in FP32, tiles are
// widened on load and rounded to nearest even on store).
template <typename state_t>
struct Tile {
  __amdgpu_buffer_rsrc_t rsrc;
  __device__ __forceinline__ explicit Tile(state_t* tile_base)
      : rsrc(__builtin_amdgcn_make_buffer_rsrc(tile_base, 0, 16384 * sizeof(state_t), 0x00020000)) {}
  // present == false: a tile of no bytes, every load from it returns zero (the range check of the buffer
  // instruction), so a kernel can issue the loads of an absent state without a branch
  __device__ __forceinline__ Tile(state_t* tile_base, bool present)
      : rsrc(__builtin_amdgcn_make_buffer_rsrc(tile_base, 0, present ? 16384 * (int)sizeof(state_t) : 0, 0x00020000)) {}
};
typedef int v2i_t __attribute__((ext_vector_type(2)));

// `lane_off` is the lane's byte offset of (rowbase + half, channel 4c) inside the
// tile; consecutive j are two rows (1 KiB) apart, so each instruction of the
// wave moves 1 KiB of contiguous memory.
template <int R>
__device__ __forceinline__ void load_state(const Tile<float>& t, int lane_off, float (&s)[R][4]) {
#pragma unroll
  for (int j = 0; j < R; ++j) {
    // Whole-vector bit cast: a bit cast applied to a single vector component reads component 0.
    const v4f_t v = __builtin_bit_cast(
        v4f_t, __builtin_amdgcn_raw_buffer_load_b128(t.rsrc, lane_off + j * 1024, 0, kLoadPolicy));
    s[j][0] = v.x; s[j][1] = v.y; s[j][2] = v.z; s[j][3] = v.w;
  }
}
template <int R>
__device__ __forceinline__ void store_state(const Tile<float>& t, int lane_off, const float (&s)[R][4]) {
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const v4f_t v = {s[j][0], s[j][1], s[j][2], s[j][3]};
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4i_t, v), t.rsrc, lane_off + j * 1024, 0, kStorePolicy);
  }
}

// bf16 pools: `lane_off` stays the FP32 byte offset; a bf16 tile is half as large, so an instruction
// of the wave moves two adjacent rows = 512 bytes.
template <int R>
__device__ __forceinline__ void load_state(const Tile<bf16_t>& t, int lane_off, float (&s)[R][4]) {
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const v2i_t v = __builtin_bit_cast(
        v2i_t, __builtin_amdgcn_raw_buffer_load_b64(t.rsrc, (lane_off >> 1) + j * 512, 0, kLoadPolicy));
    s[j][0] = lo16<bf16_t>((uint32_t)v.x); s[j][1] = hi16<bf16_t>((uint32_t)v.x);
    s[j][2] = lo16<bf16_t>((uint32_t)v.y); s[j][3] = hi16<bf16_t>((uint32_t)v.y);
  }
}
template <int R>
__device__ __forceinline__ void store_state(const Tile<bf16_t>& t, int lane_off, const float (&s)[R][4]) {
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const v2i_t v = {(int)pack2<bf16_t>(s[j][0], s[j][1]), (int)pack2<bf16_t>(s[j][2], s[j][3])};
    __builtin_amdgcn_raw_buffer_store_b64(v, t.rsrc, (lane_off >> 1) + j * 512, 0, kStorePolicy);
  }
}

// decay -> S.k -> delta -> rank-1 update (-> S.q) on the lane's R rows.
template <int R, bool PER_CHANNEL, bool WANT_OUT>
__device__ __forceinline__ void delta_rows(float (&s)[R][4], const float (&dec)[4], float dec_scalar,
                                           const float (&kv)[4], const float (&qv)[4],
                                           const float (&vv)[R], float beta, float (&out)[R]) {
#pragma unroll
  for (int j = 0; j < R; ++j) {
    float d = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      s[j][e] *= PER_CHANNEL ? dec[e] : dec_scalar;
      d = fmaf(s[j][e], kv[e], d);
    }
    d = row32_allreduce(d);
    const float u = (vv[j] - d) * beta;
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      s[j][e] = fmaf(u, kv[e], s[j][e]);
      if (WANT_OUT) acc = fmaf(s[j][e], qv[e], acc);
    }
    if (WANT_OUT) out[j] = row32_allreduce(acc);
  }
}

__device__ __forceinline__ float gate_decay(float a, float dt, float eA, float p0, float thr, int mode) {
  if (mode == PLA_GATE_LOG_DECAY) return __expf(a);
  const float x = a + dt;
  if (mode == PLA_GATE_LOWER_BOUND) return __expf(p0 * fast_sigmoid(eA * x));
  const float bx = p0 * x;
  const float sp = (bx <= thr) ? fast_rcp(p0) * __logf(1.0f + __expf(bx)) : x;
  return __expf(-eA * sp);
}

}  // namespace pla
