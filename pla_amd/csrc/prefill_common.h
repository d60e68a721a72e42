// Pieces shared by the GDN and KDA chunk-64 prefill kernels: MFMA wrappers, bf16 hi/lo
// splitting, operand access for v_mfma_f32_16x16x32_bf16 and the device-side chunk table.
#pragma once

#include "common.h"

namespace pla {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x8_t __attribute__((ext_vector_type(8)));
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned u32x8_t __attribute__((ext_vector_type(8)));

constexpr int CHUNK = 64;

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

// A (or B) operand of one 16x16x32 MFMA step from a row-major bf16 tile: lane (r = lane%16,
// kb = lane/16) takes columns [32s+4kb, +4) and [32s+16+4kb, +4) of row r, which is the
// contraction order in which an accumulator tile pair (row blocks 2s, 2s+1) presents its rows.
__device__ __forceinline__ bf16x8_t operand_from(const uint16_t* row_ptr, int s, int kb) {
  const uint2 p0 = *reinterpret_cast<const uint2*>(row_ptr + 32 * s + 4 * kb);
  const uint2 p1 = *reinterpret_cast<const uint2*>(row_ptr + 32 * s + 16 + 4 * kb);
  const uint4 u = make_uint4(p0.x, p0.y, p1.x, p1.y);
  return __builtin_bit_cast(bf16x8_t, u);
}

// LDS tile pitches (bf16 elements): rows stay 16-byte aligned and consecutive rows start 4 (128-wide)
// or 36 (64-wide) banks apart, which keeps the 8-byte operand reads of a wavefront conflict free.
constexpr int PITCH128 = 136;
constexpr int PITCH64 = 72;

// ---------------------------------------------------------------------------------------------
// Asynchronous global -> LDS tile copies (global_load_lds_dwordx4: no registers, no LDS store
// instructions).  Lane i of a wavefront writes its 16 bytes at (wave-uniform LDS base) + 16 i, so
// a padded tile is filled as linear memory in 1 KiB pieces; a lane whose slot falls into a row's
// padding re-reads the last 16 data bytes of that row (the padding is never read back).
//
// The copy is issued from inline assembly so that the compiler's wait-count bookkeeping does not
// see it (it would drain every outstanding copy before each LDS read).  Kernels wait by hand with
// wait_vmcnt<N>(), N = number of copies this wavefront issued after the one it needs: vector
// memory operations complete in issue order, and other memory operations issued in between only
// make such a wait longer than necessary, never shorter.
__device__ __forceinline__ void dma16(const char* gbase, uint32_t byte_offset, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :: "s"(lds_wave_base), "v"(byte_offset), "s"(gbase) : "memory", "m0");
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}
__device__ __forceinline__ uint32_t lds_address(const void* ptr) {
  return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)ptr;
}

// Copy plan for one padded LDS tile: ROWS rows of PITCH_B bytes whose first VALID_B bytes are data,
// filled from rows `row_pitch_b` apart in global memory by the WAVES wavefronts of a workgroup.
// Each wavefront issues PIECES / WAVES copies, wavefront 0 also the PIECES % WAVES left over, so the copy
// counts per wavefront are compile-time constants (EACH, FIRST).  The per-lane source offsets are
// computed once; rows beyond `last_row` re-read that row.
template <int ROWS, int PITCH_B, int VALID_B, int WAVES>
struct TileCopy {
  static constexpr int BYTES = ROWS * PITCH_B;
  static_assert(BYTES % 1024 == 0 && PITCH_B % 16 == 0 && VALID_B % 16 == 0, "tiles are filled in 1 KiB pieces");
  static constexpr int PIECES = BYTES / 1024;
  static constexpr int EACH = PIECES / WAVES;
  static constexpr int REST = PIECES % WAVES;
  static constexpr int FIRST = EACH + REST;
  uint32_t off[EACH > 0 ? EACH : 1];
  uint32_t off_rest[REST > 0 ? REST : 1];

  static __device__ __forceinline__ uint32_t source_offset(int piece, int lane, uint32_t row_pitch_b, int last_row) {
    const int at = 1024 * piece + 16 * lane;
    const int row = at / PITCH_B, cb = at - row * PITCH_B;
    return (uint32_t)min(row, last_row) * row_pitch_b + (uint32_t)min(cb, VALID_B - 16);
  }
  __device__ __forceinline__ void plan(uint32_t row_pitch_b, int last_row, int wave, int lane) {
#pragma unroll
    for (int j0 = 0; j0 < EACH; ++j0) off[j0] = source_offset(WAVES * j0 + wave, lane, row_pitch_b, last_row);
#pragma unroll
    for (int j = 0; j < REST; ++j) off_rest[j] = source_offset(WAVES * EACH + j, lane, row_pitch_b, last_row);
  }
  // `gbase` (wave-uniform) addresses row 0 of the source tile.
  __device__ __forceinline__ void issue(const void* tile, const char* gbase, int wave) const {
    const uint32_t base = lds_address(tile) + 1024u * wave;
#pragma unroll
    for (int j0 = 0; j0 < EACH; ++j0) dma16(gbase, off[j0], base + 1024u * WAVES * j0);
    if (wave == 0) {
#pragma unroll
      for (int j = 0; j < REST; ++j) dma16(gbase, off_rest[j], base + 1024u * (WAVES * EACH + j));
    }
  }
};

// Chunk table from cu_seqlens, built on the device so that no call reads offsets back to the host.
// Single workgroup.  seq_chunk_off[n] = first chunk of sequence n (seq_chunk_off[N] = total).
static __global__ void chunk_map_kernel(const int32_t* cu_seqlens, int N, int NC_max, int32_t* seq_chunk_off,
                                        int32_t* chunk_seq, int32_t* chunk_tok, int32_t* chunk_len) {
  if (threadIdx.x == 0) {
    int acc = 0;
    for (int n = 0; n < N; ++n) {
      seq_chunk_off[n] = acc;
      const int len = max(cu_seqlens[n + 1] - cu_seqlens[n], 0);
      acc += (len + CHUNK - 1) / CHUNK;
    }
    seq_chunk_off[N] = acc;
  }
  __syncthreads();
  for (int n = threadIdx.x; n < N; n += blockDim.x) {
    const int start = cu_seqlens[n];
    const int len = max(cu_seqlens[n + 1] - start, 0);
    const int c0 = seq_chunk_off[n];
    const int nc = (len + CHUNK - 1) / CHUNK;
    for (int c = 0; c < nc; ++c) {
      if (c0 + c >= NC_max) break;
      chunk_seq[c0 + c] = n;
      chunk_tok[c0 + c] = start + c * CHUNK;
      chunk_len[c0 + c] = min(CHUNK, len - c * CHUNK);
    }
  }
}

// Zero the rows of a dense [T, heads, 128] 16-bit output that lie beyond the last sequence.
static __global__ void zero_tail_kernel(uint16_t* o, const int32_t* cu_seqlens, int N, int T, int heads) {
  const int64_t first = (int64_t)cu_seqlens[N] * heads * 128;
  const int64_t total = (int64_t)T * heads * 128;
  for (int64_t i = first + (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x)
    o[i] = 0;
}

inline size_t align_up256(size_t x) { return (x + 255) & ~(size_t)255; }

}  // namespace pla
