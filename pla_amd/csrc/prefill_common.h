// Pieces shared by the GDN and KDA chunk-64 prefill kernels: MFMA wrappers, bf16 hi/lo
// splitting, operand access for v_mfma_f32_16x16x32_bf16 and the device-side chunk table.
#pragma once

#include <mutex>

#include "common.h"
#include "mfma_bf16.h"

namespace pla {

constexpr int CHUNK = 64;

typedef short i16x4_t __attribute__((ext_vector_type(4)));

// One transposing read: lane i of a group of 16 receives column i of the four rows the group addresses (lane t
// addresses columns 4 (t % 4) .. + 3 of row t / 4), packed as 16-bit (row 0, row 1), (row 2, row 3).
__device__ __forceinline__ uint2 read_tr4(const uint16_t* at) {
  const i16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4_t*)at);
  return __builtin_bit_cast(uint2, v);
}

// Element r (0..3) of what read_tr4 returned, as FP32.
template <typename T> __device__ __forceinline__ float quad_element(uint2 w, int r) {
  const uint32_t pair = r < 2 ? w.x : w.y;
  return (r & 1) ? hi16<T>(pair) : lo16<T>(pair);
}

// Pitch of a padded 128-wide LDS tile (16-bit elements): rows stay 16-byte aligned and consecutive rows start 4 banks
// apart, which keeps the 8-byte reads of a wavefront conflict free.
constexpr int PITCH128 = 136;

// ---------------------------------------------------------------------------------------------
// W = (I + L)^-1 diag(beta) for a strictly lower triangular 64 x 64 L (FP32, in LDS) on ONE wavefront, by
// 16 x 16 blocks with the off-diagonal blocks on MFMA.  With N = (I + L)^-1: the diagonal blocks D_a = (I + L_aa)^-1 come from forward substitution over 16 rows
// (lane 16 a + j owns column j of D_a), the others from N_ab = -D_a sum_{b <= c < a} L_ac N_cb in order of
// a - b = 1, 2, 3 (13 products of 16 x 16 x 16 or 16 x 16 x 32).  FP32 values cross the MFMA as bf16
// hi/lo pairs (hi.hi + hi.lo + lo.hi, error ~2^-16 per product).  L is used as workspace: D_a replaces
// L_aa, D_b^T is parked in the unused block (b, b + 1) where lanes read it as a B operand, N_ab replaces
// L_ab, and the fp16 tile leaves in 16-byte pieces (8 rows of 128 bytes per store instruction).  Only the
// strictly lower triangle of L is read.
__device__ __forceinline__ f32x4_t mfma_hilo(const HiLo& a, const HiLo& b, f32x4_t c) {
  c = mfma16(a.lo, b.hi, c);
  c = mfma16(a.hi, b.lo, c);
  return mfma16(a.hi, b.hi, c);
}

// block_inverse_inplace leaves N = (I + L)^-1 in the lower triangle of L (the blocks above the diagonal hold
// scratch); the two functions after it scale by beta and store W in one of two layouts.
__device__ __forceinline__ void block_inverse_inplace(float (*L)[68], int lane) {
  const int r16 = lane & 15, kb = lane >> 4;
  const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
  {
    // diagonal blocks: x_i = [i == j] - sum_{l < i} L_aa[i][l] x_l
    const int a = kb, j = r16;
    float x[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
      for (int l4 = 0; l4 < i; l4 += 4) {
        const float4 row = *reinterpret_cast<const float4*>(&L[16 * a + i][16 * a + l4]);
        acc0 = fmaf(row.x, x[l4], acc0);
        if (l4 + 1 < i) acc1 = fmaf(row.y, x[l4 + 1], acc1);
        if (l4 + 2 < i) acc0 = fmaf(row.z, x[l4 + 2], acc0);
        if (l4 + 3 < i) acc1 = fmaf(row.w, x[l4 + 3], acc1);
      }
      x[i] = (i == j ? 1.f : 0.f) - (acc0 + acc1);
    }
    // all reads of L_aa are done (one wavefront, LDS operations complete in order)
#pragma unroll
    for (int i = 0; i < 16; ++i) L[16 * a + i][16 * a + j] = x[i];
    if (a < 3) {
#pragma unroll
      for (int i4 = 0; i4 < 16; i4 += 4)
        *reinterpret_cast<float4*>(&L[16 * a + j][16 * (a + 1) + i4]) = make_float4(x[i4], x[i4 + 1], x[i4 + 2], x[i4 + 3]);
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  // operands: A = rows of L (blocks c0 and, if c1 >= 0, c1 of block row a); lane (m, kb) holds columns 4 kb .. 4 kb + 3 of each
  auto quad = [&](int row, int col) {
    const float4 t = *reinterpret_cast<const float4*>(&L[row][col]);
    return f32x4_t{t.x, t.y, t.z, t.w};
  };
  auto a_rows = [&](int a, int c0, int c1) {
    return split8(quad(16 * a + r16, 16 * c0 + 4 * kb), c1 >= 0 ? quad(16 * a + r16, 16 * c1 + 4 * kb) : zero);
  };
  auto negate = [](f32x4_t t) { return f32x4_t{-t.x, -t.y, -t.z, -t.w}; };
  // D_b as a B operand half: rows 4 kb .. 4 kb + 3 of column r16, read from the transposed copy
  const f32x4_t D0 = quad(r16, 16 + 4 * kb), D1 = quad(16 + r16, 32 + 4 * kb), D2 = quad(32 + r16, 48 + 4 * kb);
  const HiLo AD1 = a_rows(1, 1, -1), AD2 = a_rows(2, 2, -1), AD3 = a_rows(3, 3, -1);
  const HiLo A32 = a_rows(3, 2, -1);
  // a - b = 1
  const f32x4_t Y10 = mfma_hilo(a_rows(1, 0, -1), split8(D0, zero), zero);
  const f32x4_t Y21 = mfma_hilo(a_rows(2, 1, -1), split8(D1, zero), zero);
  const f32x4_t Y32 = mfma_hilo(A32, split8(D2, zero), zero);
  const f32x4_t X10 = negate(mfma_hilo(AD1, split8(Y10, zero), zero));
  const f32x4_t X21 = negate(mfma_hilo(AD2, split8(Y21, zero), zero));
  const f32x4_t X32 = negate(mfma_hilo(AD3, split8(Y32, zero), zero));
  // a - b = 2
  const HiLo B0 = split8(D0, X10);                        // [D_0; N_10], shared by N_20 and N_30
  const f32x4_t Y20 = mfma_hilo(a_rows(2, 0, 1), B0, zero);
  const f32x4_t Y31 = mfma_hilo(a_rows(3, 1, 2), split8(D1, X21), zero);
  const f32x4_t X20 = negate(mfma_hilo(AD2, split8(Y20, zero), zero));
  const f32x4_t X31 = negate(mfma_hilo(AD3, split8(Y31, zero), zero));
  // a - b = 3
  f32x4_t Y30 = mfma_hilo(a_rows(3, 0, 1), B0, zero);
  Y30 = mfma_hilo(A32, split8(X20, zero), Y30);
  const f32x4_t X30 = negate(mfma_hilo(AD3, split8(Y30, zero), zero));
  // N_ab replaces L_ab (accumulator layout: lane (n, kb) holds rows 4 kb + r of column n)
  auto put = [&](int a, int b, f32x4_t t) {
#pragma unroll
    for (int r = 0; r < 4; ++r) L[16 * a + 4 * kb + r][16 * b + r16] = t[r];
  };
  put(1, 0, X10); put(2, 1, X21); put(3, 2, X32); put(2, 0, X20); put(3, 1, X31); put(3, 0, X30);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
}

// A lower triangular 64 x 64 tile as the A (or B) operands of the products that contract over its columns: only six
// of the eight 16 x 32 operand blocks hold anything (row block m, column half s: s = 0 for every m, s = 1 for
// m = 2, 3).  Block b is 1 KiB: lane (r, kb) owns 16 bytes, columns 32 s + 4 kb .. + 3 and 32 s + 16 + 4 kb .. + 3 of
// row 16 m + r, which is the contraction order in which a pair of accumulator tiles presents its rows.  A consumer
// copies the blocks to LDS as they are and reads an operand with one 16-byte access per lane.
constexpr int TRI_BLOCKS = 6;
__device__ __forceinline__ constexpr int tri_block_m(int b) { return b < 4 ? b : b - 2; }
__device__ __forceinline__ constexpr int tri_block_s(int b) { return b < 4 ? 0 : 1; }
// W = N diag(beta) from the tile block_inverse_inplace leaves, as an fp16 hi + lo pair in that layout: hi blocks at
// W, lo blocks at W + TRI_BLOCKS * 512 (halves).
__device__ __forceinline__ void store_w_operand_blocks(float (*L)[68], const float* beta, int lane, uint16_t* W) {
  const int r16 = lane & 15, kb = lane >> 4;
#pragma unroll
  for (int b = 0; b < TRI_BLOCKS; ++b) {
    const int i = 16 * tri_block_m(b) + r16;
    uint32_t hi[4], lo[4];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int j0 = 32 * tri_block_s(b) + 16 * half + 4 * kb;
      const float4 n4 = *reinterpret_cast<const float4*>(&L[i][j0]);
      const float4 b4 = *reinterpret_cast<const float4*>(&beta[j0]);
      const float w0 = j0 <= i ? n4.x * b4.x : 0.f, w1 = j0 + 1 <= i ? n4.y * b4.y : 0.f;
      const float w2 = j0 + 2 <= i ? n4.z * b4.z : 0.f, w3 = j0 + 3 <= i ? n4.w * b4.w : 0.f;
      pack2_pair(w0, w1, hi[2 * half], lo[2 * half]);
      pack2_pair(w2, w3, hi[2 * half + 1], lo[2 * half + 1]);
    }
    *reinterpret_cast<uint4*>(W + b * 512 + lane * 8) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    *reinterpret_cast<uint4*>(W + (TRI_BLOCKS + b) * 512 + lane * 8) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
  }
}

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
// A pointer whose value is the same in every lane, as a scalar: where the compiler holds such a value in vector
// registers (a value merged from two branches of one kernel, say) dma16 cannot take it as its base.
template <typename T>
__device__ __forceinline__ T* uniform_pointer(T* p) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a), hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  return reinterpret_cast<T*>(((uint64_t)hi << 32) | lo);
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}
// Workgroup barrier that orders LDS traffic only: this wavefront's LDS operations are complete before it arrives
// and the compiler moves no memory access across it, but vector memory operations (copies, loads, stores that
// nobody in the workgroup waits for) stay in flight.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
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

// ---------------------------------------------------------------------------------------------
// Unpadded, swizzled 64 x 128 tiles of 16-bit values (16 KiB).  A row is sixteen 16-byte granules; granule g of row i
// lies at granule g ^ (2 (i & 7)) of that row's 256 bytes.  Measured on gfx950 with all eight wavefronts of a workgroup
// reading: 16-byte operand reads (sixteen consecutive rows, one granule index) run at the LDS peak of 256 bytes per
// cycle and the transposing 8-byte reads (four rows x four 8-byte pieces per group of sixteen lanes) at the 128 bytes
// per cycle of 8-byte reads, where rows padded to 272 bytes give 85 (two 8-byte reads per operand) and 128.
//
// Operand tiles (K, Q) also permute the columns inside each group of 32 so that the eight contraction elements a lane
// feeds to one MFMA step - columns 32 s + 4 kb .. + 3 and 32 s + 16 + 4 kb .. + 3, the order in which a pair of
// accumulator tiles presents its rows - are the two halves of ONE granule, index 4 s + kb.
constexpr int TILE128_HALVES = CHUNK * 128;
__device__ __forceinline__ int swizzled_granule(int row, int g) { return g ^ (2 * (row & 7)); }
// offset (in 16-bit elements) of granule g of row `row`
__device__ __forceinline__ int tile_offset(int row, int g) { return row * 128 + 8 * swizzled_granule(row, g); }
// A (or B) operand of contraction step s for row `row` of an operand tile: one 16-byte read
__device__ __forceinline__ bf16x8_t operand_granule(const uint16_t* tile, int row, int s, int kb) {
  return __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(tile + tile_offset(row, 4 * s + kb)));
}
// The same operand from the TRANSPOSE of an operand tile: lane (r, kb) takes rows [32 s + 4 kb, + 4) and
// [32 s + 16 + 4 kb, + 4) of original column 16 m + r.  Lane t of a group of 16 addresses the four columns
// 16 m + 4 (t % 4) .. + 3 of row base + t / 4, which are half (m & 1) of granule 4 (m / 2) + t % 4.
__device__ __forceinline__ bf16x8_t operand_granule_transposed(const uint16_t* tile, int s, int m, int kb, int r) {
  const int row = 32 * s + 4 * kb + (r >> 2);                  // (row + 16) & 7 == row & 7: both reads share the swizzle
  const uint16_t* at = tile + tile_offset(row, 4 * (m >> 1) + (r & 3)) + 4 * (m & 1);
  const i16x4_t p0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4_t*)at);
  const i16x4_t p1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4_t*)(at + 16 * 128));
  typedef short i16x8_t __attribute__((ext_vector_type(8)));
  const i16x8_t u = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
  return __builtin_bit_cast(bf16x8_t, u);
}
// Copy plan for a swizzled 64 x 128 tile whose columns keep their order (V): a 1 KiB piece is four rows, lane i of
// the issuing wavefront fills physical granule i % 16 of row 4 piece + i / 16, which holds granule
// (i % 16) ^ swizzle of that row.  Rows beyond `last_row` re-read that row.
template <int WAVES>
struct SwizzledTileCopy {
  static constexpr int PIECES = TILE128_HALVES * 2 / 1024;
  static_assert(PIECES % WAVES == 0, "every wavefront issues the same number of copies");
  static constexpr int EACH = PIECES / WAVES;
  uint32_t off[EACH];
  __device__ __forceinline__ void plan(uint32_t row_pitch_b, int last_row, int wave, int lane) {
#pragma unroll
    for (int j = 0; j < EACH; ++j) {
      const int row = 4 * (WAVES * j + wave) + (lane >> 4);
      off[j] = (uint32_t)min(row, last_row) * row_pitch_b + 16u * (uint32_t)swizzled_granule(row, lane & 15);
    }
  }
  __device__ __forceinline__ void issue(const void* tile, const char* gbase, int wave) const {
    const uint32_t base = lds_address(tile) + 1024u * wave;
#pragma unroll
    for (int j = 0; j < EACH; ++j) dma16(gbase, off[j], base + 1024u * WAVES * j);
  }
};

// Chunk table from cu_seqlens, built on the device so that no call reads offsets back to the host.
// Single workgroup.  seq_chunk_off[n] = first chunk of sequence n (seq_chunk_off[N] = total).
__device__ __forceinline__ void chunk_map(const int32_t* cu_seqlens, int N, int NC_max, int32_t* seq_chunk_off,
                                          int32_t* chunk_seq, int32_t* chunk_tok, int32_t* chunk_len) {
  // exclusive scan of the chunk counts by the first wavefront, 64 sequences per trip to memory (a serial loop
  // over the sequences would pay one memory latency per sequence)
  if (threadIdx.x < 64) {
    const int lane0 = threadIdx.x;
    int carry = 0;
    for (int base = 0; base < N; base += 64) {
      const int n = base + lane0;
      int nc = 0;
      if (n < N) nc = (max(cu_seqlens[n + 1] - cu_seqlens[n], 0) + CHUNK - 1) / CHUNK;
      int incl = nc;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d, 64);
        if (lane0 >= d) incl += up;
      }
      if (n < N) seq_chunk_off[n] = carry + incl - nc;
      carry += __shfl(incl, 63, 64);
    }
    if (lane0 == 0) seq_chunk_off[N] = carry;
  }
  __syncthreads();
  // one wavefront per sequence, its lanes stride over the chunks
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  for (int n = wave; n < N; n += waves) {
    const int start = cu_seqlens[n];
    const int len = max(cu_seqlens[n + 1] - start, 0);
    const int c0 = seq_chunk_off[n];
    const int nc = (len + CHUNK - 1) / CHUNK;
    for (int c = lane; c < nc && c0 + c < NC_max; c += 64) {
      chunk_seq[c0 + c] = n;
      chunk_tok[c0 + c] = start + c * CHUNK;
      chunk_len[c0 + c] = min(CHUNK, len - c * CHUNK);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Splitting long sequences into segments, for calls with too few (sequence, head) chains to fill the
// chip.  The per-token recurrence is affine in the state, S_out = S_in M + B, where for one segment
// B is the state the segment produces from a zero state and M (K x K) is what it produces from the
// identity with all values v = 0 (rows of the k-last state transform independently).  So:
//   pass 1   no output.  A first segment runs from the caller's state, keeps a copy of it and delivers the state it
//            ends in (its B); every segment between the first and the last of its sequence runs twice, from zero
//            (-> B) and from the identity with v = 0 (-> M); the last segment does not run: nothing needs its summary
//   combine  per (sequence, head): S_in of every later segment, S <- S M + B in FP32
//   pass 2   every segment runs from its true S_in and writes o; the last one delivers the final state
// which costs three sweeps over a middle segment instead of one but runs them all concurrently.
struct SegmentTable {
  int32_t* seq_seg_off;   // [N + 1] first segment of each sequence
  int32_t* seg_seq;       // [segments] sequence of a segment
  int32_t* seg_c0;        // first chunk (global chunk index)
  int32_t* seg_nc;        // number of chunks
  float* M;               // [segment, head, 128, 128] transition matrices
  float* B;               // [segment, head, V, K] zero-state results (first segments: the state they end in)
  float* S;               // [segment, head, V, K] state entering the segment
  float* identity;        // [128, 128]
  int seg_chunks;         // chunks per segment (0: sequences are not split)
  int max_segments;
};

// ---------------------------------------------------------------------------------------------
// Stages: with enough chains to fill the chip the per-chunk preparation (which every CU works on) and
// the sequential sweep (one workgroup per chain, most of a CU idle) are pipelined.  Each sequence is cut
// into `stages` consecutive parts; stage s of the sweep needs only the preparation of stage s, so the
// preparation of stage s + 1 runs on a second stream underneath the sweep of stage s.  The state is
// carried from stage to stage through one [V, K] tile per chain.
struct StageTable {
  int32_t* order;         // [chunks] global chunk ids, all of stage 0 first, then stage 1, ...
  int32_t* stage_begin;   // [MAX_STAGES + 2]: offsets into `order` per stage, then (last word) the number of stages in effect
  float* carry;           // [N, heads, V, K] (whole sequences; segments carry in their own tiles)
  int stages;             // 0: not staged
};
constexpr int MAX_STAGES = 2;
// Chunks [stage_cut(nc, s, S), stage_cut(nc, s + 1, S)) of an item of `nc` chunks belong to stage s of the S stages in
// effect (stages beyond S are empty).
// The cut is described by a plan word: the number of stages in effect in its low byte and, above it, the sixteenths of
// an item's chunks that the first of TWO stages takes.  Whoever sees the lengths on the device makes the plan
// (stage_plan): one stage when the chains are of nearly equal length (their chunks fill 80 % or more of `items x
// longest chain`: no CU falls idle before a sweep ends, so a later preparation would not run underneath it); else
// the stages the host allowed, the first of two stages taking 3/8 of every chain when the chains fill less than
// 5/8 of that rectangle and half otherwise: the preparation of the first stage is exposed, that of the second hides
// under the first sweep only as far as chains that have ended leave CUs to it (measured, ms per call, first stage of
// 8 / 7 / 6 / 5 / 4 sixteenths: 0.440 / 0.434 / 0.428 / 0.434 / 0.443 at a fill of 0.57; at fills of 0.66 half is the
// better cut by 0.4-1.1 %, at 0.31 and 0.61 three eighths by 1.4-1.9 %).
__host__ __device__ __forceinline__ int stage_plan(int64_t total, int n_items, int longest, int S) {
  const int64_t rectangle = (int64_t)n_items * longest;
  if (S <= 0 || 5 * total >= 4 * rectangle) return 1 | (8 << 8);
  return S | ((S == 2 && 8 * total < 5 * rectangle ? 6 : 8) << 8);
}
__host__ __device__ __forceinline__ int plan_stages(int plan) { return plan & 0xff; }
__host__ __device__ __forceinline__ int stage_cut(int nc, int s, int plan) {
  const int S = plan & 0xff;
  if (S == 2 && s == 1) return (int)((int64_t)nc * (plan >> 8) / 16);
  return (int)((int64_t)nc * (s < S ? s : S) / S);
}

// Single workgroup of 256 threads with (stages + 1) * n_items_max + 1 words of LDS at `pair_begin`.  The items are sequences (`counts` null: item i holds chunks
// starts[i] .. starts[i + 1]) or segments (chunks starts[i] .. starts[i] + counts[i]); `n_items` is read
// on the device.  (Stage, item) pairs count their chunks, a serial prefix places them, then every pair
// writes its own chunk ids.
__device__ __forceinline__ void stage_map(const int32_t* starts, const int32_t* counts, const int32_t* n_items_ptr,
                                          int n_items_max, int NC_max, StageTable t, int32_t* pair_begin) {
  // pair_begin: [stages * n_items_max + 1], then n_items_max chunk counts
  const int S = t.stages;
  const int n_items = n_items_ptr ? min(*n_items_ptr, n_items_max) : n_items_max;
  int32_t* const count = pair_begin + S * n_items_max + 1;
  __shared__ int stages_in_effect;
  for (int i = threadIdx.x; i < n_items; i += blockDim.x) count[i] = counts ? counts[i] : starts[i + 1] - starts[i];
  __syncthreads();
  auto count_of = [&](int i) { return count[i]; };
  if (threadIdx.x == 0) {
    // The stages pay where chains of unequal length leave CUs idle for the later preparation to run on: with
    // chains of (nearly) equal length the chip stays full to the end of a sweep, the preparation of the next stage
    // runs after it either way, and the second pair of launches is pure overhead (measured on 8 x 2048 tokens:
    // 0.24 ms in one stage, 0.27 ms in two; on eight ragged sequences of 32 810 tokens 0.50 against 0.48 ms).
    // One stage then takes everything, the others stay empty.
    int64_t total = 0;
    int longest = 0;
    for (int i = 0; i < n_items; ++i) { total += count_of(i); longest = max(longest, count_of(i)); }
    const int E = stage_plan(total, n_items, longest, S);                  // the plan word: stages in effect and the cut
    stages_in_effect = E;
    t.stage_begin[MAX_STAGES + 1] = E;
    int k = 0;
    for (int s = 0; s < S; ++s) {
      t.stage_begin[s] = k;
      for (int i = 0; i < n_items; ++i) {
        const int nc = count_of(i);
        pair_begin[s * n_items + i] = k;
        k += stage_cut(nc, s + 1, E) - stage_cut(nc, s, E);
      }
    }
    t.stage_begin[S] = k;
  }
  __syncthreads();
  const int E = stages_in_effect;
  for (int pair = threadIdx.x >> 3; pair < S * n_items; pair += blockDim.x >> 3) {      // eight threads per pair
    const int s = pair / n_items, i = pair - s * n_items;
    const int nc = count_of(i), lo = stage_cut(nc, s, E), hi = stage_cut(nc, s + 1, E);
    const int base = pair_begin[pair];
    for (int cc = lo + (threadIdx.x & 7); cc < hi; cc += 8)
      if (base + cc - lo < NC_max) t.order[base + cc - lo] = starts[i] + cc;
  }
}
// Chunk handled by workgroup `index` of a per-chunk kernel: all chunks in order, or those of one stage.
__device__ __forceinline__ int staged_chunk(const StageTable& t, int stage, int index, int total_chunks) {
  if (t.stages == 0) return index < total_chunks ? index : -1;
  const int begin = t.stage_begin[stage], end = t.stage_begin[stage + 1];
  return begin + index < end ? t.order[begin + index] : -1;
}

// Workgroups are handed to the eight XCDs (each with an L2 of its own) round robin by index.  Workgroups that read
// the same tiles at the same time - the `group` value heads of one q/k head sweep the same K and Q - fetch them
// from memory once if they share an L2: this maps the hardware index onto a logical one such that the members
// of a group get indices that are equal modulo 8.  The grid must be xcd_grouped_grid(total, group); indices
// beyond `total` come back as -1.
constexpr int XCDS = 8;
inline unsigned xcd_grouped_grid(unsigned total, unsigned group) {
  const unsigned groups = (total + group - 1) / group;
  return (groups + XCDS - 1) / XCDS * XCDS * group;
}
__device__ __forceinline__ int xcd_grouped_index(int hw_index, int group, int total) {
  const int xcd = hw_index % XCDS, t = hw_index / XCDS;
  const int member = t % group, g = (t / group) * XCDS + xcd;
  const int logical = g * group + member;
  return logical < total ? logical : -1;
}

// What one workgroup of a sequential kernel sweeps: a whole sequence (pass 0, blockIdx = (sequence,
// head)) or one segment in one of the roles above (pass 1: blockIdx = (segment, head, from-identity
// flag); pass 2: (segment, head)); with stages (passes 0 and 1) only the part of it that belongs to
// `stage`, which may hold no chunk at all, the state being carried from stage to stage in a tile.
struct SweepRole {
  int n, head, c_begin, c_end;
  const float* init;      // [V, K] tile the state starts from (nullptr: zero)
  float* fin;             // [V, K] tile that receives the state at the end (nullptr: none)
  float* keep_init;       // [V, K] tile that receives a copy of the start state (nullptr: none)
  bool zero_v, active;
};
__device__ __forceinline__ SweepRole select_sweep(int pass, int heads, int N, const int32_t* seq_chunk_off,
                                                  const SegmentTable& seg, const StageTable& stg, int stage,
                                                  const float* h0, const int32_t* h0_indices,
                                                  int64_t h0_slot_stride, float* ht, const int32_t* ht_indices,
                                                  int64_t ht_slot_stride, int block = -1,
                                                  const int3 inline_chunks = int3{-1, 0, 0}) {
  // inline_chunks (pass 0 only, x >= 0): (first chunk, end chunk, stages in effect) of the workgroup's sequence worked
  // out by the caller (inline_sequences) instead of read from the tables
  // block: the logical workgroup index when the caller remaps blockIdx (see xcd_grouped_index), else blockIdx.x
  // Segments: the first sweep publishes no output at all (a first segment keeps a copy of its start state and only
  // delivers the state it ends in), the second sweep runs every segment with output.  The LAST segment of a sequence
  // has no part in the first sweep - nothing needs its summary -: the second sweep takes it from the state the combine
  // step (or, for a sequence of one segment, the caller) provides and delivers the final state itself.
  SweepRole r{};
  auto state_in = [&](int n, int head) -> const float* {
    const int slot = (h0 != nullptr) ? (h0_indices ? h0_indices[n] : n) : -1;
    return slot >= 0 ? h0 + (int64_t)slot * h0_slot_stride + (int64_t)head * 16384 : nullptr;
  };
  auto state_out = [&](int n, int head) -> float* {
    const int slot = (ht != nullptr) ? (ht_indices ? ht_indices[n] : n) : -1;
    return slot >= 0 ? ht + (int64_t)slot * ht_slot_stride + (int64_t)head * 16384 : nullptr;
  };
  float* carry = nullptr;
  if (pass == 0) {
    const int logical = block >= 0 ? block : (int)blockIdx.x;
    r.n = logical / heads;
    r.head = logical - r.n * heads;
    r.c_begin = inline_chunks.x >= 0 ? inline_chunks.x : seq_chunk_off[r.n];
    r.c_end = inline_chunks.x >= 0 ? inline_chunks.y : seq_chunk_off[r.n + 1];
    if (r.c_begin >= r.c_end) return r;              // empty sequence: state untouched, no output
    r.init = state_in(r.n, r.head);
    r.fin = state_out(r.n, r.head);
    if (stg.stages > 0) carry = stg.carry + ((int64_t)r.n * heads + r.head) * 16384;
  } else {
    const int logical = block >= 0 ? block : (int)blockIdx.x;
    const int item = pass == 1 ? (logical >> 1) : logical;
    const bool from_identity = pass == 1 && (logical & 1);
    const int s = item / heads;
    r.head = item - s * heads;
    if (s >= seg.seq_seg_off[N]) return r;
    r.n = seg.seg_seq[s];
    const bool first = s == seg.seq_seg_off[r.n], last = s + 1 == seg.seq_seg_off[r.n + 1];
    r.c_begin = seg.seg_c0[s];
    r.c_end = r.c_begin + seg.seg_nc[s];
    const int64_t tile = ((int64_t)s * heads + r.head) * 16384;
    if (pass == 1) {
      if (last) return r;
      if (first) {
        if (from_identity) return r;
        r.init = state_in(r.n, r.head);
        r.fin = seg.B + tile;                           // B of a first segment: the state entering the second
        carry = seg.B + tile;
        r.keep_init = seg.S + tile;
      } else {
        if (from_identity) { r.init = seg.identity; r.zero_v = true; r.fin = seg.M + tile; }
        else r.fin = seg.B + tile;
        carry = r.fin;
      }
    } else {
      // the state entering the segment: the caller's for a sequence of one segment, else the copy its first segment
      // kept or what the combine step stored
      r.init = (first && last) ? state_in(r.n, r.head) : seg.S + tile;
      if (last) r.fin = state_out(r.n, r.head);
    }
  }
  if (carry != nullptr && stg.stages > 0) {
    const int E = inline_chunks.x >= 0 ? inline_chunks.z : stg.stage_begin[MAX_STAGES + 1];   // the plan word (stage_plan)
    if (stage >= plan_stages(E)) return r;                                      // an empty stage: the one before it delivered the state
    const int nc = r.c_end - r.c_begin, c0 = r.c_begin;
    r.c_begin = c0 + stage_cut(nc, stage, E);
    r.c_end = c0 + stage_cut(nc, stage + 1, E);
    if (stage > 0) { r.init = carry; r.keep_init = nullptr; }      // the start state is kept by stage 0 only
    if (stage < plan_stages(E) - 1) r.fin = carry;
  }
  r.active = true;
  return r;
}

// ---------------------------------------------------------------------------------------------
// The same tables worked out by ONE wavefront in registers, for calls of whole sequences with at most 64
// sequences: lane n holds sequence n, prefix sums run over the lanes.  A kernel that does this at its start needs no
// table kernel before it (one launch and its gap less on the critical path of a call) and no dependent trips to
// memory for its tile: one load of cu_seqlens per lane.  The results equal chunk_map / stage_map / staged_chunk /
// select_sweep(pass 0) for the same offsets, including the rule that keeps a single stage for chains of nearly equal
// length.  All 64 lanes of the wavefront must call these functions together.
constexpr int INLINE_TABLE_SEQUENCES = 64;
__device__ __forceinline__ int wave_inclusive_scan(int x, int lane) {
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int up = __shfl_up(x, d, 64);
    if (lane >= d) x += up;
  }
  return x;
}
struct InlineSequences {
  int start, len, nc, off;      // this lane's sequence: first token, tokens, chunks, first chunk (global index)
  int total, E;                 // chunks of the call; the plan word (stage_plan)
};
__device__ __forceinline__ InlineSequences inline_sequences(const int32_t* cu_seqlens, int N, int stages, int lane) {
  InlineSequences q;
  const int a = lane < N ? cu_seqlens[lane] : 0, b = lane < N ? cu_seqlens[lane + 1] : 0;
  q.start = a;
  q.len = max(b - a, 0);
  q.nc = (q.len + CHUNK - 1) / CHUNK;
  const int incl = wave_inclusive_scan(q.nc, lane);
  q.off = incl - q.nc;
  q.total = __builtin_amdgcn_readlane(incl, 63);
  int longest = q.nc;
#pragma unroll
  for (int d = 32; d > 0; d >>= 1) longest = max(longest, __shfl_xor(longest, d, 64));
  longest = __builtin_amdgcn_readfirstlane(longest);
  q.E = stage_plan(q.total, N, longest, stages);
  return q;
}
// Chunk `index` of stage `stage` (all chunks in order when the call is not staged): its global chunk id, first token
// and length, or id -1 when the stage holds fewer chunks.
struct InlineTile { int cb, t0, len; };
__device__ __forceinline__ InlineTile inline_tile(const InlineSequences& q, int stage, int index, int NC_max, int lane) {
  InlineTile t{-1, 0, 0};
  if (stage >= plan_stages(q.E)) return t;
  const int lo = stage_cut(q.nc, stage, q.E), hi = stage_cut(q.nc, stage + 1, q.E);
  const int cnt = hi - lo;
  const int before = wave_inclusive_scan(cnt, lane) - cnt;
  const unsigned long long owner = __ballot(index >= before && index < before + cnt);
  if (owner == 0) return t;
  const int n = __builtin_amdgcn_readfirstlane(__ffsll((long long)owner) - 1);
  const int cc = __builtin_amdgcn_readlane(lo, n) + index - __builtin_amdgcn_readlane(before, n);
  const int cb = __builtin_amdgcn_readlane(q.off, n) + cc;
  if (cb >= NC_max) return t;                   // offsets that do not fit the workspace: the tile is skipped
  t.cb = cb;
  t.t0 = __builtin_amdgcn_readlane(q.start, n) + cc * CHUNK;
  t.len = min(CHUNK, __builtin_amdgcn_readlane(q.len, n) - cc * CHUNK);
  return t;
}

// Segments per sequence and the 128 x 128 identity.  Single workgroup, after chunk_map.
__device__ __forceinline__ void segment_map(const int32_t* seq_chunk_off, int N, SegmentTable t) {
  if (threadIdx.x < 64) {                     // exclusive scan of the segment counts, as in chunk_map
    const int lane0 = threadIdx.x;
    int carry = 0;
    for (int base = 0; base < N; base += 64) {
      const int n = base + lane0;
      int ns = 0;
      if (n < N) ns = (seq_chunk_off[n + 1] - seq_chunk_off[n] + t.seg_chunks - 1) / t.seg_chunks;
      int incl = ns;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d, 64);
        if (lane0 >= d) incl += up;
      }
      if (n < N) t.seq_seg_off[n] = carry + incl - ns;
      carry += __shfl(incl, 63, 64);
    }
    if (lane0 == 0) t.seq_seg_off[N] = carry;
  }
  for (int i = threadIdx.x; i < 128 * 128; i += blockDim.x) t.identity[i] = (i >> 7) == (i & 127) ? 1.f : 0.f;
  __syncthreads();
  for (int n = threadIdx.x; n < N; n += blockDim.x) {
    const int c0 = seq_chunk_off[n], nc = seq_chunk_off[n + 1] - c0, s0 = t.seq_seg_off[n];
    const int ns = (nc + t.seg_chunks - 1) / t.seg_chunks;
    for (int i = 0; i < ns; ++i) {
      if (s0 + i >= t.max_segments) break;
      t.seg_seq[s0 + i] = n;
      t.seg_c0[s0 + i] = c0 + i * t.seg_chunks;
      t.seg_nc[s0 + i] = min(t.seg_chunks, nc - i * t.seg_chunks);
    }
  }
}

// Eight workgroups of 256 threads per (sequence, head), each owning 16 rows of the state (rows transform
// independently): walks the sequence's segments and stores the state entering every later segment (the last one
// included: the second sweep carries it to the final state).  A step S <- S M + B is a 16 x 128 x 128 product per workgroup on the FP32 MFMA
// (v_mfma_f32_16x16x4_f32, exact products, FP32 accumulation): wavefront w owns columns 32 w .. 32 w + 31 as two
// accumulator tiles that start from B; the A operand is the workgroup's 16 rows of S from LDS (lane (r, kb) takes
// S[r][16 s + 4 kb + e] for step (s, e)), the B operand the matching row of M straight from memory (lane (c, kb):
// M[16 s + 4 kb + e][column c], 64 contiguous bytes per group of 16 lanes), all 64 loads of a step requested before
// the first product.
constexpr int COMBINE_SPLIT = 8;
static __global__ __launch_bounds__(256) void segment_combine_kernel(SegmentTable t, int heads, int chains) {
  // the eight workgroups of a chain read the same M tiles: on one XCD they come from memory once (xcd_grouped_index)
  const int logical = xcd_grouped_index(blockIdx.x, COMBINE_SPLIT, chains * COMBINE_SPLIT);
  if (logical < 0) return;
  const int part = logical % COMBINE_SPLIT;
  const int chain = logical / COMBINE_SPLIT;
  const int n = chain / heads, h = chain - n * heads;
  const int first = t.seq_seg_off[n], end = t.seq_seg_off[n + 1];
  if (end - first < 2) return;                 // a single segment starts from the caller's state
  __shared__ __align__(16) float S[16][132];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, kb = lane >> 4;
  const int col0 = 32 * wave + c;              // this lane's column of accumulator tile 0 (tile 1: + 16)
  // place of accumulator element (tile cb, row v) inside a [128, 128] tile
  auto at = [&](int cb, int v) { return (int64_t)(16 * part + 4 * kb + v) * 128 + col0 + 16 * cb; };
  f32x4_t acc[2];
  {
    const float* src = t.B + ((int64_t)first * heads + h) * 16384;
#pragma unroll
    for (int cb = 0; cb < 2; ++cb)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[cb][v] = src[at(cb, v)];
  }
  for (int seg = first + 1; seg < end; ++seg) {
    const int64_t tile = ((int64_t)seg * heads + h) * 16384;
    // the state entering this segment: to memory for the second sweep, to LDS as the A operand of this step
#pragma unroll
    for (int cb = 0; cb < 2; ++cb)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        t.S[tile + at(cb, v)] = acc[cb][v];
        S[4 * kb + v][col0 + 16 * cb] = acc[cb][v];
      }
    if (seg + 1 == end) break;                 // the last segment: nothing follows it
    // M rows and the B tile of this segment, requested before the barrier
    const float* Mt = t.M + tile;
    float m[2][32];
#pragma unroll
    for (int s8 = 0; s8 < 8; ++s8)
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int cb = 0; cb < 2; ++cb) m[cb][4 * s8 + e] = Mt[(int64_t)(16 * s8 + 4 * kb + e) * 128 + col0 + 16 * cb];
#pragma unroll
    for (int cb = 0; cb < 2; ++cb)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[cb][v] = t.B[tile + at(cb, v)];
    __syncthreads();
    float4 a[8];
#pragma unroll
    for (int s8 = 0; s8 < 8; ++s8) a[s8] = *reinterpret_cast<const float4*>(&S[c][16 * s8 + 4 * kb]);
#pragma unroll
    for (int s8 = 0; s8 < 8; ++s8)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float av = e == 0 ? a[s8].x : e == 1 ? a[s8].y : e == 2 ? a[s8].z : a[s8].w;
#pragma unroll
        for (int cb = 0; cb < 2; ++cb)
          acc[cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, m[cb][4 * s8 + e], acc[cb], 0, 0, 0);
      }
    __syncthreads();                           // every wavefront has read S before the next step overwrites it
  }
}

// Chunks per segment for a call of T tokens, N sequences and `heads` value heads: 0 (no split) unless
// the call has at most 64 chains and the segments would be at least 16 chunks long and at least two.
inline int pick_segment_chunks(int T, int N, int heads) {
  if ((int64_t)N * heads > 64) return 0;
  const int nc = T / CHUNK;
  int seg = (int)(((int64_t)nc * heads + 255) / 256);
  if (seg < 16) seg = 16;
  return 2 * seg > nc ? 0 : seg;
}
inline int max_segments(int T, int N, int seg_chunks) { return seg_chunks > 0 ? T / CHUNK / seg_chunks + N + 1 : 0; }

// Zero the rows of a dense [T, heads, 128] 16-bit output that lie beyond the last sequence (workgroup `block` of `blocks`).
__device__ __forceinline__ void zero_tail(uint16_t* o, const int32_t* cu_seqlens, int N, int T, int heads, int block, int blocks) {
  const int64_t first = (int64_t)cu_seqlens[N] * heads * 128;
  const int64_t total = (int64_t)T * heads * 128;
  for (int64_t i = first + (int64_t)block * blockDim.x + threadIdx.x; i < total; i += (int64_t)blocks * blockDim.x)
    o[i] = 0;
}

// All tables of a call in one launch.  Workgroup 0 builds the chunk table, then (split calls) the segment
// table, then (pipelined calls) the stage table; each step reads what the previous one wrote, through
// memory, after a device-scope fence and a barrier of that one workgroup.  The other workgroups zero the
// output rows beyond the last sequence.  Dynamic LDS: (stages + 1) * stage_items + 1 words.
constexpr int TABLE_WORKGROUPS = 1 + 64;
static __global__ __launch_bounds__(256) void prefill_tables_kernel(
    const int32_t* cu_seqlens, int N, int T, int NC_max, int32_t* seq_chunk_off, int32_t* chunk_seq,
    int32_t* chunk_tok, int32_t* chunk_len, SegmentTable seg, StageTable stg, int stage_items, uint16_t* o, int heads) {
  extern __shared__ int32_t table_lds[];
  if (blockIdx.x > 0) {
    zero_tail(o, cu_seqlens, N, T, heads, blockIdx.x - 1, gridDim.x - 1);
    return;
  }
  chunk_map(cu_seqlens, N, NC_max, seq_chunk_off, chunk_seq, chunk_tok, chunk_len);
  const bool segmented = seg.seg_chunks > 0;
  if (segmented) {
    __threadfence();
    __syncthreads();
    segment_map(seq_chunk_off, N, seg);
  }
  if (stg.stages > 0) {
    __threadfence();
    __syncthreads();
    stage_map(segmented ? seg.seg_c0 : seq_chunk_off, segmented ? seg.seg_nc : nullptr,
              segmented ? seg.seq_seg_off + N : nullptr, stage_items, NC_max, stg, table_lds);
  }
}
inline void launch_tables(hipStream_t s, const int32_t* cu_seqlens, int N, int T, int NC_max, int32_t* seq_chunk_off,
                          int32_t* chunk_seq, int32_t* chunk_tok, int32_t* chunk_len, const SegmentTable& seg,
                          const StageTable& stg, int stage_items, void* o, int heads) {
  const size_t lds = stg.stages > 0 ? (size_t)((stg.stages + 1) * stage_items + 1) * 4 : 0;
  hipLaunchKernelGGL(prefill_tables_kernel, dim3(TABLE_WORKGROUPS), dim3(256), lds, s, cu_seqlens, N, T, NC_max,
                     seq_chunk_off, chunk_seq, chunk_tok, chunk_len, seg, stg, stage_items,
                     reinterpret_cast<uint16_t*>(o), heads);
}

inline size_t align_up256(size_t x) { return (x + 255) & ~(size_t)255; }

// Side streams (default priority, non-blocking), each with its own fork / ready events.  A call takes one from
// its device's pool for the time it enqueues its launches and puts it back before it returns, so calls that
// are enqueued concurrently (host threads launching on different streams) never share a stream or an event,
// while consecutive calls reuse the same few objects: an event wait binds to the record that precedes it in
// the calling thread, and work queued on a reused side stream simply runs after the previous call's.  A side
// stream that has joined a graph capture stays part of it until the capture ends: only calls of that same
// capture may take it again (every staged call of one capture then shares one side stream), any other call
// passes it over.  Streams and events are created on first need and kept for the life of the process.  A call
// that finds no side stream (the pool is exhausted, or creation failed) is not staged: the lease is taken
// before the first launch, so nothing has been enqueued by then.
struct SideStream {
  hipStream_t stream;
  hipEvent_t fork;
  hipEvent_t ready[MAX_STAGES];
  bool busy;
};
class SideStreamLease {
 public:
  // caller: the stream the call launches on; wanted: false leaves the lease empty
  SideStreamLease(hipStream_t caller, bool wanted) : taken_(nullptr) {
    int dev = 0;
    if (!wanted || hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return;
    unsigned long long caller_capture = 0;
    const bool caller_capturing = capture_of(caller, &caller_capture);
    std::lock_guard<std::mutex> lock(guard());
    SideStream* const pool = pools()[dev];
    SideStream* idle = nullptr;
    for (int i = 0; i < POOL && taken_ == nullptr; ++i) {
      if (pool[i].stream == nullptr || pool[i].busy) continue;
      unsigned long long id = 0;
      if (!capture_of(pool[i].stream, &id)) { if (idle == nullptr) idle = &pool[i]; }
      else if (caller_capturing && id == caller_capture) taken_ = &pool[i];      // already part of the caller's capture
    }
    if (taken_ == nullptr) taken_ = idle;
    if (taken_ == nullptr)
      for (int i = 0; i < POOL; ++i)
        if (pool[i].stream == nullptr) {
          if (create(pool[i])) taken_ = &pool[i];
          break;
        }
    if (taken_ != nullptr) taken_->busy = true;
  }
  ~SideStreamLease() {
    if (taken_ == nullptr) return;
    std::lock_guard<std::mutex> lock(guard());
    taken_->busy = false;
  }
  SideStreamLease(const SideStreamLease&) = delete;
  SideStreamLease& operator=(const SideStreamLease&) = delete;
  SideStream* get() const { return taken_; }     // nullptr: not wanted, none could be created, or the pool is in use

 private:
  static constexpr int MAX_DEVICES = 64, POOL = 16;
  static std::mutex& guard() { static std::mutex m; return m; }
  static SideStream (*pools())[POOL] { static SideStream table[MAX_DEVICES][POOL] = {}; return table; }
  // true (and the capture's id) while the stream is part of an unfinished graph capture; a stream whose state
  // cannot be read counts as capturing with an id no caller has
  static bool capture_of(hipStream_t stream, unsigned long long* id) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamGetCaptureInfo(stream, &status, id) != hipSuccess) { *id = ~0ull; return true; }
    return status != hipStreamCaptureStatusNone;
  }
  static bool create(SideStream& t) {
    SideStream made{};
    if (hipStreamCreateWithFlags(&made.stream, hipStreamNonBlocking) != hipSuccess) return false;
    bool ok = hipEventCreateWithFlags(&made.fork, hipEventDisableTiming) == hipSuccess;
    for (int i = 0; i < MAX_STAGES && ok; ++i) ok = hipEventCreateWithFlags(&made.ready[i], hipEventDisableTiming) == hipSuccess;
    if (!ok) {                                   // give back what was created
      for (int i = 0; i < MAX_STAGES; ++i)
        if (made.ready[i] != nullptr) (void)hipEventDestroy(made.ready[i]);
      if (made.fork != nullptr) (void)hipEventDestroy(made.fork);
      (void)hipStreamDestroy(made.stream);
      return false;
    }
    t = made;
    return true;
  }
  SideStream* taken_;
};

// Plan of a mixed sweep (gdn_fused_sweep_mixed_kernel, kda_sweep_mixed_kernel: the chains of the longest sequences as
// two workgroups of 64 V columns each, first in the grid, the others whole, longest first, in one launch) for sequences that sweep `r[n]` chunks in one launch:
// order[] receives the sequences longest first, the return value is the number of leading ones whose chains are swept
// as two halves (0: sweep all chains whole).  The launch is priced in chunk times of a whole chain on an idle chip:
// a half takes `half_cost` (0.9 measured for GDN) of that, the launch lasts as long as its longest chain (or as the whole chains need on the CUs the
// halves leave them, or as all the work needs on all CUs), and a chunk takes up to `fill_cost` (17 % for GDN) longer as the chip fills (3.0
// us with a third of the CUs busy, 3.5 us with all of them: the sweeps share the memory system).  The split is taken
// where the price falls by 5 % or more.
constexpr int CUS = 256;
inline int mixed_sweep_plan(const int* r, int N, int HV, unsigned char* order, double half_cost = 0.9, double fill_cost = 0.17) {
  for (int n = 0; n < N; ++n) {
    int at = n;
    for (; at > 0 && r[order[at - 1]] < r[n]; --at) order[at] = order[at - 1];
    order[at] = (unsigned char)n;
  }
  double rest = 0, halves = 0;
  for (int n = 0; n < N; ++n) rest += r[n];
  if (rest == 0) return 0;
  double whole_price = 0, best = 0;
  int best_k = 0;
  for (int k = 0; k <= N && 2 * k * HV <= CUS; ++k) {
    if (k > 0) { halves += r[order[k - 1]]; rest -= r[order[k - 1]]; }
    const double work = (2 * half_cost * halves + rest) * HV;
    double span = std::max(k > 0 ? half_cost * r[order[0]] : 0.0, work / CUS);
    if (k < N) {
      span = std::max(span, (double)r[order[k]]);
      if ((int64_t)(N + k) * HV > CUS) {          // whole chains wait for CUs: longest first on those the halves leave
        const int free_cus = CUS - 2 * k * HV;
        if (free_cus <= 0) break;
        span = std::max(span, rest * HV / free_cus + 0.5 * r[order[N - 1]]);
      }
    }
    const double price = span * (1.0 + fill_cost * std::min(1.0, work / (CUS * span)));
    if (k == 0) whole_price = best = price;
    else if (price < best) { best = price; best_k = k; }
  }
  return best <= 0.95 * whole_price ? best_k : 0;
}

// Stages for a call of whole sequences: two, where there are enough chains to fill the chip and 16 chunks per
// sequence on average; the table kernel then keeps both only for chains of unequal length (stage_map).  Measured on
// GDN, eight ragged sequences of 32 810 tokens: 0.50 ms in one stage, 0.48 in two, 0.52 in four - every further stage
// costs about 25 us (two more launches, an event between two streams, the state through memory, a pipeline that
// fills again), and the preparation only hides under a sweep on CUs that chains which ended early have left.
// (Segmented calls already keep every CU busy with sweeps - staging them was measured for GDN: 0.57 -> 0.66 ms for
// one sequence of 16 384 tokens -; and staging only pays where the preparation is bound by memory latency and leaves
// the sweeps their issue slots, which holds for GDN and not for KDA, whose preparation is instruction bound: the KDA
// path does not call this.)
inline int pick_stages(int T, int N, int heads, int seg_chunks) {
  if (seg_chunks > 0) return 0;
  // (the stage map keeps (stages + 1) counters per sequence in LDS: at most 2048 sequences)
  return ((int64_t)N * heads >= 128 && T / CHUNK >= 16 * N && N <= 2048) ? MAX_STAGES : 0;
}

// Launch order of a prefill call, shared by both paths.  `prepare(stream)` launches the per-chunk
// kernels of stage *stage_field, `sweep(grid)` the sequential kernel for (*pass_field, *stage_field).
// Stage 0 is prepared on the caller's stream, alone; the side stream (a SideStreamLease the caller holds for the
// time of the call) prepares the other stages underneath the sweeps and is joined before the last sweep starts.
template <typename Prepare, typename Sweep>
inline bool launch_pipeline(hipStream_t s, int stages, SideStream* side, bool segmented, unsigned grid_whole,
                            unsigned grid_segments, int* pass_field, int* stage_field, Prepare prepare, Sweep sweep) {
  *pass_field = segmented ? 1 : 0;
  const unsigned grid = segmented ? 2 * grid_segments : grid_whole;
  if (stages == 0) {
    *stage_field = 0;
    prepare(s);
    sweep(grid);
    return true;
  }
  if (side == nullptr) return false;             // (callers stage a call only with a side stream in hand)
  bool ok = true;
  for (int st = 0; st < stages; ++st) {
    *stage_field = st;
    prepare(st == 0 ? s : side->stream);
    if (st == 0) {
      ok = ok && hipEventRecord(side->fork, s) == hipSuccess;
      ok = ok && hipStreamWaitEvent(side->stream, side->fork, 0) == hipSuccess;
    } else {
      ok = ok && hipEventRecord(side->ready[st], side->stream) == hipSuccess;
    }
  }
  for (int st = 0; st < stages; ++st) {
    *stage_field = st;
    if (st > 0) ok = ok && hipStreamWaitEvent(s, side->ready[st], 0) == hipSuccess;
    sweep(grid);
  }
  return ok;
}

}  // namespace pla
