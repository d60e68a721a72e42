// Chunk-64 gated delta-rule prefill for GDN (scalar gate per value head) on gfx950.
//
// Per chunk of C = 64 tokens (G = inclusive cumulative log-decay inside the chunk, S the
// FP32 state, k-last):
//     L   = I + strict_tril(beta_i (k_i . k_j) e^{G_i - G_j})
//     W   = L^-1 diag(beta)                                   (parallel over chunks)
//     P   = scale * tril(q_i . k_j e^{G_i - G_j})             (parallel over chunks)
//     X   = V - e^{G} (.) (K S^T)         U = W X             (sequential)
//     O   = scale e^{G} (.) (Q S^T) + P U
//     S^T = e^{G_last} S^T + K^T (e^{G_last - G} (.) U)
// which is the WY/UT form of the token recurrence (reference algebra:
// scripts/prefill/flashqla/private/ref_gdr.py:78-298; kernels
// src/prefill/flashqla/kernels/chunk_cumsum_cute.cu:232-330, kkt_solve_cute_impl.cuh:34-60,
// fused_fwd_cute.cu:34-66).  Because the gate is a scalar per (token, head) every decay is a
// row or column scaling of a GEMM result, and every factor lies in (0, 1].  All MFMA operands are
// fp16 (v_mfma_f32_16x16x32_f16, the rate of the bf16 instruction): normalised q / k (rounded to the
// activation dtype first, as the reference does, which fp16 then holds exactly) and the FP32
// quantities S, X, W, U, P rounded to fp16 (11 significant bits; accumulation and the state stay
// FP32).  W and the U of the state update travel as hi + lo pairs: when keys nearly repeat and beta is
// near 1, U = W X cancels heavily and the state is the work of the last few tokens, so a single rounding of
// those two shows unaveraged (final-state rel-L2 1e-3 .. 3.5e-3 in a float64 simulation of the rounding
// points, 2.5e-4 .. 2.7e-4 with the pairs; random keys: 3.7e-4 .. 4.8e-4 single, bound 1e-3).  Every rounding
// saturates at +-65504, the fp16 range, instead of producing infinities.
//
// Kernels:
//   prefill_tables_kernel    chunk / segment / stage tables from cu_seqlens (device side, graph-capturable)
//   gdn_align_rows_kernel    q / k rows that start on 4-byte boundaries only are copied into dense buffers first
//   gdn_wsolve_kernel        preparation, one wavefront per (chunk, value head): gate, beta and their chunk-local
//                            cumsum, the decay-factor tile, normalised K, K K^T on MFMA, the inverse of I + L by
//                            16 x 16 blocks, W (hi, lo) in the six-block operand layout; for calls split into
//                            segments also the normalised K rows and (one appended workgroup) the tables
//   gdn_fused_sweep_kernel   sequential kernel with output, over whole sequences or (second sweep) over segments: one
//                            workgroup per (sequence or segment, value head) of four computing wavefronts (32 V
//                            columns of S^T each, in MFMA accumulator layout, the chain K S^T -> X -> U -> S^T in
//                            registers) and four feeding wavefronts that normalise the raw q / k rows into LDS
//                            tiles, form P and issue the global -> LDS copies of V, W and the decay factors; two
//                            barriers per chunk; with NB = 1 two workgroups per chain, 64 V columns each (calls
//                            of at most 128 chains)
//   gdn_fused_sweep_mixed_kernel  the same sweep for ragged whole sequences: the chains of the longest sequences as
//                            two halves, the others whole, in one launch (plan from the host offsets)
//   gdn_lean_sweep_kernel    first sweep over segments (no output): the zero-state and the identity sweep of a
//                            segment side by side in one workgroup of eight wavefronts that share every tile

#include <algorithm>
#include <type_traits>

#include "prefill_common.h"

namespace pla {

// Floats per (chunk, value head) tile of decay factors: scale e^G | e^G | e^{G_last - G} | e^{G_last} (x 64) | G
constexpr int GTILE_FLOATS = 320;

struct GdnPrefillParams {
  // inputs
  const void* q; const void* k; const void* v;        // activation dtype, token strides below
  int64_t stride_q, stride_k, stride_v;               // elements
  const void* a; const void* b; int64_t stride_a, stride_b;   // raw gate / beta logits [T, HV]
  const float* A_log; const float* dt_bias;           // [HV]
  const float* g_in; const float* beta_in;            // optional precomputed log-decay / beta [T, HV]
  const int32_t* cu_seqlens; int N; int T;            // packed offsets, sequences, physical tokens
  float scale; int normalize_qk;
  // state
  const float* h0; const int32_t* h0_indices; int64_t h0_slot_stride;   // read (may be null)
  float* ht; const int32_t* ht_indices; int64_t ht_slot_stride;         // written (may be null)
  // output
  void* o;                                            // [T, HV, 128] dense
  // workspace
  int32_t* seq_chunk_off; int32_t* chunk_seq; int32_t* chunk_tok; int32_t* chunk_len;
  uint16_t* kn;                                       // [T, H, 128] normalised K rows in operand column order (calls split into segments)
  float* kinv;                                        // [H, T] 1 / |k| per row (a head's tokens are contiguous)
  float* gcum; float* beta;
  uint16_t* W;                                        // fp16 [chunk, HV, 12 blocks of 1 KiB]: W = hi + lo, six-block operand layout
  float* gtile;          // [chunk, HV, 320]: scale e^{G} | e^{G} | e^{G_last - G} | e^{G_last} | G
  SegmentTable seg;      // split long sequences (seg.seg_chunks > 0)
  StageTable stg;        // pipelined preparation and sweep (stg.stages > 0)
  int pass;              // 0: whole sequences; 1, 2: the two sweeps over segments
  int stage;             // stage handled by this launch (per-chunk kernels and pass 3)
  int H, HV, NC_max;
  int inline_tables;     // at most 64 whole sequences: kernels work the chunk tables out themselves (no table kernel)
  int tail_blocks;       // workgroups appended to the preparation grid that zero the output rows beyond the last sequence
  int store_kn;          // gdn_wsolve_kernel also stores the normalised K rows (kn): the first sweep over segments copies them
  // gdn_fused_sweep_mixed_kernel: the first `split_grid` workgroups sweep the chains of sequences seq_order[0 .. n_long)
  // as two halves, the others those of seq_order[n_long .. N) whole
  unsigned split_grid; int n_long;
  unsigned char seq_order[INLINE_TABLE_SEQUENCES];
};

// q and k rows that start on 4-byte boundaries only (a packed view shifted inside its buffer) are copied into dense
// [T, H, 128] buffers first, which the kernels below read in 16-byte pieces: one piece per thread and trip.
static __global__ __launch_bounds__(256) void gdn_align_rows_kernel(const uint16_t* q, const uint16_t* k, int64_t stride_q,
                                                                    int64_t stride_k, int T, int H, uint16_t* q_out,
                                                                    uint16_t* k_out) {
  const int64_t pieces = (int64_t)T * H * 16;                  // 16-byte pieces per tensor
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < 2 * pieces; i += (int64_t)gridDim.x * 256) {
    const bool keys = i >= pieces;
    const int64_t j = keys ? i - pieces : i;
    const int64_t t = j / (H * 16);
    const int c = (int)(j - t * (H * 16));                     // piece c of token t
    const uint32_t* src = reinterpret_cast<const uint32_t*>((keys ? k : q) + t * (keys ? stride_k : stride_q) + 8 * c);
    *reinterpret_cast<uint4*>((keys ? k_out : q_out) + 8 * j) = make_uint4(src[0], src[1], src[2], src[3]);
  }
}

// The value that lane ^ 32 holds.
__device__ __forceinline__ uint32_t from_other_half(uint32_t x) {
  uint32_t a = x, b = x;                // after the swap: a = the value of lanes 0-31 in both halves, b = that of lanes 32-63
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return (threadIdx.x & 32) ? a : b;
}

// ---------------------------------------------------------------------------------------------
// Preparation of a chunk: what does not depend on the state and needs the triangular solve.  The sweep
// (gdn_fused_sweep_kernel) normalises q and k and forms P itself, so only the key side is here.  One wavefront per
// (chunk, value head); the WAVES wavefronts of a workgroup take consecutive value heads of one q/k head:
// gate, beta and their cumulative sum (lane j = token j: g_j = -exp(A_log) softplus(a_j + dt_bias), beta_j =
// sigmoid(b_j), or the caller's g / beta; a scan over the lanes; g_cum and beta as the call returns them, the chunk's
// tile of decay factors with the raw cumulative log-decay appended for the sweep's P), normalised K in registers (rows
// loaded directly in MFMA operand layout, L2-normalised, rounded to the activation dtype - the reference's operand -
// and held as fp16, which represents those values exactly), K K^T on MFMA, the
// inverse of I + L by 16 x 16 blocks, and W = (I + L)^-1 diag(beta) as an fp16 hi + lo pair in the six-block
// operand layout (12 KiB per (chunk, value head)).
// The blocks of L below the diagonal never leave the registers: the accumulators of K K^T are the operands of the
// transposed block recursion as they stand, and its results are the lane's pieces of the W blocks.  The wavefronts
// of a workgroup (the value heads of one q/k head) share the loading and normalising of the keys through LDS: a
// quarter fewer vector instructions per tile and half the registers for raw rows, which brings three wavefronts
// to a SIMD without spills (config 3 0.450 -> 0.440 ms, 8 x 2048 tokens 0.233 -> 0.224 ms; four per SIMD by a launch
// bound measure the same: the kernel is bound by its vector instructions now, not by latency).  For a call split
// into segments (store_kn) the wavefront that normalised a row block also stores it: the first sweep over segments
// copies its K tiles from those rows.
template <typename act_t, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void gdn_wsolve_kernel(const GdnPrefillParams p) {
  const int groups = p.HV / WAVES;
  const int lane = threadIdx.x & 63;
  const int main_blocks = gridDim.x - p.tail_blocks;
  if ((int)blockIdx.x >= main_blocks) {
    // Appended workgroups: they zero the padded rows of o and, for a call split into segments, the first of them
    // builds the chunk and segment tables the sweeps read (this kernel works its own tiles out by itself, so the
    // tables only have to be complete when it ends).
    const int extra = blockIdx.x - main_blocks;
    const int builders = p.seg.seg_chunks > 0 ? 1 : 0;
    if (extra < builders) {
      chunk_map(p.cu_seqlens, p.N, p.NC_max, p.seq_chunk_off, p.chunk_seq, p.chunk_tok, p.chunk_len);
      __threadfence();
      __syncthreads();
      segment_map(p.seq_chunk_off, p.N, p.seg);
    } else {
      zero_tail(reinterpret_cast<uint16_t*>(p.o), p.cu_seqlens, p.N, p.T, p.HV, extra - builders, p.tail_blocks - builders);
    }
    return;
  }
  int cb, t0, len;
  if (p.inline_tables) {
    const InlineSequences seqs = inline_sequences(p.cu_seqlens, p.N, p.stg.stages, lane);
    const InlineTile tile = inline_tile(seqs, p.stage, blockIdx.x / groups, p.NC_max, lane);
    cb = tile.cb; t0 = tile.t0; len = tile.len;
    if (cb < 0) return;
  } else {
    cb = staged_chunk(p.stg, p.stage, blockIdx.x / groups, p.seq_chunk_off[p.N]);
    if (cb < 0) return;
    t0 = p.chunk_tok[cb];
    len = p.chunk_len[cb];
  }
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int hv = (blockIdx.x % groups) * WAVES + wave;
  const int h = hv / (p.HV / p.H);
  const int r16 = lane & 15, kb = lane >> 4;

  // Per wavefront only the four diagonal 16 x 16 blocks of L pass through LDS (rows of 20 floats, blocks 336 floats
  // apart: the four groups of 16 lanes that walk one block each in the forward substitution stay on different banks);
  // the six blocks below the diagonal stay in the accumulators of K K^T.  5.9 KB instead of a 64 x 68 FP32 tile.
  constexpr int DIAG_PITCH = 20, DIAG_BLOCK = 336;
  // One buffer serves two purposes in turn: first the normalised keys the wavefronts hand each other ([row block][step]
  // [lane], 16 KiB), then, behind a barrier, every wavefront's diagonal blocks.
  constexpr int SHARE_BYTES = WAVES * 4 * DIAG_BLOCK * 4 > 16 * 64 * 16 ? WAVES * 4 * DIAG_BLOCK * 4 : 16 * 64 * 16;
  __shared__ __align__(16) unsigned char share[SHARE_BYTES];
  __shared__ __align__(16) float Gs_all[WAVES][CHUNK];
  __shared__ __align__(16) float Bs_all[WAVES][CHUNK];
  uint4* const Kshare = reinterpret_cast<uint4*>(share);
  float* const Ld = reinterpret_cast<float*>(share) + wave * 4 * DIAG_BLOCK;
  float* const Gs = Gs_all[wave];
  float* const Bs = Bs_all[wave];

  // gate inputs of the lane's token, requested ahead of the K rows: memory returns in issue order, so the gate math
  // below starts as soon as these few words are here and runs while the rows are still in flight
  float gate_in = 0.f, beta_raw = 0.f, dt_b = 0.f, a_log = 0.f;
  if (lane < len) {
    const int64_t t = t0 + lane;
    if (p.g_in) {
      gate_in = p.g_in[t * p.HV + hv];
      beta_raw = p.beta_in[t * p.HV + hv];
    } else {
      gate_in = to_float(reinterpret_cast<const act_t*>(p.a)[t * p.stride_a + hv]);
      beta_raw = to_float(reinterpret_cast<const act_t*>(p.b)[t * p.stride_b + hv]);
      dt_b = p.dt_bias[hv];
      a_log = p.A_log[hv];
    }
  }
  // Raw K operands.  The wavefronts of a workgroup work on the value heads of ONE q/k head and need the same
  // normalised keys: each loads and normalises 4 / WAVES of the four row blocks and hands them to the others through
  // LDS.  All loads of a lane are requested before the first use (rows are 16-byte aligned on this path).
  constexpr int PER = 4 / WAVES;
  static_assert(WAVES == 1 || WAVES == 2 || WAVES == 4, "row blocks are dealt evenly");
  uint4 kraw[PER][4];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int row = 16 * (wave * PER + i) + r16;
    const int64_t t = t0 + (row < len ? row : 0);
    const uint16_t* kr = reinterpret_cast<const uint16_t*>(p.k) + t * p.stride_k + h * 128 + 8 * kb;
#pragma unroll
    for (int s = 0; s < 4; ++s) kraw[i][s] = *reinterpret_cast<const uint4*>(kr + 32 * s);
  }

  // ---- gate: lane = token ----
  {
    float g = 0.f, bt = 0.f;
    if (lane < len) {
      if (p.g_in) {
        g = gate_in;
        bt = beta_raw;
      } else {
        const float x = gate_in + dt_b;
        const float sp = x <= 20.0f ? log1pf(expf(x)) : x;
        g = -expf(a_log) * sp;
        bt = 1.0f / (1.0f + expf(-beta_raw));
      }
    }
    float cum = g;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
      const float up = __shfl_up(cum, d, 64);
      if (lane >= d) cum += up;
    }
    const float glast = __shfl(cum, 63, 64);
    Gs[lane] = cum;
    Bs[lane] = bt;
    float* gt = p.gtile + ((int64_t)cb * p.HV + hv) * GTILE_FLOATS;
    const float e = __expf(cum);
    gt[lane] = p.scale * e;
    gt[64 + lane] = e;
    gt[128 + lane] = __expf(glast - cum);
    gt[192 + lane] = __expf(glast);
    gt[256 + lane] = cum;
  }

  // ---- k: normalise, round to the activation dtype, hold as fp16 ----
  bf16x8_t Kop[4][4];
  {
    const uint4 zero4 = make_uint4(0, 0, 0, 0);
    const bool first_group = (hv - wave) % (p.HV / p.H) == 0;           // this workgroup holds the head's first value heads
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int mb = wave * PER + i;
      const bool ok = 16 * mb + r16 < len;
      float inv = 1.f;
      if (p.normalize_qk) {
        float ss = 0.f;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const uint32_t w[4] = {kraw[i][s].x, kraw[i][s].y, kraw[i][s].z, kraw[i][s].w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float a0 = lo16<act_t>(w[e]), a1 = hi16<act_t>(w[e]);
            ss += a0 * a0 + a1 * a1;
          }
        }
        const LanePair r1 = swap_rows16(ss);
        const LanePair r2 = swap_halves(r1.lo + r1.hi);
        inv = rsqrtf(r2.lo + r2.hi + 1e-6f);
        // the sweep scales the raw rows by the same factor, so both kernels hold the same rounded keys
        if (ok && kb == 0 && first_group) p.kinv[(int64_t)h * p.T + t0 + 16 * mb + r16] = inv;
      }
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const uint32_t in[4] = {kraw[i][s].x, kraw[i][s].y, kraw[i][s].z, kraw[i][s].w};
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t a = pack2<act_t>(lo16<act_t>(in[e]) * inv, hi16<act_t>(in[e]) * inv);
          w[e] = pack2_rtz(lo16<act_t>(a), hi16<act_t>(a));
        }
        const uint4 row_op = ok ? make_uint4(w[0], w[1], w[2], w[3]) : zero4;
        if constexpr (WAVES == 1) Kop[i][s] = __builtin_bit_cast(bf16x8_t, row_op);
        else Kshare[(mb * 4 + s) * 64 + lane] = row_op;
        if (p.store_kn && first_group) {
          // The rows leave in the column order of an operand tile (prefill_common.h): granule 4 s + g of a row holds
          // columns 32 s + 4 g .. + 3 and 32 s + 16 + 4 g .. + 3.  The lane's columns 32 s + 8 kb .. + 7 are one half of
          // granules 2 (kb % 2) and 2 (kb % 2) + 1; lane kb ^ 2 (32 lanes away) holds the other halves, so the two
          // exchange 8 bytes and each stores one whole granule.
          const bool upper = kb >= 2;
          const uint32_t r0 = from_other_half(upper ? row_op.x : row_op.z), r1 = from_other_half(upper ? row_op.y : row_op.w);
          const uint4 granule = upper ? make_uint4(r0, r1, row_op.z, row_op.w) : make_uint4(row_op.x, row_op.y, r0, r1);
          if (ok)
            *reinterpret_cast<uint4*>(p.kn + ((int64_t)(t0 + 16 * mb + r16) * p.H + h) * 128 + 8 * (4 * s + 2 * (kb & 1) + (kb >> 1))) = granule;
        }
      }
    }
  }
  __syncthreads();
  // Copies for the caller, [T, HV] FP32, only on request: the words of a token's other value heads are written by other
  // workgroups at other times, so every store here is a piece of a line of its own (measured: 1.5 % of a call per copy
  // with 4-byte stores).  The first wavefront writes the values of all WAVES heads of the workgroup as one piece per
  // token.  (Measured as well: workgroups of their own that write a chunk's 64 x HV words as one contiguous block
  // cost as much as they save.)
  if (wave == 0 && lane < len) {
    const int64_t at = (int64_t)(t0 + lane) * p.HV + hv;        // hv: the workgroup's first head, a multiple of WAVES
    auto put = [&](float* out, const float (&all)[WAVES][CHUNK]) {
      if constexpr (WAVES == 4) *reinterpret_cast<float4*>(out + at) = make_float4(all[0][lane], all[1][lane], all[2][lane], all[3][lane]);
      else if constexpr (WAVES == 2) *reinterpret_cast<float2*>(out + at) = make_float2(all[0][lane], all[1][lane]);
      else out[at] = all[0][lane];
    };
    if (p.gcum != nullptr) put(p.gcum, Gs_all);
    if (p.beta != nullptr) put(p.beta, Bs_all);
  }
  if constexpr (WAVES > 1) {
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
      for (int s = 0; s < 4; ++s) Kop[mb][s] = __builtin_bit_cast(bf16x8_t, Kshare[(mb * 4 + s) * 64 + lane]);
    __syncthreads();                    // every wavefront holds the keys: the buffer is free for the diagonal blocks
  }

  // L = strict_tril(beta_i (k_i . k_j) e^{G_i - G_j}) by 16 x 16 blocks.  The accumulators of block (mi, ni) hold rows
  // i = 4 kb + r of column j = r16: for a block below the diagonal that is the A operand of L_ab^T as it stands
  // (Lr[mi][ni]); the diagonal blocks go to LDS, row major, for the forward substitution.
  const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
  f32x4_t Lr[4][4];
#pragma unroll
  for (int mi = 0; mi < 4; ++mi) {
    const float4 Gi = *reinterpret_cast<const float4*>(&Gs[16 * mi + 4 * kb]);
    const float4 Bi = *reinterpret_cast<const float4*>(&Bs[16 * mi + 4 * kb]);
    const float gi[4] = {Gi.x, Gi.y, Gi.z, Gi.w}, bi[4] = {Bi.x, Bi.y, Bi.z, Bi.w};
#pragma unroll
    for (int ni = 0; ni <= mi; ++ni) {
      f32x4_t kk = zero;
#pragma unroll
      for (int s = 0; s < 4; ++s) kk = mfma16h(Kop[mi][s], Kop[ni][s], kk);
      const float Gj = Gs[16 * ni + r16];
      if (ni < mi) {
#pragma unroll
        for (int r = 0; r < 4; ++r) Lr[mi][ni][r] = bi[r] * kk[r] * __expf(gi[r] - Gj);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          Ld[mi * DIAG_BLOCK + (4 * kb + r) * DIAG_PITCH + r16] = 4 * kb + r > r16 ? bi[r] * kk[r] * __expf(gi[r] - Gj) : 0.f;
      }
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  // Diagonal blocks D_a = (I + L_aa)^-1: lane (a = kb, j = r16) solves column j by forward substitution over the 16
  // rows, x_i = [i == j] - sum_{l < i} L_aa[i][l] x_l, and writes it over row j of the block (the block then holds
  // D_a^T; every read of L_aa precedes the writes: one wavefront, LDS operations complete in order).
  {
    float* const La = Ld + kb * DIAG_BLOCK;
    float x[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
      for (int l4 = 0; l4 < i; l4 += 4) {
        const float4 row = *reinterpret_cast<const float4*>(&La[i * DIAG_PITCH + l4]);
        acc0 = fmaf(row.x, x[l4], acc0);
        if (l4 + 1 < i) acc1 = fmaf(row.y, x[l4 + 1], acc1);
        if (l4 + 2 < i) acc0 = fmaf(row.z, x[l4 + 2], acc0);
        if (l4 + 3 < i) acc1 = fmaf(row.w, x[l4 + 3], acc1);
      }
      x[i] = (i == r16 ? 1.f : 0.f) - (acc0 + acc1);
    }
#pragma unroll
    for (int i4 = 0; i4 < 16; i4 += 4)
      *reinterpret_cast<float4*>(&La[r16 * DIAG_PITCH + i4]) = make_float4(x[i4], x[i4 + 1], x[i4 + 2], x[i4 + 3]);
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  // Dq[a]: D_a[r16][4 kb + r], the lane's piece of D_a as the operand of a product that contracts over its columns
  // and, as it stands, of the W blocks; DTq[b]: D_b[4 kb + r][r16], the same for D_b^T.
  f32x4_t Dq[4], DTq[3];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int r = 0; r < 4; ++r) Dq[a][r] = Ld[a * DIAG_BLOCK + (4 * kb + r) * DIAG_PITCH + r16];
#pragma unroll
  for (int b = 0; b < 3; ++b) {
    const float4 t = *reinterpret_cast<const float4*>(&Ld[b * DIAG_BLOCK + r16 * DIAG_PITCH + 4 * kb]);
    DTq[b] = f32x4_t{t.x, t.y, t.z, t.w};
  }
  // The blocks of N = (I + L)^-1 below the diagonal, transposed: N_ab^T = -D_b^T sum_{b < c <= a} L_cb^T N_ac^T with
  // N_aa = D_a, in order of a - b = 1, 2, 3.  Every product has the earlier result on its right, where an accumulator
  // tile is an operand as it stands, and leaves N_ab^T in accumulator layout: rows j = 4 kb + r of column i = r16,
  // which is the lane's piece N_ab[r16][4 kb + r] of a W block.  The products run on the FP32 MFMA
  // (v_mfma_f32_16x16x4_f32, exact products): lane (r16, kb) supplies one element of row r16 per instruction, and with
  // the contraction index taken as 4 kb + r for instruction r both operands are the lane's own quads, element r of
  // each.  (As bf16 hi / lo pairs on the 16 x 16 x 32 instruction the same products cost a third of the matrix-pipe
  // time but about 900 vector instructions per tile for the splits, in a kernel that its vector instructions bound.)
  auto negate = [](f32x4_t t) { return f32x4_t{-t.x, -t.y, -t.z, -t.w}; };
  auto product = [](const f32x4_t& a, const f32x4_t& b, f32x4_t acc) {       // acc += A B over one 16-wide block
#pragma unroll
    for (int r = 0; r < 4; ++r) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[r], b[r], acc, 0, 0, 0);
    return acc;
  };
  auto solve = [&](int b, const f32x4_t& y) { return negate(product(DTq[b], y, zero)); };
  f32x4_t Nq[4][4];
  Nq[1][0] = solve(0, product(Lr[1][0], Dq[1], zero));
  Nq[2][1] = solve(1, product(Lr[2][1], Dq[2], zero));
  Nq[3][2] = solve(2, product(Lr[3][2], Dq[3], zero));
  Nq[2][0] = solve(0, product(Lr[2][0], Dq[2], product(Lr[1][0], Nq[2][1], zero)));
  Nq[3][1] = solve(1, product(Lr[3][1], Dq[3], product(Lr[2][1], Nq[3][2], zero)));
  Nq[3][0] = solve(0, product(Lr[3][0], Dq[3], product(Lr[2][0], Nq[3][2], product(Lr[1][0], Nq[3][1], zero))));
  // W = N diag(beta) as an fp16 hi + lo pair in the six-block operand layout: block (row block m, column half s) holds
  // the lane's pieces of blocks (m, 2 s) and (m, 2 s + 1)
  uint16_t* const Wt = p.W + ((int64_t)cb * p.HV + hv) * (2 * TRI_BLOCKS * 512);
#pragma unroll
  for (int b = 0; b < TRI_BLOCKS; ++b) {
    const int m = tri_block_m(b), sh = tri_block_s(b);
    uint32_t hi[4], lo[4];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int cbk = 2 * sh + half;                       // column block
      f32x4_t n4 = zero;
      if (cbk < m) n4 = Nq[m][cbk];
      else if (cbk == m) n4 = Dq[m];
      const float4 b4 = *reinterpret_cast<const float4*>(&Bs[16 * cbk + 4 * kb]);
      const bool diag = cbk == m;                          // a diagonal block keeps columns j <= i
      const float w0 = !diag || 4 * kb <= r16 ? n4[0] * b4.x : 0.f, w1 = !diag || 4 * kb + 1 <= r16 ? n4[1] * b4.y : 0.f;
      const float w2 = !diag || 4 * kb + 2 <= r16 ? n4[2] * b4.z : 0.f, w3 = !diag || 4 * kb + 3 <= r16 ? n4[3] * b4.w : 0.f;
      pack2_pair(w0, w1, hi[2 * half], lo[2 * half]);
      pack2_pair(w2, w3, hi[2 * half + 1], lo[2 * half + 1]);
    }
    *reinterpret_cast<uint4*>(Wt + b * 512 + lane * 8) = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    *reinterpret_cast<uint4*>(Wt + (TRI_BLOCKS + b) * 512 + lane * 8) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
  }
}

// ---------------------------------------------------------------------------------------------
// First sweep over segments, both roles in one workgroup.  A later segment is swept twice without output - from a
// zero state (its B summary) and from the identity with v = 0 (its transition matrix M) - and both sweeps multiply
// the same K and W tiles.  One workgroup of eight wavefronts per (segment, value head) runs them side by side:
// wavefronts 0-3 carry the B columns (32 each), wavefronts 4-7 the M columns and, having no values to subtract,
// also issue every global -> LDS copy, so each tile crosses memory and LDS once for the two sweeps and two
// wavefronts share a SIMD.  A first segment has no M role: its wavefronts 4-7 only copy, wavefronts 0-3 sweep it
// from its real start state (of which they keep a copy for the second sweep).  All tiles are double buffered by
// chunk parity (90 KB of LDS: K and V in swizzled unpadded tiles, 134 us -> 124 us per sweep of 32 chunks against rows
// padded to 272 bytes) and there is one barrier per chunk: at the barrier that opens chunk c its tiles have landed (every
// wavefront waited for its own copies) and the buffers of chunk c - 1 are free for the copies of chunk c + 1.
template <typename act_t>
__global__ __launch_bounds__(512, 1) void gdn_lean_sweep_kernel(const GdnPrefillParams p) {
  constexpr int NB = 2;
  // what gdn_wsolve_kernel left per (chunk, value head): W (six blocks hi, six lo) and the tile of decay factors
  constexpr int W_BYTES = 2 * TRI_BLOCKS * 1024, G_BYTES = GTILE_FLOATS * 4;
  // K and V tiles, filled by the four copying wavefronts: swizzled and unpadded (the K rows come in the column order
  // of an operand tile, V with its columns in order)
  using CopyWide = SwizzledTileCopy<4>;
  constexpr int KV_HALVES = TILE128_HALVES;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, kb = lane >> 4;
  const bool m_side = wave >= 4;                               // wavefronts 4-7: transition-matrix columns + copies
  const int cw = wave & 3;                                     // position among the four wavefronts of a role
  const int vcol = 32 * cw + r16;

  // the two roles of this (segment, head): logical workgroups 2 i (zero state / real state) and 2 i + 1 (identity)
  // the value heads of a q/k head copy the same K rows: on one XCD they come from memory once
  const int pair = xcd_grouped_index(blockIdx.x, p.HV / p.H, p.seg.max_segments * p.HV);
  if (pair < 0) return;
  const SweepRole lead = select_sweep(1, p.HV, p.N, p.seq_chunk_off, p.seg, p.stg, p.stage, p.h0, p.h0_indices, p.h0_slot_stride,
                                      p.ht, p.ht_indices, p.ht_slot_stride, 2 * pair);
  if (!lead.active) return;
  const SweepRole mrole = select_sweep(1, p.HV, p.N, p.seq_chunk_off, p.seg, p.stg, p.stage, p.h0, p.h0_indices, p.h0_slot_stride,
                                       p.ht, p.ht_indices, p.ht_slot_stride, 2 * pair + 1);
  const SweepRole& role = m_side ? mrole : lead;
  const bool computing = role.active;                          // wave-uniform; false: wavefronts 4-7 of a first segment
  const int n = lead.n, hv = lead.head, c_begin = lead.c_begin, c_end = lead.c_end;
  const int h = hv / (p.HV / p.H);
  const int seq_start = p.cu_seqlens[n] + (c_begin - p.seq_chunk_off[n]) * CHUNK;
  const int seq_len = min(p.cu_seqlens[n + 1] - seq_start, (c_end - c_begin) * CHUNK);
  const int n_chunks = c_end - c_begin;
  auto chunk_len = [&](int c) { return min(CHUNK, seq_len - c * CHUNK); };

  __shared__ __align__(1024) uint16_t tK[2][KV_HALVES];
  __shared__ __align__(1024) uint16_t tV[2][KV_HALVES];
  // W [parity]: the six-block operand layout (hi blocks, then lo blocks)
  __shared__ __align__(16) uint16_t tW[2][2 * TRI_BLOCKS * 512];
  // decay factors: [64,128) e^{G}, [128,192) e^{G_last - G}, [192] e^{G_last}
  __shared__ __align__(16) float tG[2][256];

  // S^T slices in accumulator layout: St[nb][mc][r] = S[v = vcol + 16 nb][c = 16 mc + 4 kb + r]
  f32x4_t St[NB][8];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
    if (computing && role.init != nullptr) {
      const float* src = role.init + (int64_t)(vcol + 16 * nb) * 128 + 4 * kb;
#pragma unroll
      for (int mc = 0; mc < 8; ++mc) {
        const float4 t4 = *reinterpret_cast<const float4*>(src + 16 * mc);
        St[nb][mc] = f32x4_t{t4.x, t4.y, t4.z, t4.w};
      }
    } else {
#pragma unroll
      for (int mc = 0; mc < 8; ++mc) St[nb][mc] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
  if (computing && role.keep_init != nullptr) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      float* dst = role.keep_init + (int64_t)(vcol + 16 * nb) * 128 + 4 * kb;
#pragma unroll
      for (int mc = 0; mc < 8; ++mc)
        *reinterpret_cast<float4*>(dst + 16 * mc) = make_float4(St[nb][mc].x, St[nb][mc].y, St[nb][mc].z, St[nb][mc].w);
    }
  }
  const bool use_v = computing && !role.zero_v;                // the identity sweep runs with v = 0
  // LDS reads.  K operand of contraction step s for row block mi; the lane's V values of rows 16 mi + 4 kb .. + 3, column
  // vcol + 16 nb, by one transposing read: lane t of a group of 16 addresses columns 32 cw + 16 nb + 4 (t % 4) .. + 3 of
  // row 16 mi + 4 kb + t / 4, which in a swizzled tile is half (t % 2) of granule 4 cw + 2 nb + (t % 4) / 2; the
  // swizzle 8 (kb & 1) + 2 (t / 4) of that row does not depend on mi, and nb = 1 differs in one bit of the granule index.
  auto k_operand = [&](const uint16_t* K, int mi, int s) { return operand_granule(K, 16 * mi + r16, s, kb); };
  const int trV = (4 * kb + (r16 >> 2)) * 128 + 8 * ((4 * cw + ((r16 & 3) >> 1)) ^ (8 * (kb & 1) + 2 * (r16 >> 2))) + 4 * (r16 & 1);
  auto v_at = [&](const uint16_t* V, int mi, int nb) { return V + ((trV + 16 * 128 * mi) ^ (16 * nb)); };

  // ---- copies (wavefronts 4-7) ----
  const int64_t tok_pitch_b = (int64_t)p.H * 256;              // bytes between tokens of kn
  const char* const kn_b = reinterpret_cast<const char*>(p.kn) + ((int64_t)seq_start * p.H + h) * 256;
  const char* const v_b = reinterpret_cast<const char*>(p.v) + ((int64_t)seq_start * p.stride_v + hv * 128) * 2;
  const char* const w_b = reinterpret_cast<const char*>(p.W) + ((int64_t)c_begin * p.HV + hv) * W_BYTES;
  const char* const gt_b = reinterpret_cast<const char*>(p.gtile) + ((int64_t)c_begin * p.HV + hv) * G_BYTES;
  CopyWide plan_k, plan_v;
  if (m_side) {
    plan_k.plan((uint32_t)tok_pitch_b, CHUNK - 1, cw, lane);
    plan_v.plan((uint32_t)(p.stride_v * 2), CHUNK - 1, cw, lane);
  }
  // A wavefront that issues copies is held until the memory pipeline has taken them, so the two wavefronts of a SIMD
  // issue at different times and one of them always computes: wavefronts 4-7 request the decay tile, K and V right
  // after the barrier, wavefronts 0-3 the W pair between the two phases of the chunk.
  auto issue_w = [&](int c) {
    const int par = c & 1;
    const char* const ws = w_b + (int64_t)c * p.HV * W_BYTES;
#pragma unroll
    for (int j = 0; j < 2 * TRI_BLOCKS / 4; ++j)     // twelve 1 KiB blocks, three per wavefront, as they lie in memory
      dma16(ws, 1024u * (4 * j + cw) + 16u * lane, lds_address(&tW[par][0]) + 1024u * (4 * j + cw));
  };
  auto issue = [&](int c) {
    const int par = c & 1;
    const char* ks = kn_b + (int64_t)c * CHUNK * tok_pitch_b;
    const char* vs = v_b + (int64_t)c * CHUNK * p.stride_v * 2;
    const int len = chunk_len(c);
    if (cw == 0) dma16(gt_b + (int64_t)c * p.HV * G_BYTES, 16u * lane, lds_address(&tG[par][0]));
    if (len == CHUNK) {
      plan_k.issue(tK[par], ks, cw);
      plan_v.issue(tV[par], vs, cw);
    } else {                                         // rows past the sequence end re-read its last row
      CopyWide tail;
      tail.plan((uint32_t)tok_pitch_b, len - 1, cw, lane);
      tail.issue(tK[par], ks, cw);
      tail.plan((uint32_t)(p.stride_v * 2), len - 1, cw, lane);
      tail.issue(tV[par], vs, cw);
    }
  };
  if (n_chunks > 0) {
    if (m_side) issue(0); else issue_w(0);
  }

  for (int ci = 0; ci < n_chunks; ++ci) {
    const int par = ci & 1;
    wait_vmcnt<0>();                                 // this wavefront's copies for chunk ci have landed
    __syncthreads();                                 // ... and chunk ci - 1 is finished: its buffers are free
    if (m_side && ci + 1 < n_chunks) issue(ci + 1);
    if (!computing) continue;
    const uint16_t* const K = tK[par];
    const uint16_t* const V = tV[par];
    const float* const G = tG[par];
    // ---- KS = K S^T ----
    f32x4_t KS[NB][4];
    bf16x8_t wa[2][4], wl[2][4];
    float4 eg[4];
    uint2 vraw[NB][4];        // rows 16 mi + 4 kb .. + 3 of the lane's V column, one transposing read each
    {
      bf16x8_t ka[2][4], sb[2][NB];
#pragma unroll
      for (int mi = 0; mi < 4; ++mi) ka[0][mi] = k_operand(K, mi, 0);
      __builtin_amdgcn_sched_barrier(0x000F);        // LDS requests stay above this line; ALU and MFMA work may cross it
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mi = 0; mi < 4; ++mi) KS[nb][mi] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) sb[0][nb] = half8_rtz(St[nb][0], St[nb][1]);
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        if (s < 3) {
#pragma unroll
          for (int mi = 0; mi < 4; ++mi) ka[(s + 1) & 1][mi] = k_operand(K, mi, s + 1);
        } else {
          // under the last step: V and e^G
#pragma unroll
          for (int mi = 0; mi < 4; ++mi) {
            eg[mi] = *reinterpret_cast<const float4*>(&G[64 + 16 * mi + 4 * kb]);
            if (use_v) {
#pragma unroll
              for (int nb = 0; nb < NB; ++nb) {
                vraw[nb][mi] = read_tr4(v_at(V, mi, nb));
              }
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0x000F);
        if (s < 3) {
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) sb[(s + 1) & 1][nb] = half8_rtz(St[nb][2 * s + 2], St[nb][2 * s + 3]);
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int mi = 0; mi < 4; ++mi) KS[nb][mi] = mfma16h(ka[s & 1][mi], sb[s & 1][nb], KS[nb][mi]);
      }
    }
    // ---- X = V - e^G (.) KS,  U = W X ----
    f32x4_t U[NB][4];
    bf16x8_t kt[2][8];
    float4 dg[2][2];
    float egl;
    {
      // W is requested here: the arithmetic of X covers the LDS latency
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int mi = 0; mi < 4; ++mi) {
          // block (row block mi, contraction half s2) of the lower triangle: 0-3 for s2 = 0, 4 and 5 (mi 2, 3) for s2 = 1;
          // the two blocks above the diagonal (s2 = 1, mi < 2) are zero and cost neither a read nor an MFMA
          if (s2 == 1 && mi < 2) continue;
          const int b = s2 == 0 ? mi : mi + 2;
          wa[s2][mi] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(&tW[par][b * 512 + lane * 8]));
          wl[s2][mi] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(&tW[par][(TRI_BLOCKS + b) * 512 + lane * 8]));
        }
      __builtin_amdgcn_sched_barrier(0x000F);
      f32x4_t X[NB][4];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mi = 0; mi < 4; ++mi) {
          X[nb][mi][0] = (use_v ? lo16<act_t>(vraw[nb][mi].x) : 0.f) - eg[mi].x * KS[nb][mi][0];
          X[nb][mi][1] = (use_v ? hi16<act_t>(vraw[nb][mi].x) : 0.f) - eg[mi].y * KS[nb][mi][1];
          X[nb][mi][2] = (use_v ? lo16<act_t>(vraw[nb][mi].y) : 0.f) - eg[mi].z * KS[nb][mi][2];
          X[nb][mi][3] = (use_v ? hi16<act_t>(vraw[nb][mi].y) : 0.f) - eg[mi].w * KS[nb][mi][3];
        }
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mi = 0; mi < 4; ++mi) U[nb][mi] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        bf16x8_t xb[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) xb[nb] = half8_sat(X[nb][2 * s], X[nb][2 * s + 1]);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int mi = s == 1 ? 2 : 0; mi < 4; ++mi) U[nb][mi] = mfma16h(wl[s][mi], xb[nb], U[nb][mi]);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int mi = s == 1 ? 2 : 0; mi < 4; ++mi) U[nb][mi] = mfma16h(wa[s][mi], xb[nb], U[nb][mi]);
      }
    }
    if (!m_side && ci + 1 < n_chunks) issue_w(ci + 1);
    // ---- S^T = e^{G_last} S^T + K^T (e^{G_last - G} (.) U) ----
    {
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
#pragma unroll
        for (int mc = 0; mc < 8; ++mc) kt[s2][mc] = operand_granule_transposed(K, s2, mc, kb, r16);
        dg[s2][0] = *reinterpret_cast<const float4*>(&G[128 + 32 * s2 + 4 * kb]);
        dg[s2][1] = *reinterpret_cast<const float4*>(&G[128 + 32 * s2 + 16 + 4 * kb]);
      }
      egl = G[192];
      __builtin_amdgcn_sched_barrier(0x000F);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mc = 0; mc < 8; ++mc) St[nb][mc] *= egl;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        HalfPair ub[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const f32x4_t u0 = {U[nb][2 * s][0] * dg[s][0].x, U[nb][2 * s][1] * dg[s][0].y, U[nb][2 * s][2] * dg[s][0].z,
                              U[nb][2 * s][3] * dg[s][0].w};
          const f32x4_t u1 = {U[nb][2 * s + 1][0] * dg[s][1].x, U[nb][2 * s + 1][1] * dg[s][1].y,
                              U[nb][2 * s + 1][2] * dg[s][1].z, U[nb][2 * s + 1][3] * dg[s][1].w};
          ub[nb] = half8_pair(u0, u1);
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int mc = 0; mc < 8; ++mc) St[nb][mc] = mfma16h(kt[s][mc], ub[nb].lo, St[nb][mc]);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int mc = 0; mc < 8; ++mc) St[nb][mc] = mfma16h(kt[s][mc], ub[nb].hi, St[nb][mc]);
      }
    }
  }

  if (computing && role.fin != nullptr) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      float* dst = role.fin + (int64_t)(vcol + 16 * nb) * 128 + 4 * kb;
#pragma unroll
      for (int mc = 0; mc < 8; ++mc)
        *reinterpret_cast<float4*>(dst + 16 * mc) = make_float4(St[nb][mc].x, St[nb][mc].y, St[nb][mc].z, St[nb][mc].w);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Fused sweep, over whole sequences or as the second sweep over segments (pass 2): one workgroup of EIGHT wavefronts
// per (sequence or segment, value head) with NB = 2; with NB = 1 two workgroups per chain, each on 64 of the 128 V
// columns (16 per computing wavefront), for calls whose chains would leave half of the CUs idle.  Per chunk:
//     KS = K S^T,  X = V - e^G (.) KS,  U = W X                  (W as an fp16 hi + lo pair)
//     O^T = scale e^G (.) (S Q^T) + U^T P^T  -> rows of o         (the output product is formed transposed: a lane
//                                                                  then holds four adjacent V columns of one token
//                                                                  and stores them as 8 bytes, no LDS tile)
//     S^T = e^{G_last} S^T + K^T (e^{G_last - G} (.) U)          (U as an fp16 hi + lo pair)
// Wavefronts 0-3 compute, each on its own 32 V columns of S^T, nothing crossing wavefronts (the chain K S^T -> X -> U
// -> S^T stays in registers; the query product is formed after U, so its accumulators and those of K S^T never live
// together).
// Wavefronts 4-7 feed them, so that neither the normalised rows nor P cross memory:
//   rows   wavefronts 4, 5 take the raw K rows of the next chunk (32 rows each), 6, 7 the raw Q rows: loaded one
//          chunk ahead into registers (16 lanes per row, 16 bytes per lane).  K rows are scaled by the row's 1 / |k|
//          (from the preparation kernel, so that both kernels round the very same normalised keys), rounded to the
//          activation dtype and written to the LDS tile as fp16.  Q only enters the output, so its rows are written
//          unscaled and 1 / |q| (summed here) joins the row factors of the output and of P instead
//   P      scale tril(q_i . k_j e^{G_i - G_j}) of the current chunk from those tiles: the products are formed
//          transposed (A = K rows, B = Q rows), which leaves a lane with four consecutive j of one token i, i.e. with
//          8 of the 16 bytes it owns in the six-block operand layout (prefill_common.h) that phase 3 reads
//   copies V, W (12 KiB, six-block layout, hi then lo) and the decay-factor tile by global -> LDS copies
// Two barriers per chunk: A opens the chunk (all tiles of it are complete, those of the chunk before are free),
// B precedes the product with P (P is complete).  The computing wavefronts run a hand-ordered schedule: every LDS
// operand is requested a fixed number of steps before the MFMA that uses it and the VALU work (conversions, X, the
// hi / lo split of U, the decay of S) is placed under the MFMAs; scheduling barriers keep that order.
#define SB() __builtin_amdgcn_sched_barrier(0)
// LDS of one workgroup of the fused sweep (layout in fused_sweep below)
constexpr int FUSED_W_HALVES = 2 * TRI_BLOCKS * 512;       // hi blocks, then lo blocks
constexpr int FUSED_OFF_P = 0, FUSED_OFF_G = FUSED_OFF_P + TRI_BLOCKS * 1024, FUSED_OFF_RQ = FUSED_OFF_G + 2 * 2048;
constexpr int FUSED_OFF_W = (FUSED_OFF_RQ + 2 * CHUNK * 4 + 1023) / 1024 * 1024, FUSED_OFF_Q = FUSED_OFF_W + 2 * FUSED_W_HALVES * 2;
constexpr int FUSED_OFF_K = FUSED_OFF_Q + 2 * TILE128_HALVES * 2, FUSED_OFF_V = FUSED_OFF_K + 2 * TILE128_HALVES * 2;
constexpr int FUSED_LDS_BYTES = FUSED_OFF_V + 2 * TILE128_HALVES * 2;

// The sweep of one workgroup.  `wide`: 2 / NB x the chain's logical index (sequence x HV + value head, or segment x
// HV + value head in the second sweep over segments) plus, for NB = 1, the half of the V columns it takes.
template <typename act_t, int NB>
__device__ __forceinline__ void fused_sweep(const GdnPrefillParams& p, unsigned char* const lds_all, const int wide) {
  constexpr int CW = 4, AUX = 4;
  constexpr int HALVES = 2 / NB;             // workgroups per chain: NB = 1 sweeps 64 of the 128 V columns
  using CopyV = SwizzledTileCopy<AUX>;
  const int block = wide / HALVES, v_half = wide % HALVES;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  // the chunks of this workgroup's sequence: from the tables, or worked out here (every wavefront for itself)
  int3 inline_chunks{-1, 0, 0};
  int seq_first_chunk = 0, seq_first_token = 0, seq_end_token = 0;
  const bool inline_tables = p.inline_tables && p.pass == 0;         // segments are looked up in the segment table
  if (inline_tables) {
    const InlineSequences seqs = inline_sequences(p.cu_seqlens, p.N, p.stg.stages, lane);
    const int n0 = __builtin_amdgcn_readfirstlane(block / p.HV);
    seq_first_chunk = __builtin_amdgcn_readlane(seqs.off, n0);
    seq_first_token = __builtin_amdgcn_readlane(seqs.start, n0);
    seq_end_token = seq_first_token + __builtin_amdgcn_readlane(seqs.len, n0);
    inline_chunks = int3{seq_first_chunk, min(seq_first_chunk + __builtin_amdgcn_readlane(seqs.nc, n0), p.NC_max), seqs.E};
  }
  const SweepRole role = select_sweep(p.pass, p.HV, p.N, p.seq_chunk_off, p.seg, p.stg, p.stage, p.h0, p.h0_indices, p.h0_slot_stride,
                                      p.ht, p.ht_indices, p.ht_slot_stride, block, inline_chunks);
  if (!role.active) return;
  const int n = role.n, hv = role.head, c_begin = role.c_begin, c_end = role.c_end;
  const int h = hv / (p.HV / p.H);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, kb = lane >> 4;
  if (!inline_tables) {
    seq_first_chunk = p.seq_chunk_off[n];
    seq_first_token = p.cu_seqlens[n];
    seq_end_token = p.cu_seqlens[n + 1];
  }
  const int seq_start = seq_first_token + (c_begin - seq_first_chunk) * CHUNK;
  const int seq_len = min(seq_end_token - seq_start, (c_end - c_begin) * CHUNK);
  const int n_chunks = c_end - c_begin;
  auto chunk_len = [&](int c) { return min(CHUNK, seq_len - c * CHUNK); };

  // K and Q: swizzled operand tiles (columns permuted inside groups of 32); V: swizzled, columns in order.  All of the
  // workgroup's LDS is ONE array with a fixed layout: what is read at many constant offsets from one per-lane address
  // (the blocks of P and W, the decay factors) lies in the first 64 KiB, where those offsets fit the 16-bit offset
  // field of an LDS instruction; above that every distinct offset would cost a register for its address.
  constexpr int W_HALVES = FUSED_W_HALVES;
  constexpr int OFF_P = FUSED_OFF_P, OFF_G = FUSED_OFF_G, OFF_RQ = FUSED_OFF_RQ, OFF_W = FUSED_OFF_W, OFF_Q = FUSED_OFF_Q;
  constexpr int OFF_K = FUSED_OFF_K, OFF_V = FUSED_OFF_V;
  uint16_t* const tP = reinterpret_cast<uint16_t*>(lds_all + OFF_P);
  // decay factors: [0,64) scale e^{G}, [64,128) e^{G}, [128,192) e^{G_last - G}, [192] e^{G_last}, [256,320) G
  float (*const tG)[512] = reinterpret_cast<float (*)[512]>(lds_all + OFF_G);                       // [2][512]
  float (*const tRq)[CHUNK] = reinterpret_cast<float (*)[CHUNK]>(lds_all + OFF_RQ);                 // [2][64]: 1 / |q| per row of the Q tile
  uint16_t (*const tW)[W_HALVES] = reinterpret_cast<uint16_t (*)[W_HALVES]>(lds_all + OFF_W);       // [parity][hi blocks, lo blocks]
  uint16_t (*const tQ)[TILE128_HALVES] = reinterpret_cast<uint16_t (*)[TILE128_HALVES]>(lds_all + OFF_Q);
  uint16_t (*const tK)[TILE128_HALVES] = reinterpret_cast<uint16_t (*)[TILE128_HALVES]>(lds_all + OFF_K);
  uint16_t (*const tV)[TILE128_HALVES] = reinterpret_cast<uint16_t (*)[TILE128_HALVES]>(lds_all + OFF_V);

  if (wave >= CW) {
    // ---- the feeding wavefronts: one instance of this code per wavefront (its role is a compile-time constant) ----
    auto feed = [&](auto role_tag) __attribute__((always_inline)) {
      constexpr int a = decltype(role_tag)::value;
      constexpr bool q_side = a >= 2;
      constexpr int row0 = 32 * (a & 1);                  // this wavefront's rows of a chunk: row0 .. row0 + 31
      const int lr = lane >> 4, lc = lane & 15;           // piece j: row row0 + 4 j + lr, columns 8 lc .. 8 lc + 7
      const int64_t row_pitch = q_side ? p.stride_q : p.stride_k;
      // bases of the sequence part (wave-uniform, 64-bit) and offsets inside a chunk (per lane, 32-bit)
      const char* const rows_b = reinterpret_cast<const char*>(q_side ? p.q : p.k) + ((int64_t)seq_start * row_pitch + h * 128) * 2;
      const char* const kinv_b = reinterpret_cast<const char*>(p.kinv + (int64_t)h * p.T + seq_start);
      const int64_t chunk_pitch_b = (int64_t)CHUNK * row_pitch * 2;
      const char* const v_b = reinterpret_cast<const char*>(p.v) + ((int64_t)seq_start * p.stride_v + hv * 128) * 2;
      const char* const w_b = reinterpret_cast<const char*>(p.W) + ((int64_t)c_begin * p.HV + hv) * (2 * TRI_BLOCKS * 1024);
      const char* const gt_b = reinterpret_cast<const char*>(p.gtile) + ((int64_t)c_begin * p.HV + hv) * (GTILE_FLOATS * 4);
      CopyV plan_v;
      plan_v.plan((uint32_t)(p.stride_v * 2), CHUNK - 1, a, lane);

      // global -> LDS copies of chunk c (its buffers are free): V, W and the decay-factor tile
      auto issue_copies = [&](int c) {
        const int par = c & 1;
        const char* vs = v_b + (int64_t)c * CHUNK * p.stride_v * 2;
        const int len = chunk_len(c);
        if (len == CHUNK) plan_v.issue(tV[par], vs, a);
        else {                                           // rows past the sequence end re-read its last row
          CopyV tail;
          tail.plan((uint32_t)(p.stride_v * 2), len - 1, a, lane);
          tail.issue(tV[par], vs, a);
        }
        const char* ws = w_b + (int64_t)c * p.HV * (2 * TRI_BLOCKS * 1024);
#pragma unroll
        for (int j = 0; j < 2 * TRI_BLOCKS / AUX; ++j)
          dma16(ws, 1024u * (AUX * j + a) + 16u * lane, lds_address(&tW[par][0]) + 1024u * (AUX * j + a));
        const char* gs = gt_b + (int64_t)c * p.HV * (GTILE_FLOATS * 4);
        if (a == 1) dma16(gs, 16u * lane, lds_address(&tG[par][0]));
        if (a == 2) dma16(gs, 1024u + 16u * (lane & 15), lds_address(&tG[par][256]));   // 64 floats; lanes 16-63 repeat them
      };
      // raw rows of chunk c into registers (rows past the end of the sequence part re-read its last row)
      auto load_rows = [&](int c, uint4 (&raw)[8], float (&inv)[8]) {
        const char* const cb = rows_b + (int64_t)c * chunk_pitch_b;
        const char* const ib = kinv_b + (int64_t)c * CHUNK * 4;
        const int last = seq_len - 1 - c * CHUNK;          // last valid row of this chunk (>= 63 for a full one)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const uint32_t row = (uint32_t)min(row0 + 4 * j + lr, last);
          raw[j] = *reinterpret_cast<const uint4*>(cb + row * (uint32_t)(row_pitch * 2) + 16u * lc);
          // without normalisation the preparation never writes 1 / |k|: the workspace words are not read at all
          inv[j] = (q_side || !p.normalize_qk) ? 1.f : *reinterpret_cast<const float*>(ib + row * 4u);
        }
      };
      // K rows: scaled by 1 / |k|, rounded to the activation dtype (the operand of the reference), written as fp16,
      // which holds those values exactly; rows past the end of the sequence are zero.  Q rows feed the output only:
      // they are written as they are (fp16 of the raw value) and 1 / |q| goes to tRq, from where it enters the
      // output through the row factor scale e^G and P through its row factor.
      auto write_rows = [&](int c, const uint4 (&raw)[8], const float (&inv_in)[8]) {
        // The lane's 16 bytes are columns 8 lc .. 8 lc + 7 of row row0 + lr + 4 j: the first 8 bytes belong to granule
        // 4 (lc / 4) + 2 (lc % 2), half (lc / 2) % 2, the other 8 to the granule after it (same half).  The row's swizzle
        // 2 (row & 7) = 2 lr + 8 (j & 1) is even, so the second granule lies 16 bytes after the first.
        uint16_t* const tile = q_side ? tQ[c & 1] : tK[c & 1];
        const int g0 = 4 * (lc >> 2) + 2 * (lc & 1), half = (lc >> 1) & 1;
        uint16_t* const T_even = tile + (row0 + lr) * 128 + 8 * (g0 ^ (2 * lr)) + 4 * half;        // j even
        uint16_t* const T_odd = tile + (row0 + lr) * 128 + 8 * (g0 ^ (2 * lr + 8)) + 4 * half;     // j odd
        auto put = [&](int j, uint32_t w0, uint32_t w1, uint32_t w2, uint32_t w3) {
          uint16_t* const at = ((j & 1) ? T_odd : T_even) + 4 * j * 128;
          *reinterpret_cast<uint2*>(at) = make_uint2(w0, w1);
          *reinterpret_cast<uint2*>(at + 8) = make_uint2(w2, w3);
        };
        const int len = chunk_len(c);
        if constexpr (q_side) {
          float ss[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const uint32_t in[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
            uint32_t w[4];
            float acc = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float a0 = lo16<act_t>(in[e]), a1 = hi16<act_t>(in[e]);
              acc += a0 * a0 + a1 * a1;
              w[e] = pack2_rtz(a0, a1);
            }
            ss[j] = acc;
            put(j, w[0], w[1], w[2], w[3]);
          }
#pragma unroll
          for (int j = 0; j < 8; ++j) ss[j] = row16_allreduce(ss[j]);
          float* const rq = &tRq[c & 1][row0 + lr];
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const float r = rsqrtf(ss[j] + 1e-6f);
            if (lc == 0) rq[4 * j] = p.normalize_qk ? r : 1.f;
          }
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const uint32_t in[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
            const float inv = row0 + 4 * j + lr < len ? inv_in[j] : 0.f;
            uint32_t w[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const uint32_t r = pack2<act_t>(lo16<act_t>(in[e]) * inv, hi16<act_t>(in[e]) * inv);
              w[e] = pack2_rtz(lo16<act_t>(r), hi16<act_t>(r));
            }
            put(j, w[0], w[1], w[2], w[3]);
          }
        }
      };
      // P of chunk c from its K and Q tiles: this wavefront's blocks of the six
      auto form_p = [&](int c) {
        const uint16_t* const K = tK[c & 1];
        const uint16_t* const Q = tQ[c & 1];
        const float* const G = &tG[c & 1][256];
        auto block = [&](auto b_tag) {
          constexpr int b = decltype(b_tag)::value;
          constexpr int ni = tri_block_m(b), s = tri_block_s(b);
          constexpr int halves = 2 * s + 1 > ni ? 1 : 2;        // (nj, ni) products of this block that are not all zero
          bf16x8_t qb[4], kb_op[halves][4];
#pragma unroll
          for (int s2 = 0; s2 < 4; ++s2) qb[s2] = operand_granule(Q, 16 * ni + r16, s2, kb);
#pragma unroll
          for (int half = 0; half < halves; ++half)
#pragma unroll
            for (int s2 = 0; s2 < 4; ++s2) kb_op[half][s2] = operand_granule(K, 16 * (2 * s + half) + r16, s2, kb);
          const int i = 16 * ni + r16;
          const float Gi = G[i];
          const float pre = p.scale * tRq[c & 1][i];
          float4 Gj[halves];
#pragma unroll
          for (int half = 0; half < halves; ++half) Gj[half] = *reinterpret_cast<const float4*>(&G[16 * (2 * s + half) + 4 * kb]);
          f32x4_t acc[halves];
#pragma unroll
          for (int half = 0; half < halves; ++half) acc[half] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s2 = 0; s2 < 4; ++s2)
#pragma unroll
            for (int half = 0; half < halves; ++half) acc[half] = mfma16h(kb_op[half][s2], qb[s2], acc[half]);
          uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
          for (int half = 0; half < halves; ++half) {
            const int j0 = 16 * (2 * s + half) + 4 * kb;
            const float p0 = j0 <= i ? pre * acc[half][0] * __expf(Gi - Gj[half].x) : 0.f;
            const float p1 = j0 + 1 <= i ? pre * acc[half][1] * __expf(Gi - Gj[half].y) : 0.f;
            const float p2 = j0 + 2 <= i ? pre * acc[half][2] * __expf(Gi - Gj[half].z) : 0.f;
            const float p3 = j0 + 3 <= i ? pre * acc[half][3] * __expf(Gi - Gj[half].w) : 0.f;
            w[2 * half] = pack2_rtz(p0, p1);
            w[2 * half + 1] = pack2_rtz(p2, p3);
          }
          *reinterpret_cast<uint4*>(tP + b * 512 + lane * 8) = make_uint4(w[0], w[1], w[2], w[3]);
        };
        // three (nj, ni) products on each wavefront of the Q side, two on each of the K side (whose rows cost more)
        if constexpr (a == 0) block(std::integral_constant<int, 1>{});
        else if constexpr (a == 1) block(std::integral_constant<int, 5>{});
        else if constexpr (a == 2) { block(std::integral_constant<int, 0>{}); block(std::integral_constant<int, 3>{}); }
        else { block(std::integral_constant<int, 2>{}); block(std::integral_constant<int, 4>{}); }
      };

      // `raw` holds the rows of the chunk that is written next; the rows after those are requested right after
      // barrier A (behind the copies) into `ahead` and change over at the end of the iteration.
      uint4 raw[8], ahead[8];
      float inv[8], inv_ahead[8];
      if (n_chunks > 0) {
        issue_copies(0);
        load_rows(0, raw, inv);
        write_rows(0, raw, inv);
        if (n_chunks > 1) load_rows(1, raw, inv);
      }
      for (int ci = 0; ci < n_chunks; ++ci) {
        wait_vmcnt<0>();                               // this wavefront's copies for chunk ci have landed
        lds_barrier();                                 // barrier A (the rows this wavefront wrote are in LDS)
        if (ci + 1 < n_chunks) issue_copies(ci + 1);
        if (ci + 2 < n_chunks) load_rows(ci + 2, ahead, inv_ahead);
        form_p(ci);
        lds_barrier();                                 // barrier B (P is in LDS; copies and loads stay in flight)
        if (ci + 1 < n_chunks) write_rows(ci + 1, raw, inv);
        if (ci + 2 < n_chunks) {
#pragma unroll
          for (int j = 0; j < 8; ++j) { raw[j] = ahead[j]; inv[j] = inv_ahead[j]; }
        }
      }
    };
    if (wave == CW) feed(std::integral_constant<int, 0>{});
    else if (wave == CW + 1) feed(std::integral_constant<int, 1>{});
    else if (wave == CW + 2) feed(std::integral_constant<int, 2>{});
    else feed(std::integral_constant<int, 3>{});
    return;
  }

  // ---- the computing wavefronts ----
  const int vbase = 64 * v_half + 16 * NB * wave;
  const int vcol = vbase + r16;
  f32x4_t St[NB][8];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
    if (role.init != nullptr) {
      const float* src = role.init + (int64_t)(vcol + 16 * nb) * 128 + 4 * kb;
#pragma unroll
      for (int mc = 0; mc < 8; ++mc) {
        const float4 t4 = *reinterpret_cast<const float4*>(src + 16 * mc);
        St[nb][mc] = f32x4_t{t4.x, t4.y, t4.z, t4.w};
      }
    } else {
#pragma unroll
      for (int mc = 0; mc < 8; ++mc) St[nb][mc] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
  if (role.keep_init != nullptr) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      float* dst = role.keep_init + (int64_t)(vcol + 16 * nb) * 128 + 4 * kb;
#pragma unroll
      for (int mc = 0; mc < 8; ++mc)
        *reinterpret_cast<float4*>(dst + 16 * mc) = make_float4(St[nb][mc].x, St[nb][mc].y, St[nb][mc].z, St[nb][mc].w);
    }
  }
  uint16_t* const o_lane = reinterpret_cast<uint16_t*>(p.o) + ((int64_t)(seq_start + r16) * p.HV + hv) * 128 + vbase + 4 * kb;
  // V through the transposing read: lane t of a group addresses columns vbase + 16 nb + 4 (t % 4) .. + 3 of row
  // 16 mi + 4 kb + t / 4, i.e. half (t % 2) of granule 4 wave + 2 nb + (t % 4) / 2; the swizzle 8 (kb & 1) + 2 (t / 4)
  // of that row does not depend on mi, and block nb = 1 differs from nb = 0 in one bit of the granule index
  const int trV = (4 * kb + (r16 >> 2)) * 128 + 8 * ((vbase / 8 + ((r16 & 3) >> 1)) ^ (8 * (kb & 1) + 2 * (r16 >> 2))) + 4 * (r16 & 1);
  auto v_at = [&](const uint16_t* V, int mi, int nb) { return V + ((trV + 16 * 128 * mi) ^ (16 * nb)); };
  // Byte offsets of this lane's operand reads inside an operand tile.  The granule index enters the address in bits 4-7
  // and the swizzle is an exclusive or, so a step (or a group of 32 columns) further is one exclusive or of the WHOLE
  // address with 64 s (tile bases are multiples of 256); row blocks and halves are constant offsets of the read.
  // Only these two values are kept across chunks: a chunk derives its addresses from them behind an opaque
  // statement, so that the compiler does not carry one register per (tile, step) through the whole loop.
  const uint32_t offA0 = 2 * tile_offset(r16, kb);                          // row r16, granule kb (step 0)
  const uint32_t offT0 = 2 * tile_offset(4 * kb + (r16 >> 2), r16 & 3);     // transposing reads: row 4 kb + r16 / 4, granule r16 % 4
  typedef const __attribute__((address_space(3))) unsigned char* lds_bytes_t;
  auto opaque = [](uint32_t x) { asm volatile("" : "+v"(x)); return x; };
  auto read_operand = [](uint32_t base, int step, int byte_offset) {
    const lds_bytes_t at = (lds_bytes_t)(uintptr_t)(base ^ (64u * step));
    return __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const __attribute__((address_space(3))) u32x4_t*>(at + byte_offset));
  };
  // K^T operand (contraction half s2, column block m) = two transposing reads 16 rows apart
  auto read_transposed = [](uint32_t base, int s2, int m) {
    const lds_bytes_t at = (lds_bytes_t)(uintptr_t)(base ^ (64u * (m >> 1)));
    typedef __attribute__((address_space(3))) i16x4_t* tr_ptr_t;
    const i16x4_t p0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr_t)(at + 8192 * s2 + 8 * (m & 1)));
    const i16x4_t p1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr_t)(at + 8192 * s2 + 8 * (m & 1) + 4096));
    typedef short i16x8_t __attribute__((ext_vector_type(8)));
    const i16x8_t u = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
    return __builtin_bit_cast(bf16x8_t, u);
  };
  const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};

  auto pk = [](float x, float y) { return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(x, y)); };
  auto pk_sat = [](float x, float y) {
    const f32x2_t c = {__builtin_amdgcn_fmed3f(x, -65504.f, 65504.f), __builtin_amdgcn_fmed3f(y, -65504.f, 65504.f)};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(c, f16x2_t));
  };
  // hi = x rounded toward zero (which saturates at the largest finite fp16 value by itself), lo = the rest,
  // again toward zero: hi + lo carries x to about 21 bits
  auto pk_pair = [](float x, float y) {
    const auto hh = __builtin_amdgcn_cvt_pkrtz(x, y);
    return make_uint2(__builtin_bit_cast(uint32_t, hh),
                      __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(x - (float)hh[0], y - (float)hh[1])));
  };
  auto op = [](u32x4_t w) { return __builtin_bit_cast(bf16x8_t, w); };

  // One chunk.  FULL: all 64 rows are tokens (no store masks).
  auto chunk = [&](int ci, auto full_tag) __attribute__((always_inline)) {
    constexpr bool FULL = decltype(full_tag)::value;
    const int par = ci & 1;
    const uint16_t* const K = tK[par];
    const uint16_t* const Q = tQ[par];
    const uint16_t* const V = tV[par];
    const uint16_t* const Wt = tW[par];
    const uint16_t* const Pt = tP;
    const float* const G = tG[par];
    const uint32_t kA = opaque(lds_address(K) + offA0), qA = opaque(lds_address(Q) + offA0), kT = opaque(lds_address(K) + offT0);
    auto ldK = [&](int j) { return read_operand(kA, j >> 2, 4096 * (j & 3)); };
    auto ldQ = [&](int j) { return read_operand(qA, j >> 2, 4096 * (j & 3)); };
    // W operands in the order they are used: 0-3 lo (s 0, m 0..3), 4-7 hi (s 0), 8-9 lo (s 1, m 2, 3), 10-11 hi (s 1);
    // block b = m for s 0, 4 and 5 for s 1 (tri_block_m / tri_block_s), hi blocks first in the tile, then lo
    auto w_blk = [](int w) { return w < 8 ? (w & 3) : 4 + (w & 1); };
    auto w_mi = [](int w) { return tri_block_m(w < 8 ? (w & 3) : 4 + (w & 1)); };
    auto w_s = [](int w) { return w < 8 ? 0 : 1; };
    auto ldW = [&](int w) {
      const bool lo = (w < 4) || (w == 8) || (w == 9);
      return __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(Wt + ((lo ? TRI_BLOCKS : 0) + w_blk(w)) * 512 + lane * 8));
    };
    // P operands: block i (token rows tri_block_m(i), contraction half tri_block_s(i))
    auto p_ni = [](int i) { return tri_block_m(i); };
    auto p_s = [](int i) { return tri_block_s(i); };
    auto ldP = [&](int i) { return __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(Pt + i * 512 + lane * 8)); };

    // ================= phase 1: KS = K S^T =================
    bf16x8_t ka[16];
    u32x4_t sb[4][NB];
#pragma unroll
    for (int j = 0; j < 6; ++j) ka[j] = ldK(j);
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
      sb[0][nb] = u32x4_t{pk(St[nb][0][0], St[nb][0][1]), pk(St[nb][0][2], St[nb][0][3]), pk(St[nb][1][0], St[nb][1][1]),
                          pk(St[nb][1][2], St[nb][1][3])};
    SB();
    f32x4_t KS[NB][4];
    uint2 vraw[4][NB];
    float4 eg[4];
    float sq[4], egl;
    bf16x8_t qa[16];
    u32x4_t sq_[4][NB];          // the state operands again for the query product
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int s = j >> 2, mi = j & 3;
      if (j + 6 < 16) ka[j + 6] = ldK(j + 6);
      else if (j == 10) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) { vraw[0][nb] = read_tr4(v_at(V, 0, nb)); vraw[1][nb] = read_tr4(v_at(V, 1, nb)); }
      } else if (j == 11) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) { vraw[2][nb] = read_tr4(v_at(V, 2, nb)); vraw[3][nb] = read_tr4(v_at(V, 3, nb)); }
      } else if (j == 12) {
#pragma unroll
        for (int m2 = 0; m2 < 4; ++m2) eg[m2] = *reinterpret_cast<const float4*>(&G[64 + 16 * m2 + 4 * kb]);
      } else {
        qa[2 * (j - 13)] = ldQ(2 * (j - 13));
        qa[2 * (j - 13) + 1] = ldQ(2 * (j - 13) + 1);
      }
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        KS[nb][mi] = mfma16h(ka[j], op(sb[s][nb]), s == 0 ? zero4 : KS[nb][mi]);
      if (s < 3) {
        // dword mi of the next step's state operands
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const f32x4_t src = St[nb][2 * s + 2 + (mi >> 1)];
          sb[s + 1][nb][mi] = (mi & 1) ? pk(src[2], src[3]) : pk(src[0], src[1]);
        }
      } else {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const f32x4_t src = St[nb][mi >> 1];
          sq_[0][nb][mi] = (mi & 1) ? pk(src[2], src[3]) : pk(src[0], src[1]);
        }
      }
      SB();
    }

    // ================= phase 2a: O^T = S Q^T (query product) under X = V - e^G (.) KS =================
    f32x4_t OT[NB][4];
    bf16x8_t wq[12];
    u32x4_t xb[2][NB];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int s = j >> 2, ni = j & 3;
      if (j + 6 < 16) qa[j + 6] = ldQ(j + 6);
      else wq[j - 10] = ldW(j - 10);
      if (j == 8) {
#pragma unroll
        for (int n2 = 0; n2 < 4; ++n2) sq[n2] = G[16 * n2 + r16] * tRq[par][16 * n2 + r16];
        egl = G[192];
      }
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        OT[nb][ni] = mfma16h(op(sq_[s][nb]), qa[j], s == 0 ? zero4 : OT[nb][ni]);
      if (s < 3) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const f32x4_t src = St[nb][2 * s + 2 + (ni >> 1)];
          sq_[s + 1][nb][ni] = (ni & 1) ? pk(src[2], src[3]) : pk(src[0], src[1]);
        }
      }
      if (j < 8 * NB) {
        // half an X tile: tile t = (mi, nb), elements 2 h, 2 h + 1
        const int t = j >> 1, mi = NB == 2 ? t >> 1 : t, nb = NB == 2 ? t & 1 : 0, hh = j & 1;
        const uint32_t w = hh ? vraw[mi][nb].y : vraw[mi][nb].x;
        const float v0 = lo16<act_t>(w), v1 = hi16<act_t>(w);
        const float e0 = hh ? eg[mi].z : eg[mi].x, e1 = hh ? eg[mi].w : eg[mi].y;
        const float x0 = v0 - e0 * KS[nb][mi][2 * hh], x1 = v1 - e1 * KS[nb][mi][2 * hh + 1];
        xb[mi >> 1][nb][2 * (mi & 1) + hh] = pk_sat(x0, x1);
      }
      SB();
    }

    // ================= phase 2b: U = W X (lower triangular W: 6 of the 8 operand blocks) =================
    f32x4_t U[NB][4];
    bf16x8_t pa[6];
    float4 dg[2][2];
#pragma unroll
    for (int w = 0; w < 12; ++w) {
      const int s = w_s(w), mi = w_mi(w);
      if (w + 6 < 12) wq[w + 6] = ldW(w + 6);
      else if (w == 9) {
        dg[0][0] = *reinterpret_cast<const float4*>(&G[128 + 4 * kb]);
        dg[0][1] = *reinterpret_cast<const float4*>(&G[128 + 16 + 4 * kb]);
      }
      const bool first = w < 4;        // first product into this accumulator (lo, s 0)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        U[nb][mi] = mfma16h(wq[w], op(xb[s][nb]), first ? zero4 : U[nb][mi]);
      // VALU underneath: the query product scaled by scale e^G (w 0..5), then the decay of the first half of S
      if (w < 4) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) OT[nb][w] *= sq[w];
      } else if (NB == 2 || w < 8) {
        const int mc = NB == 2 ? (w - 4) >> 1 : w - 4, nb = NB == 2 ? (w - 4) & 1 : 0;      // (mc, nb) for w = 4..11 -> mc 0..3
        St[nb][mc] *= egl;
      }
      SB();
    }

    // ================= phase 3: O^T += U^T P^T (6 operand blocks), under the hi/lo split of e^{G_last - G} (.) U =================
    // Barrier B: P of this chunk is complete (the other four wavefronts formed it while phases 1 to 2b ran, which
    // take them about as long); its operands are requested at once and arrive under the conversions of U.
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_barrier();
    SB();
#pragma unroll
    for (int i = 0; i < TRI_BLOCKS; ++i) pa[i] = ldP(i);
    SB();
    u32x4_t ur[2][NB];
    u32x4_t ubh[2][NB], ubl[2][NB];
    bf16x8_t kt[16];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      ur[0][nb] = u32x4_t{pk(U[nb][0][0], U[nb][0][1]), pk(U[nb][0][2], U[nb][0][3]), pk(U[nb][1][0], U[nb][1][1]), pk(U[nb][1][2], U[nb][1][3])};
      ur[1][nb] = u32x4_t{pk(U[nb][2][0], U[nb][2][1]), pk(U[nb][2][2], U[nb][2][3]), pk(U[nb][3][0], U[nb][3][1]), pk(U[nb][3][2], U[nb][3][3])};
    }
    SB();
#pragma unroll
    for (int i = 0; i < 6; ++i) {
      const int s = p_s(i), ni = p_ni(i);
      if (i >= 2) kt[i - 2] = read_transposed(kT, 0, i - 2);       // kt[0..3]: (s 0, mc 0..3)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) OT[nb][ni] = mfma16h(op(ur[s][nb]), pa[i], OT[nb][ni]);
      if (i < 4) {
        // ub[0][nb] dword i: from U tile (i >> 1), elements 2 (i & 1), +1
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const int tl = i >> 1, e = 2 * (i & 1);
          const float4 d = dg[0][tl];
          const float d0 = e ? d.z : d.x, d1 = e ? d.w : d.y;
          const uint2 hl = pk_pair(U[nb][tl][e] * d0, U[nb][tl][e + 1] * d1);
          ubh[0][nb][i] = hl.x; ubl[0][nb][i] = hl.y;
        }
      } else {
        // the decay of S, rows mc 4, 5 (both nb) under the last two steps
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) St[nb][i] *= egl;
      }
      SB();
    }

    // ================= phase 4: S^T = e^{G_last} S^T + K^T (e^{G_last - G} (.) U), output under it =================
    const int len = FULL ? CHUNK : chunk_len(ci);
    uint16_t* const dst = o_lane + (int64_t)ci * CHUNK * p.HV * 128;
    // The K^T operands go through in pairs: the lo products of both, then the hi products, so that two products into
    // the same accumulator are four MFMAs apart (the accumulator changes registers between them, which makes the
    // second wait for the first to retire).  Step k handles pair k / 2: even k the lo products, odd k the hi ones.
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int pair = k >> 1, s = pair >> 2, mc0 = 2 * (pair & 3);
      const bool hi_part = k & 1;
      if (!hi_part && 2 * pair + 4 < 16) {
        kt[2 * pair + 4] = read_transposed(kT, (2 * pair + 4) >> 3, (2 * pair + 4) & 7);
        kt[2 * pair + 5] = read_transposed(kT, (2 * pair + 5) >> 3, (2 * pair + 5) & 7);
      }
      if (k == 0) {
        dg[1][0] = *reinterpret_cast<const float4*>(&G[128 + 32 + 4 * kb]);
        dg[1][1] = *reinterpret_cast<const float4*>(&G[128 + 48 + 4 * kb]);
      }
      if (k == 0) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) St[nb][6] *= egl;
      } else if (k == 1) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) St[nb][7] *= egl;
      }
#pragma unroll
      for (int m2 = 0; m2 < 2; ++m2)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
          St[nb][mc0 + m2] = mfma16h(kt[2 * pair + m2], op(hi_part ? ubh[s][nb] : ubl[s][nb]), St[nb][mc0 + m2]);
      if (k >= 2 && k < 6) {
        // ub[1][nb] dword (k - 2)
        const int i = k - 2;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
          const int tl = i >> 1, e = 2 * (i & 1);
          const float4 d = dg[1][tl];
          const float d0 = e ? d.z : d.x, d1 = e ? d.w : d.y;
          const uint2 hl = pk_pair(U[nb][2 + tl][e] * d0, U[nb][2 + tl][e + 1] * d1);
          ubh[1][nb][i] = hl.x; ubl[1][nb][i] = hl.y;
        }
      } else if (k >= 8 && k < 12) {
        // output rows of token block ni = k - 8
        const int ni = k - 8;
        if (FULL || 16 * ni + r16 < len) {
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) {
            const uint2 packed = make_uint2(pack2<act_t>(OT[nb][ni][0], OT[nb][ni][1]), pack2<act_t>(OT[nb][ni][2], OT[nb][ni][3]));
            *reinterpret_cast<uint2*>(dst + (int64_t)16 * ni * p.HV * 128 + 16 * nb) = packed;
          }
        }
      }
      SB();
    }
  };

  wait_vmcnt<0>();                                   // the start state has arrived: no wait for it inside the loop
  for (int ci = 0; ci < n_chunks; ++ci) {
    __builtin_amdgcn_s_waitcnt(0xc07f);              // lgkmcnt(0) only: output stores may stay in flight
    __builtin_amdgcn_s_barrier();                    // barrier A: the tiles of chunk ci are complete
    if (ci + 1 < n_chunks || seq_len - ci * CHUNK == CHUNK) chunk(ci, std::true_type{});
    else chunk(ci, std::false_type{});
  }

  if (role.fin != nullptr) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      float* dst = role.fin + (int64_t)(vcol + 16 * nb) * 128 + 4 * kb;
#pragma unroll
      for (int mc = 0; mc < 8; ++mc)
        *reinterpret_cast<float4*>(dst + 16 * mc) = make_float4(St[nb][mc].x, St[nb][mc].y, St[nb][mc].z, St[nb][mc].w);
    }
  }
}
#undef SB

// One workgroup per (sequence, value head), or per (segment, value head) in the second sweep over segments (NB = 2);
// NB = 1: two per chain, 64 V columns each (the columns of V are independent: same bits).
template <typename act_t, int NB>
__global__ __launch_bounds__(512, 1) void gdn_fused_sweep_kernel(const GdnPrefillParams p) {
  constexpr int HALVES = 2 / NB;
  __shared__ __align__(1024) unsigned char lds_all[FUSED_LDS_BYTES];
  const int wide = xcd_grouped_index(blockIdx.x, HALVES * (p.HV / p.H), HALVES * (p.pass == 2 ? p.seg.max_segments : p.N) * p.HV);
  if (wide < 0) return;
  fused_sweep<act_t, NB>(p, lds_all, wide);
}

// Whole sequences of unequal length, swept in one launch whose longest chains decide how long it lasts while the CUs
// of chains that have ended stand idle: the chains of the longest sequences are swept as two halves (which start
// first: workgroups are dispatched in index order), those of the others whole, longest first.
template <typename act_t>
__global__ __launch_bounds__(512, 1) void gdn_fused_sweep_mixed_kernel(const GdnPrefillParams p) {
  __shared__ __align__(1024) unsigned char lds_all[FUSED_LDS_BYTES];
  const int ratio = p.HV / p.H;
  if (blockIdx.x < p.split_grid) {
    const int wide = xcd_grouped_index(blockIdx.x, 2 * ratio, 2 * p.n_long * p.HV);
    if (wide < 0) return;
    const int chain = wide >> 1, k = chain / p.HV;
    fused_sweep<act_t, 1>(p, lds_all, 2 * (p.seq_order[k] * p.HV + chain - k * p.HV) + (wide & 1));
  } else {
    const int chain = xcd_grouped_index(blockIdx.x - p.split_grid, ratio, (p.N - p.n_long) * p.HV);
    if (chain < 0) return;
    const int k = chain / p.HV;
    fused_sweep<act_t, 2>(p, lds_all, p.seq_order[p.n_long + k] * p.HV + chain - k * p.HV);
  }
}

struct GdnWorkspaceLayout {
  size_t seq_chunk_off, chunk_seq, chunk_tok, chunk_len, q_rows, k_rows, kn, kinv, gtile, W;
  size_t seq_seg_off, seg_seq, seg_c0, seg_nc, segM, segB, segS, identity;
  size_t order, stage_begin, carry, total;
  int NC_max, seg_chunks, max_segments, stages;
};
// The plan for a call of N <= INLINE_TABLE_SEQUENCES whole sequences run in `stages` stages (0: unstaged): *stage
// receives the stage whose sweep is the last one.
static int mixed_sweep_from_offsets(const int32_t* raw_cu_seqlens, int N, int HV, int stages, unsigned char* order, int* stage) {
  int nc[INLINE_TABLE_SEQUENCES], r[INLINE_TABLE_SEQUENCES];
  int64_t total = 0;
  int longest = 0;
  for (int n = 0; n < N; ++n) {
    nc[n] = (std::max(raw_cu_seqlens[n + 1] - raw_cu_seqlens[n], 0) + CHUNK - 1) / CHUNK;
    total += nc[n];
    longest = std::max(longest, nc[n]);
  }
  const int plan = stage_plan(total, N, longest, stages);
  const int last = plan_stages(plan) - 1;
  for (int n = 0; n < N; ++n) r[n] = stage_cut(nc[n], last + 1, plan) - stage_cut(nc[n], last, plan);
  *stage = last;
  return mixed_sweep_plan(r, N, HV, order);
}

static GdnWorkspaceLayout gdn_layout(int T, int N, int H, int HV, bool allow_stages = true) {
  GdnWorkspaceLayout L;
  L.NC_max = T / CHUNK + N;
  size_t off = 0;
  auto take = [&](size_t bytes) { const size_t at = off; off = align_up256(off + bytes); return at; };
  L.seq_chunk_off = take((size_t)(N + 1) * 4);
  L.chunk_seq = take((size_t)L.NC_max * 4);
  L.chunk_tok = take((size_t)L.NC_max * 4);
  L.chunk_len = take((size_t)L.NC_max * 4);
  L.q_rows = take((size_t)T * H * 128 * 2);              // aligned copies of q and k rows that are not
  L.k_rows = take((size_t)T * H * 128 * 2);
  L.kn = take((size_t)T * H * 128 * 2);
  L.kinv = take((size_t)T * H * 4);
  L.gtile = take((size_t)L.NC_max * HV * GTILE_FLOATS * 4);
  L.W = take((size_t)L.NC_max * HV * 2 * TRI_BLOCKS * 1024);
  L.seg_chunks = pick_segment_chunks(T, N, HV);
  L.max_segments = max_segments(T, N, L.seg_chunks);
  if (L.seg_chunks > 0) {
    L.seq_seg_off = take((size_t)(N + 1) * 4);
    L.seg_seq = take((size_t)L.max_segments * 4);
    L.seg_c0 = take((size_t)L.max_segments * 4);
    L.seg_nc = take((size_t)L.max_segments * 4);
    const size_t states = (size_t)L.max_segments * HV * 16384 * 4;
    L.segM = take(states); L.segB = take(states); L.segS = take(states);
    L.identity = take(16384 * 4);
  }
  // pipeline the preparation with the sweeps in stages where that pays
  L.stages = allow_stages ? pick_stages(T, N, HV, L.seg_chunks) : 0;
  if (L.stages > 0) {
    L.order = take((size_t)L.NC_max * 4);
    L.stage_begin = take((size_t)(MAX_STAGES + 2) * 4);
    L.carry = L.seg_chunks > 0 ? 0 : take((size_t)N * HV * 16384 * 4);
  }
  L.total = off;
  return L;
}


// Workspace of pla_gdn_prefill_launch_static: one array per GPU, held until the process ends.  In host code the
// array's name is only a handle for the runtime, not a device address; the address on the current device comes from
// hipGetSymbolAddress, is looked up once per device and is what kernels and launches receive.
static __device__ __align__(256) unsigned char scratch[PLA_GDN_PREFILL_STATIC_BYTES];
// The first look-up on a device may load the code object, which must not happen while `stream` captures a graph: a
// capturing caller that has not called the entry point on this device before gets CAPTURE_BEFORE_LOOKUP back.
static void* const CAPTURE_BEFORE_LOOKUP = reinterpret_cast<void*>(1);
static void* static_scratch_address(hipStream_t stream) {
  static void* address[64] = {};
  static std::mutex guard;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  std::lock_guard<std::mutex> lock(guard);
  if (address[dev] == nullptr) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess || status != hipStreamCaptureStatusNone) return CAPTURE_BEFORE_LOOKUP;
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
    address[dev] = ptr;
  }
  return address[dev];
}

}  // namespace pla

using namespace pla;

extern "C" int64_t pla_gdn_prefill_workspace_bytes(int T, int N, int H, int HV) {
  if (T <= 0 || N <= 0 || H <= 0 || HV <= 0) return 0;
  return (int64_t)gdn_layout(T, N, H, HV).total;
}

// Checks and launches shared by the entry points below.  static_scratch: the workspace is the library's own
// array (sized by the unstaged layout, which needs no side stream), else the caller's buffer.
static int gdn_prefill_run(
    const void* q, const void* k, const void* v, int64_t stride_q, int64_t stride_k, int64_t stride_v,
    const void* a, const void* b, int64_t stride_a, int64_t stride_b,
    const float* A_log, const float* dt_bias, const float* g_in, const float* beta_in,
    const int32_t* cu_seqlens, int N, int T, float scale, int normalize_qk,
    const float* h0, const int32_t* h0_indices, int64_t h0_slot_stride,
    float* ht, const int32_t* ht_indices, int64_t ht_slot_stride,
    void* o, void* workspace, int64_t workspace_bytes, bool static_scratch,
    float* gcum_out, float* beta_out,
    int H, int HV, int K, int V, int act_dtype, void* stream, const int32_t* raw_cu_seqlens = nullptr) {
  PLA_REQUIRE(K == 128 && V == 128, "GDN prefill requires head_dim K == V == 128, got K=%d, V=%d", K, V);
  PLA_REQUIRE(T > 0 && N > 0, "GDN prefill needs at least one token and one sequence");
  PLA_REQUIRE(H > 0 && HV >= H && HV % H == 0, "HV must be a positive multiple of H, got H=%d, HV=%d", H, HV);
  PLA_REQUIRE(act_dtype == PLA_BF16 || act_dtype == PLA_F16, "GDN prefill takes bf16 or fp16 activations");
  const bool half_act = act_dtype == PLA_F16;
  PLA_REQUIRE(q && k && v && o && cu_seqlens, "null tensor pointer");
  PLA_REQUIRE((g_in != nullptr) == (beta_in != nullptr), "g and beta must be given together");
  PLA_REQUIRE(g_in != nullptr || (a && b && A_log && dt_bias), "raw gating needs a, b, A_log and dt_bias");
  PLA_REQUIRE(((uintptr_t)q % 4 == 0) && ((uintptr_t)k % 4 == 0) && stride_q % 2 == 0 && stride_k % 2 == 0,
              "q/k rows require 4-byte alignment");
  PLA_REQUIRE((uintptr_t)v % 16 == 0 && stride_v % 8 == 0, "v rows require 16-byte alignment (they are copied to LDS in 16-byte pieces)");
  PLA_REQUIRE((uintptr_t)o % 16 == 0, "o requires 16-byte alignment");
  PLA_REQUIRE((uintptr_t)gcum_out % 16 == 0 && (uintptr_t)beta_out % 16 == 0, "gcum_out and beta_out require 16-byte alignment");
  const GdnWorkspaceLayout L = gdn_layout(T, N, H, HV, !static_scratch);
  if (static_scratch) {
    PLA_REQUIRE((int64_t)L.total <= PLA_GDN_PREFILL_STATIC_BYTES,
                "call too large for the built-in scratch array: it needs %zu bytes of workspace, the array holds %lld "
                "(use pla_gdn_prefill_launch with a caller workspace)", L.total, (long long)PLA_GDN_PREFILL_STATIC_BYTES);
    workspace = static_scratch_address(reinterpret_cast<hipStream_t>(stream));
    PLA_REQUIRE(workspace != CAPTURE_BEFORE_LOOKUP,
                "the first call of pla_gdn_prefill_launch_static on a device looks up the scratch array's address and must "
                "not be captured: call it once on this device before capturing");
    PLA_REQUIRE(workspace != nullptr, "hipGetSymbolAddress failed for the built-in scratch array");
  } else {
    PLA_REQUIRE(workspace != nullptr, "null tensor pointer");
    PLA_REQUIRE(workspace_bytes >= (int64_t)L.total, "workspace too small: need %zu bytes", L.total);
  }
  PLA_REQUIRE((uintptr_t)workspace % 256 == 0, "workspace requires 256-byte alignment");
  if (h0) PLA_REQUIRE((uintptr_t)h0 % 16 == 0 && h0_slot_stride % 4 == 0, "state requires 16-byte alignment");
  if (ht) PLA_REQUIRE((uintptr_t)ht % 16 == 0 && ht_slot_stride % 4 == 0, "state requires 16-byte alignment");

  char* ws = reinterpret_cast<char*>(workspace);
  GdnPrefillParams p{};
  p.q = q; p.k = k; p.v = v; p.stride_q = stride_q; p.stride_k = stride_k; p.stride_v = stride_v;
  p.a = a; p.b = b; p.stride_a = stride_a; p.stride_b = stride_b;
  p.A_log = A_log; p.dt_bias = dt_bias; p.g_in = g_in; p.beta_in = beta_in;
  p.cu_seqlens = cu_seqlens; p.N = N; p.T = T; p.scale = scale; p.normalize_qk = normalize_qk;
  p.h0 = h0; p.h0_indices = h0_indices; p.h0_slot_stride = h0_slot_stride;
  p.ht = ht; p.ht_indices = ht_indices; p.ht_slot_stride = ht_slot_stride;
  p.o = o;
  p.seq_chunk_off = reinterpret_cast<int32_t*>(ws + L.seq_chunk_off);
  p.chunk_seq = reinterpret_cast<int32_t*>(ws + L.chunk_seq);
  p.chunk_tok = reinterpret_cast<int32_t*>(ws + L.chunk_tok);
  p.chunk_len = reinterpret_cast<int32_t*>(ws + L.chunk_len);
  p.kn = reinterpret_cast<uint16_t*>(ws + L.kn);
  p.kinv = reinterpret_cast<float*>(ws + L.kinv);
  p.gcum = gcum_out;
  p.beta = beta_out;
  p.gtile = reinterpret_cast<float*>(ws + L.gtile);
  p.W = reinterpret_cast<uint16_t*>(ws + L.W);
  p.H = H; p.HV = HV; p.NC_max = L.NC_max;

  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const bool segmented = L.seg_chunks > 0;
  // the kernels read q and k rows in 16-byte pieces: rows that start on 4-byte boundaries only are copied first
  if (!((uintptr_t)q % 16 == 0 && (uintptr_t)k % 16 == 0 && stride_q % 8 == 0 && stride_k % 8 == 0)) {
    uint16_t* const q_rows = reinterpret_cast<uint16_t*>(ws + L.q_rows);
    uint16_t* const k_rows = reinterpret_cast<uint16_t*>(ws + L.k_rows);
    const int64_t threads = (int64_t)T * H * 32;
    hipLaunchKernelGGL(gdn_align_rows_kernel, dim3((unsigned)std::min<int64_t>((threads + 255) / 256, 8192)), dim3(256), 0, s,
                       reinterpret_cast<const uint16_t*>(q), reinterpret_cast<const uint16_t*>(k), stride_q, stride_k, T, H,
                       q_rows, k_rows);
    p.q = q_rows; p.k = k_rows;
    p.stride_q = p.stride_k = (int64_t)H * 128;
  }
  // a call split into segments: the preparation also stores the normalised K rows, which the first sweep copies
  p.store_kn = segmented;
  const bool v_halves = !segmented && (int64_t)N * HV <= 128;
  if (segmented) {
    // few, long sequences: sweep their segments concurrently (two sweeps and a combine step)
    p.seg.seq_seg_off = reinterpret_cast<int32_t*>(ws + L.seq_seg_off);
    p.seg.seg_seq = reinterpret_cast<int32_t*>(ws + L.seg_seq);
    p.seg.seg_c0 = reinterpret_cast<int32_t*>(ws + L.seg_c0);
    p.seg.seg_nc = reinterpret_cast<int32_t*>(ws + L.seg_nc);
    p.seg.M = reinterpret_cast<float*>(ws + L.segM);
    p.seg.B = reinterpret_cast<float*>(ws + L.segB);
    p.seg.S = reinterpret_cast<float*>(ws + L.segS);
    p.seg.identity = reinterpret_cast<float*>(ws + L.identity);
    p.seg.seg_chunks = L.seg_chunks;
    p.seg.max_segments = L.max_segments;
  }
  // the staged pipeline needs a side stream: without one (pool exhausted) the call runs unstaged, decided before
  // anything is launched
  // With the offsets on the host as well the host applies the device's own rule (stage_plan) ahead of it: chains of
  // nearly equal length run in one stage, and then nothing is enqueued for a second one (no side stream, no events,
  // no launches that find nothing to do).
  bool staged = L.stages > 0;
  if (staged && raw_cu_seqlens != nullptr) {
    int64_t total = 0;
    int longest = 0;
    for (int n = 0; n < N; ++n) {
      const int nc = (std::max(raw_cu_seqlens[n + 1] - raw_cu_seqlens[n], 0) + CHUNK - 1) / CHUNK;
      total += nc;
      longest = std::max(longest, nc);
    }
    staged = 5 * total < 4 * (int64_t)N * longest;
  }
  const SideStreamLease lease(s, staged);
  const int stages = lease.get() != nullptr ? L.stages : 0;
  if (stages > 0) {
    p.stg.order = reinterpret_cast<int32_t*>(ws + L.order);
    p.stg.stage_begin = reinterpret_cast<int32_t*>(ws + L.stage_begin);
    p.stg.carry = segmented ? nullptr : reinterpret_cast<float*>(ws + L.carry);
    p.stg.stages = stages;
  }
  // Ragged whole sequences whose offsets the host holds: the last (or only) sweep runs the chains of the longest
  // sequences as two halves where that shortens it (mixed_sweep_plan)
  // More chains than CUs: every sweep of the call also starts its chains longest first (in the order of the
  // sequences the last chain to find a CU may be the longest one, and the launch then ends that much later).
  int mixed_stage = -1, halved = 0;
  bool longest_first = false;
  if (!segmented && !v_halves && raw_cu_seqlens != nullptr && N <= INLINE_TABLE_SEQUENCES) {
    halved = mixed_sweep_from_offsets(raw_cu_seqlens, N, HV, stages, p.seq_order, &mixed_stage);
    if (halved == 0) mixed_stage = -1;
    longest_first = (int64_t)N * HV > CUS;
  }
  // At most 64 sequences: no table kernel runs ahead of the preparation, whose first launch also zeroes the padded
  // rows of o.  Whole sequences: every kernel works its chunks out by itself.  Segments: the
  // preparation does, and one workgroup appended to it writes the chunk and segment tables for the sweeps.
  p.inline_tables = N <= INLINE_TABLE_SEQUENCES;
  if (!p.inline_tables)
    launch_tables(s, cu_seqlens, N, T, L.NC_max, p.seq_chunk_off, p.chunk_seq, p.chunk_tok, p.chunk_len, p.seg, p.stg,
                  segmented ? L.max_segments : N, o, HV);
  const bool ok = launch_pipeline(
      s, stages, lease.get(), segmented, (unsigned)N * HV, (unsigned)L.max_segments * HV, &p.pass, &p.stage,
      [&](hipStream_t ps) {
        const int ratio = HV / H;       // value heads per q/k head: as many wavefronts of a workgroup share K and Q
        const int waves = ratio % 4 == 0 ? 4 : ratio % 2 == 0 ? 2 : 1;
        p.tail_blocks = (p.inline_tables && p.stage == 0) ? TABLE_WORKGROUPS - (segmented ? 0 : 1) : 0;
        const dim3 grid((unsigned)L.NC_max * (HV / waves) + p.tail_blocks), block(64 * waves);
        if (half_act) {
          if (waves == 4) hipLaunchKernelGGL((gdn_wsolve_kernel<f16_t, 4>), grid, block, 0, ps, p);
          else if (waves == 2) hipLaunchKernelGGL((gdn_wsolve_kernel<f16_t, 2>), grid, block, 0, ps, p);
          else hipLaunchKernelGGL((gdn_wsolve_kernel<f16_t, 1>), grid, block, 0, ps, p);
        } else {
          if (waves == 4) hipLaunchKernelGGL((gdn_wsolve_kernel<bf16_t, 4>), grid, block, 0, ps, p);
          else if (waves == 2) hipLaunchKernelGGL((gdn_wsolve_kernel<bf16_t, 2>), grid, block, 0, ps, p);
          else hipLaunchKernelGGL((gdn_wsolve_kernel<bf16_t, 1>), grid, block, 0, ps, p);
        }
      },
      [&](unsigned grid) {
        if (p.pass == 1) {        // first sweep over segments: no output, both roles in one workgroup per (segment, head)
          const unsigned g = xcd_grouped_grid(grid / 2, (unsigned)(HV / H));
          if (half_act) hipLaunchKernelGGL(gdn_lean_sweep_kernel<f16_t>, dim3(g), dim3(512), 0, s, p);
          else hipLaunchKernelGGL(gdn_lean_sweep_kernel<bf16_t>, dim3(g), dim3(512), 0, s, p);
        } else {
          // Whole sequences that give at most 128 chains (few long ones are split into segments instead) leave half of the CUs idle: two
          // workgroups then sweep a chain, 64 V columns each - the columns of V are independent, so the results are the
          // same bits.  A half costs 0.86 to 0.93 of a whole chain's chunk time (K, Q, W and P are fetched and formed once
          // per workgroup whatever its width): 4 x 4096 tokens of 32 value heads 0.248 -> 0.236 ms, 3 x 4096 0.227 -> 0.205.
          if (p.stage == mixed_stage || longest_first) {
            p.n_long = p.stage == mixed_stage ? halved : 0;
            p.split_grid = xcd_grouped_grid(2 * (unsigned)p.n_long * HV, 2 * (unsigned)(HV / H));
            const unsigned g = p.split_grid + xcd_grouped_grid((unsigned)(N - p.n_long) * HV, (unsigned)(HV / H));
            if (half_act) hipLaunchKernelGGL(gdn_fused_sweep_mixed_kernel<f16_t>, dim3(g), dim3(512), 0, s, p);
            else hipLaunchKernelGGL(gdn_fused_sweep_mixed_kernel<bf16_t>, dim3(g), dim3(512), 0, s, p);
          } else if (v_halves) {
            const unsigned g = xcd_grouped_grid(2 * grid, 2 * (unsigned)(HV / H));
            if (half_act) hipLaunchKernelGGL((gdn_fused_sweep_kernel<f16_t, 1>), dim3(g), dim3(512), 0, s, p);
            else hipLaunchKernelGGL((gdn_fused_sweep_kernel<bf16_t, 1>), dim3(g), dim3(512), 0, s, p);
          } else {
            const unsigned g = xcd_grouped_grid(grid, (unsigned)(HV / H));
            if (half_act) hipLaunchKernelGGL((gdn_fused_sweep_kernel<f16_t, 2>), dim3(g), dim3(512), 0, s, p);
            else hipLaunchKernelGGL((gdn_fused_sweep_kernel<bf16_t, 2>), dim3(g), dim3(512), 0, s, p);
          }
        }
      });
  PLA_REQUIRE(ok, "an event call of the staged prefill failed: %s", hipGetErrorString(hipGetLastError()));
  if (segmented) {
    hipLaunchKernelGGL(segment_combine_kernel, dim3(xcd_grouped_grid((unsigned)N * HV * COMBINE_SPLIT, COMBINE_SPLIT)), dim3(256), 0, s, p.seg, HV,
                       N * HV);
    p.pass = 2;
    // Segments are at least 16 chunks long, so short calls and calls of few heads give fewer (segment, head) pairs than
    // half of the CUs: the second sweep then runs two workgroups per pair, 64 V columns each, as above.  The number of
    // segments is known exactly where the caller passed the offsets on the host, else from the tokens alone.
    int64_t segments = N == 1 ? ((T + CHUNK - 1) / CHUNK + L.seg_chunks - 1) / L.seg_chunks : (int64_t)(T / CHUNK + N) / L.seg_chunks + N;
    if (raw_cu_seqlens != nullptr) {
      segments = 0;
      for (int n = 0; n < N; ++n) {
        const int nc = (std::max(raw_cu_seqlens[n + 1] - raw_cu_seqlens[n], 0) + CHUNK - 1) / CHUNK;
        segments += (nc + L.seg_chunks - 1) / L.seg_chunks;
      }
    }
    if (segments * HV <= 128) {
      const unsigned g = xcd_grouped_grid(2 * (unsigned)L.max_segments * HV, 2 * (unsigned)(HV / H));
      if (half_act) hipLaunchKernelGGL((gdn_fused_sweep_kernel<f16_t, 1>), dim3(g), dim3(512), 0, s, p);
      else hipLaunchKernelGGL((gdn_fused_sweep_kernel<bf16_t, 1>), dim3(g), dim3(512), 0, s, p);
    } else {
      const unsigned g = xcd_grouped_grid((unsigned)L.max_segments * HV, (unsigned)(HV / H));
      if (half_act) hipLaunchKernelGGL((gdn_fused_sweep_kernel<f16_t, 2>), dim3(g), dim3(512), 0, s, p);
      else hipLaunchKernelGGL((gdn_fused_sweep_kernel<bf16_t, 2>), dim3(g), dim3(512), 0, s, p);
    }
  }
  return check_launch("gdn prefill launch");
}

extern "C" int pla_gdn_prefill_launch(
    const void* q, const void* k, const void* v, int64_t stride_q, int64_t stride_k, int64_t stride_v,
    const void* a, const void* b, int64_t stride_a, int64_t stride_b,
    const float* A_log, const float* dt_bias, const float* g_in, const float* beta_in,
    const int32_t* cu_seqlens, int N, int T, float scale, int normalize_qk,
    const float* h0, const int32_t* h0_indices, int64_t h0_slot_stride,
    float* ht, const int32_t* ht_indices, int64_t ht_slot_stride,
    void* o, void* workspace, int64_t workspace_bytes,
    float* gcum_out, float* beta_out,
    int H, int HV, int K, int V, int act_dtype, void* stream) {
  return gdn_prefill_run(q, k, v, stride_q, stride_k, stride_v, a, b, stride_a, stride_b, A_log, dt_bias, g_in, beta_in,
                         cu_seqlens, N, T, scale, normalize_qk, h0, h0_indices, h0_slot_stride, ht, ht_indices,
                         ht_slot_stride, o, workspace, workspace_bytes, false, gcum_out, beta_out, H, HV, K, V, act_dtype,
                         stream);
}

extern "C" int pla_gdn_prefill_launch_raw(
    const void* q, const void* k, const void* v, int64_t stride_q, int64_t stride_k, int64_t stride_v,
    const void* a, const void* b, int64_t stride_a, int64_t stride_b,
    const float* A_log, const float* dt_bias, const float* g_in, const float* beta_in,
    const int32_t* cu_seqlens, int N, int T, float scale, int normalize_qk,
    const float* h0, const int32_t* h0_indices, int64_t h0_slot_stride,
    float* ht, const int32_t* ht_indices, int64_t ht_slot_stride,
    void* o, void* workspace, int64_t workspace_bytes,
    float* gcum_out, float* beta_out,
    int H, int HV, int K, int V, int act_dtype, void* stream, const int32_t* raw_cu_seqlens) {
  return gdn_prefill_run(q, k, v, stride_q, stride_k, stride_v, a, b, stride_a, stride_b, A_log, dt_bias, g_in, beta_in,
                         cu_seqlens, N, T, scale, normalize_qk, h0, h0_indices, h0_slot_stride, ht, ht_indices,
                         ht_slot_stride, o, workspace, workspace_bytes, false, gcum_out, beta_out, H, HV, K, V, act_dtype,
                         stream, raw_cu_seqlens);
}

extern "C" int pla_gdn_prefill_halved_sequences(const int32_t* raw_cu_seqlens, int N, int T, int H, int HV) {
  if (raw_cu_seqlens == nullptr || N <= 0 || N > INLINE_TABLE_SEQUENCES || T <= 0 || H <= 0 || HV < H || HV % H != 0) return 0;
  const GdnWorkspaceLayout L = gdn_layout(T, N, H, HV);
  if (L.seg_chunks > 0 || (int64_t)N * HV <= 128) return 0;
  unsigned char order[INLINE_TABLE_SEQUENCES];
  int stage = 0;
  return mixed_sweep_from_offsets(raw_cu_seqlens, N, HV, L.stages, order, &stage);
}

extern "C" int pla_gdn_prefill_launch_static(
    const void* q, const void* k, const void* v, int64_t stride_q, int64_t stride_k, int64_t stride_v,
    const void* a, const void* b, int64_t stride_a, int64_t stride_b,
    const float* A_log, const float* dt_bias, const float* g_in, const float* beta_in,
    const int32_t* cu_seqlens, int N, int T, float scale, int normalize_qk,
    const float* h0, const int32_t* h0_indices, int64_t h0_slot_stride,
    float* ht, const int32_t* ht_indices, int64_t ht_slot_stride,
    void* o, float* gcum_out, float* beta_out,
    int H, int HV, int K, int V, int act_dtype, void* stream) {
  return gdn_prefill_run(q, k, v, stride_q, stride_k, stride_v, a, b, stride_a, stride_b, A_log, dt_bias, g_in, beta_in,
                         cu_seqlens, N, T, scale, normalize_qk, h0, h0_indices, h0_slot_stride, ht, ht_indices,
                         ht_slot_stride, o, nullptr, 0, true, gcum_out, beta_out, H, HV, K, V, act_dtype, stream);
}
