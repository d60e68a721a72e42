// Chunk-64 gated delta-rule prefill for KDA (per-channel gate) on gfx950.
//
// Per chunk of C = 64 tokens, with G_i[c] the inclusive cumulative log-decay of channel c inside
// the chunk (g <= 0, so G decreases along the chunk) and S the FP32 k-last state:
//     M_ij = sum_c k_i[c] k_j[c] e^{G_i[c] - G_j[c]}   (i > j)      L = I + diag(beta) M
//     P_ij = scale sum_c q_i[c] k_j[c] e^{G_i[c] - G_j[c]}   (i >= j)
//     W    = L^-1 diag(beta)
//     X    = V - (K (.) e^{G}) S^T            U = W X
//     O    = scale (Q (.) e^{G}) S^T + P U
//     S^T  = e^{G_last} (.) S^T + (K (.) e^{G_last - G})^T U
// (reference pipeline: src/prefill/flashkdapro/tc01/fla/runtime.cc:474-545 - gate, token, inter,
// recompute, recurrence, output; public contract pla/prefill/flashkdapro/ops.py:68-219).
// The gate cannot be factored out of the products here, so the decayed operands are formed in
// FP32.  In M / P every exponent is <= 0 except inside a 16-row diagonal block, where the reference row
// is the block's first row and the exponent is bounded by 15 tokens of decay (|lower_bound| <= 5
// gives e^75, well inside the bf16 / FP32 range) - the same sub-chunk scheme as the reference's
// FLA kernels (scripts/prefill/private/ref/chunk_intra.py:170-202); those operands are split into
// bf16 hi + lo parts (bf16 has the range, the pair the precision).  The operands of the sequential
// sweep (k e^{G}, q e^{G}, k e^{G_last - G}, W, P, S, X, U) all carry factors in (0, 1] and go to the
// MFMA as fp16, rounded once.
//
// Kernels:
//   kda_prep_solve_kernel   one workgroup per (chunk, head): q/k L2 norm (rounded to bf16), lower-bound
//                           gate, cumulative decay, decayed operand tiles (fp16), M / P on MFMA, the
//                           inverse of I + L by 16 x 16 blocks, W and P (fp16)
//   kda_sweep_kernel        one workgroup per (sequence, head) or second segment sweep: four computing
//                           wavefronts x 32 V columns with a register-chained MFMA pipeline, two wavefronts
//                           that issue the asynchronous global -> LDS tile copies; writes o; with NB = 1 two
//                           workgroups per chain, 64 V columns each (calls of at most 128 chains)
//   kda_sweep_mixed_kernel  the same sweep for ragged whole sequences: the chains of the longest sequences as two
//                           halves, the others whole, in one launch (plan from the host offsets)
//   kda_lean_sweep_kernel   first sweep over segments: the zero-state sweep and the transition-matrix
//                           sweep of two segments in one workgroup of eight wavefronts, no output
// The operands of every sweep product are fp16 (v_mfma_f32_16x16x32_f16): the decayed tiles hold factors in
// (0, 1].  W, K e^{G_last-G} and the U of the state update are hi + lo pairs; a float64 simulation of these
// rounding points gives a final-state rel-L2 below 5e-4 from strong to weak decay (bound 1e-3); the pairs are
// what keeps keys that repeat within a chunk inside the same bound (measured on such keys: 3.3e-4 .. 3.7e-4 with the
// pairs, 1.7e-3 with K e^{G_last-G} rounded once).  The K e^{G_last-G} tile is stored row major like the others; its transposed
// operands come from ds_read_b64_tr_b16.

#include "prefill_common.h"

namespace pla {

// Wavefronts of kda_sweep_kernel that issue its global -> LDS copies.  One wavefront holds at most 63 memory
// operations in flight (1 KiB each here); two share the issue work and that limit (config 4: 2.46 -> 2.44 ms, 2.43 ms
// with three).
constexpr int KDA_SWEEP_COPIERS = 2;
struct KdaPrefillParams {
  const void* q; const void* k; const void* v; const void* g; const void* beta;   // bf16
  int64_t stride_q, stride_k, stride_v, stride_g, stride_beta;                    // token pitches (elements)
  const float* A_log; const float* dt_bias;                                       // [H], [H*128]
  float lower_bound, scale;
  const int32_t* cu_seqlens; int N; int T;
  const float* h0; const int32_t* h0_indices; int64_t h0_slot_stride;
  float* ht; const int32_t* ht_indices; int64_t ht_slot_stride;
  void* o;
  int32_t* seq_chunk_off; int32_t* chunk_seq; int32_t* chunk_tok; int32_t* chunk_len;
  // operand tiles of the sweeps, fp16 (every factor lies in (0, 1]; values below 6e-8 vanish)
  uint16_t* Kg; uint16_t* Qg;                      // [chunk, H, 64, 128]: k e^{G}, scale q e^{G}
  uint16_t* Kt;                                    // [chunk, H, 2, 64, 128]: k e^{G_last - G} as an fp16 hi + lo pair
  uint16_t* W;                                     // [chunk, H, 2, 6 blocks]: W = hi + lo in the six-block operand layout (prefill_common.h)
  uint16_t* P;                                     // [chunk, H, 6 blocks]: P in the same layout
  float* eGlast;                                   // [chunk, H, 128]: e^{G_last}
  SegmentTable seg;                                // split long sequences (seg.seg_chunks > 0)
  StageTable stg;                                  // pipelined preparation and sweep (stg.stages > 0)
  int pass;                                        // 0: whole sequences; 1, 2: the two sweeps over segments
  int stage;                                       // stage handled by this launch (prep kernel, passes 0 and 1)
  int H, NC_max;
  // kda_sweep_mixed_kernel: the first `split_grid` workgroups sweep the chains of sequences seq_order[0 .. n_long) as
  // two halves, the others those of seq_order[n_long .. N) whole
  unsigned split_grid; int n_long;
  unsigned char seq_order[INLINE_TABLE_SEQUENCES];
};

// 52 KB, so that three workgroups share a CU.  The normalised q never goes through LDS: the thread that
// normalised a piece of it also forms that piece of the decayed tile, and the wavefront that needs a row block
// as an MFMA operand reads those rows again (they were fetched a moment ago) and scales them by the row's
// inverse norm.  L takes over Kn's storage once every wavefront is done with its k operands (the M blocks wait
// in registers for the barrier).
struct __align__(16) KdaPrepShared {
  float G[CHUNK][132];
  union {
    uint16_t Kn[CHUNK][PITCH128];
    float L[CHUNK][68];
  };
  float B[CHUNK];
  float QI[CHUNK];         // 1 / |q_row|
};
static_assert(sizeof(float[CHUNK][68]) <= sizeof(uint16_t[CHUNK][PITCH128]), "L must fit into Kn's storage");

// Eight decayed elements of a bf16 row: x[c] * exp(sign * (G[c] - R[c])) for the lane's two
// channel quads of contraction step s.
__device__ __forceinline__ void decayed8(const uint16_t* xrow, const float* grow, const float* rrow, float sign,
                                         int s, int kb, f32x4_t& a, f32x4_t& b) {
  const int c0 = 32 * s + 4 * kb, c1 = c0 + 16;
  const uint2 x0 = *reinterpret_cast<const uint2*>(xrow + c0);
  const uint2 x1 = *reinterpret_cast<const uint2*>(xrow + c1);
  const float4 g0 = *reinterpret_cast<const float4*>(grow + c0);
  const float4 g1 = *reinterpret_cast<const float4*>(grow + c1);
  const float4 r0 = *reinterpret_cast<const float4*>(rrow + c0);
  const float4 r1 = *reinterpret_cast<const float4*>(rrow + c1);
  a = f32x4_t{lo16<bf16_t>(x0.x) * __expf(sign * (g0.x - r0.x)), hi16<bf16_t>(x0.x) * __expf(sign * (g0.y - r0.y)),
              lo16<bf16_t>(x0.y) * __expf(sign * (g0.z - r0.z)), hi16<bf16_t>(x0.y) * __expf(sign * (g0.w - r0.w))};
  b = f32x4_t{lo16<bf16_t>(x1.x) * __expf(sign * (g1.x - r1.x)), hi16<bf16_t>(x1.x) * __expf(sign * (g1.y - r1.y)),
              lo16<bf16_t>(x1.y) * __expf(sign * (g1.z - r1.z)), hi16<bf16_t>(x1.y) * __expf(sign * (g1.w - r1.w))};
}

__global__ __launch_bounds__(256) void kda_prep_solve_kernel(const KdaPrefillParams p) {
  const int cb = staged_chunk(p.stg, p.stage, blockIdx.x, p.seq_chunk_off[p.N]);
  const int h = blockIdx.y;
  if (cb < 0) return;
  const int t0 = p.chunk_tok[cb];
  const int len = p.chunk_len[cb];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kb = lane >> 4;
  __shared__ KdaPrepShared sh;
  const int64_t tile = (int64_t)cb * p.H + h;

  uint32_t qn[4][4], kn[4][4];   // normalised bf16 pairs of rows tid / 16 + 16 u, channels 8 (tid % 16) .. + 7
  uint2 qraw[4][2];
  // ---- phase 1: normalised q / k, per-channel log-decay, beta ---------------------------------
  {
    // q, k: thread handles eight channels of rows tid / 16 + 16 u (a row is one 16-lane DPP row, so its
    // sum of squares is a row reduction); all eight 16-byte loads are in flight at once
    const int nrow = tid >> 4, nc0 = 8 * (tid & 15);
    uint4 qv[4], kv[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = nrow + 16 * u;
      const int64_t t = t0 + (j < len ? j : 0);
      qv[u] = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.q) + t * p.stride_q + h * 128 + nc0);
      kv[u] = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.k) + t * p.stride_k + h * 128 + nc0);
    }
    // gate: thread handles eight channels of rows tid / 16 + 16 u; requested together with q and k, so the
    // phase costs one trip to memory
    const int gc0 = 8 * (tid & 15);
    uint4 graw[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = (tid >> 4) + 16 * u;
      graw[u] = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.g) +
                                                (int64_t)(t0 + (j < len ? j : 0)) * p.stride_g + h * 128 + gc0);
    }
    float dtb[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) dtb[e] = p.dt_bias[h * 128 + gc0 + e];
    const float a_log = p.A_log[h];
    float braw = 0.f;
    if (tid < len) braw = to_float(reinterpret_cast<const bf16_t*>(p.beta)[(int64_t)(t0 + tid) * p.stride_beta + h]);
    // the q rows of this wavefront's row block in MFMA operand layout (phase 3), raw
    {
      const int i_row = 16 * wave + r16;
      const uint16_t* qrow = reinterpret_cast<const uint16_t*>(p.q) + (int64_t)(t0 + (i_row < len ? i_row : 0)) * p.stride_q + h * 128;
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        qraw[s][0] = *reinterpret_cast<const uint2*>(qrow + 32 * s + 4 * kb);
        qraw[s][1] = *reinterpret_cast<const uint2*>(qrow + 32 * s + 4 * kb + 16);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = nrow + 16 * u;
      const uint32_t qw[4] = {qv[u].x, qv[u].y, qv[u].z, qv[u].w}, kw[4] = {kv[u].x, kv[u].y, kv[u].z, kv[u].w};
      float qs = 0.f, ks = 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float q0 = lo16<bf16_t>(qw[e]), q1 = hi16<bf16_t>(qw[e]), k0 = lo16<bf16_t>(kw[e]), k1 = hi16<bf16_t>(kw[e]);
        qs += q0 * q0 + q1 * q1;
        ks += k0 * k0 + k1 * k1;
      }
      const float qi = rsqrtf(row16_allreduce(qs) + 1e-6f), ki = rsqrtf(row16_allreduce(ks) + 1e-6f);
      const bool ok = j < len;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        qn[u][e] = ok ? pack2<bf16_t>(lo16<bf16_t>(qw[e]) * qi, hi16<bf16_t>(qw[e]) * qi) : 0u;
        kn[u][e] = ok ? pack2<bf16_t>(lo16<bf16_t>(kw[e]) * ki, hi16<bf16_t>(kw[e]) * ki) : 0u;
      }
      *reinterpret_cast<uint4*>(&sh.Kn[j][nc0]) = make_uint4(kn[u][0], kn[u][1], kn[u][2], kn[u][3]);
      if ((tid & 15) == 0) sh.QI[j] = ok ? qi : 0.f;
    }
    const float eA = expf(a_log);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = (tid >> 4) + 16 * u;
      const uint32_t w[4] = {graw[u].x, graw[u].y, graw[u].z, graw[u].w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float g0 = p.lower_bound * fast_rcp(1.0f + __expf(-eA * (lo16<bf16_t>(w[e]) + dtb[2 * e])));
        const float g1 = p.lower_bound * fast_rcp(1.0f + __expf(-eA * (hi16<bf16_t>(w[e]) + dtb[2 * e + 1])));
        sh.G[j][gc0 + 2 * e] = j < len ? g0 : 0.f;
        sh.G[j][gc0 + 2 * e + 1] = j < len ? g1 : 0.f;
      }
    }
    if (tid < CHUNK) {
      sh.B[tid] = tid < len ? 1.0f / (1.0f + expf(-braw)) : 0.f;
    }
  }
  __syncthreads();
  if (tid < 128) {
    float cum = 0.f;
    for (int j = 0; j < CHUNK; ++j) {
      cum += sh.G[j][tid];
      sh.G[j][tid] = cum;                 // rows beyond the chunk repeat G_last (their g is zero)
    }
    p.eGlast[tile * 128 + tid] = __expf(cum);
  }
  __syncthreads();

  // ---- phase 2: decayed operand tiles for the sequential kernel (fp16, row major) ---------------
  {
    const float* const glast = &sh.G[CHUNK - 1][0];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = (tid >> 4) + 16 * u, c0 = 8 * (tid & 15);   // the rows and channels this thread normalised
      const uint32_t* const kwv = kn[u];
      const uint32_t* const qwv = qn[u];
      uint32_t kg[4], qg[4], kt[4], ktl[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float g0 = sh.G[j][c0 + 2 * e], g1 = sh.G[j][c0 + 2 * e + 1];
        const float e0 = __expf(g0), e1 = __expf(g1);
        const float k0 = lo16<bf16_t>(kwv[e]), k1 = hi16<bf16_t>(kwv[e]);
        kg[e] = pack2<f16_t>(k0 * e0, k1 * e1);
        qg[e] = pack2<f16_t>(p.scale * lo16<bf16_t>(qwv[e]) * e0, p.scale * hi16<bf16_t>(qwv[e]) * e1);
        pack2_pair(k0 * __expf(glast[c0 + 2 * e] - g0), k1 * __expf(glast[c0 + 2 * e + 1] - g1), kt[e], ktl[e]);
      }
      // The tiles leave in the layout the sweeps read from LDS (they copy them as linear memory): unpadded rows of
      // 256 bytes with the swizzle of prefill_common.h, columns permuted inside groups of 32 so that an operand granule
      // holds channels 32 s + 4 kb .. + 3 and 32 s + 16 + 4 kb .. + 3.  The thread's channels c0 .. c0 + 3 and
      // c0 + 4 .. c0 + 7 are the same half of two neighbouring granules, and the thread two lanes away holds the other
      // halves: the two exchange one piece each (a quad permutation) and then each stores one whole granule, so a
      // wavefront still writes whole rows with one 16-byte store per lane.
      const int lc = tid & 15;
      const bool upper = lc & 2;                       // this thread holds the second halves of its granules
      const int granule = 4 * (lc >> 2) + 2 * (lc & 1) + (upper ? 1 : 0);
      auto whole_granule = [&](const uint32_t (&x)[4]) {
        const uint32_t s0 = upper ? x[0] : x[2], s1 = upper ? x[1] : x[3];
        const uint32_t r0 = (uint32_t)__builtin_amdgcn_mov_dpp((int)s0, 0x4E, 0xF, 0xF, true);      // lane ^ 2
        const uint32_t r1 = (uint32_t)__builtin_amdgcn_mov_dpp((int)s1, 0x4E, 0xF, 0xF, true);
        return upper ? make_uint4(r0, r1, x[2], x[3]) : make_uint4(x[0], x[1], r0, r1);
      };
      const int64_t at = tile * 8192 + tile_offset(j, granule), at2 = tile * 16384 + tile_offset(j, granule);
      *reinterpret_cast<uint4*>(p.Kg + at) = whole_granule(kg);
      *reinterpret_cast<uint4*>(p.Qg + at) = whole_granule(qg);
      *reinterpret_cast<uint4*>(p.Kt + at2) = whole_granule(kt);
      *reinterpret_cast<uint4*>(p.Kt + at2 + 8192) = whole_granule(ktl);
    }
  }

  // ---- phase 3: M and P, wavefront w owns row block w (reference row = first row of the block) --
  {
    const int bi = wave;
    const float* const R = &sh.G[16 * bi][0];
    const int i_row = 16 * bi + r16;
    HiLo Al[4];
    bf16x8_t Ql[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      // the decay factors e^{G_i - R} of the lane's eight channels serve both the k and the q rows
      const int c0 = 32 * s + 4 * kb, c1 = c0 + 16;
      const float4 g0 = *reinterpret_cast<const float4*>(&sh.G[i_row][c0]), g1 = *reinterpret_cast<const float4*>(&sh.G[i_row][c1]);
      const float4 r0 = *reinterpret_cast<const float4*>(R + c0), r1 = *reinterpret_cast<const float4*>(R + c1);
      const f32x4_t e0 = {__expf(g0.x - r0.x), __expf(g0.y - r0.y), __expf(g0.z - r0.z), __expf(g0.w - r0.w)};
      const f32x4_t e1 = {__expf(g1.x - r1.x), __expf(g1.y - r1.y), __expf(g1.z - r1.z), __expf(g1.w - r1.w)};
      const uint2 k0 = *reinterpret_cast<const uint2*>(&sh.Kn[i_row][c0]), k1 = *reinterpret_cast<const uint2*>(&sh.Kn[i_row][c1]);
      f32x4_t a = {lo16<bf16_t>(k0.x) * e0[0], hi16<bf16_t>(k0.x) * e0[1], lo16<bf16_t>(k0.y) * e0[2], hi16<bf16_t>(k0.y) * e0[3]};
      f32x4_t b = {lo16<bf16_t>(k1.x) * e1[0], hi16<bf16_t>(k1.x) * e1[1], lo16<bf16_t>(k1.y) * e1[2], hi16<bf16_t>(k1.y) * e1[3]};
      Al[s] = split8(a, b);
      // the same normalised bf16 values as phase 1 formed: raw q times the row's inverse norm, rounded to bf16
      const float qi = sh.QI[i_row];
      const uint2 x0 = qraw[s][0], x1 = qraw[s][1];
      const uint32_t n0 = pack2<bf16_t>(lo16<bf16_t>(x0.x) * qi, hi16<bf16_t>(x0.x) * qi);
      const uint32_t n1 = pack2<bf16_t>(lo16<bf16_t>(x0.y) * qi, hi16<bf16_t>(x0.y) * qi);
      const uint32_t n2 = pack2<bf16_t>(lo16<bf16_t>(x1.x) * qi, hi16<bf16_t>(x1.x) * qi);
      const uint32_t n3 = pack2<bf16_t>(lo16<bf16_t>(x1.y) * qi, hi16<bf16_t>(x1.y) * qi);
      a = f32x4_t{lo16<bf16_t>(n0) * e0[0], hi16<bf16_t>(n0) * e0[1], lo16<bf16_t>(n1) * e0[2], hi16<bf16_t>(n1) * e0[3]};
      b = f32x4_t{lo16<bf16_t>(n2) * e1[0], hi16<bf16_t>(n2) * e1[1], lo16<bf16_t>(n3) * e1[2], hi16<bf16_t>(n3) * e1[3]};
      Ql[s] = round8(a, b);
    }
    // P leaves in the six-block operand layout (prefill_common.h): its product is formed transposed (A = k rows j,
    // B = q rows i), so a lane holds four consecutive j of token i = 16 bi + r16, which is half of the 16 bytes it owns
    // in block (row block bi, contraction half s = bj / 2); the halves of blocks above the diagonal are zero.
    uint16_t* const Pt = p.P + tile * (TRI_BLOCKS * 512);
    f32x4_t mblock[4];
    uint32_t ppk[4][2] = {{0u, 0u}, {0u, 0u}, {0u, 0u}, {0u, 0u}};
#pragma unroll
    for (int bj = 0; bj < 4; ++bj) {
      const int j = 16 * bj + r16;
      if (bj > bi) continue;
      f32x4_t m = {0.f, 0.f, 0.f, 0.f}, pq = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        f32x4_t a, b;
        decayed8(&sh.Kn[j][0], &sh.G[j][0], R, -1.0f, s, kb, a, b);     // k_j e^{R - G_j}
        const HiLo Br = split8(a, b);
        m = mfma16(Al[s].hi, Br.hi, m);
        m = mfma16(Al[s].lo, Br.hi, m);
        m = mfma16(Al[s].hi, Br.lo, m);
        pq = mfma16(Br.hi, Ql[s], pq);        // pq[r] = P[i = 16 bi + r16][j = 16 bj + 4 kb + r] / scale
      }
      mblock[bj] = m;
      {
        const int i = 16 * bi + r16, j0 = 16 * bj + 4 * kb;
        ppk[bj][0] = pack2<f16_t>(i >= j0 ? p.scale * pq[0] : 0.f, i >= j0 + 1 ? p.scale * pq[1] : 0.f);
        ppk[bj][1] = pack2<f16_t>(i >= j0 + 2 ? p.scale * pq[2] : 0.f, i >= j0 + 3 ? p.scale * pq[3] : 0.f);
      }
    }
    *reinterpret_cast<uint4*>(Pt + bi * 512 + lane * 8) = make_uint4(ppk[0][0], ppk[0][1], ppk[1][0], ppk[1][1]);
    if (bi >= 2) *reinterpret_cast<uint4*>(Pt + (2 + bi) * 512 + lane * 8) = make_uint4(ppk[2][0], ppk[2][1], ppk[3][0], ppk[3][1]);
    __syncthreads();                     // Kn is dead from here on: L reuses its storage
#pragma unroll
    for (int bj = 0; bj < 4; ++bj) {
      if (bj > bi) continue;
      const int j = 16 * bj + r16;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = 16 * bi + 4 * kb + r;
        sh.L[i][j] = i > j ? sh.B[i] * mblock[bj][r] : 0.f;
      }
    }
  }
  __syncthreads();

  // ---- phase 4: W = L^-1 diag(beta) by blocks on one wavefront (which one rotates with the workgroup, so
  // that co-resident workgroups keep different SIMDs busy) -----------------------------------------
  if (wave == (int)(blockIdx.x & 3)) {
    block_inverse_inplace(sh.L, lane);
    store_w_operand_blocks(sh.L, sh.B, lane, p.W + tile * (2 * TRI_BLOCKS * 512));
  }
}

// ---------------------------------------------------------------------------------------------
// Sequential kernel with output (whole sequences, and the second sweep over segments): one workgroup per
// (sequence or segment, head) of SIX wavefronts.  Wavefronts 0-3 compute, each on its own 32 V columns, and touch
// memory only to store their output rows; wavefronts 4 and 5 issue the global -> LDS copies of the workgroup, every
// tile dealt between them in 1 KiB pieces (an LDS copy occupies its issuer for tens of cycles, about 2.5 k cycles
// per chunk in all, and a wavefront holds at most 63 of them in flight).  S^T stays in MFMA
// accumulator layout (an accumulator tile pair is already a valid operand of the next product); the output product
// is formed transposed, so that a lane holds four adjacent V columns of one token and stores them as 8 bytes.
// 133 KiB of LDS: K e^G and W (hi, lo) are double buffered by chunk parity, everything else is single, with two
// barriers per chunk:
//   barrier A   K e^G, W, V of chunk c landed; chunk c - 1 finished     copy scale Q e^G, P, K e^{G_last-G} (hi, lo),
//               KS = (K e^G) S^T,  X = V - KS,  U = W X                 e^{G_last} of c, then K e^G and W of c + 1
//   barrier B   the tiles requested at A landed; V is free              copy V of c + 1
//               O^T = S (scale Q e^G)^T + U^T P^T -> rows of o
//               S^T = e^{G_last} (.) S^T + (K e^{G_last-G})^T U         (pairs: hi.lo + lo.hi + hi.hi)
// LDS of one workgroup of kda_sweep
constexpr int KDA_W_HALVES = 2 * TRI_BLOCKS * 512;               // W: hi blocks, then lo blocks (six-block operand layout)
struct KdaSweepLds {
  __align__(1024) uint16_t tK[2][TILE128_HALVES];       // swizzled operand tiles, as the preparation stored them
  __align__(16) uint16_t tW[2][KDA_W_HALVES];           // [parity][hi blocks, lo blocks]
  __align__(16) uint16_t tV[CHUNK * PITCH128];
  __align__(1024) uint16_t tQ[TILE128_HALVES];
  __align__(16) uint16_t tP[TRI_BLOCKS * 512];
  __align__(1024) uint16_t tKt[2][TILE128_HALVES];      // hi, lo: the same layout, read transposed
  __align__(16) float tE[128];
};

// The sweep of one workgroup.  `wide`: 2 / NB x the chain's logical index (sequence x H + head, or segment x H + head
// in the second sweep over segments) plus, for NB = 1, the half of the V columns it takes.
template <int NB>
__device__ __forceinline__ void kda_sweep(const KdaPrefillParams& p, KdaSweepLds& lds, const int wide) {
  constexpr int HALVES = 2 / NB;             // workgroups per chain: NB = 1 sweeps 64 of the 128 V columns
  constexpr int NCOPY = KDA_SWEEP_COPIERS;
  using CopyWide = TileCopy<CHUNK, 2 * PITCH128, 256, NCOPY>;  // 64 x 128 tile, its pieces dealt to the copying wavefronts
  constexpr int W_HALVES = KDA_W_HALVES;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, kb = lane >> 4;
  const int v_half = wide % HALVES;
  const SweepRole role = select_sweep(p.pass, p.H, p.N, p.seq_chunk_off, p.seg, p.stg, p.stage, p.h0, p.h0_indices, p.h0_slot_stride,
                                      p.ht, p.ht_indices, p.ht_slot_stride, wide / HALVES);
  if (!role.active) return;
  const int n = role.n, h = role.head, c_begin = role.c_begin, c_end = role.c_end;
  const int seq_start = p.cu_seqlens[n] + (c_begin - p.seq_chunk_off[n]) * CHUNK;
  const int seq_len = min(p.cu_seqlens[n + 1] - seq_start, (c_end - c_begin) * CHUNK);
  const int n_chunks = c_end - c_begin;
  auto chunk_len = [&](int c) { return min(CHUNK, seq_len - c * CHUNK); };

  auto& tK = lds.tK; auto& tW = lds.tW; auto& tV = lds.tV; auto& tQ = lds.tQ; auto& tP = lds.tP; auto& tKt = lds.tKt; auto& tE = lds.tE;

  if (wave >= 4) {
    const int cw = wave - 4;                         // which of the copying wavefronts
    // ---- the copying wavefront -------------------------------------------------------------
    const int64_t tile0 = (int64_t)c_begin * p.H + h;
    const char* const kg_b = uniform_pointer(reinterpret_cast<const char*>(p.Kg) + tile0 * 16384);
    const char* const qg_b = uniform_pointer(reinterpret_cast<const char*>(p.Qg) + tile0 * 16384);
    const char* const kt_b = uniform_pointer(reinterpret_cast<const char*>(p.Kt) + tile0 * 32768);
    const char* const w_b = uniform_pointer(reinterpret_cast<const char*>(p.W) + tile0 * (W_HALVES * 2));
    const char* const pp_b = uniform_pointer(reinterpret_cast<const char*>(p.P) + tile0 * (TRI_BLOCKS * 1024));
    const char* const eg_b = uniform_pointer(reinterpret_cast<const char*>(p.eGlast) + tile0 * 512);
    const char* const v_b = uniform_pointer(reinterpret_cast<const char*>(p.v) + ((int64_t)seq_start * p.stride_v + h * 128) * 2);
    const int64_t big_step = (int64_t)p.H * 16384, w_step = (int64_t)p.H * (W_HALVES * 2), p_step = (int64_t)p.H * (TRI_BLOCKS * 1024);
    const int64_t e_step = (int64_t)p.H * 512;
    CopyWide plan_v;
    plan_v.plan((uint32_t)(p.stride_v * 2), CHUNK - 1, cw, lane);
    // a 16 KiB operand tile is copied as it lies in memory, its sixteen 1 KiB pieces dealt to the copying wavefronts
    auto copy_tile = [&](const uint16_t* dst, const char* src) {
#pragma unroll
      for (int j0 = 0; j0 < 16 / NCOPY; ++j0) {
        const int j = NCOPY * j0 + cw;
        dma16(src, 1024u * j + 16u * lane, lds_address(dst) + 1024u * j);
      }
    };
    auto issue_kw = [&](int c) {                     // K e^G and W (hi, lo) into the buffers of c's parity
      const int par = c & 1;
      copy_tile(tK[par], kg_b + c * big_step);
#pragma unroll
      for (int j0 = 0; j0 < 2 * TRI_BLOCKS / NCOPY; ++j0) {
        const int j = NCOPY * j0 + cw;
        dma16(w_b + c * w_step, 1024u * j + 16u * lane, lds_address(tW[par]) + 1024u * j);
      }
    };
    auto issue_v = [&](int c) {
      const char* vs = v_b + (int64_t)c * CHUNK * p.stride_v * 2;
      const int len = chunk_len(c);
      if (len == CHUNK) {
        plan_v.issue(tV, vs, cw);
      } else {                                       // rows past the sequence re-read its last row
        CopyWide tail_v;
        tail_v.plan((uint32_t)(p.stride_v * 2), len - 1, cw, lane);
        tail_v.issue(tV, vs, cw);
      }
    };
    auto issue_second = [&](int c) {                 // scale Q e^G, P, K e^{G_last-G} (hi, lo), e^{G_last}
      copy_tile(tQ, qg_b + c * big_step);
#pragma unroll
      for (int j0 = 0; j0 < TRI_BLOCKS / NCOPY; ++j0) {
        const int j = NCOPY * j0 + cw;
        dma16(pp_b + c * p_step, 1024u * j + 16u * lane, lds_address(tP) + 1024u * j);
      }
      copy_tile(tKt[0], kt_b + c * 2 * big_step);
      copy_tile(tKt[1], kt_b + c * 2 * big_step + 16384);
      if (cw == NCOPY - 1 && lane < 32) dma16(eg_b + c * e_step, 16u * lane, lds_address(tE));
    };
    static_assert(2 * TRI_BLOCKS % NCOPY == 0 && TRI_BLOCKS % NCOPY == 0 && 16 % NCOPY == 0, "pieces are dealt evenly");
    constexpr int KW_COPIES = (16 + 2 * TRI_BLOCKS) / NCOPY;                 // copies of one issue_kw by one wavefront
    if (n_chunks > 0) {
      issue_kw(0);
      issue_v(0);
    }
    for (int ci = 0; ci < n_chunks; ++ci) {
      const bool more = ci + 1 < n_chunks;
      wait_vmcnt<0>();                               // K e^G, W, V of chunk ci have landed
      __syncthreads();                               // barrier A: ... and chunk ci - 1 is finished
      issue_second(ci);
      if (more) {
        issue_kw(ci + 1);
        // the second-half tiles of ci have landed (what follows may be in flight)
        wait_vmcnt<KW_COPIES>();
      } else {
        wait_vmcnt<0>();
      }
      __syncthreads();                               // barrier B: ... and V is free
      if (more) issue_v(ci + 1);
    }
    return;
  }

  // ---- the computing wavefronts ------------------------------------------------------------
  const int vbase = 64 * v_half + 16 * NB * wave;
  const int vcol = vbase + r16;                      // state / KS / U layout: the lane's column (second block: + 16)
  // S^T slices in accumulator layout: St[nb][mc][r] = S[v = vcol + 16 nb][c = 16 mc + 4 kb + r]
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
  // output rows: in the transposed product a lane holds V columns vbase + 16 nb + 4 kb .. + 3 of token 16 ni + r16
  uint16_t* const o_lane = reinterpret_cast<uint16_t*>(p.o) + ((int64_t)(seq_start + r16) * p.H + h) * 128 + vbase + 4 * kb;

  for (int ci = 0; ci < n_chunks; ++ci) {
    const int par = ci & 1;
    // barrier A (bare: the tiles come from the copying wavefront's LDS copies, which it waited for)
    __builtin_amdgcn_s_waitcnt(0xc07f);              // lgkmcnt(0) only
    __builtin_amdgcn_s_barrier();
    const uint16_t* const K = tK[par];
    // ---- KS = (K e^G) S^T ----
    f32x4_t KS[NB][4];
    // W operands: block b of the six (row block tri_block_m(b), contraction half tri_block_s(b)), hi at block b, lo at
    // block TRI_BLOCKS + b; one 16-byte read per lane
    bf16x8_t wa[TRI_BLOCKS], wl[TRI_BLOCKS];
    auto ldW = [&](int b, bool lo) {
      return __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(&tW[par][((lo ? TRI_BLOCKS : 0) + b) * 512 + lane * 8]));
    };
    uint2 vraw[NB][4];        // rows 16 mi + 4 kb .. + 3 of the lane's V column, one transposing read each
    {
      bf16x8_t ka[2][4], sb[2][NB];
#pragma unroll
      for (int mi = 0; mi < 4; ++mi) ka[0][mi] = operand_granule(K, 16 * mi + r16, 0, kb);
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
          for (int mi = 0; mi < 4; ++mi) ka[(s + 1) & 1][mi] = operand_granule(K, 16 * mi + r16, s + 1, kb);
        } else {
          // under the last step: V and the first half of W
#pragma unroll
          for (int mi = 0; mi < 4; ++mi)
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
              vraw[nb][mi] = read_tr4(&tV[(16 * mi + 4 * kb + (r16 >> 2)) * PITCH128 + (vcol - r16) + 16 * nb + 4 * (r16 & 3)]);
            }
#pragma unroll
          for (int b = 0; b < 4; ++b) { wa[b] = ldW(b, false); wl[b] = ldW(b, true); }
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
    // ---- X = V - KS,  U = W X ----
    f32x4_t U[NB][4];
    {
#pragma unroll
      for (int b = 4; b < TRI_BLOCKS; ++b) { wa[b] = ldW(b, false); wl[b] = ldW(b, true); }
      __builtin_amdgcn_sched_barrier(0x000F);
      f32x4_t X[NB][4];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mi = 0; mi < 4; ++mi)
#pragma unroll
          for (int r = 0; r < 4; ++r) X[nb][mi][r] = quad_element<bf16_t>(vraw[nb][mi], r) - KS[nb][mi][r];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mi = 0; mi < 4; ++mi) U[nb][mi] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        bf16x8_t xb[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) xb[nb] = half8_sat(X[nb][2 * s], X[nb][2 * s + 1]);
        // lower triangular W: contraction half 1 only reaches row blocks 2 and 3
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int b = (s == 0 ? 0 : 4); b < (s == 0 ? 4 : TRI_BLOCKS); ++b) U[nb][tri_block_m(b)] = mfma16h(wl[b], xb[nb], U[nb][tri_block_m(b)]);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int b = (s == 0 ? 0 : 4); b < (s == 0 ? 4 : TRI_BLOCKS); ++b) U[nb][tri_block_m(b)] = mfma16h(wa[b], xb[nb], U[nb][tri_block_m(b)]);
      }
    }
    // barrier B: Q, P, the K e^{G_last-G} pair and e^{G_last} of this chunk have landed
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_barrier();
    // ---- O^T = S (scale Q e^G)^T + U^T P^T -> o ----
    bf16x8_t kt[8], ktl[8];
    {
      f32x4_t OT[NB][4];                             // OT[nb][ni][r] = o[token 16 ni + r16][v = vbase + 16 nb + 4 kb + r]
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int ni = 0; ni < 4; ++ni) OT[nb][ni] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      bf16x8_t qa[2][4], sb[2][NB], pa[TRI_BLOCKS];
#pragma unroll
      for (int ni = 0; ni < 4; ++ni) qa[0][ni] = operand_granule(tQ, 16 * ni + r16, 0, kb);
      __builtin_amdgcn_sched_barrier(0x000F);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) sb[0][nb] = half8_rtz(St[nb][0], St[nb][1]);
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        if (s < 3) {
#pragma unroll
          for (int ni = 0; ni < 4; ++ni) qa[(s + 1) & 1][ni] = operand_granule(tQ, 16 * ni + r16, s + 1, kb);
        } else {
#pragma unroll
          for (int b = 0; b < TRI_BLOCKS; ++b) pa[b] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(&tP[b * 512 + lane * 8]));
        }
        __builtin_amdgcn_sched_barrier(0x000F);
        if (s < 3) {
#pragma unroll
          for (int nb = 0; nb < NB; ++nb) sb[(s + 1) & 1][nb] = half8_rtz(St[nb][2 * s + 2], St[nb][2 * s + 3]);
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int ni = 0; ni < 4; ++ni) OT[nb][ni] = mfma16h(sb[s & 1][nb], qa[s & 1][ni], OT[nb][ni]);
      }
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        bf16x8_t ur[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) ur[nb] = half8_rtz(U[nb][2 * s], U[nb][2 * s + 1]);
        if (s == 1) {
          // under the last step: the first transposed key operands of the state update
#pragma unroll
          for (int mc = 0; mc < 8; ++mc) {
            kt[mc] = operand_granule_transposed(tKt[0], 0, mc, kb, r16);
            ktl[mc] = operand_granule_transposed(tKt[1], 0, mc, kb, r16);
          }
          __builtin_amdgcn_sched_barrier(0x000F);
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int b = (s == 0 ? 0 : 4); b < (s == 0 ? 4 : TRI_BLOCKS); ++b) OT[nb][tri_block_m(b)] = mfma16h(ur[nb], pa[b], OT[nb][tri_block_m(b)]);
      }
      {
        const int len = chunk_len(ci);
        uint16_t* const dst = o_lane + (int64_t)ci * CHUNK * p.H * 128;
#pragma unroll
        for (int ni = 0; ni < 4; ++ni)
          if (16 * ni + r16 < len) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
              const uint2 packed = make_uint2(pack2<bf16_t>(OT[nb][ni][0], OT[nb][ni][1]), pack2<bf16_t>(OT[nb][ni][2], OT[nb][ni][3]));
              *reinterpret_cast<uint2*>(dst + (int64_t)16 * ni * p.H * 128 + 16 * nb) = packed;
            }
          }
      }
    }
    // ---- S^T = e^{G_last} (.) S^T + (K e^{G_last - G})^T U ----
    {
      float4 eg[8];
#pragma unroll
      for (int mc = 0; mc < 8; ++mc) eg[mc] = *reinterpret_cast<const float4*>(&tE[16 * mc + 4 * kb]);
      __builtin_amdgcn_sched_barrier(0x000F);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mc = 0; mc < 8; ++mc)
          St[nb][mc] = f32x4_t{St[nb][mc][0] * eg[mc].x, St[nb][mc][1] * eg[mc].y, St[nb][mc][2] * eg[mc].z,
                               St[nb][mc][3] * eg[mc].w};
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        HalfPair ub[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) ub[nb] = half8_pair(U[nb][2 * s], U[nb][2 * s + 1]);
        // hi . lo and lo . hi first, the large term last
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int mc = 0; mc < 8; ++mc) St[nb][mc] = mfma16h(ktl[mc], ub[nb].hi, St[nb][mc]);
        if (s == 0) {
#pragma unroll
          for (int mc = 0; mc < 8; ++mc) ktl[mc] = operand_granule_transposed(tKt[1], 1, mc, kb, r16);
          __builtin_amdgcn_sched_barrier(0x000F);
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int mc = 0; mc < 8; ++mc) St[nb][mc] = mfma16h(kt[mc], ub[nb].lo, St[nb][mc]);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int mc = 0; mc < 8; ++mc) St[nb][mc] = mfma16h(kt[mc], ub[nb].hi, St[nb][mc]);
        if (s == 0) {
#pragma unroll
          for (int mc = 0; mc < 8; ++mc) kt[mc] = operand_granule_transposed(tKt[0], 1, mc, kb, r16);
          __builtin_amdgcn_sched_barrier(0x000F);
        }
      }
    }
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

// One workgroup per (sequence, head) or per (segment, head) in the second sweep over segments (NB = 2); NB = 1: two
// per chain, 64 V columns each, on one XCD: they copy the same tiles, which then come from memory once.
template <int NB>
__global__ __launch_bounds__(64 * (4 + KDA_SWEEP_COPIERS), 1) void kda_sweep_kernel(const KdaPrefillParams p) {
  constexpr int HALVES = 2 / NB;
  __shared__ KdaSweepLds lds;
  const int wide = HALVES == 1 ? (int)blockIdx.x
                               : xcd_grouped_index(blockIdx.x, HALVES, HALVES * (p.pass == 2 ? p.seg.max_segments : p.N) * p.H);
  if (wide < 0) return;
  kda_sweep<NB>(p, lds, wide);
}

// Ragged whole sequences: the chains of the longest sequences as two halves (first in the grid: workgroups are
// dispatched in index order), those of the others whole, longest first (mixed_sweep_plan).
__global__ __launch_bounds__(64 * (4 + KDA_SWEEP_COPIERS), 1) void kda_sweep_mixed_kernel(const KdaPrefillParams p) {
  __shared__ KdaSweepLds lds;
  if (blockIdx.x < p.split_grid) {
    const int wide = xcd_grouped_index(blockIdx.x, 2, 2 * p.n_long * p.H);
    if (wide < 0) return;
    const int chain = wide >> 1, k = chain / p.H;
    kda_sweep<1>(p, lds, __builtin_amdgcn_readfirstlane(2 * (p.seq_order[k] * p.H + chain - k * p.H) + (wide & 1)));
  } else {
    const int chain = blockIdx.x - p.split_grid;
    if (chain >= (p.N - p.n_long) * p.H) return;
    const int k = chain / p.H;
    kda_sweep<2>(p, lds, __builtin_amdgcn_readfirstlane(p.seq_order[p.n_long + k] * p.H + chain - k * p.H));
  }
}

// ---------------------------------------------------------------------------------------------
// First sweep over segments, both roles in one workgroup.  A later segment is swept twice without output - from a
// zero state (its B summary) and from the identity with v = 0 (its transition matrix M) - and both sweeps multiply
// the same operand tiles.  One workgroup of eight wavefronts per (segment, head) therefore runs them side by side:
// wavefronts 0-3 carry the B columns (32 each), wavefronts 4-7 the M columns; all eight issue the global -> LDS
// copies, so each tile crosses memory and LDS once for the two sweeps and two wavefronts share a SIMD.  A first
// segment has no M role: its wavefronts 4-7 only copy, wavefronts 0-3 sweep it
// from its real start state (of which they keep a copy for the second sweep).
//
// Every tile of a chunk (K e^G, V, W hi / lo, the hi / lo pair of K e^{G_last - G}, e^{G_last}) is double buffered by
// chunk parity (155 KiB of LDS: the operand tiles are unpadded), so there is ONE barrier per chunk: at the barrier
// that opens chunk c its tiles have landed and the buffers of chunk c - 1 are free; the wavefronts fill them
// with chunk c + 1 during chunk c, a whole chunk ahead of their use:
//     KS = (K e^G) S^T,  X = V - KS (or -KS),  U = W X
//     S^T = e^{G_last} (.) S^T + (K e^{G_last-G})^T U              (pairs: hi.lo + lo.hi + hi.hi)
// (With the pair single buffered and requested half a chunk ahead, behind a second barrier, copies and computation
// overlapped badly: 0.73 ms for config 4's first sweep where the copies alone take 0.47 and the computation 0.36.)
__global__ __launch_bounds__(512, 1) void kda_lean_sweep_kernel(const KdaPrefillParams p) {
  constexpr int NB = 2;
  using CopyWide = TileCopy<CHUNK, 2 * PITCH128, 256, 4>;      // 64 x 128 tile, issued by the four copying wavefronts
  constexpr int W_HALVES = 2 * TRI_BLOCKS * 512;               // W: hi blocks, then lo blocks (six-block operand layout)
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, kb = lane >> 4;
  const bool m_side = wave >= 4;                               // wavefronts 4-7: transition-matrix columns + copies
  const int cw = wave & 3;                                     // position among the four wavefronts of a role
  const int vcol = 32 * cw + r16;

  // the two roles of this (segment, head): logical workgroups 2 i (zero state / real state) and 2 i + 1 (identity)
  const SweepRole lead = select_sweep(1, p.H, p.N, p.seq_chunk_off, p.seg, p.stg, 0, p.h0, p.h0_indices, p.h0_slot_stride,
                                      p.ht, p.ht_indices, p.ht_slot_stride, 2 * (int)blockIdx.x);
  if (!lead.active) return;
  const SweepRole mrole = select_sweep(1, p.H, p.N, p.seq_chunk_off, p.seg, p.stg, 0, p.h0, p.h0_indices, p.h0_slot_stride,
                                       p.ht, p.ht_indices, p.ht_slot_stride, 2 * (int)blockIdx.x + 1);
  const SweepRole& role = m_side ? mrole : lead;
  const bool computing = role.active;                          // wave-uniform; false: wavefronts 4-7 of a first segment
  const int n = lead.n, h = lead.head, c_begin = lead.c_begin, c_end = lead.c_end;
  const int seq_start = p.cu_seqlens[n] + (c_begin - p.seq_chunk_off[n]) * CHUNK;
  const int seq_len = min(p.cu_seqlens[n + 1] - seq_start, (c_end - c_begin) * CHUNK);
  const int n_chunks = c_end - c_begin;
  auto chunk_len = [&](int c) { return min(CHUNK, seq_len - c * CHUNK); };

  __shared__ __align__(1024) uint16_t tK[2][TILE128_HALVES];       // swizzled operand tiles, as the preparation stored them
  __shared__ __align__(16) uint16_t tV[2][CHUNK * PITCH128];
  __shared__ __align__(16) uint16_t tW[2][W_HALVES];                // [parity][hi blocks, lo blocks]
  __shared__ __align__(1024) uint16_t tKt[2][2][TILE128_HALVES];   // [parity][hi, lo]: the same layout, read transposed
  __shared__ __align__(16) float tE[2][128];

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

  // ---- copies ----
  const int64_t tile0 = (int64_t)c_begin * p.H + h;
  const char* const kg_b = reinterpret_cast<const char*>(p.Kg) + tile0 * 16384;
  const char* const kt_b = reinterpret_cast<const char*>(p.Kt) + tile0 * 32768;
  const char* const w_b = reinterpret_cast<const char*>(p.W) + tile0 * (W_HALVES * 2);
  const char* const eg_b = reinterpret_cast<const char*>(p.eGlast) + tile0 * 512;
  const char* const v_b = reinterpret_cast<const char*>(p.v) + ((int64_t)seq_start * p.stride_v + h * 128) * 2;
  const int64_t big_step = (int64_t)p.H * 16384, w_step = (int64_t)p.H * (W_HALVES * 2), e_step = (int64_t)p.H * 512;
  CopyWide plan_v;
  if (m_side) plan_v.plan((uint32_t)(p.stride_v * 2), CHUNK - 1, cw, lane);
  // a 16 KiB operand tile is copied as it lies in memory, four of its sixteen 1 KiB pieces per copying wavefront
  auto copy_tile = [&](const uint16_t* dst, const char* src) {
#pragma unroll
    for (int j0 = 0; j0 < 4; ++j0) {
      const int j = 4 * j0 + cw;
      dma16(src, 1024u * j + 16u * lane, lds_address(dst) + 1024u * j);
    }
  };
  // Every tile of chunk c into the buffers of its parity, in four parts.  A wavefront that issues copies is held until
  // the memory pipeline has taken them, so the two wavefronts of a SIMD issue at different times and one of them always
  // computes: wavefronts 4-7 request K e^G, V and W right after the barrier that frees the buffers, wavefronts 0-3 the
  // pair and e^{G_last} between the two phases of the chunk; everybody waits for its own copies before the next
  // barrier.  Config 4's first sweep, ms: 0.59 this way; 0.62 with both groups issuing after the barrier; 0.63 with
  // wavefronts 4-7 issuing everything there, 0.68 with them issuing half between the phases; 0.66 with the pair
  // requested at a second barrier; the parts spread over four points of the chunk spill registers (1.3).  With
  // wavefronts 4-7 only copying (a timing probe) the sweep takes the 0.48 ms of its copies alone, and its computation
  // alone 0.36 ms.
  auto issue_part = [&](int c, int part) {
    const int par = c & 1;
    if (part == 0) {                                 // K e^G
      copy_tile(tK[par], kg_b + c * big_step);
    } else if (part == 1) {                          // V, W (hi, lo)
      const char* vs = v_b + (int64_t)c * CHUNK * p.stride_v * 2;
      const int len = chunk_len(c);
      if (len == CHUNK) {
        plan_v.issue(tV[par], vs, cw);
      } else {                                       // rows past the sequence re-read its last row
        CopyWide tail_v;
        tail_v.plan((uint32_t)(p.stride_v * 2), len - 1, cw, lane);
        tail_v.issue(tV[par], vs, cw);
      }
#pragma unroll
      for (int j = 0; j < 2 * TRI_BLOCKS / 4; ++j)    // twelve 1 KiB blocks, three per copying wavefront
        dma16(w_b + c * w_step, 1024u * (4 * j + cw) + 16u * lane, lds_address(tW[par]) + 1024u * (4 * j + cw));
    } else if (part == 2) {                          // K e^{G_last-G}, hi
      copy_tile(tKt[par][0], kt_b + c * 2 * big_step);
    } else {                                         // K e^{G_last-G}, lo; e^{G_last}
      copy_tile(tKt[par][1], kt_b + c * 2 * big_step + 16384);
      if (cw == 0 && lane < 32) dma16(eg_b + c * e_step, 16u * lane, lds_address(tE[par]));
    }
  };

  if (n_chunks > 0) {
    if (m_side) { issue_part(0, 0); issue_part(0, 1); } else { issue_part(0, 2); issue_part(0, 3); }
  }

  for (int ci = 0; ci < n_chunks; ++ci) {
    const int par = ci & 1;
    const bool more = ci + 1 < n_chunks;
    // the one barrier of a chunk: its tiles have landed, chunk ci - 1 is finished and its buffers are free
    wait_vmcnt<0>();
    __syncthreads();
    if (more && m_side) { issue_part(ci + 1, 0); issue_part(ci + 1, 1); }
    f32x4_t U[NB][4];
    if (computing) {
      const uint16_t* const K = tK[par];
      const uint16_t* const V = tV[par];
      // ---- KS = (K e^G) S^T ----
      f32x4_t KS[NB][4];
      bf16x8_t wa[TRI_BLOCKS], wl[TRI_BLOCKS];          // W operand blocks (hi, lo), one 16-byte read per lane each
      auto ldW = [&](int b, bool lo) {
        return __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(&tW[par][((lo ? TRI_BLOCKS : 0) + b) * 512 + lane * 8]));
      };
      uint2 vraw[NB][4];        // rows 16 mi + 4 kb .. + 3 of the lane's V column, one transposing read each
      {
        bf16x8_t ka[2][4], sb[2][NB];
#pragma unroll
        for (int mi = 0; mi < 4; ++mi) ka[0][mi] = operand_granule(K, 16 * mi + r16, 0, kb);
        __builtin_amdgcn_sched_barrier(0x000F);      // LDS requests stay above this line; ALU and MFMA work may cross it
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
            for (int mi = 0; mi < 4; ++mi) ka[(s + 1) & 1][mi] = operand_granule(K, 16 * mi + r16, s + 1, kb);
          } else {
            // under the last step: V and the first half of W
            if (use_v) {
#pragma unroll
              for (int mi = 0; mi < 4; ++mi)
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                  vraw[nb][mi] = read_tr4(&V[(16 * mi + 4 * kb + (r16 >> 2)) * PITCH128 + (vcol - r16) + 16 * nb + 4 * (r16 & 3)]);
                }
            }
#pragma unroll
            for (int b = 0; b < 4; ++b) { wa[b] = ldW(b, false); wl[b] = ldW(b, true); }
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
      // ---- X = V - KS,  U = W X ----
#pragma unroll
      for (int b = 4; b < TRI_BLOCKS; ++b) { wa[b] = ldW(b, false); wl[b] = ldW(b, true); }
      __builtin_amdgcn_sched_barrier(0x000F);
      f32x4_t X[NB][4];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mi = 0; mi < 4; ++mi)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            X[nb][mi][r] = (use_v ? quad_element<bf16_t>(vraw[nb][mi], r) : 0.f) - KS[nb][mi][r];
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mi = 0; mi < 4; ++mi) U[nb][mi] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        bf16x8_t xb[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) xb[nb] = half8_sat(X[nb][2 * s], X[nb][2 * s + 1]);
        // lower triangular W: contraction half 1 only reaches row blocks 2 and 3
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int b = (s == 0 ? 0 : 4); b < (s == 0 ? 4 : TRI_BLOCKS); ++b) U[nb][tri_block_m(b)] = mfma16h(wl[b], xb[nb], U[nb][tri_block_m(b)]);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int b = (s == 0 ? 0 : 4); b < (s == 0 ? 4 : TRI_BLOCKS); ++b) U[nb][tri_block_m(b)] = mfma16h(wa[b], xb[nb], U[nb][tri_block_m(b)]);
      }
    }
    if (more && !m_side) { issue_part(ci + 1, 2); issue_part(ci + 1, 3); }
    if (computing) {
      // ---- S^T = e^{G_last} (.) S^T + (K e^{G_last - G})^T U ----
      bf16x8_t kt[8], ktl[8];
#pragma unroll
      for (int mc = 0; mc < 8; ++mc) {
        kt[mc] = operand_granule_transposed(tKt[par][0], 0, mc, kb, r16);
        ktl[mc] = operand_granule_transposed(tKt[par][1], 0, mc, kb, r16);
      }
      float4 eg[8];
#pragma unroll
      for (int mc = 0; mc < 8; ++mc) eg[mc] = *reinterpret_cast<const float4*>(&tE[par][16 * mc + 4 * kb]);
      __builtin_amdgcn_sched_barrier(0x000F);
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int mc = 0; mc < 8; ++mc)
          St[nb][mc] = f32x4_t{St[nb][mc][0] * eg[mc].x, St[nb][mc][1] * eg[mc].y, St[nb][mc][2] * eg[mc].z,
                               St[nb][mc][3] * eg[mc].w};
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        HalfPair ub[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) ub[nb] = half8_pair(U[nb][2 * s], U[nb][2 * s + 1]);
        // hi . lo and lo . hi first, the large term last
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int mc = 0; mc < 8; ++mc) St[nb][mc] = mfma16h(ktl[mc], ub[nb].hi, St[nb][mc]);
        if (s == 0) {
#pragma unroll
          for (int mc = 0; mc < 8; ++mc) ktl[mc] = operand_granule_transposed(tKt[par][1], 1, mc, kb, r16);
          __builtin_amdgcn_sched_barrier(0x000F);
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int mc = 0; mc < 8; ++mc) St[nb][mc] = mfma16h(kt[mc], ub[nb].lo, St[nb][mc]);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int mc = 0; mc < 8; ++mc) St[nb][mc] = mfma16h(kt[mc], ub[nb].hi, St[nb][mc]);
        if (s == 0) {
#pragma unroll
          for (int mc = 0; mc < 8; ++mc) kt[mc] = operand_granule_transposed(tKt[par][0], 1, mc, kb, r16);
          __builtin_amdgcn_sched_barrier(0x000F);
        }
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

struct KdaWorkspaceLayout {
  size_t seq_chunk_off, chunk_seq, chunk_tok, chunk_len, Kg, Qg, Kt, W, P, eGlast;
  size_t seq_seg_off, seg_seq, seg_c0, seg_nc, segM, segB, segS, identity;
  size_t order, stage_begin, carry, total;
  int NC_max, seg_chunks, max_segments, stages;
};
static KdaWorkspaceLayout kda_layout(int T, int N, int H) {
  KdaWorkspaceLayout L;
  L.NC_max = T / CHUNK + N;
  size_t off = 0;
  auto take = [&](size_t bytes) { const size_t at = off; off = align_up256(off + bytes); return at; };
  L.seq_chunk_off = take((size_t)(N + 1) * 4);
  L.chunk_seq = take((size_t)L.NC_max * 4);
  L.chunk_tok = take((size_t)L.NC_max * 4);
  L.chunk_len = take((size_t)L.NC_max * 4);
  const size_t big = (size_t)L.NC_max * H * 8192 * 2, tri = (size_t)L.NC_max * H * TRI_BLOCKS * 1024;
  L.Kg = take(big); L.Qg = take(big); L.Kt = take(2 * big);
  L.W = take(2 * tri); L.P = take(tri);
  L.eGlast = take((size_t)L.NC_max * H * 128 * 4);
  L.seg_chunks = pick_segment_chunks(T, N, H);
  L.max_segments = max_segments(T, N, L.seg_chunks);
  if (L.seg_chunks > 0) {
    L.seq_seg_off = take((size_t)(N + 1) * 4);
    L.seg_seq = take((size_t)L.max_segments * 4);
    L.seg_c0 = take((size_t)L.max_segments * 4);
    L.seg_nc = take((size_t)L.max_segments * 4);
    const size_t states = (size_t)L.max_segments * H * 16384 * 4;
    L.segM = take(states); L.segB = take(states); L.segS = take(states);
    L.identity = take(16384 * 4);
  }
  // pipeline the preparation with the sweeps in stages where that pays
  // Not staged: a sweep (104 KB of LDS) and a preparation workgroup (51 KB) fit a CU together and the staged call
  // is correct (bit-identical per sequence), but the instruction-bound preparation slows the sweeps more than its
  // overlap saves: 8 x 2048 tokens, 32 heads 0.50 -> 0.57 ms, 18 x 1100 tokens, 12 heads 0.24 -> 0.31 ms.
  L.stages = 0;
  if (L.stages > 0) {
    L.order = take((size_t)L.NC_max * 4);
    L.stage_begin = take((size_t)(MAX_STAGES + 2) * 4);
    L.carry = L.seg_chunks > 0 ? 0 : take((size_t)N * H * 16384 * 4);
  }
  L.total = off;
  return L;
}

}  // namespace pla

using namespace pla;

extern "C" int64_t pla_kda_prefill_workspace_bytes(int T, int N, int H) {
  if (T <= 0 || N <= 0 || H <= 0) return 0;
  return (int64_t)kda_layout(T, N, H).total;
}

// The share of a KDA chain's chunk time that one of its two half workgroups takes, and how much longer a chunk takes
// on a full chip than on an idle one (mixed_sweep_plan).  Measured, ms per call of 32 heads without / with the plan
// at (0.9, 0.17) / at (0.8, 0.05): 8000 + 7000 + 1000 + 2000 + 3000 tokens 0.793 / 0.749 / 0.701; eight ragged
// sequences of 32 810 tokens 0.997 / - / 0.948; twelve of 700 to 6000 tokens 0.757 / 0.712 / 0.676.
constexpr double KDA_HALF_COST = 0.8, KDA_FILL_COST = 0.05;

static int kda_prefill_run(
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    int64_t stride_q, int64_t stride_k, int64_t stride_v, int64_t stride_g, int64_t stride_beta,
    const float* A_log, const float* dt_bias, float lower_bound, float scale,
    const int32_t* cu_seqlens, int N, int T,
    const float* h0, const int32_t* h0_indices, int64_t h0_slot_stride,
    float* ht, const int32_t* ht_indices, int64_t ht_slot_stride,
    void* o, void* workspace, int64_t workspace_bytes,
    int H, int K, int V, int act_dtype, void* stream, const int32_t* raw_cu_seqlens) {
  PLA_REQUIRE(K == 128 && V == 128, "KDA prefill requires head_dim K == V == 128, got K=%d, V=%d", K, V);
  PLA_REQUIRE(T > 0 && N > 0 && H > 0, "KDA prefill needs at least one token, sequence and head");
  PLA_REQUIRE(act_dtype == PLA_BF16, "KDA prefill takes bf16 activations (the MFMA operands are bf16)");
  PLA_REQUIRE(q && k && v && g && beta && A_log && dt_bias && o && cu_seqlens && workspace, "null tensor pointer");
  PLA_REQUIRE(lower_bound <= 0.f && lower_bound >= -5.f, "lower_bound must lie in [-5, 0], got %g", (double)lower_bound);
  PLA_REQUIRE(((uintptr_t)q % 16 == 0) && ((uintptr_t)k % 16 == 0) && ((uintptr_t)g % 16 == 0) && stride_q % 8 == 0 &&
                  stride_k % 8 == 0 && stride_g % 8 == 0,
              "q/k/g rows require 16-byte alignment");
  PLA_REQUIRE(((uintptr_t)v % 16 == 0) && stride_v % 8 == 0, "v rows require 16-byte alignment");
  PLA_REQUIRE(((uintptr_t)o % 16 == 0), "out requires 16-byte alignment");
  const KdaWorkspaceLayout L = kda_layout(T, N, H);
  PLA_REQUIRE(workspace_bytes >= (int64_t)L.total, "workspace too small: need %zu bytes", L.total);
  PLA_REQUIRE((uintptr_t)workspace % 256 == 0, "workspace requires 256-byte alignment");
  if (h0) PLA_REQUIRE((uintptr_t)h0 % 16 == 0 && h0_slot_stride % 4 == 0, "state requires 16-byte alignment");
  if (ht) PLA_REQUIRE((uintptr_t)ht % 16 == 0 && ht_slot_stride % 4 == 0, "state requires 16-byte alignment");

  char* ws = reinterpret_cast<char*>(workspace);
  KdaPrefillParams p{};
  p.q = q; p.k = k; p.v = v; p.g = g; p.beta = beta;
  p.stride_q = stride_q; p.stride_k = stride_k; p.stride_v = stride_v; p.stride_g = stride_g; p.stride_beta = stride_beta;
  p.A_log = A_log; p.dt_bias = dt_bias; p.lower_bound = lower_bound; p.scale = scale;
  p.cu_seqlens = cu_seqlens; p.N = N; p.T = T;
  p.h0 = h0; p.h0_indices = h0_indices; p.h0_slot_stride = h0_slot_stride;
  p.ht = ht; p.ht_indices = ht_indices; p.ht_slot_stride = ht_slot_stride;
  p.o = o;
  p.seq_chunk_off = reinterpret_cast<int32_t*>(ws + L.seq_chunk_off);
  p.chunk_seq = reinterpret_cast<int32_t*>(ws + L.chunk_seq);
  p.chunk_tok = reinterpret_cast<int32_t*>(ws + L.chunk_tok);
  p.chunk_len = reinterpret_cast<int32_t*>(ws + L.chunk_len);
  p.Kg = reinterpret_cast<uint16_t*>(ws + L.Kg); p.Qg = reinterpret_cast<uint16_t*>(ws + L.Qg);
  p.Kt = reinterpret_cast<uint16_t*>(ws + L.Kt);
  p.W = reinterpret_cast<uint16_t*>(ws + L.W);
  p.P = reinterpret_cast<uint16_t*>(ws + L.P);
  p.eGlast = reinterpret_cast<float*>(ws + L.eGlast);
  p.H = H; p.NC_max = L.NC_max;

  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const bool segmented = L.seg_chunks > 0;
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
  const bool v_halves = !segmented && (int64_t)N * H <= 128;
  // Ragged whole sequences whose offsets the host holds: the chains of the longest sequences run as two halves where
  // that shortens the sweep (mixed_sweep_plan; the KDA path runs in one stage)
  bool mixed = false;
  if (!segmented && !v_halves && raw_cu_seqlens != nullptr && N <= INLINE_TABLE_SEQUENCES && L.stages == 0) {
    int nc[INLINE_TABLE_SEQUENCES];
    for (int n = 0; n < N; ++n) nc[n] = (std::max(raw_cu_seqlens[n + 1] - raw_cu_seqlens[n], 0) + CHUNK - 1) / CHUNK;
    p.n_long = mixed_sweep_plan(nc, N, H, p.seq_order, KDA_HALF_COST, KDA_FILL_COST);
    // (more chains than CUs: the chains also start longest first - in the order of the sequences the last chain to
    // find a CU may be the longest one -, with or without halves)
    mixed = p.n_long > 0 || (int64_t)N * H > CUS;
    p.split_grid = xcd_grouped_grid(2 * (unsigned)p.n_long * H, 2);
  }
  const SideStreamLease lease(s, L.stages > 0);
  const int stages = lease.get() != nullptr ? L.stages : 0;
  if (stages > 0) {
    p.stg.order = reinterpret_cast<int32_t*>(ws + L.order);
    p.stg.stage_begin = reinterpret_cast<int32_t*>(ws + L.stage_begin);
    p.stg.carry = segmented ? nullptr : reinterpret_cast<float*>(ws + L.carry);
    p.stg.stages = stages;
  }
  launch_tables(s, cu_seqlens, N, T, L.NC_max, p.seq_chunk_off, p.chunk_seq, p.chunk_tok, p.chunk_len, p.seg, p.stg,
                segmented ? L.max_segments : N, o, H);
  const bool ok = launch_pipeline(
      s, stages, lease.get(), segmented, (unsigned)N * H, (unsigned)L.max_segments * H, &p.pass, &p.stage,
      [&](hipStream_t ps) { hipLaunchKernelGGL(kda_prep_solve_kernel, dim3(L.NC_max, H), dim3(256), 0, ps, p); },
      [&](unsigned grid) {
        // the first sweep over segments publishes no output: the lean variant, two workgroups per CU
        // the first sweep over segments publishes no output: both of its roles in one workgroup per (segment, head)
        if (p.pass == 1) hipLaunchKernelGGL(kda_lean_sweep_kernel, dim3(grid / 2), dim3(512), 0, s, p);
        // Whole sequences that give at most 128 chains (few long ones are split into segments instead) leave half of the CUs idle: two
        // workgroups then sweep a chain, 64 V columns each (the columns of V are independent: the same bits).
        else if (mixed) hipLaunchKernelGGL(kda_sweep_mixed_kernel, dim3(p.split_grid + (unsigned)(N - p.n_long) * H), dim3(64 * (4 + KDA_SWEEP_COPIERS)), 0, s, p);
        else if (v_halves) hipLaunchKernelGGL(kda_sweep_kernel<1>, dim3(xcd_grouped_grid(2 * grid, 2)), dim3(64 * (4 + KDA_SWEEP_COPIERS)), 0, s, p);
        else hipLaunchKernelGGL(kda_sweep_kernel<2>, dim3(grid), dim3(64 * (4 + KDA_SWEEP_COPIERS)), 0, s, p);
      });
  PLA_REQUIRE(ok, "an event call of the staged prefill failed: %s", hipGetErrorString(hipGetLastError()));
  if (segmented) {
    hipLaunchKernelGGL(segment_combine_kernel, dim3(xcd_grouped_grid((unsigned)N * H * COMBINE_SPLIT, COMBINE_SPLIT)), dim3(256), 0, s, p.seg, H,
                       N * H);
    p.pass = 2;
    // fewer (segment, head) pairs than half of the CUs (segments are at least 16 chunks long): two workgroups per pair
    // (an upper bound of their number from the token count alone: exact for a single sequence)
    if ((N == 1 ? ((T + CHUNK - 1) / CHUNK + L.seg_chunks - 1) / L.seg_chunks : (int64_t)(T / CHUNK + N) / L.seg_chunks + N) * H <= 128)
      hipLaunchKernelGGL(kda_sweep_kernel<1>, dim3(xcd_grouped_grid(2 * (unsigned)L.max_segments * H, 2)), dim3(64 * (4 + KDA_SWEEP_COPIERS)), 0, s, p);
    else
      hipLaunchKernelGGL(kda_sweep_kernel<2>, dim3((unsigned)L.max_segments * H), dim3(64 * (4 + KDA_SWEEP_COPIERS)), 0, s, p);
  }
  return check_launch("kda prefill launch");
}

extern "C" int pla_kda_prefill_launch(
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    int64_t stride_q, int64_t stride_k, int64_t stride_v, int64_t stride_g, int64_t stride_beta,
    const float* A_log, const float* dt_bias, float lower_bound, float scale,
    const int32_t* cu_seqlens, int N, int T,
    const float* h0, const int32_t* h0_indices, int64_t h0_slot_stride,
    float* ht, const int32_t* ht_indices, int64_t ht_slot_stride,
    void* o, void* workspace, int64_t workspace_bytes,
    int H, int K, int V, int act_dtype, void* stream) {
  return kda_prefill_run(q, k, v, g, beta, stride_q, stride_k, stride_v, stride_g, stride_beta, A_log, dt_bias, lower_bound, scale,
                         cu_seqlens, N, T, h0, h0_indices, h0_slot_stride, ht, ht_indices, ht_slot_stride, o, workspace,
                         workspace_bytes, H, K, V, act_dtype, stream, nullptr);
}

extern "C" int pla_kda_prefill_launch_raw(
    const void* q, const void* k, const void* v, const void* g, const void* beta,
    int64_t stride_q, int64_t stride_k, int64_t stride_v, int64_t stride_g, int64_t stride_beta,
    const float* A_log, const float* dt_bias, float lower_bound, float scale,
    const int32_t* cu_seqlens, int N, int T,
    const float* h0, const int32_t* h0_indices, int64_t h0_slot_stride,
    float* ht, const int32_t* ht_indices, int64_t ht_slot_stride,
    void* o, void* workspace, int64_t workspace_bytes,
    int H, int K, int V, int act_dtype, void* stream, const int32_t* raw_cu_seqlens) {
  return kda_prefill_run(q, k, v, g, beta, stride_q, stride_k, stride_v, stride_g, stride_beta, A_log, dt_bias, lower_bound, scale,
                         cu_seqlens, N, T, h0, h0_indices, h0_slot_stride, ht, ht_indices, ht_slot_stride, o, workspace,
                         workspace_bytes, H, K, V, act_dtype, stream, raw_cu_seqlens);
}

extern "C" int pla_kda_prefill_halved_sequences(const int32_t* raw_cu_seqlens, int N, int T, int H) {
  if (raw_cu_seqlens == nullptr || N <= 0 || N > INLINE_TABLE_SEQUENCES || T <= 0 || H <= 0) return 0;
  const KdaWorkspaceLayout L = kda_layout(T, N, H);
  if (L.seg_chunks > 0 || L.stages > 0 || (int64_t)N * H <= 128) return 0;
  int nc[INLINE_TABLE_SEQUENCES];
  unsigned char order[INLINE_TABLE_SEQUENCES];
  for (int n = 0; n < N; ++n) nc[n] = (std::max(raw_cu_seqlens[n + 1] - raw_cu_seqlens[n], 0) + CHUNK - 1) / CHUNK;
  return mixed_sweep_plan(nc, N, H, order, KDA_HALF_COST, KDA_FILL_COST);
}
