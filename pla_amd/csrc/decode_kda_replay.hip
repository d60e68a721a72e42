// KDA speculative verify with replay records (SGLang ReplaySSM, ring mode) and the conv-window
// rollback of the commit, for gfx950.
//
// Verify (reference: src/decode/kda_replayssm/kda_mtp_verify.cu:700-1100, contract
// src/decode/kda_replayssm_sglang/kda_mtp_verify_host.cpp:50-243, Python model
// scripts/decode/kda_mtp_sglang/private/_reference.py:88-177): for every request the T draft tokens
// run through the width-4 causal convolution + SiLU (seeded from the request's conv state, which
// is read-only here), the lower-bound gate and the delta-rule recurrence starting from the
// request's FP32 state, which is read once and never written.  Side effects besides the output:
// the conv window after every token goes to the request's scratch row, and the per-token records
// (post-conv k and v in bf16, log-decay and beta in FP32) go to the slot's rings, from which the
// commit later replays the accepted prefix.
//
// One workgroup of four wavefronts per (request, head).  The state tile is requested first, in
// MFMA A-operand layout.  Threads 0-127 then run the convolution of one q and one k channel
// through all tokens, threads 128-255 that of one v channel plus the channel's gate; everything
// the recurrence needs meets in LDS.  The recurrence itself is not stepped: with
//     o_t = S_0 w_t + sum_{j <= t} c_{j,t} v_j,  w_t = A_1 .. A_t q_t,  A_j = D_j (I - beta_j k_j k_j^T)
// wavefront w works out w_t and c_{.,t} for tokens t = w, w + 4 from K-vectors alone, and the tile
// is used once as the A operand of S_0 [w_0 .. w_{T-1}] on v_mfma_f32_16x16x32_bf16 (FP32 data split
// into bf16 hi + lo, three products), sixteen tokens per pass.  Up to 32 draft tokens (the reference's
// limit); windows of up to eight keep all K-vectors in registers, wider ones re-read them from LDS.
//
// Conv-window scatter (reference: conv_scatter_kernel, src/decode/kda_replayssm/kda_mtp_fold.cu:595-635):
// dst[layer, dst_idx[r], :, :] = src[layer, r, step_idx[r], :, :] for every request r with a
// non-negative step and an in-range destination.

#include "decode_common.h"
#include "readonce_verify.h"

namespace pla {

struct ReplayVerifyParams {
  const uint16_t* x_q; const uint16_t* x_k; const uint16_t* x_v; const uint16_t* g; const uint16_t* beta;
  const float* w_q; const float* w_k; const float* w_v;
  const uint16_t* cs_q; const uint16_t* cs_k; const uint16_t* cs_v;
  const float* a_log; const float* dt_bias; float* h0;
  uint16_t* out; uint16_t* ic_q; uint16_t* ic_k; uint16_t* ic_v;
  uint16_t* ring_rawv; uint16_t* ring_rawk; float* ring_g; float* ring_beta;
  const void* slot_idx; const void* scratch_idx; const void* cu;
  int slot_wide, scratch_wide, cu_wide;
  int H, N, T, L;
  float scale, lower_bound;
  int64_t sx_q, sx_k, sx_v, sg, sbeta;
  int64_t cs[3][3];        // q, k, v conv state: slot, channel, window strides
  int64_t ic[3][4];        // q, k, v scratch windows: row, step, channel, window strides
  const uint16_t* onorm_gate; const float* onorm_weight; int64_t onorm_gate_stride; float onorm_eps;
  // Paged (vLLM) mode: records and scratch windows are indexed by the request row instead of the slot,
  // the checkpoint pool has a slot pitch, slots <= null_block_id are padding and malformed query
  // intervals are skipped (src/decode/kda_replayssm/kda_mtp_verify.cu:721-741).
  int native, null_block_id, slots, tokens;
  int64_t state_slot;
  // Scratch windows with the layout [row, step, channel, 3] (window contiguous, channel pitch 3) and
  // 16-byte aligned rows: records and windows leave through LDS as 16-byte vectors.
  int wide_stores;
};

__device__ __forceinline__ int64_t index_at(const void* p, int wide, int64_t i) {
  return wide ? reinterpret_cast<const int64_t*>(p)[i] : (int64_t) reinterpret_cast<const int32_t*>(p)[i];
}
__device__ __forceinline__ float bf(uint16_t x) { return to_float(bf16_t{x}); }
__device__ __forceinline__ uint16_t to_bf(float x) { return from_float<bf16_t>(x).bits; }

// Convolution of one channel over the draft tokens.  `taps` holds the window (oldest first) and is
// advanced; returns silu(conv).  Same operation order as the reference (:815-818).
__device__ __forceinline__ float conv_step(float (&taps)[3], float x, const float4 w) {
  float acc = x * w.w;
  acc = fmaf(taps[0], w.x, acc);
  acc = fmaf(taps[1], w.y, acc);
  acc = fmaf(taps[2], w.z, acc);
  taps[0] = taps[1]; taps[1] = taps[2]; taps[2] = x;
  return acc * fast_sigmoid(acc);
}

// (windows of up to four tokens: the compiler is held to 128 registers, four workgroups per CU instead of three - 124
// without a spill, 42.3 -> 40.2 us for 64 requests of 32 heads; the eight-token kernel spills under that bound)
template <int TMAX, bool ONORM>
__global__ __launch_bounds__(256, TMAX <= 4 ? 4 : 1) void kda_verify_dspark_kernel(const ReplayVerifyParams p) {
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, c = lane & 31;
  const int r16 = lane & 15, kb = lane >> 4;
  const int n = blockIdx.x / p.H, h = blockIdx.x - n * p.H;
  int64_t slot = index_at(p.slot_idx, p.slot_wide, n);
  const int64_t bos = index_at(p.cu, p.cu_wide, n);
  const int64_t eos = index_at(p.cu, p.cu_wide, n + 1);
  if (p.native) {
    if (index_at(p.cu, p.cu_wide, 0) != 0 || bos < 0 || eos <= bos || eos > p.tokens || eos - bos > p.T || slot >= p.slots)
      return;
    if (slot <= p.null_block_id) slot = -1;
  }
  const int n_tok = (int)min((int64_t)p.T, eos - bos);
  if (bos < 0 || n_tok <= 0) return;
  const int rowbase = 32 * wave;

  if (slot < 0) {                                   // padded request: zero output rows, nothing else
    for (int i = tid; i < n_tok * 128; i += 256)
      p.out[((bos + i / 128) * p.H + h) * 128 + (i & 127)] = 0;
    return;
  }
  const int64_t srow = p.native ? n : index_at(p.scratch_idx, p.scratch_wide, n);

  // sQ[t] holds q_t after the convolution and the effective query w_t after the algebra (only the
  // wavefront that owns token t touches the row in between).
  __shared__ __align__(16) float sQ[TMAX][128], sK[TMAX][128], sV[TMAX][128], sD[TMAX][128];
  __shared__ __align__(16) float sC[TMAX][TMAX];    // sC[t][j] = c_{j,t}
  float (*const sW)[128] = sQ;
  __shared__ float sBeta[TMAX], sNorm[2][2][TMAX], sSq[4][TMAX];
  // Staging of what the workgroup writes besides o (draft windows of up to eight tokens): the raw q / k / v
  // channel sequences [state taps, tokens] the conv windows are cut from, and the log-decay records.
  constexpr bool STAGED = TMAX <= 8;
  constexpr int SEQ = TMAX + 3;
  __shared__ __align__(16) uint16_t sSeq[STAGED ? 3 : 1][STAGED ? 128 : 1][STAGED ? SEQ : 1];
  __shared__ __align__(16) float sG[STAGED ? TMAX : 1][STAGED ? 128 : 1];
  const bool staged = STAGED && p.wide_stores;

  // Small inputs first, the state tile after them: memory returns in issue order, so the convolution
  // starts as soon as its inputs are there while the 64 KiB tile is still in flight.  Wavefronts 0-1
  // (threads 0-127) own one q and one k channel each, wavefronts 2-3 one v channel and its gate.
  const bool qk_side = tid < 128;
  const int i128 = tid & 127;
  const int64_t ch = (int64_t)h * 128 + i128;
  const float4 cwa = reinterpret_cast<const float4*>(qk_side ? p.w_q : p.w_v)[ch];
  const float4 cwb = reinterpret_cast<const float4*>(p.w_k)[ch];
  const uint16_t* const cs_a = qk_side ? p.cs_q : p.cs_v;
  const int ia = qk_side ? 0 : 2;
  uint16_t ta[3], tb[3], xa[TMAX], xb[TMAX], xc[TMAX];
#pragma unroll
  for (int j = 0; j < 3; ++j) {
    ta[j] = cs_a[slot * p.cs[ia][0] + ch * p.cs[ia][1] + j * p.cs[ia][2]];
    tb[j] = p.cs_k[slot * p.cs[1][0] + ch * p.cs[1][1] + j * p.cs[1][2]];
  }
#pragma unroll
  for (int t = 0; t < TMAX; ++t) {                   // absent tokens repeat the last one
    const int64_t tok = bos + min(t, n_tok - 1);
    xa[t] = qk_side ? p.x_q[tok * p.sx_q + ch] : p.x_v[tok * p.sx_v + ch];
    xb[t] = qk_side ? p.x_k[tok * p.sx_k + ch] : p.g[tok * p.sg + ch];
    xc[t] = p.beta[tok * p.sbeta + h];
  }
  const float a_log_h = p.a_log[h];
  const float bias = p.dt_bias[ch];
  // state tile, lane (r16, kb) holds S[32 w + 16 m + r16][32 ks + 8 kb .. + 7]: requested before anything looks at
  // the small inputs (the staging below waits for them, and would hold the tile back by one trip to memory)
  const Tile<float> h_tile(p.h0 + slot * p.state_slot + (int64_t)h * 16384);
  f32x4_t sa[2][4][2];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int hf = 0; hf < 2; ++hf)
        // (no non-temporal hint: the two loads of a contraction step take interleaved 16-byte pieces of the same
        // 128-byte lines, and the second finds them in the vector cache; with the hint it fetched them from the L2
        // again: 48.6 -> 42.2 us for 64 requests of 32 heads)
        sa[m][ks][hf] = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(
            h_tile.rsrc, ((rowbase + 16 * m + r16) * 128 + 32 * ks + 8 * kb) * 4 + 16 * hf, 0, 0));

  const float eA = __expf(a_log_h);
  if constexpr (STAGED) {
    if (staged) {
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        sSeq[ia][i128][j] = ta[j];
        if (qk_side) sSeq[1][i128][j] = tb[j];
      }
#pragma unroll
      for (int t = 0; t < TMAX; ++t) {
        sSeq[ia][i128][3 + t] = xa[t];
        if (qk_side) sSeq[1][i128][3 + t] = xb[t];
      }
    }
  }

  const int64_t ring_row = ((p.native ? n : slot) * p.H + h) * p.L;   // first record of this (slot or request, head)
  if (qk_side) {
    float cq[3] = {bf(ta[0]), bf(ta[1]), bf(ta[2])}, ck[3] = {bf(tb[0]), bf(tb[1]), bf(tb[2])};
#pragma unroll
    for (int t = 0; t < TMAX; ++t) {
      if (t >= n_tok) break;
      const float q = conv_step(cq, bf(xa[t]), cwa);
      const float k = conv_step(ck, bf(xb[t]), cwb);
      sQ[t][tid] = q;
      sK[t][tid] = k;
      if (!staged) {
        p.ring_rawk[(ring_row + t) * 128 + tid] = to_bf(k);
#pragma unroll
        for (int j = 0; j < 3; ++j) {
          p.ic_q[srow * p.ic[0][0] + t * p.ic[0][1] + ch * p.ic[0][2] + j * p.ic[0][3]] = to_bf(cq[j]);
          p.ic_k[srow * p.ic[1][0] + t * p.ic[1][1] + ch * p.ic[1][2] + j * p.ic[1][3]] = to_bf(ck[j]);
        }
      }
      const float q2 = wave64_allreduce(q * q), k2 = wave64_allreduce(k * k);
      if (lane == 0) { sNorm[0][wave][t] = q2; sNorm[1][wave][t] = k2; }
    }
  } else {
    float cv[3] = {bf(ta[0]), bf(ta[1]), bf(ta[2])};
#pragma unroll
    for (int t = 0; t < TMAX; ++t) {
      if (t >= n_tok) break;
      const float v = conv_step(cv, bf(xa[t]), cwa);
      sV[t][i128] = v;
      const float gk = p.lower_bound * fast_sigmoid(eA * (bf(xb[t]) + bias));
      if (!staged) {
        p.ring_rawv[(ring_row + t) * 128 + i128] = to_bf(v);
#pragma unroll
        for (int j = 0; j < 3; ++j)
          p.ic_v[srow * p.ic[2][0] + t * p.ic[2][1] + ch * p.ic[2][2] + j * p.ic[2][3]] = to_bf(cv[j]);
        p.ring_g[(ring_row + t) * 128 + i128] = gk;
      } else if constexpr (STAGED) {
        sG[t][i128] = gk;
      }
      sD[t][i128] = __expf(gk);
      if (i128 == 0) {
        const float b = fast_sigmoid(bf(xc[t]));
        sBeta[t] = b;
        p.ring_beta[ring_row + t] = b;
      }
    }
  }
  __syncthreads();

  // K-vector algebra: wavefront w handles tokens w, w + 4, ...
  if constexpr (TMAX <= 8) {                        // all K-vectors in registers
    float kv[TMAX][4], dec[TMAX][4], beta[TMAX];
#pragma unroll
    for (int j = 0; j < TMAX; ++j) {
      const int jj = min(j, n_tok - 1);
      const float kn = fast_rsqrt(sNorm[1][0][jj] + sNorm[1][1][jj] + 1e-6f);
      const float4 k4 = *reinterpret_cast<const float4*>(&sK[jj][4 * c]);
      const float4 d4 = *reinterpret_cast<const float4*>(&sD[jj][4 * c]);
      kv[j][0] = k4.x * kn; kv[j][1] = k4.y * kn; kv[j][2] = k4.z * kn; kv[j][3] = k4.w * kn;
      dec[j][0] = d4.x; dec[j][1] = d4.y; dec[j][2] = d4.z; dec[j][3] = d4.w;
      beta[j] = sBeta[jj];
    }
#pragma unroll
    for (int tt = 0; tt < TMAX / 4; ++tt) {
      const int t = wave + 4 * tt;
      if (t >= n_tok) break;
      const float qn = fast_rsqrt(sNorm[0][0][t] + sNorm[0][1][t] + 1e-6f) * p.scale;
      const float4 q4 = *reinterpret_cast<const float4*>(&sQ[t][4 * c]);
      float w[4] = {q4.x * qn, q4.y * qn, q4.z * qn, q4.w * qn};
      float cf[TMAX];
      effective_query<TMAX>(t, w, kv, dec, beta, cf);
      if (half == 0) *reinterpret_cast<float4*>(&sW[t][4 * c]) = make_float4(w[0], w[1], w[2], w[3]);
      if (lane == 0) {
#pragma unroll
        for (int j = 0; j < TMAX; ++j) sC[t][j] = cf[j];
      }
    }
  } else {                                          // wide draft windows: K-vectors stay in LDS
    for (int t = wave; t < n_tok; t += 4) {
      const float qn = fast_rsqrt(sNorm[0][0][t] + sNorm[0][1][t] + 1e-6f) * p.scale;
      const float4 q4 = *reinterpret_cast<const float4*>(&sQ[t][4 * c]);
      float w[4] = {q4.x * qn, q4.y * qn, q4.z * qn, q4.w * qn};
      if (lane > t && lane < TMAX) sC[t][lane] = 0.f;
      for (int j = t; j >= 0; --j) {
        const float kn = fast_rsqrt(sNorm[1][0][j] + sNorm[1][1][j] + 1e-6f);
        const float4 k4 = *reinterpret_cast<const float4*>(&sK[j][4 * c]);
        const float4 d4 = *reinterpret_cast<const float4*>(&sD[j][4 * c]);
        const float kj[4] = {k4.x * kn, k4.y * kn, k4.z * kn, k4.w * kn};
        float dot = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) dot = fmaf(kj[e], w[e], dot);
        const float cf = sBeta[j] * row32_allreduce(dot);
        w[0] = d4.x * fmaf(-cf, kj[0], w[0]);
        w[1] = d4.y * fmaf(-cf, kj[1], w[1]);
        w[2] = d4.z * fmaf(-cf, kj[2], w[2]);
        w[3] = d4.w * fmaf(-cf, kj[3], w[3]);
        if (lane == 0) sC[t][j] = cf;
      }
      if (half == 0) *reinterpret_cast<float4*>(&sW[t][4 * c]) = make_float4(w[0], w[1], w[2], w[3]);
    }
  }
  __syncthreads();

  // Tile pass, sixteen tokens (MFMA columns) at a time: column r16 of [w_0 .. w_{T-1} 0 .. 0]
  constexpr int NCOL = (TMAX + 15) / 16;
  float o[NCOL][2][4];
  float ss[NCOL];
#pragma unroll
  for (int cg = 0; cg < NCOL; ++cg) {
    const int token = 16 * cg + r16;
    const int tcol = min(token, n_tok - 1);
    const float keep = token < n_tok ? 1.f : 0.f;
    HiLo wb[4];
    query_operands(sW, tcol, keep, kb, wb);
    ss[cg] = 0.f;
    if (16 * cg >= n_tok) continue;                 // uniform: no token in this column group
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      const f32x4_t acc = rows_times_queries(sa[m], wb);
      // lane (r16 = token, kb): rows 32 w + 16 m + 4 kb .. + 3 of S_0 w_token, plus the bias terms
      o[cg][m][0] = acc[0]; o[cg][m][1] = acc[1]; o[cg][m][2] = acc[2]; o[cg][m][3] = acc[3];
    }
    const int last = min(n_tok, 16 * cg + 16);      // c_{j,t} = 0 for j > t
#pragma unroll(TMAX <= 8 ? TMAX : 4)
    for (int jt = 0; jt < (TMAX <= 8 ? TMAX : last); ++jt) {
      if (TMAX <= 8 && jt >= n_tok) break;
      const float cj = sC[tcol][jt];
#pragma unroll
      for (int m = 0; m < 2; ++m) {
        const float4 v4 = *reinterpret_cast<const float4*>(&sV[jt][rowbase + 16 * m + 4 * kb]);
        o[cg][m][0] = fmaf(cj, v4.x, o[cg][m][0]);
        o[cg][m][1] = fmaf(cj, v4.y, o[cg][m][1]);
        o[cg][m][2] = fmaf(cj, v4.z, o[cg][m][2]);
        o[cg][m][3] = fmaf(cj, v4.w, o[cg][m][3]);
      }
    }
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int r = 0; r < 4; ++r) ss[cg] = fmaf(o[cg][m][r], o[cg][m][r], ss[cg]);
  }

  if constexpr (ONORM) {
    // sum of squares of a token's 128 outputs: over the four 16-lane rows of the wavefront, then over
    // the four wavefronts through LDS
#pragma unroll
    for (int cg = 0; cg < NCOL; ++cg) {
      const LanePair rows = swap_rows16(ss[cg]);
      const LanePair halves = swap_halves(rows.lo + rows.hi);
      if (lane < 16 && 16 * cg + lane < TMAX) sSq[wave][16 * cg + lane] = halves.lo + halves.hi;
    }
    __syncthreads();
  }
#pragma unroll
  for (int cg = 0; cg < NCOL; ++cg) {
    const int token = 16 * cg + r16;
    if (token >= n_tok) continue;
    float rstd = 1.f;
    if constexpr (ONORM) {
      const float total = sSq[0][token] + sSq[1][token] + sSq[2][token] + sSq[3][token];
      rstd = fast_rsqrt(total * (1.0f / 128.0f) + p.onorm_eps);
    }
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      const int row = rowbase + 16 * m + 4 * kb;
      float val[4] = {o[cg][m][0], o[cg][m][1], o[cg][m][2], o[cg][m][3]};
      if constexpr (ONORM) {
        const uint2 gw = *reinterpret_cast<const uint2*>(p.onorm_gate + (bos + token) * p.onorm_gate_stride + h * 128 + row);
        const float4 w4 = *reinterpret_cast<const float4*>(p.onorm_weight + row);
        val[0] *= rstd * w4.x * fast_sigmoid(lo16<bf16_t>(gw.x));
        val[1] *= rstd * w4.y * fast_sigmoid(hi16<bf16_t>(gw.x));
        val[2] *= rstd * w4.z * fast_sigmoid(lo16<bf16_t>(gw.y));
        val[3] *= rstd * w4.w * fast_sigmoid(hi16<bf16_t>(gw.y));
      }
      *reinterpret_cast<uint2*>(p.out + ((bos + token) * p.H + h) * 128 + row) =
          make_uint2(pack2<bf16_t>(val[0], val[1]), pack2<bf16_t>(val[2], val[3]));
    }
  }

  // Records and windows last: nothing in this workgroup waits for them.
  if constexpr (STAGED) {
    if (staged) {
      // Per token 208 vectors of 16 bytes.  Wavefront 0: post-conv k and v as bf16 (lanes 0-15, 16-31) and
      // the log-decay (lanes 32-63); wavefront 1 + x: the window of tensor x (q, k, v) after the token,
      // 48 vectors = 128 channels x 3 taps, taps t + 1 .. t + 3 of the channel's sequence.
      if (wave == 0) {
        for (int t = 0; t < n_tok; ++t) {
          if (lane < 32) {
            const bool is_v = lane >= 16;
            const float* src = (is_v ? sV[t] : sK[t]) + 8 * (lane & 15);
            const float4 a = *reinterpret_cast<const float4*>(src), b = *reinterpret_cast<const float4*>(src + 4);
            uint16_t* dst = (is_v ? p.ring_rawv : p.ring_rawk) + (ring_row + t) * 128 + 8 * (lane & 15);
            *reinterpret_cast<uint4*>(dst) = make_uint4(pack2<bf16_t>(a.x, a.y), pack2<bf16_t>(a.z, a.w),
                                                        pack2<bf16_t>(b.x, b.y), pack2<bf16_t>(b.z, b.w));
          } else {
            *reinterpret_cast<float4*>(p.ring_g + (ring_row + t) * 128 + 4 * (lane - 32)) =
                *reinterpret_cast<const float4*>(&sG[t][4 * (lane - 32)]);
          }
        }
      } else if (lane < 48) {
        const int x = wave - 1;
        const uint16_t* src[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) src[e] = &sSeq[x][(8 * lane + e) / 3][1 + (8 * lane + e) % 3];
        uint16_t* const dst = (x == 0 ? p.ic_q : x == 1 ? p.ic_k : p.ic_v) + srow * p.ic[x][0] + (int64_t)h * 384 + 8 * lane;
        for (int t = 0; t < n_tok; ++t) {
          uint32_t w[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = (uint32_t)src[2 * e][t] | ((uint32_t)src[2 * e + 1][t] << 16);
          *reinterpret_cast<uint4*>(dst + t * p.ic[x][1]) = make_uint4(w[0], w[1], w[2], w[3]);
        }
      }
    }
  }
}

// One thread per channel: copies the window of the selected step into the destination slot.
template <typename T>
__global__ __launch_bounds__(256) void conv_window_scatter_kernel(
    const T* src, T* dst, const void* dst_idx, int dst_wide, const void* step_idx, int step_wide,
    int dim, int km1, int64_t s_layer, int64_t s_req, int64_t s_step, int64_t s_dim, int64_t s_win,
    int64_t d_layer, int64_t d_req, int64_t d_dim, int64_t d_win, int src_reqs, int src_steps, int dst_reqs) {
  const int r = blockIdx.x;
  const int64_t layer = blockIdx.y;
  const int64_t step = index_at(step_idx, step_wide, r);
  const int64_t d_i = index_at(dst_idx, dst_wide, r);
  if (step < 0 || d_i < 0 || d_i >= dst_reqs || r >= src_reqs || step >= src_steps) return;
  const int d = blockIdx.z * 256 + threadIdx.x;
  if (d >= dim) return;
  const T* sp = src + layer * s_layer + (int64_t)r * s_req + step * s_step + (int64_t)d * s_dim;
  T* dp = dst + layer * d_layer + d_i * d_req + (int64_t)d * d_dim;
  for (int w = 0; w < km1; ++w) dp[w * d_win] = sp[w * s_win];
}

// Conv windows of a commit plan into the paged conv histories of all layers: request r copies the window
// after its boundary_lengths[r]-th token to slot boundary[r] (if any) and then the window after its
// lengths[r]-th token to slot final[r]; one thread per channel does both, in this order.  Layer pointers
// and strides come from the layer table (entries 6-14).
__global__ __launch_bounds__(256) void conv_window_native_kernel(
    const int64_t* layer_table, const int32_t* lengths, const int32_t* final_idx, const int32_t* boundary_idx,
    const int32_t* boundary_lengths, int channels, int steps, int rows, int slots) {
  const int r = blockIdx.x;
  const int d = blockIdx.z * 256 + threadIdx.x;
  if (d >= channels || r >= rows) return;
  const int64_t* const e = layer_table + (int64_t)blockIdx.y * PLA_LAYER_TABLE_ENTRIES;
  uint16_t* const conv = reinterpret_cast<uint16_t*>(e[6]);
  const uint16_t* const win = reinterpret_cast<const uint16_t*>(e[10]);
  const int64_t c_slot = e[7], c_ch = e[8], c_tap = e[9], w_row = e[11], w_step = e[12], w_ch = e[13], w_tap = e[14];
  const int count[2] = {boundary_lengths[r], lengths[r]};
  const int dest[2] = {boundary_idx[r], final_idx[r]};
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int step = count[i] - 1;
    if (step < 0 || step >= steps || dest[i] < 0 || dest[i] >= slots) continue;
    const uint16_t* sp = win + r * w_row + step * w_step + d * w_ch;
    uint16_t* dp = conv + dest[i] * c_slot + d * c_ch;
#pragma unroll
    for (int w = 0; w < 3; ++w) dp[w * c_tap] = sp[w * w_tap];
  }
}

static bool aligned_at(const void* ptr, size_t a) { return (reinterpret_cast<uintptr_t>(ptr) % a) == 0; }

}  // namespace pla

namespace pla {
// Shared by the ring-mode and the paged entry points.
static int launch_replay_verify(ReplayVerifyParams& p, const int64_t* strides, int t_loop, hipStream_t s) {
  PLA_REQUIRE(p.H > 0 && p.N > 0 && t_loop > 0, "verify requires H > 0, N > 0 and at least one token per request");
  PLA_REQUIRE(t_loop <= 32, "the verify handles up to 32 draft tokens per request, got %d", t_loop);
  PLA_REQUIRE(p.L >= t_loop, "record rings shorter than the draft window");
  PLA_REQUIRE((int64_t)p.N * p.H <= 0x7fffffffLL, "N * H exceeds the grid limit");
  PLA_REQUIRE(aligned_at(p.h0, 16) && p.state_slot % 4 == 0 && aligned_at(p.w_q, 16) && aligned_at(p.w_k, 16) &&
              aligned_at(p.w_v, 16) && aligned_at(p.out, 8), "state, conv weights and out require vector alignment");
  const bool onorm = p.onorm_gate != nullptr;
  PLA_REQUIRE(!onorm || (p.onorm_weight != nullptr && aligned_at(p.onorm_weight, 16) && aligned_at(p.onorm_gate, 8) &&
                         p.onorm_gate_stride % 4 == 0 && p.onorm_eps >= 0.f),
              "fused output norm requires an aligned gate (token stride a multiple of 4), a weight and eps >= 0");
  for (int i = 0; i < 26; ++i) PLA_REQUIRE(strides[i] > 0, "stride %d must be positive", i);
  p.T = t_loop;
  p.wide_stores = 1;
  {
    void* const windows[3] = {p.ic_q, p.ic_k, p.ic_v};
    for (int x = 0; x < 3; ++x)
      if (strides[14 + 4 * x + 2] != 3 || strides[14 + 4 * x + 3] != 1 || strides[14 + 4 * x] % 8 != 0 ||
          strides[14 + 4 * x + 1] % 8 != 0 || !aligned_at(windows[x], 16))
        p.wide_stores = 0;
    if (!aligned_at(p.ring_rawk, 16) || !aligned_at(p.ring_rawv, 16) || !aligned_at(p.ring_g, 16)) p.wide_stores = 0;
  }
  p.sx_q = strides[0]; p.sx_k = strides[1]; p.sx_v = strides[2]; p.sg = strides[3]; p.sbeta = strides[4];
  for (int t = 0; t < 3; ++t)
    for (int j = 0; j < 3; ++j) p.cs[t][j] = strides[5 + 3 * t + j];
  for (int t = 0; t < 3; ++t)
    for (int j = 0; j < 4; ++j) p.ic[t][j] = strides[14 + 4 * t + j];
  const dim3 grid((unsigned)p.N * (unsigned)p.H), block(256);
  if (t_loop <= 4) {
    if (onorm) kda_verify_dspark_kernel<4, true><<<grid, block, 0, s>>>(p);
    else kda_verify_dspark_kernel<4, false><<<grid, block, 0, s>>>(p);
  } else if (t_loop <= 8) {
    if (onorm) kda_verify_dspark_kernel<8, true><<<grid, block, 0, s>>>(p);
    else kda_verify_dspark_kernel<8, false><<<grid, block, 0, s>>>(p);
  } else if (t_loop <= 16) {
    if (onorm) kda_verify_dspark_kernel<16, true><<<grid, block, 0, s>>>(p);
    else kda_verify_dspark_kernel<16, false><<<grid, block, 0, s>>>(p);
  } else {
    if (onorm) kda_verify_dspark_kernel<32, true><<<grid, block, 0, s>>>(p);
    else kda_verify_dspark_kernel<32, false><<<grid, block, 0, s>>>(p);
  }
  return check_launch("kda_verify_dspark_kernel");
}
}  // namespace pla

extern "C" int pla_kda_verify_dspark_launch(
    const void* x_q, const void* x_k, const void* x_v, const void* g_in, const void* beta_in,
    const float* w_q, const float* w_k, const float* w_v,
    const void* cs_q, const void* cs_k, const void* cs_v,
    const float* a_log, const float* dt_bias, const float* h0,
    void* out, void* ic_q, void* ic_k, void* ic_v,
    void* ring_rawv, void* ring_rawk, float* ring_g, float* ring_beta,
    const void* slot_idx, int slot_idx_wide, const void* scratch_idx, int scratch_idx_wide,
    const void* cu_seqlens, int cu_seqlens_wide,
    int H, int N, int t_loop, int ring_len, float scale, float lower_bound,
    const int64_t* strides,
    const void* onorm_gate, const float* onorm_weight, int64_t onorm_gate_stride, float onorm_eps,
    void* stream) {
  using namespace pla;
  PLA_REQUIRE(x_q && x_k && x_v && g_in && beta_in && w_q && w_k && w_v && cs_q && cs_k && cs_v && a_log && dt_bias && h0 &&
              out && ic_q && ic_k && ic_v && ring_rawv && ring_rawk && ring_g && ring_beta && slot_idx && scratch_idx &&
              cu_seqlens && strides, "null tensor pointer");
  ReplayVerifyParams p{};
  p.x_q = (const uint16_t*)x_q; p.x_k = (const uint16_t*)x_k; p.x_v = (const uint16_t*)x_v;
  p.g = (const uint16_t*)g_in; p.beta = (const uint16_t*)beta_in;
  p.w_q = w_q; p.w_k = w_k; p.w_v = w_v;
  p.cs_q = (const uint16_t*)cs_q; p.cs_k = (const uint16_t*)cs_k; p.cs_v = (const uint16_t*)cs_v;
  p.a_log = a_log; p.dt_bias = dt_bias; p.h0 = const_cast<float*>(h0);
  p.out = (uint16_t*)out; p.ic_q = (uint16_t*)ic_q; p.ic_k = (uint16_t*)ic_k; p.ic_v = (uint16_t*)ic_v;
  p.ring_rawv = (uint16_t*)ring_rawv; p.ring_rawk = (uint16_t*)ring_rawk; p.ring_g = ring_g; p.ring_beta = ring_beta;
  p.slot_idx = slot_idx; p.scratch_idx = scratch_idx; p.cu = cu_seqlens;
  p.slot_wide = slot_idx_wide; p.scratch_wide = scratch_idx_wide; p.cu_wide = cu_seqlens_wide;
  p.H = H; p.N = N; p.L = ring_len; p.scale = scale; p.lower_bound = lower_bound;
  p.onorm_gate = (const uint16_t*)onorm_gate; p.onorm_weight = onorm_weight;
  p.onorm_gate_stride = onorm_gate_stride; p.onorm_eps = onorm_eps;
  p.native = 0; p.null_block_id = -1; p.slots = 0; p.tokens = 0; p.state_slot = (int64_t)H * 16384;
  return launch_replay_verify(p, strides, t_loop, static_cast<hipStream_t>(stream));
}

extern "C" int pla_kda_replay_verify_native_launch(
    const void* x_q, const void* x_k, const void* x_v, const void* g_in, const void* beta_in,
    const float* w_q, const float* w_k, const float* w_v,
    const void* cs_q, const void* cs_k, const void* cs_v,
    const float* a_log, const float* dt_bias, const float* h0,
    void* out, void* ic_q, void* ic_k, void* ic_v,
    void* rawv, void* rawk, float* gate, float* beta,
    const void* slot_idx, int slot_idx_wide, const void* cu_seqlens, int cu_seqlens_wide,
    int H, int N, int Q, float scale, float lower_bound, const int64_t* strides,
    int64_t state_slot_stride, int slots, int tokens, int null_block_id, void* stream) {
  using namespace pla;
  PLA_REQUIRE(x_q && x_k && x_v && g_in && beta_in && w_q && w_k && w_v && cs_q && cs_k && cs_v && a_log && dt_bias && h0 &&
              out && ic_q && ic_k && ic_v && rawv && rawk && gate && beta && slot_idx && cu_seqlens && strides,
              "null tensor pointer");
  PLA_REQUIRE(null_block_id == -1 || null_block_id == 0, "null_block_id must be -1 or 0");
  PLA_REQUIRE(slots > 0 && tokens >= 0 && state_slot_stride >= (int64_t)H * 16384,
              "paged state requires slots > 0 and a slot pitch of at least H * 128 * 128");
  if (N == 0) return 0;
  ReplayVerifyParams p{};
  p.x_q = (const uint16_t*)x_q; p.x_k = (const uint16_t*)x_k; p.x_v = (const uint16_t*)x_v;
  p.g = (const uint16_t*)g_in; p.beta = (const uint16_t*)beta_in;
  p.w_q = w_q; p.w_k = w_k; p.w_v = w_v;
  p.cs_q = (const uint16_t*)cs_q; p.cs_k = (const uint16_t*)cs_k; p.cs_v = (const uint16_t*)cs_v;
  p.a_log = a_log; p.dt_bias = dt_bias; p.h0 = const_cast<float*>(h0);
  p.out = (uint16_t*)out; p.ic_q = (uint16_t*)ic_q; p.ic_k = (uint16_t*)ic_k; p.ic_v = (uint16_t*)ic_v;
  p.ring_rawv = (uint16_t*)rawv; p.ring_rawk = (uint16_t*)rawk; p.ring_g = gate; p.ring_beta = beta;
  p.slot_idx = slot_idx; p.scratch_idx = slot_idx; p.cu = cu_seqlens;
  p.slot_wide = slot_idx_wide; p.scratch_wide = slot_idx_wide; p.cu_wide = cu_seqlens_wide;
  p.H = H; p.N = N; p.L = Q; p.scale = scale; p.lower_bound = lower_bound;
  p.onorm_gate = nullptr; p.onorm_weight = nullptr; p.onorm_gate_stride = 0; p.onorm_eps = 0.f;
  p.native = 1; p.null_block_id = null_block_id; p.slots = slots; p.tokens = tokens; p.state_slot = state_slot_stride;
  return launch_replay_verify(p, strides, Q, static_cast<hipStream_t>(stream));
}

extern "C" int pla_conv_window_scatter_launch(
    int elem_bytes, int km1, const void* src, void* dst,
    const void* dst_idx, int dst_idx_wide, const void* step_idx, int step_idx_wide,
    int layers, int dim, int reqs,
    int64_t src_s0, int64_t src_s1, int64_t src_s2, int64_t src_s3, int64_t src_s4,
    int64_t dst_s0, int64_t dst_s1, int64_t dst_s2, int64_t dst_s3,
    int src_reqs, int src_steps, int dst_reqs, void* stream) {
  using namespace pla;
  PLA_REQUIRE(elem_bytes == 2 || elem_bytes == 4, "conv scatter: element size must be 2 or 4 bytes, got %d", elem_bytes);
  PLA_REQUIRE(km1 >= 1 && km1 <= 4, "conv scatter: unsupported conv window %d", km1);
  if (reqs == 0) return 0;
  PLA_REQUIRE(src && dst && dst_idx && step_idx, "null tensor pointer");
  PLA_REQUIRE(layers > 0 && dim > 0 && reqs > 0 && layers <= 65535, "conv scatter: layers, dim and reqs must be positive");
  const dim3 grid((unsigned)reqs, (unsigned)layers, (unsigned)((dim + 255) / 256)), block(256);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (elem_bytes == 2)
    conv_window_scatter_kernel<uint16_t><<<grid, block, 0, s>>>(
        (const uint16_t*)src, (uint16_t*)dst, dst_idx, dst_idx_wide, step_idx, step_idx_wide, dim, km1,
        src_s0, src_s1, src_s2, src_s3, src_s4, dst_s0, dst_s1, dst_s2, dst_s3, src_reqs, src_steps, dst_reqs);
  else
    conv_window_scatter_kernel<uint32_t><<<grid, block, 0, s>>>(
        (const uint32_t*)src, (uint32_t*)dst, dst_idx, dst_idx_wide, step_idx, step_idx_wide, dim, km1,
        src_s0, src_s1, src_s2, src_s3, src_s4, dst_s0, dst_s1, dst_s2, dst_s3, src_reqs, src_steps, dst_reqs);
  return check_launch("conv_window_scatter_kernel");
}

extern "C" int pla_kda_conv_native_launch(
    const int64_t* layer_table, int layers, const int32_t* lengths, const int32_t* final_indices,
    const int32_t* boundary_indices, const int32_t* boundary_lengths,
    int batch, int channels, int Q, int rows, int slots, void* stream) {
  using namespace pla;
  PLA_REQUIRE(layer_table && lengths && final_indices && boundary_indices && boundary_lengths, "null table or plan pointer");
  PLA_REQUIRE(layers >= 1 && layers <= 65535 && channels > 0 && Q >= 1 && slots > 0 && batch <= rows,
              "conv commit requires 1..65535 layers, channels > 0, Q >= 1, slots > 0 and batch <= record rows");
  if (batch == 0) return 0;
  const dim3 grid((unsigned)batch, (unsigned)layers, (unsigned)((channels + 255) / 256)), block(256);
  conv_window_native_kernel<<<grid, block, 0, static_cast<hipStream_t>(stream)>>>(
      layer_table, lengths, final_indices, boundary_indices, boundary_lengths, channels, Q, rows, slots);
  return check_launch("conv_window_native_kernel");
}
