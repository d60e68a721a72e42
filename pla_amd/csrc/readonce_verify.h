// Building blocks of the read-once speculative verify (state read once, never written).
//
// With A_j = D_j (I - beta_j k_j k_j^T) the stepped recurrence over draft tokens 0 .. t unrolls to
//     o_t = S_0 w_t + sum_{j <= t} c_{j,t} v_j,    w_t = A_0 A_1 .. A_t q_t,
//     c_{j,t} = beta_j k_j^T (A_{j+1} .. A_t q_t),
// so the effective queries w_t and the coefficients need only K-vectors, and the state tile enters once,
// as the A operand of S_0 [w_0 .. w_{T-1}] on v_mfma_f32_16x16x32_bf16 (FP32 data carried as bf16 hi + lo:
// hi*hi + lo*hi + hi*lo keeps 16 mantissa bits).  Reference algebra:
// src/decode/kda_replayssm/kda_mtp_verify.cu:630-652.
#pragma once

#include "common.h"
#include "mfma_bf16.h"

namespace pla {

// Effective query and coefficients of token t.  A lane holds four K channels of every vector (both
// halves of the wavefront hold the same data); `w` enters as the scaled, normalised q_t and leaves as
// w_t; cf[j] = c_{j,t} (zero for j > t).  kv: normalised keys, dec: decays exp(g_j), beta: activated.
template <int TMAX>
__device__ __forceinline__ void effective_query(int t, float (&w)[4], const float (&kv)[TMAX][4],
                                                const float (&dec)[TMAX][4], const float (&beta)[TMAX],
                                                float (&cf)[TMAX]) {
#pragma unroll
  for (int j = TMAX - 1; j >= 0; --j) {
    cf[j] = 0.f;
    if (j > t) continue;                       // uniform over the wavefront
    float dot = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) dot = fmaf(kv[j][e], w[e], dot);
    cf[j] = beta[j] * row32_allreduce(dot);
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = dec[j][e] * fmaf(-cf[j], kv[j][e], w[e]);
  }
}

// B operands of the tile pass from the effective queries in LDS (`sw[t][128]`): lane (r16, kb) takes
// column r16 of [w_0 .. w_{T-1} 0 .. 0], contraction elements 32 ks + 8 kb .. + 7.  Lanes whose column
// holds no token (keep == 0) read token `tcol` and zero it.
__device__ __forceinline__ void query_operands(const float (*sw)[128], int tcol, float keep, int kb, HiLo (&wb)[4]) {
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    const float4 w0 = *reinterpret_cast<const float4*>(&sw[tcol][32 * ks + 8 * kb]);
    const float4 w1 = *reinterpret_cast<const float4*>(&sw[tcol][32 * ks + 8 * kb + 4]);
    wb[ks] = split8(f32x4_t{w0.x * keep, w0.y * keep, w0.z * keep, w0.w * keep},
                    f32x4_t{w1.x * keep, w1.y * keep, w1.z * keep, w1.w * keep});
  }
}

// Sixteen state rows times the effective queries.  `rows[ks][hf]`: the lane's (r16, kb) eight FP32 state
// values S[row0 + r16][32 ks + 8 kb + 4 hf .. + 3].  Result: lane (r16 = token, kb) holds rows
// row0 + 4 kb .. + 3 of S_0 w_token.
__device__ __forceinline__ f32x4_t rows_times_queries(const f32x4_t (&rows)[4][2], const HiLo (&wb)[4]) {
  f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    const HiLo a = split8(rows[ks][0], rows[ks][1]);
    acc = mfma16(a.hi, wb[ks].hi, acc);
    acc = mfma16(a.lo, wb[ks].hi, acc);
    acc = mfma16(a.hi, wb[ks].lo, acc);
  }
  return acc;
}

}  // namespace pla
