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
// row or column scaling of a GEMM result, so the bf16 MFMA operands q, k, v stay exact;
// the FP32 quantities that feed the state (S, X, W, U) are split into bf16 hi + lo parts
// (16 mantissa bits), which keeps the FP32 final state within 1e-5 of a float64 evaluation.
//
// Kernels:
//   chunk_map_kernel         chunk table from cu_seqlens (device side, graph-capturable)
//   gdn_prep_kernel          gate, beta, chunk-local cumsum, q/k L2 norm (rounded to bf16), K^T tiles
//   gdn_gram_solve_kernel    one wavefront per (chunk, value head): K K^T, Q K^T on MFMA, FP32
//                            forward substitution in LDS, W (hi/lo) and P to the workspace
//   gdn_chunk_seq_kernel     one workgroup per (sequence, value head), 8 wavefronts each owning a
//                            16-wide V slice of S^T in MFMA accumulator layout; the chain
//                            K S^T -> X -> U -> O, S^T runs on v_mfma_f32_16x16x32_bf16 with every
//                            intermediate staying in registers (an accumulator tile is already a
//                            valid B operand of the next product), A operands staged through LDS.

#include "prefill_common.h"

namespace pla {

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
  uint16_t* qn; uint16_t* kn; uint16_t* knT;
  float* gcum; float* beta;
  uint16_t* Whi; uint16_t* Wlo; uint16_t* P;
  int H, HV, NC_max;
};

// ---------------------------------------------------------------------------------------------
// grid (chunk, H + 1), 256 threads.  blockIdx.y < H: L2 norm of q and k of one head for the
// chunk's 64 tokens (each wavefront owns 16 rows and requests all of them before reducing) and
// the transposed K tile; blockIdx.y == H: gate, beta and the chunk-local cumulative log-decay.
template <typename act_t>
__global__ __launch_bounds__(256) void gdn_prep_kernel(const GdnPrefillParams p) {
  const int cb = blockIdx.x;
  if (cb >= p.seq_chunk_off[p.N]) return;
  const int t0 = p.chunk_tok[cb];
  const int len = p.chunk_len[cb];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __shared__ union {
    uint16_t tile[CHUNK][130];        // normalised k of one head, for the transposed copy
    float g[CHUNK][129];              // per-token log-decay of up to 128 value heads
  } sh;

  if ((int)blockIdx.y == p.H) {
    for (int hv0 = 0; hv0 < p.HV; hv0 += 128) {
      const int nh = min(128, p.HV - hv0);
      for (int idx = threadIdx.x; idx < CHUNK * nh; idx += 256) {
        const int j = idx / nh, hv = hv0 + idx - j * nh;
        float g = 0.f;
        if (j < len) {
          const int64_t t = t0 + j;
          float bt;
          if (p.g_in) {
            g = p.g_in[t * p.HV + hv];
            bt = p.beta_in[t * p.HV + hv];
          } else {
            const float x = to_float(reinterpret_cast<const act_t*>(p.a)[t * p.stride_a + hv]) + p.dt_bias[hv];
            const float sp = x <= 20.0f ? log1pf(expf(x)) : x;
            g = -expf(p.A_log[hv]) * sp;
            const float braw = to_float(reinterpret_cast<const act_t*>(p.b)[t * p.stride_b + hv]);
            bt = 1.0f / (1.0f + expf(-braw));
          }
          p.beta[t * p.HV + hv] = bt;
        }
        sh.g[j][hv - hv0] = g;
      }
      __syncthreads();
      if ((int)threadIdx.x < nh) {
        float cum = 0.f;
        for (int j = 0; j < len; ++j) {
          cum += sh.g[j][threadIdx.x];
          p.gcum[(int64_t)(t0 + j) * p.HV + hv0 + threadIdx.x] = cum;
        }
      }
      __syncthreads();
    }
    return;
  }

  const int h = blockIdx.y;
  uint32_t qw[16], kw[16];
#pragma unroll
  for (int x = 0; x < 16; ++x) {
    const int j = 16 * wave + x;
    const int64_t t = t0 + (j < len ? j : 0);
    qw[x] = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const act_t*>(p.q) + t * p.stride_q + h * 128 + 2 * lane);
    kw[x] = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const act_t*>(p.k) + t * p.stride_k + h * 128 + 2 * lane);
  }
#pragma unroll
  for (int x = 0; x < 16; ++x) {
    const int j = 16 * wave + x;
    float q0 = lo16<act_t>(qw[x]), q1 = hi16<act_t>(qw[x]), k0 = lo16<act_t>(kw[x]), k1 = hi16<act_t>(kw[x]);
    if (p.normalize_qk) {
      const float qs = wave64_allreduce(q0 * q0 + q1 * q1);
      const float ks = wave64_allreduce(k0 * k0 + k1 * k1);
      const float qi = rsqrtf(qs + 1e-6f), ki = rsqrtf(ks + 1e-6f);
      q0 *= qi; q1 *= qi; k0 *= ki; k1 *= ki;
    }
    uint32_t ko = 0;
    if (j < len) {
      ko = pack2<bf16_t>(k0, k1);
      const int64_t t = t0 + j;
      *reinterpret_cast<uint32_t*>(p.qn + (t * p.H + h) * 128 + 2 * lane) = pack2<bf16_t>(q0, q1);
      *reinterpret_cast<uint32_t*>(p.kn + (t * p.H + h) * 128 + 2 * lane) = ko;
    }
    *reinterpret_cast<uint32_t*>(&sh.tile[j][2 * lane]) = ko;       // zero rows beyond the chunk
  }
  __syncthreads();
  // K^T tile [128][64]: thread (c, half) gathers 32 tokens of column c
  {
    const int c = threadIdx.x >> 1, half = threadIdx.x & 1;
    uint16_t* dst = p.knT + (((int64_t)cb * p.H + h) * 128 + c) * CHUNK + 32 * half;
    uint32_t w[16];
#pragma unroll
    for (int jj = 0; jj < 16; ++jj)
      w[jj] = (uint32_t)sh.tile[32 * half + 2 * jj][c] | ((uint32_t)sh.tile[32 * half + 2 * jj + 1][c] << 16);
#pragma unroll
    for (int x = 0; x < 4; ++x)
      reinterpret_cast<uint4*>(dst)[x] = make_uint4(w[4 * x], w[4 * x + 1], w[4 * x + 2], w[4 * x + 3]);
  }
}

// ---------------------------------------------------------------------------------------------
// One wavefront per (chunk, value head).
__global__ __launch_bounds__(64) void gdn_gram_solve_kernel(const GdnPrefillParams p) {
  const int cb = blockIdx.x / p.HV;
  const int hv = blockIdx.x - cb * p.HV;
  if (cb >= p.seq_chunk_off[p.N]) return;
  const int h = hv / (p.HV / p.H);
  const int t0 = p.chunk_tok[cb];
  const int len = p.chunk_len[cb];
  const int lane = threadIdx.x;
  const int r16 = lane & 15, kb = lane >> 4;

  __shared__ float Lm[CHUNK][68];
  __shared__ float Gs[CHUNK];
  __shared__ float Bs[CHUNK];

  {
    const bool ok = lane < len;
    const float glast = p.gcum[(int64_t)(t0 + len - 1) * p.HV + hv];
    Gs[lane] = ok ? p.gcum[(int64_t)(t0 + lane) * p.HV + hv] : glast;
    Bs[lane] = ok ? p.beta[(int64_t)(t0 + lane) * p.HV + hv] : 0.f;
  }

  // K operands: 4 row blocks x 4 contraction steps (rows beyond the chunk are zero)
  const uint4 zero4 = make_uint4(0, 0, 0, 0);
  bf16x8_t Kop[4][4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb) {
    const int row = 16 * mb + r16;
    const bool ok = row < len;
    const uint16_t* kr = p.kn + ((int64_t)(t0 + (ok ? row : 0)) * p.H + h) * 128;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const bf16x8_t kz = operand_from(kr, s, kb);
      Kop[mb][s] = ok ? kz : __builtin_bit_cast(bf16x8_t, zero4);
    }
  }
  __syncthreads();

  // L = strict_tril(beta_i (k_i . k_j) e^{G_i - G_j})
#pragma unroll
  for (int mi = 0; mi < 4; ++mi) {
#pragma unroll
    for (int ni = 0; ni <= mi; ++ni) {
      f32x4_t kk = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 4; ++s) kk = mfma16(Kop[mi][s], Kop[ni][s], kk);
      const int j = 16 * ni + r16;
      const float Gj = Gs[j];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = 16 * mi + 4 * kb + r;
        Lm[i][j] = i > j ? Bs[i] * kk[r] * __expf(Gs[i] - Gj) : 0.f;
      }
    }
  }

  // P = scale * tril(q_i . k_j e^{G_i - G_j}); one row block of Q at a time keeps registers low
  uint16_t* const Pt = p.P + ((int64_t)cb * p.HV + hv) * 4096;
#pragma unroll
  for (int mi = 0; mi < 4; ++mi) {
    const int row = 16 * mi + r16;
    const bool ok = row < len;
    const uint16_t* qr = p.qn + ((int64_t)(t0 + (ok ? row : 0)) * p.H + h) * 128;
    bf16x8_t Qop[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const bf16x8_t qz = operand_from(qr, s, kb);
      Qop[s] = ok ? qz : __builtin_bit_cast(bf16x8_t, zero4);
    }
#pragma unroll
    for (int ni = 0; ni < 4; ++ni) {
      const int j = 16 * ni + r16;
      if (ni > mi) {
#pragma unroll
        for (int r = 0; r < 4; ++r) Pt[(16 * mi + 4 * kb + r) * 64 + j] = 0;
        continue;
      }
      f32x4_t qk = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 4; ++s) qk = mfma16(Qop[s], Kop[ni][s], qk);
      const float Gj = Gs[j];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = 16 * mi + 4 * kb + r;
        const float gam = i >= j ? __expf(Gs[i] - Gj) : 0.f;
        Pt[i * 64 + j] = from_float<bf16_t>(p.scale * qk[r] * gam).bits;
      }
    }
  }
  __syncthreads();

  // forward substitution, one column per lane: x_i = beta_j [i == j] - sum_{l < i} L[i][l] x_l
  float x[CHUNK];
  const float bj = Bs[lane];
#pragma unroll
  for (int i = 0; i < CHUNK; ++i) {
    // four independent partial sums keep the FMA pipeline full
    float a0 = (i == lane) ? bj : 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
    for (int l4 = 0; l4 < i; l4 += 4) {
      const float4 row = *reinterpret_cast<const float4*>(&Lm[i][l4]);
      a0 = fmaf(-row.x, x[l4], a0);
      if (l4 + 1 < i) a1 = fmaf(-row.y, x[l4 + 1], a1);
      if (l4 + 2 < i) a2 = fmaf(-row.z, x[l4 + 2], a2);
      if (l4 + 3 < i) a3 = fmaf(-row.w, x[l4 + 3], a3);
    }
    x[i] = (a0 + a1) + (a2 + a3);
  }
  uint16_t* const Wh = p.Whi + ((int64_t)cb * p.HV + hv) * 4096;
  uint16_t* const Wl = p.Wlo + ((int64_t)cb * p.HV + hv) * 4096;
#pragma unroll
  for (int i = 0; i < CHUNK; ++i) {
    const bf16_t hi = from_float<bf16_t>(x[i]);
    Wh[i * 64 + lane] = hi.bits;
    Wl[i * 64 + lane] = from_float<bf16_t>(x[i] - to_float(hi)).bits;
  }
}

// ---------------------------------------------------------------------------------------------
// LDS tiles of the sequential kernel (bf16 elements, padded pitches keep 16-byte row alignment
// and spread rows over banks).
struct __align__(16) SeqTiles {
  uint16_t K[CHUNK][PITCH128];
  uint16_t Q[CHUNK][PITCH128];
  uint16_t V[CHUNK][PITCH128];
  uint16_t O[CHUNK][PITCH128];
  uint16_t Kt[128][PITCH64];
  uint16_t Whi[CHUNK][PITCH64];
  uint16_t Wlo[CHUNK][PITCH64];
  uint16_t P[CHUNK][PITCH64];
  float sQ[CHUNK];     // scale * e^{G_i}
  float eG[CHUNK];     // e^{G_i}
  float dG[CHUNK];     // e^{G_last - G_i}
  float eGlast;
};

// Everything the next chunk needs is requested from global memory one chunk ahead and parked
// in registers (eleven 16-byte vectors per thread), every per-chunk address is a running
// pointer, V and O travel through LDS tiles (coalesced 16-byte global accesses, immediate-offset
// LDS accesses), so the chunk-to-chunk critical path holds only LDS reads, conversions and MFMAs.
template <typename act_t>
__global__ __launch_bounds__(512) void gdn_chunk_seq_kernel(const GdnPrefillParams p) {
  const int n = blockIdx.x / p.HV;
  const int hv = blockIdx.x - n * p.HV;
  const int h = hv / (p.HV / p.H);
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kb = lane >> 4;
  const int vcol = 16 * wave + r16;                  // this lane's V column
  const int c_begin = p.seq_chunk_off[n], c_end = p.seq_chunk_off[n + 1];
  if (c_begin >= c_end) return;                      // empty sequence: state untouched, no output
  const int seq_start = p.cu_seqlens[n];
  const int seq_len = p.cu_seqlens[n + 1] - seq_start;

  __shared__ SeqTiles T;

  // S^T slice in accumulator layout: St[mc][r] = S[v = vcol][c = 16 mc + 4 kb + r]
  f32x4_t St[8];
  {
    const int slot = (p.h0 != nullptr) ? (p.h0_indices ? p.h0_indices[n] : n) : -1;
    if (slot >= 0) {
      const float* src = p.h0 + (int64_t)slot * p.h0_slot_stride + ((int64_t)hv * 128 + vcol) * 128 + 4 * kb;
#pragma unroll
      for (int mc = 0; mc < 8; ++mc) {
        const float4 t4 = *reinterpret_cast<const float4*>(src + 16 * mc);
        St[mc] = f32x4_t{t4.x, t4.y, t4.z, t4.w};
      }
    } else {
#pragma unroll
      for (int mc = 0; mc < 8; ++mc) St[mc] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
  }

  // cooperative copy coordinates: 64-row x 128-column tiles are 1024 16-byte vectors (two per
  // thread: rows krow and krow + 32), 64 x 64 and the 128 x 64 K^T tiles 512 / 1024 vectors.
  const int krow = tid >> 4, kcv = tid & 15;
  const int srow = tid >> 3, scv = tid & 7;
  const int64_t tok_pitch = (int64_t)p.H * 128;                // elements between tokens of kn / qn
  const int64_t half_k = 32 * tok_pitch, half_v = 32 * p.stride_v;
  const uint16_t* kptr = p.kn + ((int64_t)(seq_start + krow) * p.H + h) * 128 + 8 * kcv;
  const uint16_t* qptr = p.qn + ((int64_t)(seq_start + krow) * p.H + h) * 128 + 8 * kcv;
  const uint16_t* vptr = reinterpret_cast<const uint16_t*>(p.v) + (int64_t)(seq_start + krow) * p.stride_v + hv * 128 + 8 * kcv;
  const uint16_t* ktptr = p.knT + ((int64_t)c_begin * p.H + h) * 8192 + 8 * tid;
  const uint16_t* whptr = p.Whi + ((int64_t)c_begin * p.HV + hv) * 4096 + 8 * tid;
  const uint16_t* wlptr = p.Wlo + ((int64_t)c_begin * p.HV + hv) * 4096 + 8 * tid;
  const uint16_t* ppptr = p.P + ((int64_t)c_begin * p.HV + hv) * 4096 + 8 * tid;
  const float* gptr = p.gcum + (int64_t)seq_start * p.HV + hv;
  uint16_t* optr = reinterpret_cast<uint16_t*>(p.o) + ((int64_t)(seq_start + krow) * p.HV + hv) * 128 + 8 * kcv;
  const int64_t o_half = (int64_t)32 * p.HV * 128;
  const uint4 zero4 = make_uint4(0, 0, 0, 0);

  uint4 pk0, pk1, pq0, pq1, pv0, pv1, pt0, pt1, pwh, pwl, ppp;
  float pg;
  // `len` rows of the chunk are real; rows beyond are read from row 0 of the chunk and zeroed.
  auto prefetch = [&](int len) {
    const bool ok0 = krow < len, ok1 = krow + 32 < len;
    const int64_t back0 = ok0 ? 0 : -(int64_t)krow, back1 = ok1 ? 32 : -(int64_t)krow;
    pk0 = *reinterpret_cast<const uint4*>(kptr + back0 * tok_pitch);
    pq0 = *reinterpret_cast<const uint4*>(qptr + back0 * tok_pitch);
    pv0 = *reinterpret_cast<const uint4*>(vptr + back0 * p.stride_v);
    pk1 = *reinterpret_cast<const uint4*>(kptr + back1 * tok_pitch);
    pq1 = *reinterpret_cast<const uint4*>(qptr + back1 * tok_pitch);
    pv1 = *reinterpret_cast<const uint4*>(vptr + back1 * p.stride_v);
    pt0 = *reinterpret_cast<const uint4*>(ktptr);
    pt1 = *reinterpret_cast<const uint4*>(ktptr + 4096);
    pwh = *reinterpret_cast<const uint4*>(whptr);
    pwl = *reinterpret_cast<const uint4*>(wlptr);
    ppp = *reinterpret_cast<const uint4*>(ppptr);
    pg = gptr[(int64_t)(lane < len ? lane : len - 1) * p.HV];
    if (!ok0) { pk0 = zero4; pq0 = zero4; pv0 = zero4; }
    if (!ok1) { pk1 = zero4; pq1 = zero4; pv1 = zero4; }
    (void)half_k; (void)half_v;
  };
  auto advance = [&]() {
    kptr += CHUNK * tok_pitch; qptr += CHUNK * tok_pitch; vptr += CHUNK * p.stride_v;
    ktptr += (int64_t)p.H * 8192; whptr += (int64_t)p.HV * 4096; wlptr += (int64_t)p.HV * 4096;
    ppptr += (int64_t)p.HV * 4096; gptr += (int64_t)CHUNK * p.HV;
  };
  // coalesced write of the previous chunk's output tile
  auto flush_output = [&](int len) {
    if (krow < len) *reinterpret_cast<uint4*>(optr) = *reinterpret_cast<const uint4*>(&T.O[krow][8 * kcv]);
    if (krow + 32 < len) *reinterpret_cast<uint4*>(optr + o_half) = *reinterpret_cast<const uint4*>(&T.O[krow + 32][8 * kcv]);
    optr += (int64_t)CHUNK * p.HV * 128;
  };

  const int n_chunks = c_end - c_begin;
  prefetch(min(CHUNK, seq_len));
  advance();
  int prev_len = 0;
  for (int ci = 0; ci < n_chunks; ++ci) {
    const int len = min(CHUNK, seq_len - ci * CHUNK);

    __syncthreads();                 // everyone finished with the previous chunk's tiles
    if (ci > 0) flush_output(prev_len);
    *reinterpret_cast<uint4*>(&T.K[krow][8 * kcv]) = pk0;
    *reinterpret_cast<uint4*>(&T.K[krow + 32][8 * kcv]) = pk1;
    *reinterpret_cast<uint4*>(&T.Q[krow][8 * kcv]) = pq0;
    *reinterpret_cast<uint4*>(&T.Q[krow + 32][8 * kcv]) = pq1;
    *reinterpret_cast<uint4*>(&T.V[krow][8 * kcv]) = pv0;
    *reinterpret_cast<uint4*>(&T.V[krow + 32][8 * kcv]) = pv1;
    *reinterpret_cast<uint4*>(&T.Kt[srow][8 * scv]) = pt0;
    *reinterpret_cast<uint4*>(&T.Kt[64 + srow][8 * scv]) = pt1;
    *reinterpret_cast<uint4*>(&T.Whi[srow][8 * scv]) = pwh;
    *reinterpret_cast<uint4*>(&T.Wlo[srow][8 * scv]) = pwl;
    *reinterpret_cast<uint4*>(&T.P[srow][8 * scv]) = ppp;
    if (wave == 0) {
      const float glast = __shfl(pg, len - 1, 64);
      const float e = __expf(pg);
      T.eG[lane] = e;
      T.sQ[lane] = p.scale * e;
      T.dG[lane] = __expf(glast - pg);
      if (lane == 0) T.eGlast = __expf(glast);
    }
    __syncthreads();
    if (ci + 1 < n_chunks) {
      prefetch(min(CHUNK, seq_len - (ci + 1) * CHUNK));
      advance();
    }

    // (1) KS = K S^T and (3a) QS = Q S^T : contraction over the 128 K channels
    f32x4_t KS[4], QS[4];
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) { KS[mi] = f32x4_t{0.f, 0.f, 0.f, 0.f}; QS[mi] = KS[mi]; }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const HiLo sb = split8(St[2 * s], St[2 * s + 1]);
#pragma unroll
      for (int mi = 0; mi < 4; ++mi) {
        const bf16x8_t ka = operand_from(&T.K[16 * mi + r16][0], s, kb);
        const bf16x8_t qa = operand_from(&T.Q[16 * mi + r16][0], s, kb);
        KS[mi] = mfma16(ka, sb.hi, KS[mi]);
        QS[mi] = mfma16(qa, sb.hi, QS[mi]);
        KS[mi] = mfma16(ka, sb.lo, KS[mi]);
      }
    }

    // X = V - e^{G} (.) KS   (rows of the accumulator are tokens)
    f32x4_t X[4];
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) {
      const float4 eg = *reinterpret_cast<const float4*>(&T.eG[16 * mi + 4 * kb]);
      const uint16_t* vr = &T.V[16 * mi + 4 * kb][vcol];
      X[mi][0] = to_float(act_t{vr[0]}) - eg.x * KS[mi][0];
      X[mi][1] = to_float(act_t{vr[PITCH128]}) - eg.y * KS[mi][1];
      X[mi][2] = to_float(act_t{vr[2 * PITCH128]}) - eg.z * KS[mi][2];
      X[mi][3] = to_float(act_t{vr[3 * PITCH128]}) - eg.w * KS[mi][3];
    }

    // (2) U = W X : contraction over the 64 tokens, W and X both split
    f32x4_t U[4];
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) U[mi] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const HiLo xb = split8(X[2 * s], X[2 * s + 1]);
#pragma unroll
      for (int mi = 0; mi < 4; ++mi) {
        const bf16x8_t wh = operand_from(&T.Whi[16 * mi + r16][0], s, kb);
        const bf16x8_t wl = operand_from(&T.Wlo[16 * mi + r16][0], s, kb);
        U[mi] = mfma16(wh, xb.hi, U[mi]);
        U[mi] = mfma16(wl, xb.hi, U[mi]);
        U[mi] = mfma16(wh, xb.lo, U[mi]);
      }
    }

    // (4) S^T = e^{G_last} S^T + K^T (e^{G_last - G} (.) U)   -- the next chunk waits for this
    const float egl = T.eGlast;
#pragma unroll
    for (int mc = 0; mc < 8; ++mc) St[mc] *= egl;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const float4 d0 = *reinterpret_cast<const float4*>(&T.dG[32 * s + 4 * kb]);
      const float4 d1 = *reinterpret_cast<const float4*>(&T.dG[32 * s + 16 + 4 * kb]);
      const f32x4_t u0 = {U[2 * s][0] * d0.x, U[2 * s][1] * d0.y, U[2 * s][2] * d0.z, U[2 * s][3] * d0.w};
      const f32x4_t u1 = {U[2 * s + 1][0] * d1.x, U[2 * s + 1][1] * d1.y, U[2 * s + 1][2] * d1.z, U[2 * s + 1][3] * d1.w};
      const HiLo ub = split8(u0, u1);
#pragma unroll
      for (int mc = 0; mc < 8; ++mc) {
        const bf16x8_t ka = operand_from(&T.Kt[16 * mc + r16][0], s, kb);
        St[mc] = mfma16(ka, ub.hi, St[mc]);
        St[mc] = mfma16(ka, ub.lo, St[mc]);
      }
    }

    // (3b) O = scale e^{G} (.) QS + P U   -- off the state's critical path
    f32x4_t O[4];
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) {
      const float4 sq = *reinterpret_cast<const float4*>(&T.sQ[16 * mi + 4 * kb]);
      O[mi] = f32x4_t{sq.x * QS[mi][0], sq.y * QS[mi][1], sq.z * QS[mi][2], sq.w * QS[mi][3]};
    }
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const bf16x8_t ub = round8(U[2 * s], U[2 * s + 1]);
#pragma unroll
      for (int mi = 0; mi < 4; ++mi)
        O[mi] = mfma16(operand_from(&T.P[16 * mi + r16][0], s, kb), ub, O[mi]);
    }
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) {
      uint16_t* orow = &T.O[16 * mi + 4 * kb][vcol];
      orow[0] = from_float<act_t>(O[mi][0]).bits;
      orow[PITCH128] = from_float<act_t>(O[mi][1]).bits;
      orow[2 * PITCH128] = from_float<act_t>(O[mi][2]).bits;
      orow[3 * PITCH128] = from_float<act_t>(O[mi][3]).bits;
    }
    prev_len = len;
  }
  __syncthreads();
  flush_output(prev_len);

  if (p.ht != nullptr) {
    const int slot = p.ht_indices ? p.ht_indices[n] : n;
    if (slot >= 0) {
      float* dst = p.ht + (int64_t)slot * p.ht_slot_stride + ((int64_t)hv * 128 + vcol) * 128 + 4 * kb;
#pragma unroll
      for (int mc = 0; mc < 8; ++mc)
        *reinterpret_cast<float4*>(dst + 16 * mc) = make_float4(St[mc].x, St[mc].y, St[mc].z, St[mc].w);
    }
  }
}


struct GdnWorkspaceLayout {
  size_t seq_chunk_off, chunk_seq, chunk_tok, chunk_len, qn, kn, knT, gcum, beta, Whi, Wlo, P, total;
  int NC_max;
};
static GdnWorkspaceLayout gdn_layout(int T, int N, int H, int HV) {
  GdnWorkspaceLayout L;
  L.NC_max = T / CHUNK + N;
  size_t off = 0;
  auto take = [&](size_t bytes) { const size_t at = off; off = align_up256(off + bytes); return at; };
  L.seq_chunk_off = take((size_t)(N + 1) * 4);
  L.chunk_seq = take((size_t)L.NC_max * 4);
  L.chunk_tok = take((size_t)L.NC_max * 4);
  L.chunk_len = take((size_t)L.NC_max * 4);
  L.qn = take((size_t)T * H * 128 * 2);
  L.kn = take((size_t)T * H * 128 * 2);
  L.knT = take((size_t)L.NC_max * H * 128 * CHUNK * 2);
  L.gcum = take((size_t)T * HV * 4);
  L.beta = take((size_t)T * HV * 4);
  L.Whi = take((size_t)L.NC_max * HV * 4096 * 2);
  L.Wlo = take((size_t)L.NC_max * HV * 4096 * 2);
  L.P = take((size_t)L.NC_max * HV * 4096 * 2);
  L.total = off;
  return L;
}

}  // namespace pla

using namespace pla;

extern "C" int64_t pla_gdn_prefill_workspace_bytes(int T, int N, int H, int HV) {
  if (T <= 0 || N <= 0 || H <= 0 || HV <= 0) return 0;
  return (int64_t)gdn_layout(T, N, H, HV).total;
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
  PLA_REQUIRE(K == 128 && V == 128, "GDN prefill requires head_dim K == V == 128, got K=%d, V=%d", K, V);
  PLA_REQUIRE(T > 0 && N > 0, "GDN prefill needs at least one token and one sequence");
  PLA_REQUIRE(H > 0 && HV >= H && HV % H == 0, "HV must be a positive multiple of H, got H=%d, HV=%d", H, HV);
  PLA_REQUIRE(act_dtype == PLA_BF16, "GDN prefill takes bf16 activations (the MFMA operands are bf16)");
  PLA_REQUIRE(q && k && v && o && cu_seqlens && workspace, "null tensor pointer");
  PLA_REQUIRE((g_in != nullptr) == (beta_in != nullptr), "g and beta must be given together");
  PLA_REQUIRE(g_in != nullptr || (a && b && A_log && dt_bias), "raw gating needs a, b, A_log and dt_bias");
  PLA_REQUIRE(((uintptr_t)q % 4 == 0) && ((uintptr_t)k % 4 == 0) && stride_q % 2 == 0 && stride_k % 2 == 0,
              "q/k rows require 4-byte alignment");
  const GdnWorkspaceLayout L = gdn_layout(T, N, H, HV);
  PLA_REQUIRE(workspace_bytes >= (int64_t)L.total, "workspace too small: need %zu bytes", L.total);
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
  p.qn = reinterpret_cast<uint16_t*>(ws + L.qn);
  p.kn = reinterpret_cast<uint16_t*>(ws + L.kn);
  p.knT = reinterpret_cast<uint16_t*>(ws + L.knT);
  p.gcum = gcum_out ? gcum_out : reinterpret_cast<float*>(ws + L.gcum);
  p.beta = beta_out ? beta_out : reinterpret_cast<float*>(ws + L.beta);
  p.Whi = reinterpret_cast<uint16_t*>(ws + L.Whi);
  p.Wlo = reinterpret_cast<uint16_t*>(ws + L.Wlo);
  p.P = reinterpret_cast<uint16_t*>(ws + L.P);
  p.H = H; p.HV = HV; p.NC_max = L.NC_max;

  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(chunk_map_kernel, dim3(1), dim3(256), 0, s, cu_seqlens, N, L.NC_max, p.seq_chunk_off,
                     p.chunk_seq, p.chunk_tok, p.chunk_len);
  hipLaunchKernelGGL(zero_tail_kernel, dim3(64), dim3(256), 0, s, reinterpret_cast<uint16_t*>(o), cu_seqlens, N, T, HV);
  if (act_dtype == PLA_BF16) {
    hipLaunchKernelGGL(gdn_prep_kernel<bf16_t>, dim3(L.NC_max, H + 1), dim3(256), 0, s, p);
  } else {
    hipLaunchKernelGGL(gdn_prep_kernel<f16_t>, dim3(L.NC_max, H + 1), dim3(256), 0, s, p);
  }
  hipLaunchKernelGGL(gdn_gram_solve_kernel, dim3((unsigned)L.NC_max * HV), dim3(64), 0, s, p);
  if (act_dtype == PLA_BF16)
    hipLaunchKernelGGL(gdn_chunk_seq_kernel<bf16_t>, dim3((unsigned)N * HV), dim3(512), 0, s, p);
  else
    hipLaunchKernelGGL(gdn_chunk_seq_kernel<f16_t>, dim3((unsigned)N * HV), dim3(512), 0, s, p);
  return check_launch("gdn prefill launch");
}
