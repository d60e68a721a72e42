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
// FP32 and split into bf16 hi + lo parts wherever they feed the state.  Overflow never occurs:
// every exponent is <= 0 except inside a 16-row diagonal block of M / P, where the reference row
// is the block's first row and the exponent is bounded by 15 tokens of decay (|lower_bound| <= 5
// gives e^75, well inside the bf16 / FP32 range) - the same sub-chunk scheme as the reference's
// FLA kernels (scripts/prefill/private/ref/chunk_intra.py:170-202).
//
// Kernels:
//   kda_prep_solve_kernel   one workgroup per (chunk, head): q/k L2 norm (rounded to bf16), lower-bound
//                           gate, cumulative decay, decayed operand tiles, M / P on MFMA, FP32 forward
//                           substitution, W (hi/lo)
//   kda_chunk_seq_kernel    one workgroup per (sequence, head), 8 wavefronts x 16 V columns, same
//                           register-chained MFMA pipeline as the GDN kernel

#include "prefill_common.h"

namespace pla {

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
  uint16_t* Khi; uint16_t* Klo; uint16_t* Qh;      // [chunk, H, 64, 128]: k e^{G} (hi, lo), scale q e^{G}
  uint16_t* KtH; uint16_t* KtL;                    // [chunk, H, 128, 64]: (k e^{G_last - G})^T (hi, lo)
  uint16_t* Whi; uint16_t* Wlo; uint16_t* P;       // [chunk, H, 64, 64]
  float* eGlast;                                   // [chunk, H, 128]: e^{G_last}
  SegmentTable seg;                                // split long sequences (seg.seg_chunks > 0)
  int pass;                                        // 0: whole sequences; 1, 2: the two sweeps over segments
  int H, NC_max;
};

// 69 KB, so that two workgroups share a CU.  L takes over Qn's storage once every wavefront has
// formed its q operands (a barrier in phase 3 separates the two uses).
struct __align__(16) KdaPrepShared {
  float G[CHUNK][132];
  uint16_t Kn[CHUNK][PITCH128];
  union {
    uint16_t Qn[CHUNK][PITCH128];
    float L[CHUNK][68];
  };
  float B[CHUNK];
};
static_assert(sizeof(float[CHUNK][68]) <= sizeof(uint16_t[CHUNK][PITCH128]), "L must fit into Qn's storage");

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
  const int cb = blockIdx.x;
  const int h = blockIdx.y;
  if (cb >= p.seq_chunk_off[p.N]) return;
  const int t0 = p.chunk_tok[cb];
  const int len = p.chunk_len[cb];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kb = lane >> 4;
  __shared__ KdaPrepShared sh;
  const int64_t tile = (int64_t)cb * p.H + h;

#ifdef PLA_PROF
  long long tk[6]; tk[0] = clock64();
#endif
  // ---- phase 1: normalised q / k, per-channel log-decay, beta ---------------------------------
  {
    uint32_t qw[16], kw[16];
#pragma unroll
    for (int x = 0; x < 16; ++x) {
      const int j = 16 * wave + x;
      const int64_t t = t0 + (j < len ? j : 0);
      qw[x] = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint16_t*>(p.q) + t * p.stride_q + h * 128 + 2 * lane);
      kw[x] = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint16_t*>(p.k) + t * p.stride_k + h * 128 + 2 * lane);
    }
#pragma unroll
    for (int x = 0; x < 16; ++x) {
      const int j = 16 * wave + x;
      float q0 = lo16<bf16_t>(qw[x]), q1 = hi16<bf16_t>(qw[x]), k0 = lo16<bf16_t>(kw[x]), k1 = hi16<bf16_t>(kw[x]);
      const float qi = rsqrtf(wave64_allreduce(q0 * q0 + q1 * q1) + 1e-6f);
      const float ki = rsqrtf(wave64_allreduce(k0 * k0 + k1 * k1) + 1e-6f);
      const bool ok = j < len;
      *reinterpret_cast<uint32_t*>(&sh.Qn[j][2 * lane]) = ok ? pack2<bf16_t>(q0 * qi, q1 * qi) : 0u;
      *reinterpret_cast<uint32_t*>(&sh.Kn[j][2 * lane]) = ok ? pack2<bf16_t>(k0 * ki, k1 * ki) : 0u;
    }
    // gate: thread handles eight channels of rows tid / 16 + 16 u; all four 16-byte loads are in flight at once
    const float eA = expf(p.A_log[h]);
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
      float bt = 0.f;
      if (tid < len) {
        const float braw = to_float(reinterpret_cast<const bf16_t*>(p.beta)[(int64_t)(t0 + tid) * p.stride_beta + h]);
        bt = 1.0f / (1.0f + expf(-braw));
      }
      sh.B[tid] = bt;
    }
  }
  __syncthreads();
#ifdef PLA_PROF
  tk[1] = clock64();
#endif
  if (tid < 128) {
    float cum = 0.f;
    for (int j = 0; j < CHUNK; ++j) {
      cum += sh.G[j][tid];
      sh.G[j][tid] = cum;                 // rows beyond the chunk repeat G_last (their g is zero)
    }
    p.eGlast[tile * 128 + tid] = __expf(cum);
  }
  __syncthreads();

#ifdef PLA_PROF
  tk[2] = clock64();
#endif
  // ---- phase 2: decayed operand tiles for the sequential kernel -------------------------------
  {
    // row-major tiles: thread handles row j, eight channels, twice
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int vec = tid + 256 * u;                // 1024 vectors: 64 rows x 16
      const int j = vec >> 4, c0 = 8 * (vec & 15);
      const uint4 kx = *reinterpret_cast<const uint4*>(&sh.Kn[j][c0]);
      const uint4 qx = *reinterpret_cast<const uint4*>(&sh.Qn[j][c0]);
      const uint32_t kwv[4] = {kx.x, kx.y, kx.z, kx.w}, qwv[4] = {qx.x, qx.y, qx.z, qx.w};
      uint32_t khi[4], klo[4], qh[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float e0 = __expf(sh.G[j][c0 + 2 * e]), e1 = __expf(sh.G[j][c0 + 2 * e + 1]);
        const float a0 = lo16<bf16_t>(kwv[e]) * e0, a1 = hi16<bf16_t>(kwv[e]) * e1;
        khi[e] = pack2<bf16_t>(a0, a1);
        klo[e] = pack2<bf16_t>(a0 - lo16<bf16_t>(khi[e]), a1 - hi16<bf16_t>(khi[e]));
        qh[e] = pack2<bf16_t>(p.scale * lo16<bf16_t>(qwv[e]) * e0, p.scale * hi16<bf16_t>(qwv[e]) * e1);
      }
      const int64_t off = tile * 8192 + (int64_t)j * 128 + c0;
      *reinterpret_cast<uint4*>(p.Khi + off) = make_uint4(khi[0], khi[1], khi[2], khi[3]);
      *reinterpret_cast<uint4*>(p.Klo + off) = make_uint4(klo[0], klo[1], klo[2], klo[3]);
      *reinterpret_cast<uint4*>(p.Qh + off) = make_uint4(qh[0], qh[1], qh[2], qh[3]);
    }
    // transposed tile (k e^{G_last - G})^T: thread (c, half) gathers 32 tokens of channel c
    const int c = tid >> 1, half = tid & 1;
    const float gl = sh.G[CHUNK - 1][c];
    uint32_t th[16], tl[16];
#pragma unroll
    for (int jj = 0; jj < 16; ++jj) {
      const int j0 = 32 * half + 2 * jj;
      const float a0 = to_float(bf16_t{sh.Kn[j0][c]}) * __expf(gl - sh.G[j0][c]);
      const float a1 = to_float(bf16_t{sh.Kn[j0 + 1][c]}) * __expf(gl - sh.G[j0 + 1][c]);
      th[jj] = pack2<bf16_t>(a0, a1);
      tl[jj] = pack2<bf16_t>(a0 - lo16<bf16_t>(th[jj]), a1 - hi16<bf16_t>(th[jj]));
    }
    const int64_t off = tile * 8192 + (int64_t)c * CHUNK + 32 * half;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      reinterpret_cast<uint4*>(p.KtH + off)[x] = make_uint4(th[4 * x], th[4 * x + 1], th[4 * x + 2], th[4 * x + 3]);
      reinterpret_cast<uint4*>(p.KtL + off)[x] = make_uint4(tl[4 * x], tl[4 * x + 1], tl[4 * x + 2], tl[4 * x + 3]);
    }
  }

#ifdef PLA_PROF
  tk[3] = clock64();
#endif
  // ---- phase 3: M and P, wavefront w owns row block w (reference row = first row of the block) --
  {
    const int bi = wave;
    const float* const R = &sh.G[16 * bi][0];
    const int i_row = 16 * bi + r16;
    HiLo Al[4];
    bf16x8_t Ql[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      f32x4_t a, b;
      decayed8(&sh.Kn[i_row][0], &sh.G[i_row][0], R, 1.0f, s, kb, a, b);
      Al[s] = split8(a, b);
      decayed8(&sh.Qn[i_row][0], &sh.G[i_row][0], R, 1.0f, s, kb, a, b);
      Ql[s] = round8(a, b);
    }
    __syncthreads();                     // Qn is dead from here on: L reuses its storage
    uint16_t* const Pt = p.P + tile * 4096;
    for (int bj = 0; bj < 4; ++bj) {
      const int j = 16 * bj + r16;
      if (bj > bi) {
#pragma unroll
        for (int r = 0; r < 4; ++r) Pt[(16 * bi + 4 * kb + r) * 64 + j] = 0;
        continue;
      }
      f32x4_t m = {0.f, 0.f, 0.f, 0.f}, pq = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        f32x4_t a, b;
        decayed8(&sh.Kn[j][0], &sh.G[j][0], R, -1.0f, s, kb, a, b);     // k_j e^{R - G_j}
        const HiLo Br = split8(a, b);
        m = mfma16(Al[s].hi, Br.hi, m);
        m = mfma16(Al[s].lo, Br.hi, m);
        m = mfma16(Al[s].hi, Br.lo, m);
        pq = mfma16(Ql[s], Br.hi, pq);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = 16 * bi + 4 * kb + r;
        sh.L[i][solve_slot(j)] = i > j ? sh.B[i] * m[r] : 0.f;
        Pt[i * 64 + j] = from_float<bf16_t>(i >= j ? p.scale * pq[r] : 0.f).bits;
      }
    }
  }
  __syncthreads();

#ifdef PLA_PROF
  tk[4] = clock64();
#endif
  // ---- phase 4: W = L^-1 diag(beta), forward substitution on all four wavefronts ----------------
  solve_store_w(sh.L, sh.B, wave, lane, p.Whi + tile * 4096, p.Wlo + tile * 4096);
}

// ---------------------------------------------------------------------------------------------
struct __align__(16) KdaSeqTiles {
  uint16_t Khi[CHUNK][PITCH128];
  uint16_t Klo[CHUNK][PITCH128];
  uint16_t Q[CHUNK][PITCH128];
  uint16_t V[CHUNK][PITCH128];        // doubles as the output tile: wave w only touches columns [16w, 16w+16)
  uint16_t KtH[128][PITCH64];
  uint16_t KtL[128][PITCH64];
  uint16_t Whi[CHUNK][PITCH64];
  uint16_t Wlo[CHUNK][PITCH64];
  uint16_t P[CHUNK][PITCH64];
  float eGl[128];
};

__global__ __launch_bounds__(512) void kda_chunk_seq_kernel(const KdaPrefillParams p) {
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int r16 = lane & 15, kb = lane >> 4;
  const int vcol = 16 * wave + r16;

  // What this workgroup sweeps: a whole sequence, or one segment of it in one of three roles.
  int n, h, c_begin, c_end;
  const float* init = nullptr;        // [V, K] tile the state starts from (nullptr: zero)
  float* fin = nullptr;               // [V, K] tile that receives the state at the end (nullptr: none)
  bool zero_v = false, write_o = true;
  if (p.pass == 0) {
    n = blockIdx.x / p.H;
    h = blockIdx.x - n * p.H;
    c_begin = p.seq_chunk_off[n];
    c_end = p.seq_chunk_off[n + 1];
    if (c_begin >= c_end) return;
    const int slot = (p.h0 != nullptr) ? (p.h0_indices ? p.h0_indices[n] : n) : -1;
    if (slot >= 0) init = p.h0 + (int64_t)slot * p.h0_slot_stride + (int64_t)h * 16384;
    const int oslot = (p.ht != nullptr) ? (p.ht_indices ? p.ht_indices[n] : n) : -1;
    if (oslot >= 0) fin = p.ht + (int64_t)oslot * p.ht_slot_stride + (int64_t)h * 16384;
  } else {
    const int item = p.pass == 1 ? (int)(blockIdx.x >> 1) : (int)blockIdx.x;
    const int from_identity = p.pass == 1 ? (int)(blockIdx.x & 1) : 0;
    const int seg = item / p.H;
    h = item - seg * p.H;
    if (seg >= p.seg.seq_seg_off[p.N]) return;
    n = p.seg.seg_seq[seg];
    const bool first = seg == p.seg.seq_seg_off[n], last = seg + 1 == p.seg.seq_seg_off[n + 1];
    c_begin = p.seg.seg_c0[seg];
    c_end = c_begin + p.seg.seg_nc[seg];
    const int64_t tile = ((int64_t)seg * p.H + h) * 16384;
    if (p.pass == 1) {
      if (first) {
        if (from_identity) return;
        const int slot = (p.h0 != nullptr) ? (p.h0_indices ? p.h0_indices[n] : n) : -1;
        if (slot >= 0) init = p.h0 + (int64_t)slot * p.h0_slot_stride + (int64_t)h * 16384;
        if (!last) {
          fin = p.seg.B + tile;                       // the state that enters the second segment
        } else {
          const int oslot = (p.ht != nullptr) ? (p.ht_indices ? p.ht_indices[n] : n) : -1;
          if (oslot >= 0) fin = p.ht + (int64_t)oslot * p.ht_slot_stride + (int64_t)h * 16384;
        }
      } else {
        write_o = false;
        if (from_identity) { init = p.seg.identity; zero_v = true; fin = p.seg.M + tile; }
        else fin = p.seg.B + tile;
      }
    } else {
      if (first) return;
      init = p.seg.S + tile;                          // the final state came out of the combine step
    }
  }
  const int chunk_in_seq = c_begin - p.seq_chunk_off[n];
  const int seq_start = p.cu_seqlens[n] + chunk_in_seq * CHUNK;
  const int seq_len = min(p.cu_seqlens[n + 1] - seq_start, (c_end - c_begin) * CHUNK);

  __shared__ KdaSeqTiles T;

  f32x4_t St[8];
  {
    if (init != nullptr) {
      const float* src = init + (int64_t)vcol * 128 + 4 * kb;
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

  const int krow = tid >> 4, kcv = tid & 15;
  const int srow = tid >> 3, scv = tid & 7;
  const int64_t tile_stride = (int64_t)p.H * 8192, small_stride = (int64_t)p.H * 4096;
  int64_t big = ((int64_t)c_begin * p.H + h) * 8192;            // offset of this chunk's 64x128 / 128x64 tiles
  int64_t small = ((int64_t)c_begin * p.H + h) * 4096;          // offset of the 64x64 tiles
  const uint16_t* vptr = reinterpret_cast<const uint16_t*>(p.v) + (int64_t)(seq_start + krow) * p.stride_v + h * 128 + 8 * kcv;
  uint16_t* optr = reinterpret_cast<uint16_t*>(p.o) + ((int64_t)(seq_start + krow) * p.H + h) * 128 + 8 * kcv;
  const int64_t o_half = (int64_t)32 * p.H * 128;
  const uint4 zero4 = make_uint4(0, 0, 0, 0);

  uint4 pkh0, pkh1, pkl0, pkl1, pq0, pq1, pv0, pv1, pth0, pth1, ptl0, ptl1, pwh, pwl, ppp;
  float pe = 0.f;
  auto prefetch = [&](int len) {
    const int lo = krow * 128 + 8 * kcv, hi2 = lo + 32 * 128;
    pkh0 = *reinterpret_cast<const uint4*>(p.Khi + big + lo);
    pkh1 = *reinterpret_cast<const uint4*>(p.Khi + big + hi2);
    pkl0 = *reinterpret_cast<const uint4*>(p.Klo + big + lo);
    pkl1 = *reinterpret_cast<const uint4*>(p.Klo + big + hi2);
    pq0 = *reinterpret_cast<const uint4*>(p.Qh + big + lo);
    pq1 = *reinterpret_cast<const uint4*>(p.Qh + big + hi2);
    pth0 = *reinterpret_cast<const uint4*>(p.KtH + big + 8 * tid);
    pth1 = *reinterpret_cast<const uint4*>(p.KtH + big + 4096 + 8 * tid);
    ptl0 = *reinterpret_cast<const uint4*>(p.KtL + big + 8 * tid);
    ptl1 = *reinterpret_cast<const uint4*>(p.KtL + big + 4096 + 8 * tid);
    pwh = *reinterpret_cast<const uint4*>(p.Whi + small + 8 * tid);
    pwl = *reinterpret_cast<const uint4*>(p.Wlo + small + 8 * tid);
    ppp = *reinterpret_cast<const uint4*>(p.P + small + 8 * tid);
    if (tid < 128) pe = p.eGlast[(small >> 5) + tid];            // tile index * 128
    const bool ok0 = krow < len, ok1 = krow + 32 < len;
    const int64_t back0 = ok0 ? 0 : -(int64_t)krow, back1 = ok1 ? 32 : -(int64_t)krow;
    pv0 = *reinterpret_cast<const uint4*>(vptr + back0 * p.stride_v);
    pv1 = *reinterpret_cast<const uint4*>(vptr + back1 * p.stride_v);
    if (!ok0 || zero_v) pv0 = zero4;
    if (!ok1 || zero_v) pv1 = zero4;
    big += tile_stride; small += small_stride; vptr += CHUNK * p.stride_v;
  };
  auto flush_output = [&](int len) {
    if (!write_o) return;
    if (krow < len) *reinterpret_cast<uint4*>(optr) = *reinterpret_cast<const uint4*>(&T.V[krow][8 * kcv]);
    if (krow + 32 < len) *reinterpret_cast<uint4*>(optr + o_half) = *reinterpret_cast<const uint4*>(&T.V[krow + 32][8 * kcv]);
    optr += (int64_t)CHUNK * p.H * 128;
  };

  const int n_chunks = c_end - c_begin;
  prefetch(min(CHUNK, seq_len));
  int prev_len = 0;
  for (int ci = 0; ci < n_chunks; ++ci) {
    const int len = min(CHUNK, seq_len - ci * CHUNK);
    __syncthreads();
    if (ci > 0) flush_output(prev_len);          // reads exactly the vectors this thread overwrites next
    *reinterpret_cast<uint4*>(&T.Khi[krow][8 * kcv]) = pkh0;
    *reinterpret_cast<uint4*>(&T.Khi[krow + 32][8 * kcv]) = pkh1;
    *reinterpret_cast<uint4*>(&T.Klo[krow][8 * kcv]) = pkl0;
    *reinterpret_cast<uint4*>(&T.Klo[krow + 32][8 * kcv]) = pkl1;
    *reinterpret_cast<uint4*>(&T.Q[krow][8 * kcv]) = pq0;
    *reinterpret_cast<uint4*>(&T.Q[krow + 32][8 * kcv]) = pq1;
    *reinterpret_cast<uint4*>(&T.V[krow][8 * kcv]) = pv0;
    *reinterpret_cast<uint4*>(&T.V[krow + 32][8 * kcv]) = pv1;
    *reinterpret_cast<uint4*>(&T.KtH[srow][8 * scv]) = pth0;
    *reinterpret_cast<uint4*>(&T.KtH[64 + srow][8 * scv]) = pth1;
    *reinterpret_cast<uint4*>(&T.KtL[srow][8 * scv]) = ptl0;
    *reinterpret_cast<uint4*>(&T.KtL[64 + srow][8 * scv]) = ptl1;
    *reinterpret_cast<uint4*>(&T.Whi[srow][8 * scv]) = pwh;
    *reinterpret_cast<uint4*>(&T.Wlo[srow][8 * scv]) = pwl;
    *reinterpret_cast<uint4*>(&T.P[srow][8 * scv]) = ppp;
    if (tid < 128) T.eGl[tid] = pe;
    __syncthreads();
    if (ci + 1 < n_chunks) prefetch(min(CHUNK, seq_len - (ci + 1) * CHUNK));

    // KS = (K e^{G}) S^T (three split passes) and QS = (scale Q e^{G}) S^T
    f32x4_t KS[4], QS[4];
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) { KS[mi] = f32x4_t{0.f, 0.f, 0.f, 0.f}; QS[mi] = KS[mi]; }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const HiLo sb = split8(St[2 * s], St[2 * s + 1]);
#pragma unroll
      for (int mi = 0; mi < 4; ++mi) {
        const bf16x8_t kh = operand_from(&T.Khi[16 * mi + r16][0], s, kb);
        const bf16x8_t kl = operand_from(&T.Klo[16 * mi + r16][0], s, kb);
        const bf16x8_t qa = operand_from(&T.Q[16 * mi + r16][0], s, kb);
        KS[mi] = mfma16(kh, sb.hi, KS[mi]);
        QS[mi] = mfma16(qa, sb.hi, QS[mi]);
        KS[mi] = mfma16(kl, sb.hi, KS[mi]);
        KS[mi] = mfma16(kh, sb.lo, KS[mi]);
      }
    }

    f32x4_t X[4];
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) {
      const uint16_t* vr = &T.V[16 * mi + 4 * kb][vcol];
      X[mi][0] = to_float(bf16_t{vr[0]}) - KS[mi][0];
      X[mi][1] = to_float(bf16_t{vr[PITCH128]}) - KS[mi][1];
      X[mi][2] = to_float(bf16_t{vr[2 * PITCH128]}) - KS[mi][2];
      X[mi][3] = to_float(bf16_t{vr[3 * PITCH128]}) - KS[mi][3];
    }

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

    // S^T = e^{G_last} (.) S^T + (K e^{G_last - G})^T U
#pragma unroll
    for (int mc = 0; mc < 8; ++mc) {
      const float4 e = *reinterpret_cast<const float4*>(&T.eGl[16 * mc + 4 * kb]);
      St[mc] = f32x4_t{St[mc][0] * e.x, St[mc][1] * e.y, St[mc][2] * e.z, St[mc][3] * e.w};
    }
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const HiLo ub = split8(U[2 * s], U[2 * s + 1]);
#pragma unroll
      for (int mc = 0; mc < 8; ++mc) {
        const bf16x8_t th = operand_from(&T.KtH[16 * mc + r16][0], s, kb);
        const bf16x8_t tl = operand_from(&T.KtL[16 * mc + r16][0], s, kb);
        St[mc] = mfma16(th, ub.hi, St[mc]);
        St[mc] = mfma16(tl, ub.hi, St[mc]);
        St[mc] = mfma16(th, ub.lo, St[mc]);
      }
    }

    // O = QS + P U
    f32x4_t O[4];
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) O[mi] = QS[mi];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const bf16x8_t ub = round8(U[2 * s], U[2 * s + 1]);
#pragma unroll
      for (int mi = 0; mi < 4; ++mi)
        O[mi] = mfma16(operand_from(&T.P[16 * mi + r16][0], s, kb), ub, O[mi]);
    }
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) {
      uint16_t* orow = &T.V[16 * mi + 4 * kb][vcol];
      orow[0] = from_float<bf16_t>(O[mi][0]).bits;
      orow[PITCH128] = from_float<bf16_t>(O[mi][1]).bits;
      orow[2 * PITCH128] = from_float<bf16_t>(O[mi][2]).bits;
      orow[3 * PITCH128] = from_float<bf16_t>(O[mi][3]).bits;
    }
    prev_len = len;
  }
  __syncthreads();
  flush_output(prev_len);

  if (fin != nullptr) {
    float* dst = fin + (int64_t)vcol * 128 + 4 * kb;
#pragma unroll
    for (int mc = 0; mc < 8; ++mc)
      *reinterpret_cast<float4*>(dst + 16 * mc) = make_float4(St[mc].x, St[mc].y, St[mc].z, St[mc].w);
  }
}

struct KdaWorkspaceLayout {
  size_t seq_chunk_off, chunk_seq, chunk_tok, chunk_len, Khi, Klo, Qh, KtH, KtL, Whi, Wlo, P, eGlast;
  size_t seq_seg_off, seg_seq, seg_c0, seg_nc, segM, segB, segS, identity, total;
  int NC_max, seg_chunks, max_segments;
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
  const size_t big = (size_t)L.NC_max * H * 8192 * 2, small = (size_t)L.NC_max * H * 4096 * 2;
  L.Khi = take(big); L.Klo = take(big); L.Qh = take(big); L.KtH = take(big); L.KtL = take(big);
  L.Whi = take(small); L.Wlo = take(small); L.P = take(small);
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
  L.total = off;
  return L;
}

}  // namespace pla

using namespace pla;

extern "C" int64_t pla_kda_prefill_workspace_bytes(int T, int N, int H) {
  if (T <= 0 || N <= 0 || H <= 0) return 0;
  return (int64_t)kda_layout(T, N, H).total;
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
  PLA_REQUIRE(K == 128 && V == 128, "KDA prefill requires head_dim K == V == 128, got K=%d, V=%d", K, V);
  PLA_REQUIRE(T > 0 && N > 0 && H > 0, "KDA prefill needs at least one token, sequence and head");
  PLA_REQUIRE(act_dtype == PLA_BF16, "KDA prefill takes bf16 activations (the MFMA operands are bf16)");
  PLA_REQUIRE(q && k && v && g && beta && A_log && dt_bias && o && cu_seqlens && workspace, "null tensor pointer");
  PLA_REQUIRE(lower_bound <= 0.f && lower_bound >= -5.f, "lower_bound must lie in [-5, 0], got %g", (double)lower_bound);
  PLA_REQUIRE(((uintptr_t)q % 4 == 0) && ((uintptr_t)k % 4 == 0) && stride_q % 2 == 0 && stride_k % 2 == 0,
              "q/k rows require 4-byte alignment");
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
  p.Khi = reinterpret_cast<uint16_t*>(ws + L.Khi); p.Klo = reinterpret_cast<uint16_t*>(ws + L.Klo);
  p.Qh = reinterpret_cast<uint16_t*>(ws + L.Qh);
  p.KtH = reinterpret_cast<uint16_t*>(ws + L.KtH); p.KtL = reinterpret_cast<uint16_t*>(ws + L.KtL);
  p.Whi = reinterpret_cast<uint16_t*>(ws + L.Whi); p.Wlo = reinterpret_cast<uint16_t*>(ws + L.Wlo);
  p.P = reinterpret_cast<uint16_t*>(ws + L.P);
  p.eGlast = reinterpret_cast<float*>(ws + L.eGlast);
  p.H = H; p.NC_max = L.NC_max;

  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(chunk_map_kernel, dim3(1), dim3(256), 0, s, cu_seqlens, N, L.NC_max, p.seq_chunk_off,
                     p.chunk_seq, p.chunk_tok, p.chunk_len);
  hipLaunchKernelGGL(zero_tail_kernel, dim3(64), dim3(256), 0, s, reinterpret_cast<uint16_t*>(o), cu_seqlens, N, T, H);
  hipLaunchKernelGGL(kda_prep_solve_kernel, dim3(L.NC_max, H), dim3(256), 0, s, p);
  if (L.seg_chunks == 0) {
    p.pass = 0;
    hipLaunchKernelGGL(kda_chunk_seq_kernel, dim3((unsigned)N * H), dim3(512), 0, s, p);
  } else {
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
    hipLaunchKernelGGL(segment_map_kernel, dim3(1), dim3(256), 0, s, p.seq_chunk_off, N, p.seg);
    p.pass = 1;
    hipLaunchKernelGGL(kda_chunk_seq_kernel, dim3((unsigned)L.max_segments * H * 2), dim3(512), 0, s, p);
    hipLaunchKernelGGL(segment_combine_kernel, dim3((unsigned)N * H), dim3(256), 0, s, p.seg, H, ht, ht_indices, ht_slot_stride);
    p.pass = 2;
    hipLaunchKernelGGL(kda_chunk_seq_kernel, dim3((unsigned)L.max_segments * H), dim3(512), 0, s, p);
  }
  return check_launch("kda prefill launch");
}
