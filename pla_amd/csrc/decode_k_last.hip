// k-last gated delta-rule decode, MTP verify and accepted-prefix commit for gfx950.
//
// One 128x128 FP32 state tile S[v][k] per (request, value head) is streamed from
// HBM exactly once, updated in registers and written back once.  A 64-lane
// wavefront owns RPW consecutive V-rows.  Lanes 0-31 hold the even rows of the
// wave's range and lanes 32-63 the odd rows; lane c of a half holds the K
// channels [4c, 4c+4) of each of its rows, so one 16-byte load instruction of
// the wave moves two adjacent rows = 1 KiB of contiguous memory.  The two
// reductions over K (S.k and S.q) span 32 lanes: four DPP adds inside a DPP row
// plus one v_permlane16_swap across the two rows.  There is no LDS traffic and
// no barrier, so all state loads of a wave are in flight together.
//
// Semantics follow the reference kernels
//   src/decode/k-last/fused_sigmoid_gating_k_last_packed_kernel.cuh:59-384 (packed T=1)
//   src/decode/k-last/fused_sigmoid_gating_k_last_kernel.cuh:131-1058     (decode / MTP verify)
//   src/decode/kda_replayssm/kda_mtp_fold.cu:256-545                      (commit)
// with one deliberate difference: corrupt cu_seqlens (negative start, length
// above T_max) make the request a no-op instead of trapping the device.

#include "decode_common.h"
#include "readonce_verify.h"
#include "tuned_table.h"

#include <type_traits>

namespace pla {

struct KLastParams {
  const void* A_log; int alog_dtype;
  const void* a; const void* dt_bias; int dt_bias_is_f32;
  float gate_p0;            // softplus_beta or lower_bound
  float softplus_threshold; int gate_mode;
  const void* q; const void* k; const void* v; const void* b; int beta_is_activated;
  void* o; void* h0; const int32_t* cu_seqlens; void* cache;   // pools of state_t
  const int32_t* h0_indices; const int32_t* cache_indices; int cache_steps;
  const int64_t* parents; int64_t stride_parent_seq, stride_parent_token;
  float scale; int T_max;
  int64_t stride_a, stride_q, stride_k, stride_v, stride_b, h0_slot_stride;
  int B, H, HV;
  int use_qk_l2norm, disable_state_update;
  const int32_t* num_accepted; int64_t stride_h0_indices_seq; int is_sglang;
  int tuned_kernel;         // host only: which rows of the tuned table apply (TunedKernel)
};

// READONCE > 0 (verify of up to READONCE = 4 or 8 draft tokens that writes no state, no snapshots and follows no
// tree): the recurrence is unrolled algebraically instead of being stepped through the state (readonce_verify.h):
// wavefront w of the workgroup works out the effective queries w_t and the coefficients c_{.,t} of tokens w and
// w + 4 from K-vectors and publishes them in LDS; the state tile is then used once, as the MFMA A operand of
// S_0 [w_0 .. w_{T-1}].  One workgroup covers a whole tile: RPW is 32 and wavefront w owns rows
// 32 w .. 32 w + 31 as two 16-row MFMA tiles.
template <typename act_t, bool IS_KDA, bool MTP, int RPW, int READONCE = 0, typename state_t = float>
__global__ __launch_bounds__(256) void k_last_kernel(const KLastParams p) {
  state_t* const pool = reinterpret_cast<state_t*>(p.h0);
  state_t* const snapshots = reinterpret_cast<state_t*>(p.cache);
  constexpr int R = RPW / 2;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int half = lane >> 5;
  const int c = lane & 31;
  const int i_n = blockIdx.x / p.HV;
  const int i_hv = blockIdx.x - i_n * p.HV;
  const int i_h = i_hv / (p.HV / p.H);
  const int rowbase = (blockIdx.y * 4 + wave) * RPW;

  // the request's slot is requested together with its offsets: independent loads, one trip to memory instead of two
  // on the path to the tile's address
  int h0_direct = -1;
  if (p.h0_indices != nullptr && p.stride_h0_indices_seq <= 0) h0_direct = p.h0_indices[i_n];
  int bos, T;
  if (p.cu_seqlens != nullptr) {
    bos = p.cu_seqlens[i_n];
    T = p.cu_seqlens[i_n + 1] - bos;
  } else {
    bos = i_n * p.T_max;
    T = p.T_max;
  }
  // Empty requests touch no tile and write nothing.
  if (bos < 0 || T <= 0 || T > p.T_max) return;

  act_t* const o_base = reinterpret_cast<act_t*>(p.o) + ((int64_t)bos * p.HV + i_hv) * 128 + rowbase;
  int h0_idx = -1;
  if (p.h0_indices != nullptr) {
    if (p.stride_h0_indices_seq > 0) {
      const int accepted = (p.num_accepted != nullptr) ? p.num_accepted[i_n] : 1;
      const int col = accepted > 0 ? accepted - 1 : 0;
      h0_idx = p.h0_indices[(int64_t)i_n * p.stride_h0_indices_seq + col];
    } else {
      h0_idx = h0_direct;
    }
    if (p.is_sglang ? (h0_idx < 0) : (h0_idx <= 0)) {
      float z[R];
#pragma unroll
      for (int j = 0; j < R; ++j) z[j] = 0.f;
      for (int t = 0; t < T; ++t) store_row_scalars<act_t, RPW>(o_base + (int64_t)t * p.HV * 128, lane, z);
      return;
    }
  }

  const bool have_state = p.h0 != nullptr && h0_idx >= 0;
  const int64_t tile_off = (int64_t)i_hv * 16384;                 // tile of this head inside a slot
  const int lane_off = ((rowbase + half) * 128 + 4 * c) * 4;      // bytes inside the tile
  const Tile<state_t> h_tile(have_state ? pool + (int64_t)h0_idx * p.h0_slot_stride + tile_off : nullptr, have_state);

  int cidx = -1;
  if (MTP && p.cache != nullptr && p.cache_indices != nullptr) cidx = p.cache_indices[i_n];

  // Per-head constants and the first token's activations are requested BEFORE the
  // state tile and decoded after it: memory returns in issue order, so the gate /
  // norm math of the token starts while the sixteen tile loads are still in flight.
  const bool log_decay = p.gate_mode == PLA_GATE_LOG_DECAY;
  const bool dt_wide = p.dt_bias_is_f32 != 0;
  const bool beta_wide = p.beta_is_activated != 0;
  const void* const alog_src = log_decay ? p.a : p.A_log;          // any valid address when unused
  const void* const dt_src = log_decay ? p.a : p.dt_bias;
  const RawScalar alog_raw = fetch_scalar(alog_src, !log_decay && p.alog_dtype == PLA_F32, log_decay ? 0 : i_hv);
  RawK4 dt_raw_k4{make_uint2(0, 0), make_uint2(0, 0)};
  RawScalar dt_raw{0, 0};
  if constexpr (IS_KDA) {
    dt_raw_k4 = fetch_k4(reinterpret_cast<const char*>(dt_src) + (log_decay ? 0 : (int64_t)i_hv * 128 * (dt_wide ? 4 : 2)),
                         dt_wide || log_decay, log_decay ? 0 : c);
  } else {
    dt_raw = fetch_scalar(dt_src, dt_wide || log_decay, log_decay ? 0 : i_hv);
  }
  const act_t* const qp = reinterpret_cast<const act_t*>(p.q) + i_h * 128 + 4 * c;
  const act_t* const kp = reinterpret_cast<const act_t*>(p.k) + i_h * 128 + 4 * c;
  const act_t* const vp = reinterpret_cast<const act_t*>(p.v) + i_hv * 128 + rowbase;
  const int a_esz = log_decay ? 4 : 2;

  // Raw inputs of one token (decoded at use, so that issuing them never waits).
  struct TokenIn {
    uint2 qw, kw;
    RawK4 a4;            // KDA gate input, four channels
    RawScalar a1;        // GDN gate input
    RawScalar b1;        // beta input
    uint32_t vw[R];
  };
  auto fetch = [&](int t) {
    TokenIn in{};
    const int64_t tok = (int64_t)bos + t;
    in.qw = *reinterpret_cast<const uint2*>(qp + tok * p.stride_q);
    in.kw = *reinterpret_cast<const uint2*>(kp + tok * p.stride_k);
    in.a4 = RawK4{make_uint2(0, 0), make_uint2(0, 0)};
    in.a1 = RawScalar{0, 0};
    if constexpr (IS_KDA) {
      in.a4 = fetch_k4(reinterpret_cast<const char*>(p.a) + (tok * p.stride_a + (int64_t)i_hv * 128) * a_esz, log_decay, c);
    } else {
      in.a1 = fetch_scalar(p.a, log_decay, tok * p.stride_a + i_hv);
    }
    in.b1 = fetch_scalar(p.b, beta_wide, tok * p.stride_b + i_hv);
    if constexpr (READONCE == 0) load_row_words<RPW>(vp + tok * p.stride_v, in.vw);
    return in;
  };

  TokenIn cur = fetch(0);
  // read-once verify: wavefront w takes tokens w and w + 4; they are requested ahead of the state tile, so that
  // the K-vector algebra runs while the tile is in flight (memory returns in issue order).  Tokens the request
  // does not have repeat its last one (their results are never stored).
  constexpr int TM = READONCE > 0 ? READONCE : 1;      // draft tokens the read-once verify is built for
  // Windows of more than four tokens keep fewer values in registers next to the tile in flight (each step's K-vectors
  // re-read from LDS, the query operands read per contraction step, v requested after half of the products): 188 ->
  // 120 registers, four wavefronts per SIMD instead of two (B = 64: 5 tokens 41.7 -> 37.7 us, 8 tokens 42.2 -> 38.8 us).
  // The four-token kernel is faster as it is (31.5 us against 32.8).
  constexpr bool LEAN = TM > 4;
  constexpr int NT = TM > 4 ? TM / 4 : 1;              // tokens per wavefront
  TokenIn mine[NT];
  if constexpr (READONCE > 0) {
#pragma unroll
    for (int u = 0; u < NT; ++u) mine[u] = fetch(min(wave + 4 * u, T - 1));
  }
  float s[R][4];
  // read-once verify: the tile in MFMA A-operand layout, lane (r16, kb) holds eight elements of row 32 w + 16 m + r16
  // per contraction step ks
  const int r16 = lane & 15, kb = lane >> 4;
  constexpr bool POOL_BF16 = sizeof(state_t) == 2;      // a bf16 tile is an MFMA operand as it is
  f32x4_t sa[2][4][2];
  bf16x8_t sb16[2][4];
  uint2 vq[2][TM];
  if constexpr (READONCE > 0) {
    static_assert(READONCE == 0 || RPW == 32, "the read-once verify covers a whole tile per workgroup");
    static_assert(READONCE == 0 || READONCE == 4 || READONCE == 8, "the read-once verify is built for 4 or 8 draft tokens");
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        // bf16 pool: the lane's eight elements 32 ks + 8 kb .. + 7 are 16 contiguous bytes.  FP32 pool: two loads of
        // 16 bytes, elements 32 ks + 4 kb .. + 3 and 32 ks + 16 + 4 kb .. + 3, so that the four lanes of a row read 64
        // contiguous bytes per instruction
        const int at = ((rowbase + 16 * m + r16) * 128 + 32 * ks + (POOL_BF16 ? 8 : 4) * kb) * (int)sizeof(state_t);
        if constexpr (POOL_BF16) {
          // (an absent state is a tile of no bytes: its loads return zero)
          // (no non-temporal hint, as for the FP32 tile below: consecutive contraction steps take pieces of the same lines)
          sb16[m][ks] = __builtin_bit_cast(bf16x8_t, __builtin_amdgcn_raw_buffer_load_b128(h_tile.rsrc, at, 0, 0));
        } else {
#pragma unroll
          for (int hf = 0; hf < 2; ++hf)
            // (no non-temporal hint here: the two loads of a contraction step take the two halves of the same 128-byte
            // lines, and the second finds them in the vector cache; B = 128: 60.4 -> 57.7 us, B = 64: 31.4 -> 31.2)
            sa[m][ks][hf] = __builtin_bit_cast(f32x4_t, __builtin_amdgcn_raw_buffer_load_b128(h_tile.rsrc, at + 64 * hf, 0, 0));
        }
      }
    if constexpr (!LEAN) {
      // v of every token for the lane's output rows 16 m + 4 kb .. + 3 (absent tokens repeat the last one)
  #pragma unroll
      for (int m = 0; m < 2; ++m)
  #pragma unroll
        for (int t = 0; t < TM; ++t)
          vq[m][t] = *reinterpret_cast<const uint2*>(reinterpret_cast<const act_t*>(p.v) + i_hv * 128 + rowbase + 16 * m + 4 * kb +
                                                     ((int64_t)bos + min(t, T - 1)) * p.stride_v);
    }
  } else if (have_state) {
    load_state<R>(h_tile, lane_off, s);
  } else {
#pragma unroll
    for (int j = 0; j < R; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) s[j][e] = 0.f;
  }

  // (decoded whether it is used or not, both halves named as used here: under `if (!log_decay)`, or for the half
  // that only an FP32 A_log has, the compiler moves the load itself into that branch, behind the tile loads, where
  // waiting for it means waiting for the whole tile)
  RawScalar alog_here = alog_raw;
  asm volatile("" : "+v"(alog_here.lo), "+v"(alog_here.hi));
  const float eA_any = __expf(decode_scalar(alog_here, p.alog_dtype));
  const float eA = log_decay ? 0.f : eA_any;
  float dt[4] = {0.f, 0.f, 0.f, 0.f};
  float dt_scalar = 0.f;
  if constexpr (IS_KDA) decode_k4<act_t>(dt_raw_k4, dt_wide || log_decay, dt);
  else dt_scalar = decode_scalar_act<act_t>(dt_raw, dt_wide || log_decay);

  if constexpr (READONCE > 0) {
    __shared__ __align__(16) float sW[TM][128];    // effective queries w_t
    __shared__ __align__(16) float sC[TM][TM];     // sC[t][j] = c_{j,t}
    __shared__ __align__(16) float sK[TM][128];    // normalised keys
    __shared__ __align__(16) float sD[TM][128];    // decays exp(g)
    __shared__ float sB[TM];                       // activated beta
    // each wavefront prepares the K-vectors of its own tokens once and shares them through LDS (every wavefront
    // working them out for every token cost four times the instructions)
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      const int t = wave + 4 * u;
      const TokenIn& in = mine[u];
      const float k4[4] = {lo16<act_t>(in.kw.x), hi16<act_t>(in.kw.x), lo16<act_t>(in.kw.y), hi16<act_t>(in.kw.y)};
      float kn = 1.f;
      if (p.use_qk_l2norm) {
        float ks = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) ks = fmaf(k4[e], k4[e], ks);
        kn = fast_rsqrt(row32_allreduce(ks) + 1e-6f);
      }
      float d4[4];
      if constexpr (IS_KDA) {
        float av[4];
        decode_k4<act_t>(in.a4, log_decay, av);
#pragma unroll
        for (int e = 0; e < 4; ++e)
          d4[e] = gate_decay(av[e], dt[e], eA, p.gate_p0, p.softplus_threshold, p.gate_mode);
      } else {
        const float d1 = gate_decay(decode_scalar_act<act_t>(in.a1, log_decay), dt_scalar, eA, p.gate_p0,
                                    p.softplus_threshold, p.gate_mode);
#pragma unroll
        for (int e = 0; e < 4; ++e) d4[e] = d1;
      }
      const float b_in = decode_scalar_act<act_t>(in.b1, beta_wide);
      if (half == 0) {
        *reinterpret_cast<float4*>(&sK[t][4 * c]) = make_float4(k4[0] * kn, k4[1] * kn, k4[2] * kn, k4[3] * kn);
        *reinterpret_cast<float4*>(&sD[t][4 * c]) = make_float4(d4[0], d4[1], d4[2], d4[3]);
      }
      if (lane == 0) sB[t] = beta_wide ? b_in : fast_sigmoid(b_in);
    }
    __syncthreads();
    // wavefront w: effective queries w_t and bias coefficients c_{j,t} of tokens t = w and t = w + 4
#pragma unroll
    for (int t = 0; t < TM; ++t) {
      if (wave != (t & 3)) continue;
      const TokenIn& in = mine[t >> 2];
      const float q4[4] = {lo16<act_t>(in.qw.x), hi16<act_t>(in.qw.x), lo16<act_t>(in.qw.y), hi16<act_t>(in.qw.y)};
      float qn = p.scale;
      if (p.use_qk_l2norm) {
        float qs = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e) qs = fmaf(q4[e], q4[e], qs);
        qn = fast_rsqrt(row32_allreduce(qs) + 1e-6f) * p.scale;
      }
      float w[4] = {q4[0] * qn, q4[1] * qn, q4[2] * qn, q4[3] * qn};
      float cf[TM];
      if constexpr (LEAN) {
        // the recurrence of effective_query (readonce_verify.h), each step's key, decay and beta read from LDS when the
        // step needs them: held in registers for the whole window they cost eight registers per token next to the tile
        // in flight
  #pragma unroll
        for (int j = TM - 1; j >= 0; --j) {
          cf[j] = 0.f;
          if (j > t) continue;                       // tokens after t do not enter w_t
          const float4 k4 = *reinterpret_cast<const float4*>(&sK[j][4 * c]);
          const float4 d4 = *reinterpret_cast<const float4*>(&sD[j][4 * c]);
          const float kj[4] = {k4.x, k4.y, k4.z, k4.w}, dj[4] = {d4.x, d4.y, d4.z, d4.w};
          float dot = 0.f;
  #pragma unroll
          for (int e = 0; e < 4; ++e) dot = fmaf(kj[e], w[e], dot);
          cf[j] = sB[j] * row32_allreduce(dot);
  #pragma unroll
          for (int e = 0; e < 4; ++e) w[e] = dj[e] * fmaf(-cf[j], kj[e], w[e]);
        }
      } else {
        float kv[TM][4], dec[TM][4], beta[TM];
  #pragma unroll
        for (int j = 0; j < TM; ++j) {
          // tokens after t do not enter w_t; the request's tokens before t are all present
          const float4 k4 = j <= t ? *reinterpret_cast<const float4*>(&sK[j][4 * c]) : make_float4(0.f, 0.f, 0.f, 0.f);
          const float4 d4 = j <= t ? *reinterpret_cast<const float4*>(&sD[j][4 * c]) : make_float4(0.f, 0.f, 0.f, 0.f);
          kv[j][0] = k4.x; kv[j][1] = k4.y; kv[j][2] = k4.z; kv[j][3] = k4.w;
          dec[j][0] = d4.x; dec[j][1] = d4.y; dec[j][2] = d4.z; dec[j][3] = d4.w;
          beta[j] = j <= t ? sB[j] : 0.f;
        }
        effective_query<TM>(t, w, kv, dec, beta, cf);
      }
      if (half == 0) *reinterpret_cast<float4*>(&sW[t][4 * c]) = make_float4(w[0], w[1], w[2], w[3]);
      if (lane == 0) {
#pragma unroll
        for (int j4 = 0; j4 < TM; j4 += 4)
          *reinterpret_cast<float4*>(&sC[t][j4]) = make_float4(cf[j4], cf[j4 + 1], cf[j4 + 2], cf[j4 + 3]);
      }
    }
    __syncthreads();
    // B operands: column r16 of [w_0 .. w_{TM-1} 0 .. 0]
    const int tcol = min(r16, TM - 1);
    const float keep = r16 < TM ? 1.f : 0.f;
    float cs[TM];
#pragma unroll
    for (int j4 = 0; j4 < TM; j4 += 4) {
      const float4 cmine = *reinterpret_cast<const float4*>(&sC[tcol][j4]);
      cs[j4] = cmine.x; cs[j4 + 1] = cmine.y; cs[j4 + 2] = cmine.z; cs[j4 + 3] = cmine.w;
    }
    f32x4_t accs[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    if constexpr (POOL_BF16) {
      HiLo wb[4];
      query_operands(sW, tcol, keep, kb, wb);
      if constexpr (LEAN) {
  #pragma unroll
        for (int m = 0; m < 2; ++m)
  #pragma unroll
          for (int t = 0; t < TM; ++t)
            vq[m][t] = *reinterpret_cast<const uint2*>(reinterpret_cast<const act_t*>(p.v) + i_hv * 128 + rowbase + 16 * m + 4 * kb +
                                                       ((int64_t)bos + min(t, T - 1)) * p.stride_v);
      }
#pragma unroll
      for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          accs[m] = mfma16(sb16[m][ks], wb[ks].hi, accs[m]);
          accs[m] = mfma16(sb16[m][ks], wb[ks].lo, accs[m]);
        }
    } else {
      // An FP32 tile goes through the FP32 MFMA as it is (v_mfma_f32_16x16x4_f32: lane (r16, kb) supplies one
      // element of row r16 for contraction slot kb, here its own element 32 ks + 16 hf + 4 kb + e), so neither the
      // tile nor the queries are split into 16-bit pairs: 64 matrix instructions per wavefront instead of 24, but
      // about 300 vector instructions fewer, and the products are exact.  The two row blocks alternate, so that
      // consecutive instructions never wait for the same accumulator.
      if constexpr (LEAN) {
  #pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          // (columns beyond the window repeat its last token: every column of the product depends on its own column
          // of the queries only, and those columns are never stored)
          const float4 w0 = *reinterpret_cast<const float4*>(&sW[tcol][32 * ks + 4 * kb]);
          const float4 w1 = *reinterpret_cast<const float4*>(&sW[tcol][32 * ks + 16 + 4 * kb]);
          const float wq[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
  #pragma unroll
          for (int hf = 0; hf < 2; ++hf)
  #pragma unroll
            for (int e = 0; e < 4; ++e)
  #pragma unroll
              for (int m = 0; m < 2; ++m)
                accs[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(sa[m][ks][hf][e], wq[4 * hf + e], accs[m], 0, 0, 0);
          if (ks == 1) {
            // v of every token for the lane's output rows 16 m + 4 kb .. + 3 (absent tokens repeat the last one), requested
            // where half of the tile's registers are free again
  #pragma unroll
            for (int m = 0; m < 2; ++m)
  #pragma unroll
              for (int t = 0; t < TM; ++t)
                vq[m][t] = *reinterpret_cast<const uint2*>(reinterpret_cast<const act_t*>(p.v) + i_hv * 128 + rowbase + 16 * m + 4 * kb +
                                                           ((int64_t)bos + min(t, T - 1)) * p.stride_v);
          }
        }
      } else {
        float wq[4][8];
  #pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
          const float4 w0 = *reinterpret_cast<const float4*>(&sW[tcol][32 * ks + 4 * kb]);
          const float4 w1 = *reinterpret_cast<const float4*>(&sW[tcol][32 * ks + 16 + 4 * kb]);
          // (columns beyond the window repeat its last token: every column of the product depends on its own column
          // of the queries only, and those columns are never stored)
          wq[ks][0] = w0.x; wq[ks][1] = w0.y; wq[ks][2] = w0.z; wq[ks][3] = w0.w;
          wq[ks][4] = w1.x; wq[ks][5] = w1.y; wq[ks][6] = w1.z; wq[ks][7] = w1.w;
        }
  #pragma unroll
        for (int ks = 0; ks < 4; ++ks)
  #pragma unroll
          for (int hf = 0; hf < 2; ++hf)
  #pragma unroll
            for (int e = 0; e < 4; ++e)
  #pragma unroll
              for (int m = 0; m < 2; ++m)
                accs[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(sa[m][ks][hf][e], wq[ks][4 * hf + e], accs[m], 0, 0, 0);
      }
    }
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      const f32x4_t acc = accs[m];
      // lane (r16 = token, kb): rows 16 m + 4 kb .. + 3 of S_0 w_token; add the bias terms
      float o[4] = {acc[0], acc[1], acc[2], acc[3]};
#pragma unroll
      for (int j = 0; j < TM; ++j) {
        o[0] = fmaf(cs[j], lo16<act_t>(vq[m][j].x), o[0]);
        o[1] = fmaf(cs[j], hi16<act_t>(vq[m][j].x), o[1]);
        o[2] = fmaf(cs[j], lo16<act_t>(vq[m][j].y), o[2]);
        o[3] = fmaf(cs[j], hi16<act_t>(vq[m][j].y), o[3]);
      }
      if (r16 < TM && r16 < T)
        *reinterpret_cast<uint2*>(o_base + (int64_t)r16 * p.HV * 128 + 16 * m + 4 * kb) =
            make_uint2(pack2<act_t>(o[0], o[1]), pack2<act_t>(o[2], o[3]));
    }
    return;
  }

  const int steps = MTP ? T : 1;
  for (int t = 0; t < steps; ++t) {
    // Next token's activations are requested before this token's arithmetic.
    TokenIn nxt = cur;
    if (MTP && t + 1 < steps) nxt = fetch(t + 1);

    float qv[4] = {lo16<act_t>(cur.qw.x), hi16<act_t>(cur.qw.x), lo16<act_t>(cur.qw.y), hi16<act_t>(cur.qw.y)};
    float kv[4] = {lo16<act_t>(cur.kw.x), hi16<act_t>(cur.kw.x), lo16<act_t>(cur.kw.y), hi16<act_t>(cur.kw.y)};
    float qn = p.scale, kn = 1.f;
    if (p.use_qk_l2norm) {
      float qs = 0.f, ks = 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) { qs = fmaf(qv[e], qv[e], qs); ks = fmaf(kv[e], kv[e], ks); }
      qn = fast_rsqrt(row32_allreduce(qs) + 1e-6f) * p.scale;
      kn = fast_rsqrt(row32_allreduce(ks) + 1e-6f);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) { qv[e] *= qn; kv[e] *= kn; }

    float dec[4] = {1.f, 1.f, 1.f, 1.f};
    float dec_scalar = 1.f;
    if constexpr (IS_KDA) {
      float av[4];
      decode_k4<act_t>(cur.a4, log_decay, av);
#pragma unroll
      for (int e = 0; e < 4; ++e)
        dec[e] = gate_decay(av[e], dt[e], eA, p.gate_p0, p.softplus_threshold, p.gate_mode);
    } else {
      dec_scalar = gate_decay(decode_scalar_act<act_t>(cur.a1, log_decay), dt_scalar, eA, p.gate_p0,
                              p.softplus_threshold, p.gate_mode);
    }
    const float b_in = decode_scalar_act<act_t>(cur.b1, beta_wide);
    const float beta = beta_wide ? b_in : fast_sigmoid(b_in);
    float vv[R];
    row_scalars<act_t, RPW>(cur.vw, half, vv);

    if constexpr (MTP) {
      // Eagle tree: continue from the snapshot of the parent step when it is not t-1.
      if (p.parents != nullptr && t != 0 && cidx >= 0) {
        const int64_t parent = p.parents[(int64_t)i_n * p.stride_parent_seq + (int64_t)t * p.stride_parent_token];
        if (parent >= 0 && parent < t && parent != t - 1) {
          __threadfence();   // the snapshot was written by these same lanes at step `parent`
          const Tile<state_t> parent_tile(snapshots + ((int64_t)cidx * p.cache_steps + parent) * p.HV * 16384 + tile_off);
          load_state<R>(parent_tile, lane_off, s);
        }
      }
    }

    float outv[R];
    delta_rows<R, IS_KDA, true>(s, dec, dec_scalar, kv, qv, vv, beta, outv);

    if constexpr (MTP) {
      state_t* snap = nullptr;
      if (p.is_sglang) {
        if (p.cache != nullptr && cidx >= 0)
          snap = snapshots + ((int64_t)cidx * p.cache_steps + t) * p.HV * 16384 + tile_off;
      } else if (p.stride_h0_indices_seq > 0 && p.h0_indices != nullptr && p.h0 != nullptr) {
        const int step_slot = p.h0_indices[(int64_t)i_n * p.stride_h0_indices_seq + t];
        if (step_slot > 0) snap = pool + (int64_t)step_slot * p.h0_slot_stride + tile_off;
      }
      if (snap != nullptr) store_state<R>(Tile<state_t>(snap), lane_off, s);
    }
    store_row_scalars<act_t, RPW>(o_base + (int64_t)t * p.HV * 128, lane, outv);
    cur = nxt;
  }

  if (have_state && !p.disable_state_update) store_state<R>(h_tile, lane_off, s);
}

// ---- one-token decode, common case -------------------------------------------------------
// Lean specialisation used when the call is a plain T = 1 decode with float32 A_log, a
// softplus gate and activation-typed dt_bias / beta logits (what serving issues every
// step).  Same arithmetic and lane layout as k_last_kernel; the run-time generality
// (token loops, snapshots, gate / dtype variants) is compiled out, which shortens the
// instruction stream per wave by about a third.
struct DecodeParams {
  const float* A_log; const void* a; const void* dt_bias; const void* q; const void* k; const void* v;
  const void* b; void* o; void* h0; const int32_t* cu_seqlens; const int32_t* h0_indices;
  float softplus_beta, softplus_threshold, scale;
  int64_t stride_a, stride_q, stride_k, stride_v, stride_b, h0_slot_stride;
  int H, HV, use_qk_l2norm, is_sglang;
};

template <typename act_t, bool IS_KDA, int RPW, typename state_t = float>
__global__ __launch_bounds__(256) void k_last_decode_kernel(const DecodeParams p) {
  constexpr int R = RPW / 2;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int half = lane >> 5;
  const int c = lane & 31;
  const int i_n = blockIdx.x / p.HV;
  const int i_hv = blockIdx.x - i_n * p.HV;
  const int i_h = i_hv / (p.HV / p.H);
  const int rowbase = (blockIdx.y * 4 + wave) * RPW;

  int tok = i_n;
  if (p.cu_seqlens != nullptr) {
    tok = p.cu_seqlens[i_n];
    const int T = p.cu_seqlens[i_n + 1] - tok;
    if (tok < 0 || T != 1) return;        // empty (or malformed) request: nothing is touched
  }
  const int h0_idx = p.h0_indices != nullptr ? p.h0_indices[i_n] : -1;
  act_t* const o_row = reinterpret_cast<act_t*>(p.o) + ((int64_t)tok * p.HV + i_hv) * 128 + rowbase;
  if (p.h0_indices != nullptr && (p.is_sglang ? (h0_idx < 0) : (h0_idx <= 0))) {
    float z[R];
#pragma unroll
    for (int j = 0; j < R; ++j) z[j] = 0.f;
    store_row_scalars<act_t, RPW>(o_row, lane, z);
    return;
  }
  const bool have_state = h0_idx >= 0;
  const int lane_off = ((rowbase + half) * 128 + 4 * c) * 4;
  const Tile<state_t> h_tile(have_state ? reinterpret_cast<state_t*>(p.h0) + (int64_t)h0_idx * p.h0_slot_stride + (int64_t)i_hv * 16384 : nullptr);
  float s[R][4];
  if (have_state) {
    load_state<R>(h_tile, lane_off, s);
  } else {
#pragma unroll
    for (int j = 0; j < R; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) s[j][e] = 0.f;
  }

  float qv[4], kv[4];
  load_k4(reinterpret_cast<const act_t*>(p.q) + (int64_t)tok * p.stride_q + i_h * 128, c, qv);
  load_k4(reinterpret_cast<const act_t*>(p.k) + (int64_t)tok * p.stride_k + i_h * 128, c, kv);
  uint32_t vw[R];
  load_row_words<RPW>(reinterpret_cast<const act_t*>(p.v) + (int64_t)tok * p.stride_v + i_hv * 128 + rowbase, vw);
  const float eA = __expf(p.A_log[i_hv]);
  const float beta = fast_sigmoid(to_float(reinterpret_cast<const act_t*>(p.b)[(int64_t)tok * p.stride_b + i_hv]));
  float dec[4] = {1.f, 1.f, 1.f, 1.f};
  float dec_scalar = 1.f;
  if constexpr (IS_KDA) {
    float av[4], dt[4];
    load_k4(reinterpret_cast<const act_t*>(p.a) + (int64_t)tok * p.stride_a + i_hv * 128, c, av);
    load_k4(reinterpret_cast<const act_t*>(p.dt_bias) + i_hv * 128, c, dt);
#pragma unroll
    for (int e = 0; e < 4; ++e)
      dec[e] = gate_decay(av[e], dt[e], eA, p.softplus_beta, p.softplus_threshold, PLA_GATE_SOFTPLUS);
  } else {
    dec_scalar = gate_decay(to_float(reinterpret_cast<const act_t*>(p.a)[(int64_t)tok * p.stride_a + i_hv]),
                            to_float(reinterpret_cast<const act_t*>(p.dt_bias)[i_hv]), eA,
                            p.softplus_beta, p.softplus_threshold, PLA_GATE_SOFTPLUS);
  }
  float qn = p.scale, kn = 1.f;
  if (p.use_qk_l2norm) {
    float qs = 0.f, ks = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) { qs = fmaf(qv[e], qv[e], qs); ks = fmaf(kv[e], kv[e], ks); }
    qn = fast_rsqrt(row32_allreduce(qs) + 1e-6f) * p.scale;
    kn = fast_rsqrt(row32_allreduce(ks) + 1e-6f);
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) { qv[e] *= qn; kv[e] *= kn; }
  float vv[R], outv[R];
  row_scalars<act_t, RPW>(vw, half, vv);
  delta_rows<R, IS_KDA, true>(s, dec, dec_scalar, kv, qv, vv, beta, outv);
  if (have_state) store_state<R>(h_tile, lane_off, s);
  store_row_scalars<act_t, RPW>(o_row, lane, outv);
}

struct FoldParams {
  float* h0; const void* rawv; const void* rawk; const float* gk; const float* beta;
  const int32_t* slot_idx; const int32_t* accept_lens;
  int64_t h0_slot_stride, rawv_slot_stride, rawk_slot_stride, gk_slot_stride, beta_slot_stride;
  int B, H, HV, L, null_block_id;
  // Optional: the folded state goes to final_idx[n] instead of back to the source slot; the state after
  // step track_step[n] (or after track_step[n] tokens when track_is_len) is also stored to track_idx[n];
  // records indexed by the request row instead of the slot; slots > 0 bounds every slot id.
  const int32_t* final_idx; const int32_t* track_idx; const int32_t* track_step;
  int track_is_len, records_by_request, slots;
  // blockIdx.z selects the layer: every tensor has a layer pitch (elements of its own type), or, with a
  // layer table (device memory, PLA_LAYER_TABLE_ENTRIES int64 per layer), its own base pointers.
  int64_t h0_layer_stride, rawv_layer_stride, rawk_layer_stride, gk_layer_stride, beta_layer_stride;
  const int64_t* layer_table;
};

template <typename act_t, int RPW>
__global__ __launch_bounds__(256) void kda_fold_kernel(const FoldParams p) {
  constexpr int R = RPW / 2;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int half = lane >> 5;
  const int c = lane & 31;
  const int i_n = blockIdx.x / p.HV;
  const int i_hv = blockIdx.x - i_n * p.HV;
  const int i_h = i_hv / (p.HV / p.H);
  const int rowbase = (blockIdx.y * 4 + wave) * RPW;

  const int slot = p.slot_idx[i_n];
  int n_acc = p.accept_lens[i_n];
  const int final_slot = p.final_idx != nullptr ? p.final_idx[i_n] : slot;
  const int track_slot = p.track_idx != nullptr ? p.track_idx[i_n] : p.null_block_id;
  const int track_at = p.track_idx != nullptr ? p.track_step[i_n] - (p.track_is_len ? 1 : 0) : -1;
  auto usable = [&](int id) { return id > p.null_block_id && (p.slots <= 0 || id < p.slots); };
  if (!usable(slot) || !usable(final_slot) || n_acc <= 0) return;
  if (n_acc > p.L) n_acc = p.L;
  const bool tracked = track_at >= 0 && usable(track_slot);

  // Each wavefront reads its rows of the source tile before it writes any of them, so the destinations
  // may alias the source slot.
  const int64_t layer = blockIdx.z;
  float* pool = p.h0 + layer * p.h0_layer_stride;
  int64_t h0_slot_stride = p.h0_slot_stride;
  const void* rawk = p.rawk;
  const void* rawv = p.rawv;
  const float* gk = p.gk;
  const float* beta = p.beta;
  if (p.layer_table != nullptr) {
    const int64_t* const e = p.layer_table + layer * PLA_LAYER_TABLE_ENTRIES;
    pool = reinterpret_cast<float*>(e[0]);
    h0_slot_stride = e[1];
    rawv = reinterpret_cast<const void*>(e[2]);
    rawk = reinterpret_cast<const void*>(e[3]);
    gk = reinterpret_cast<const float*>(e[4]);
    beta = reinterpret_cast<const float*>(e[5]);
  }
  const Tile<float> h_tile(pool + (int64_t)slot * h0_slot_stride + (int64_t)i_hv * 16384);
  const int lane_off = ((rowbase + half) * 128 + 4 * c) * 4;
  float s[R][4];
  load_state<R>(h_tile, lane_off, s);
  const int64_t rec = p.records_by_request ? i_n : slot;
  const act_t* const kp = reinterpret_cast<const act_t*>(rawk) + layer * p.rawk_layer_stride + rec * p.rawk_slot_stride +
                          (int64_t)i_h * p.L * 128;
  const act_t* const vp = reinterpret_cast<const act_t*>(rawv) + layer * p.rawv_layer_stride + rec * p.rawv_slot_stride +
                          (int64_t)i_hv * p.L * 128 + rowbase;
  const float* const gp = gk + layer * p.gk_layer_stride + rec * p.gk_slot_stride + (int64_t)i_hv * p.L * 128;
  const float* const bp = beta + layer * p.beta_layer_stride + rec * p.beta_slot_stride + (int64_t)i_hv * p.L;

  for (int t = 0; t < n_acc; ++t) {
    float kv[4], gv[4], dec[4], vv[R], unused[R];
    load_k4(kp + t * 128, c, kv);
    load_k4(gp + t * 128, c, gv);
    uint32_t vw[R];
    load_row_words<RPW>(vp + t * 128, vw);
    row_scalars<act_t, RPW>(vw, half, vv);
    float ks = 0.f;
#pragma unroll
    for (int e = 0; e < 4; ++e) ks = fmaf(kv[e], kv[e], ks);
    const float kn = 1.0f / sqrtf(row32_allreduce(ks) + 1e-6f);
#pragma unroll
    for (int e = 0; e < 4; ++e) { kv[e] *= kn; dec[e] = __expf(gv[e]); }
    delta_rows<R, true, false>(s, dec, 1.f, kv, kv, vv, bp[t], unused);
    if (tracked && t == track_at)
      store_state<R>(Tile<float>(pool + (int64_t)track_slot * h0_slot_stride + (int64_t)i_hv * 16384), lane_off, s);
  }
  store_state<R>(Tile<float>(pool + (int64_t)final_slot * h0_slot_stride + (int64_t)i_hv * 16384), lane_off, s);
}

// ---- host side ---------------------------------------------------------------

// gfx950 tuning table: rows of the 128-row tile owned by one wavefront, chosen
// from the number of (request, value-head) tiles so that small batches still
// spread over all 256 CUs while large batches keep 64 state VGPRs in flight.
// Measured on MI355X (packed GDN decode, HV = 32, us per step at 8 / 16 / 32 rows per wavefront):
//   32 tiles 3.9 / 4.6 / 6.0    128 tiles 5.2 / 5.6 / 6.9     256 tiles 8.2 / 7.8 / 9.2
//   512 tiles 15.8 / 15.4 / 14.8    2048 tiles 53.5 / 53.5 / 50.9    8192 tiles 207.6 / 205.8 / 190.3
static int pick_rows_per_wave(int tiles) {
  if (tiles >= 512) return 32;
  if (tiles >= 192) return 16;
  return 8;
}
// A shape the auto-tuner has measured takes its tuned row count, every other shape the thresholds above.
static int pick_rows_per_wave(int kernel, int tree, int act_dtype, int state_dtype, int H, int HV, int B) {
  const int tuned = tuned_rows_per_wave(kTunedRows, kTunedRowCount, kernel, tree, act_dtype, state_dtype, H, HV, B);
  return tuned > 0 ? tuned : pick_rows_per_wave(B * HV);
}

template <typename act_t, bool IS_KDA, bool MTP, typename state_t>
static int launch_rpw(const KLastParams& p, int rpw, hipStream_t stream) {
  const dim3 block(256);
  const unsigned tiles = (unsigned)p.B * (unsigned)p.HV;
  if constexpr (MTP) {
    // a verify that leaves no trace in memory but o: the state is read once and used once
    const bool read_once = p.disable_state_update && p.T_max <= 8 && p.cache == nullptr && p.cache_indices == nullptr &&
                           p.parents == nullptr && p.stride_h0_indices_seq == 0;
    if (read_once) {
      if (p.T_max <= 4) hipLaunchKernelGGL((k_last_kernel<act_t, IS_KDA, true, 32, 4, state_t>), dim3(tiles, 1), block, 0, stream, p);
      else hipLaunchKernelGGL((k_last_kernel<act_t, IS_KDA, true, 32, 8, state_t>), dim3(tiles, 1), block, 0, stream, p);
      return check_launch("k_last_kernel launch");
    }
  }
  switch (rpw) {
    case 32: hipLaunchKernelGGL((k_last_kernel<act_t, IS_KDA, MTP, 32, 0, state_t>), dim3(tiles, 1), block, 0, stream, p); break;
    case 16: hipLaunchKernelGGL((k_last_kernel<act_t, IS_KDA, MTP, 16, 0, state_t>), dim3(tiles, 2), block, 0, stream, p); break;
    case 8:  hipLaunchKernelGGL((k_last_kernel<act_t, IS_KDA, MTP, 8, 0, state_t>),  dim3(tiles, 4), block, 0, stream, p); break;
    default: return fail("rows_per_wave must be 0, 8, 16 or 32, got %d", rpw);
  }
  return check_launch("k_last_kernel launch");
}

template <typename act_t, typename state_t>
static int launch_flags(const KLastParams& p, bool is_kda, bool mtp, int rpw, hipStream_t stream) {
  if (is_kda) return mtp ? launch_rpw<act_t, true, true, state_t>(p, rpw, stream) : launch_rpw<act_t, true, false, state_t>(p, rpw, stream);
  return mtp ? launch_rpw<act_t, false, true, state_t>(p, rpw, stream) : launch_rpw<act_t, false, false, state_t>(p, rpw, stream);
}

static int check_common(int B, int H, int HV, int K, int V, int act_dtype, int alog_dtype, int T_max) {
  PLA_REQUIRE(K == 128 && V == 128, "k-last kernels require head_dim K == V == 128, got K=%d, V=%d", K, V);
  PLA_REQUIRE(B > 0, "k-last requires at least one sequence");
  PLA_REQUIRE(H > 0 && HV >= H && HV % H == 0, "HV must be a positive multiple of H, got H=%d, HV=%d", H, HV);
  PLA_REQUIRE(act_dtype == PLA_BF16 || act_dtype == PLA_F16, "activation dtype must be bf16 or fp16");
  PLA_REQUIRE(alog_dtype == PLA_F32 || alog_dtype == PLA_BF16 || alog_dtype == PLA_F16, "A_log dtype must be fp32, bf16 or fp16");
  PLA_REQUIRE(T_max >= 1, "T_max must be positive");
  PLA_REQUIRE((int64_t)B * HV <= 0x7fffffffLL, "B*HV exceeds the grid limit");
  return 0;
}

static bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

template <typename act_t, bool IS_KDA, typename state_t>
static int launch_decode(const DecodeParams& d, unsigned tiles, int rpw, hipStream_t stream) {
  const dim3 block(256);
  switch (rpw) {
    case 32: hipLaunchKernelGGL((k_last_decode_kernel<act_t, IS_KDA, 32, state_t>), dim3(tiles, 1), block, 0, stream, d); break;
    case 16: hipLaunchKernelGGL((k_last_decode_kernel<act_t, IS_KDA, 16, state_t>), dim3(tiles, 2), block, 0, stream, d); break;
    case 8:  hipLaunchKernelGGL((k_last_decode_kernel<act_t, IS_KDA, 8, state_t>),  dim3(tiles, 4), block, 0, stream, d); break;
    default: return fail("rows_per_wave must be 0, 8, 16 or 32, got %d", rpw);
  }
  return check_launch("k_last_decode_kernel launch");
}

template <typename state_t>
static int run_k_last_typed(const KLastParams& p, bool is_kda, bool mtp, int act_dtype, int rows_per_wave, void* stream) {
  const int rpw = rows_per_wave > 0 ? rows_per_wave
                                    : pick_rows_per_wave(p.tuned_kernel, p.parents != nullptr, act_dtype,
                                                         std::is_same<state_t, float>::value ? PLA_F32 : PLA_BF16,
                                                         p.H, p.HV, p.B);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const bool lean = !mtp && p.T_max == 1 && p.alog_dtype == PLA_F32 && p.gate_mode == PLA_GATE_SOFTPLUS &&
                    !p.dt_bias_is_f32 && !p.beta_is_activated && p.h0 != nullptr;
  if (lean) {
    DecodeParams d{reinterpret_cast<const float*>(p.A_log), p.a, p.dt_bias, p.q, p.k, p.v, p.b, p.o, p.h0,
                   p.cu_seqlens, p.h0_indices, p.gate_p0, p.softplus_threshold, p.scale,
                   p.stride_a, p.stride_q, p.stride_k, p.stride_v, p.stride_b, p.h0_slot_stride,
                   p.H, p.HV, p.use_qk_l2norm, p.is_sglang};
    const unsigned tiles = (unsigned)p.B * (unsigned)p.HV;
    if (act_dtype == PLA_BF16)
      return is_kda ? launch_decode<bf16_t, true, state_t>(d, tiles, rpw, s) : launch_decode<bf16_t, false, state_t>(d, tiles, rpw, s);
    return is_kda ? launch_decode<f16_t, true, state_t>(d, tiles, rpw, s) : launch_decode<f16_t, false, state_t>(d, tiles, rpw, s);
  }
  if (act_dtype == PLA_BF16) return launch_flags<bf16_t, state_t>(p, is_kda, mtp, rpw, s);
  return launch_flags<f16_t, state_t>(p, is_kda, mtp, rpw, s);
}
static int run_k_last(const KLastParams& p, bool is_kda, bool mtp, int act_dtype, int state_dtype, int rows_per_wave,
                      void* stream) {
  return state_dtype == PLA_BF16 ? run_k_last_typed<bf16_t>(p, is_kda, mtp, act_dtype, rows_per_wave, stream)
                                 : run_k_last_typed<float>(p, is_kda, mtp, act_dtype, rows_per_wave, stream);
}
// Pool base and slot pitch: four elements (16 bytes FP32, 8 bytes bf16).
static int check_pool(const void* h0, int state_dtype, int64_t h0_slot_stride, int HV, size_t base_align) {
  PLA_REQUIRE(state_dtype == PLA_F32 || state_dtype == PLA_BF16, "state dtype must be float32 or bfloat16");
  PLA_REQUIRE(aligned(h0, base_align) && h0_slot_stride % 4 == 0, "state base and slot pitch require 16-byte alignment");
  PLA_REQUIRE(h0_slot_stride >= (int64_t)HV * 16384, "state slot pitch must cover HV*V*K");
  return 0;
}

}  // namespace pla

using namespace pla;

extern "C" int pla_k_last_packed_launch(
    const void* A_log, int alog_dtype, const void* a, const void* dt_bias,
    float softplus_beta, float softplus_threshold,
    const void* mixed_qkv, const void* b, void* o, void* h0, int state_dtype,
    const int32_t* cu_seqlens, const int32_t* h0_indices,
    float scale, int T_max,
    int64_t stride_a, int64_t stride_qkv, int64_t stride_b, int64_t h0_slot_stride,
    int B, int H, int HV, int K, int V,
    int use_qk_l2norm, int is_sglang, int is_kda, int act_dtype,
    int rows_per_wave, void* stream) {
  if (check_common(B, H, HV, K, V, act_dtype, alog_dtype, T_max)) return 1;
  PLA_REQUIRE(T_max == 1, "packed decode handles one token per request (T_max == 1)");
  PLA_REQUIRE(A_log && a && dt_bias && mixed_qkv && b && o, "null tensor pointer");
  PLA_REQUIRE(h0 != nullptr, "initial_state_source is required for k_last_packed");
  PLA_REQUIRE(aligned(mixed_qkv, 16) && stride_qkv % 8 == 0, "mixed_qkv base and token stride require 16-byte alignment");
  if (check_pool(h0, state_dtype, h0_slot_stride, HV, 16)) return 1;
  PLA_REQUIRE(aligned(o, 16), "out requires 16-byte alignment");
  PLA_REQUIRE(stride_qkv >= (int64_t)(2 * H + HV) * 128, "mixed_qkv token stride must cover its complete row");
  if (is_kda) PLA_REQUIRE(aligned(a, 8) && stride_a % 4 == 0 && aligned(dt_bias, 8), "KDA a/dt_bias require 8-byte alignment");
  KLastParams p{};
  p.A_log = A_log; p.alog_dtype = alog_dtype; p.a = a; p.dt_bias = dt_bias; p.dt_bias_is_f32 = 0;
  p.gate_p0 = softplus_beta; p.softplus_threshold = softplus_threshold; p.gate_mode = PLA_GATE_SOFTPLUS;
  const size_t esz = 2;
  p.q = mixed_qkv;
  p.k = reinterpret_cast<const char*>(mixed_qkv) + (size_t)H * 128 * esz;
  p.v = reinterpret_cast<const char*>(mixed_qkv) + (size_t)2 * H * 128 * esz;
  p.b = b; p.beta_is_activated = 0; p.o = o; p.h0 = h0; p.cu_seqlens = cu_seqlens;
  p.h0_indices = h0_indices; p.scale = scale; p.T_max = 1;
  p.stride_a = stride_a; p.stride_q = p.stride_k = p.stride_v = stride_qkv; p.stride_b = stride_b;
  p.h0_slot_stride = h0_slot_stride; p.B = B; p.H = H; p.HV = HV;
  p.use_qk_l2norm = use_qk_l2norm; p.disable_state_update = 0; p.is_sglang = is_sglang;
  p.tuned_kernel = TUNED_K_LAST_PACKED;
  return run_k_last(p, is_kda != 0, false, act_dtype, state_dtype, rows_per_wave, stream);
}

extern "C" int pla_k_last_launch(
    const void* A_log, int alog_dtype, const void* a, const void* dt_bias, int dt_bias_is_f32,
    float softplus_beta_or_lower_bound, float softplus_threshold, int gate_mode,
    const void* q, const void* k, const void* v, const void* b, int beta_is_activated,
    void* o, void* h0, int state_dtype, const int32_t* cu_seqlens, void* cache,
    const int32_t* h0_indices, const int32_t* cache_indices, int cache_steps,
    const int64_t* parents, int64_t stride_parent_seq, int64_t stride_parent_token,
    float scale, int T_max,
    int64_t stride_a, int64_t stride_q, int64_t stride_k, int64_t stride_v, int64_t stride_b,
    int64_t h0_slot_stride,
    int B, int H, int HV, int K, int V,
    int use_qk_l2norm, int disable_state_update,
    const int32_t* num_accepted, int64_t stride_h0_indices_seq, int is_sglang,
    int is_kda, int act_dtype, int rows_per_wave, void* stream) {
  if (check_common(B, H, HV, K, V, act_dtype, alog_dtype, T_max)) return 1;
  PLA_REQUIRE(gate_mode >= PLA_GATE_SOFTPLUS && gate_mode <= PLA_GATE_LOG_DECAY, "unknown gate_mode %d", gate_mode);
  PLA_REQUIRE(gate_mode != PLA_GATE_LOWER_BOUND || is_kda, "lower_bound is only supported for KDA");
  PLA_REQUIRE(a && q && k && v && b && o, "null tensor pointer");
  PLA_REQUIRE(gate_mode == PLA_GATE_LOG_DECAY || (A_log && dt_bias), "A_log and dt_bias are required unless the gate is a log-decay");
  PLA_REQUIRE(aligned(q, 8) && aligned(k, 8) && aligned(v, 16) && stride_q % 4 == 0 && stride_k % 4 == 0 && stride_v % 8 == 0,
              "q/k/v base and token stride require 16-byte alignment");
  PLA_REQUIRE(aligned(o, 16), "out requires 16-byte alignment");
  PLA_REQUIRE(state_dtype == PLA_F32 || state_dtype == PLA_BF16, "state dtype must be float32 or bfloat16");
  const size_t pool_align = state_dtype == PLA_F32 ? 16 : 8;
  if (h0 && check_pool(h0, state_dtype, h0_slot_stride, HV, pool_align)) return 1;
  if (cache) PLA_REQUIRE(aligned(cache, pool_align), "intermediate cache base requires vector alignment (four elements)");
  if (cache) PLA_REQUIRE(cache_steps > 0, "intermediate cache requires a positive step pitch");
  if (is_kda) {
    const size_t need = gate_mode == PLA_GATE_LOG_DECAY ? 16 : 8;
    PLA_REQUIRE(aligned(a, need) && stride_a % 4 == 0, "KDA gate rows require vector alignment");
    if (gate_mode != PLA_GATE_LOG_DECAY)
      PLA_REQUIRE(aligned(dt_bias, dt_bias_is_f32 ? 16 : 8), "KDA dt_bias requires vector alignment");
  }
  PLA_REQUIRE(stride_h0_indices_seq == 0 || !is_sglang, "2D initial_state_indices is the vLLM spec-decode layout; pass is_sglang=False");
  PLA_REQUIRE(parents == nullptr || (cache != nullptr && cache_indices != nullptr), "retrieve_parent_token requires the intermediate cache and its indices");
  KLastParams p{};
  p.A_log = A_log; p.alog_dtype = alog_dtype; p.a = a; p.dt_bias = dt_bias; p.dt_bias_is_f32 = dt_bias_is_f32;
  p.gate_p0 = softplus_beta_or_lower_bound; p.softplus_threshold = softplus_threshold; p.gate_mode = gate_mode;
  p.q = q; p.k = k; p.v = v; p.b = b; p.beta_is_activated = beta_is_activated;
  p.o = o; p.h0 = h0; p.cu_seqlens = cu_seqlens; p.cache = cache;
  p.h0_indices = h0_indices; p.cache_indices = cache_indices; p.cache_steps = cache_steps;
  p.parents = parents; p.stride_parent_seq = stride_parent_seq; p.stride_parent_token = stride_parent_token;
  p.scale = scale; p.T_max = T_max;
  p.stride_a = stride_a; p.stride_q = stride_q; p.stride_k = stride_k; p.stride_v = stride_v; p.stride_b = stride_b;
  p.h0_slot_stride = h0_slot_stride; p.B = B; p.H = H; p.HV = HV;
  p.use_qk_l2norm = use_qk_l2norm; p.disable_state_update = disable_state_update;
  p.num_accepted = num_accepted; p.stride_h0_indices_seq = stride_h0_indices_seq; p.is_sglang = is_sglang;
  const bool mtp = T_max > 1 || disable_state_update || cache != nullptr || cache_indices != nullptr ||
                   parents != nullptr || stride_h0_indices_seq > 0;
  p.tuned_kernel = mtp ? TUNED_K_LAST_MTP : TUNED_K_LAST;
  return run_k_last(p, is_kda != 0, mtp, act_dtype, state_dtype, rows_per_wave, stream);
}

extern "C" int pla_tuned_rows_per_wave(int kernel, int tree, int act_dtype, int state_dtype, int H, int HV, int B) {
  if (kernel < TUNED_K_LAST || kernel > TUNED_K_LAST_MTP || H <= 0 || HV <= 0 || B <= 0) return 0;
  return pick_rows_per_wave(kernel, tree != 0, act_dtype, state_dtype, H, HV, B);
}

static int launch_fold(const FoldParams& p, int act_dtype, void* stream, int layers = 1) {
  PLA_REQUIRE((p.layer_table || (p.h0 && p.rawv && p.rawk && p.gk && p.beta)) && p.slot_idx && p.accept_lens, "null tensor pointer");
  PLA_REQUIRE(p.B > 0 && p.L > 0, "fold requires B > 0 and L > 0");
  PLA_REQUIRE(p.H > 0 && p.HV >= p.H && p.HV % p.H == 0, "HV must be a positive multiple of H, got H=%d, HV=%d", p.H, p.HV);
  PLA_REQUIRE(act_dtype == PLA_BF16 || act_dtype == PLA_F16, "record dtype must be bf16 or fp16");
  PLA_REQUIRE((p.track_idx == nullptr) == (p.track_step == nullptr), "track indices and steps must be given together");
  PLA_REQUIRE(p.layer_table != nullptr ||
              (aligned(p.h0, 16) && p.h0_slot_stride % 4 == 0 && aligned(p.gk, 16) && p.gk_slot_stride % 4 == 0 &&
               aligned(p.rawk, 8) && p.rawk_slot_stride % 4 == 0 && aligned(p.rawv, 16) && p.rawv_slot_stride % 8 == 0),
              "state and record tensors require 16-byte alignment");
  PLA_REQUIRE(layers >= 1 && layers <= 65535, "fold takes 1..65535 layers per launch, got %d", layers);
  PLA_REQUIRE(layers == 1 || (p.h0_layer_stride % 4 == 0 && p.gk_layer_stride % 4 == 0 && p.rawk_layer_stride % 4 == 0 &&
                              p.rawv_layer_stride % 8 == 0), "layer pitches require 16-byte alignment");
  const unsigned tiles = (unsigned)p.B * (unsigned)p.HV;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int rpw = pick_rows_per_wave((int)tiles * layers);
  const dim3 block(256);
  const unsigned z = (unsigned)layers;
  if (act_dtype == PLA_BF16) {
    if (rpw == 32) hipLaunchKernelGGL((kda_fold_kernel<bf16_t, 32>), dim3(tiles, 1, z), block, 0, s, p);
    else if (rpw == 16) hipLaunchKernelGGL((kda_fold_kernel<bf16_t, 16>), dim3(tiles, 2, z), block, 0, s, p);
    else hipLaunchKernelGGL((kda_fold_kernel<bf16_t, 8>), dim3(tiles, 4, z), block, 0, s, p);
  } else {
    if (rpw == 32) hipLaunchKernelGGL((kda_fold_kernel<f16_t, 32>), dim3(tiles, 1, z), block, 0, s, p);
    else if (rpw == 16) hipLaunchKernelGGL((kda_fold_kernel<f16_t, 16>), dim3(tiles, 2, z), block, 0, s, p);
    else hipLaunchKernelGGL((kda_fold_kernel<f16_t, 8>), dim3(tiles, 4, z), block, 0, s, p);
  }
  return check_launch("kda_fold_kernel launch");
}

extern "C" int pla_kda_fold_launch(
    float* h0, const void* rawv, const void* rawk, const float* gk, const float* beta,
    const int32_t* slot_idx, const int32_t* accept_lens,
    const int32_t* track_idx, const int32_t* track_step,
    int64_t h0_slot_stride, int64_t rawv_slot_stride, int64_t rawk_slot_stride,
    int64_t gk_slot_stride, int64_t beta_slot_stride,
    int layers, int64_t h0_layer_stride, int64_t rawv_layer_stride, int64_t rawk_layer_stride,
    int64_t gk_layer_stride, int64_t beta_layer_stride,
    int B, int H, int HV, int L, int null_block_id, int act_dtype, void* stream) {
  FoldParams p{h0, rawv, rawk, gk, beta, slot_idx, accept_lens,
               h0_slot_stride, rawv_slot_stride, rawk_slot_stride, gk_slot_stride, beta_slot_stride,
               B, H, HV, L, null_block_id, nullptr, track_idx, track_step, 0, 0, 0,
               h0_layer_stride, rawv_layer_stride, rawk_layer_stride, gk_layer_stride, beta_layer_stride};
  return launch_fold(p, act_dtype, stream, layers);
}

extern "C" int pla_kda_fold_native_launch(
    const int64_t* layer_table, int layers,
    const int32_t* source, const int32_t* lengths, const int32_t* final_indices,
    const int32_t* boundary_indices, const int32_t* boundary_lengths,
    int batch, int heads, int Q, int slots, int null_block_id, void* stream) {
  PLA_REQUIRE(layer_table && final_indices && boundary_indices && boundary_lengths, "null table or plan pointer");
  PLA_REQUIRE(slots > 0 && (null_block_id == -1 || null_block_id == 0), "paged fold requires slots > 0 and null_block_id -1 or 0");
  if (batch == 0) return 0;
  FoldParams p{nullptr, nullptr, nullptr, nullptr, nullptr, source, lengths,
               0, (int64_t)heads * Q * 128, (int64_t)heads * Q * 128, (int64_t)heads * Q * 128,
               (int64_t)heads * Q, batch, heads, heads, Q, null_block_id,
               final_indices, boundary_indices, boundary_lengths, 1, 1, slots, 0, 0, 0, 0, 0, layer_table};
  return launch_fold(p, PLA_BF16, stream, layers);
}
