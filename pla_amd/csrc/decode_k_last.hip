// k-last gated delta-rule decode, MTP verify and accepted-prefix commit for gfx950.
//
// One 128x128 FP32 state tile S[v][k] per (request, value head) is streamed from
// HBM exactly once, updated in registers and written back once.  A 64-lane
// wavefront owns RPW consecutive V-rows; inside the wave every aligned group of
// 16 lanes owns RPW/4 consecutive rows, and lane c of a group holds the K
// channels [4c,4c+4) and [64+4c,64+4c+4) of each of its rows (two 16-byte loads
// per row, each load instruction covering four 256-byte contiguous segments).
// Both reductions over K (S.k and S.q) therefore stay inside one DPP row and
// cost four v_add_f32 DPP steps; there is no LDS traffic and no barrier, so all
// state loads of a wave are in flight together.
//
// Semantics follow the reference kernels
//   src/decode/k-last/fused_sigmoid_gating_k_last_packed_kernel.cuh:59-384 (packed T=1)
//   src/decode/k-last/fused_sigmoid_gating_k_last_kernel.cuh:131-1058     (decode / MTP verify)
//   src/decode/kda_replayssm/kda_mtp_fold.cu:256-545                      (commit)
// with one deliberate difference: corrupt cu_seqlens (negative start, length
// above T_max) make the request a no-op instead of trapping the device.

#include "common.h"

namespace pla {

struct KLastParams {
  const void* A_log; int alog_dtype;
  const void* a; const void* dt_bias; int dt_bias_is_f32;
  float gate_p0;            // softplus_beta or lower_bound
  float softplus_threshold; int gate_mode;
  const void* q; const void* k; const void* v; const void* b; int beta_is_activated;
  void* o; float* h0; const int32_t* cu_seqlens; float* cache;
  const int32_t* h0_indices; const int32_t* cache_indices; int cache_steps;
  const int64_t* parents; int64_t stride_parent_seq, stride_parent_token;
  float scale; int T_max;
  int64_t stride_a, stride_q, stride_k, stride_v, stride_b, h0_slot_stride;
  int B, H, HV;
  int use_qk_l2norm, disable_state_update;
  const int32_t* num_accepted; int64_t stride_h0_indices_seq; int is_sglang;
};

__device__ __forceinline__ float load_param(const void* p, int dtype, int i) {
  if (dtype == PLA_F32) return reinterpret_cast<const float*>(p)[i];
  if (dtype == PLA_BF16) return to_float(reinterpret_cast<const bf16_t*>(p)[i]);
  return to_float(reinterpret_cast<const f16_t*>(p)[i]);
}

// The lane's eight K channels of one 128-wide activation row.
template <typename act_t>
__device__ __forceinline__ void load_k8(const act_t* row, int c, float (&x)[8]) {
  const uint2 lo = *reinterpret_cast<const uint2*>(row + 4 * c);
  const uint2 hi = *reinterpret_cast<const uint2*>(row + 64 + 4 * c);
  x[0] = lo16<act_t>(lo.x); x[1] = hi16<act_t>(lo.x); x[2] = lo16<act_t>(lo.y); x[3] = hi16<act_t>(lo.y);
  x[4] = lo16<act_t>(hi.x); x[5] = hi16<act_t>(hi.x); x[6] = lo16<act_t>(hi.y); x[7] = hi16<act_t>(hi.y);
}
__device__ __forceinline__ void load_k8(const float* row, int c, float (&x)[8]) {
  const float4 lo = *reinterpret_cast<const float4*>(row + 4 * c);
  const float4 hi = *reinterpret_cast<const float4*>(row + 64 + 4 * c);
  x[0] = lo.x; x[1] = lo.y; x[2] = lo.z; x[3] = lo.w;
  x[4] = hi.x; x[5] = hi.y; x[6] = hi.z; x[7] = hi.w;
}

// R consecutive activations (R = 2, 4 or 8) starting at p (aligned to 2R bytes).
template <typename act_t, int R>
__device__ __forceinline__ void load_rows(const act_t* p, float (&x)[R]) {
  static_assert(R == 2 || R == 4 || R == 8, "rows per lane group");
  if constexpr (R == 8) {
    const uint4 w = *reinterpret_cast<const uint4*>(p);
    x[0] = lo16<act_t>(w.x); x[1] = hi16<act_t>(w.x); x[2] = lo16<act_t>(w.y); x[3] = hi16<act_t>(w.y);
    x[4] = lo16<act_t>(w.z); x[5] = hi16<act_t>(w.z); x[6] = lo16<act_t>(w.w); x[7] = hi16<act_t>(w.w);
  } else if constexpr (R == 4) {
    const uint2 w = *reinterpret_cast<const uint2*>(p);
    x[0] = lo16<act_t>(w.x); x[1] = hi16<act_t>(w.x); x[2] = lo16<act_t>(w.y); x[3] = hi16<act_t>(w.y);
  } else {
    const uint32_t w = *reinterpret_cast<const uint32_t*>(p);
    x[0] = lo16<act_t>(w); x[1] = hi16<act_t>(w);
  }
}
template <typename act_t, int R>
__device__ __forceinline__ void store_rows(act_t* p, const float (&x)[R]) {
  if constexpr (R == 8) {
    *reinterpret_cast<uint4*>(p) = make_uint4(pack2<act_t>(x[0], x[1]), pack2<act_t>(x[2], x[3]),
                                              pack2<act_t>(x[4], x[5]), pack2<act_t>(x[6], x[7]));
  } else if constexpr (R == 4) {
    *reinterpret_cast<uint2*>(p) = make_uint2(pack2<act_t>(x[0], x[1]), pack2<act_t>(x[2], x[3]));
  } else {
    *reinterpret_cast<uint32_t*>(p) = pack2<act_t>(x[0], x[1]);
  }
}

template <int R>
__device__ __forceinline__ void load_state(const float* base, float (&s)[R][8]) {
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const float4 lo = *reinterpret_cast<const float4*>(base + j * 128);
    const float4 hi = *reinterpret_cast<const float4*>(base + j * 128 + 64);
    s[j][0] = lo.x; s[j][1] = lo.y; s[j][2] = lo.z; s[j][3] = lo.w;
    s[j][4] = hi.x; s[j][5] = hi.y; s[j][6] = hi.z; s[j][7] = hi.w;
  }
}
template <int R>
__device__ __forceinline__ void store_state(float* base, const float (&s)[R][8]) {
#pragma unroll
  for (int j = 0; j < R; ++j) {
    *reinterpret_cast<float4*>(base + j * 128) = make_float4(s[j][0], s[j][1], s[j][2], s[j][3]);
    *reinterpret_cast<float4*>(base + j * 128 + 64) = make_float4(s[j][4], s[j][5], s[j][6], s[j][7]);
  }
}

// decay -> S.k -> delta -> rank-1 update (-> S.q) on the lane group's R rows.
template <int R, bool PER_CHANNEL, bool WANT_OUT>
__device__ __forceinline__ void delta_rows(float (&s)[R][8], const float (&dec)[8], float dec_scalar,
                                           const float (&kv)[8], const float (&qv)[8],
                                           const float (&vv)[R], float beta, float (&out)[R]) {
#pragma unroll
  for (int j = 0; j < R; ++j) {
    float d = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      s[j][e] *= PER_CHANNEL ? dec[e] : dec_scalar;
      d = fmaf(s[j][e], kv[e], d);
    }
    d = row16_allreduce(d);
    const float u = (vv[j] - d) * beta;
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      s[j][e] = fmaf(u, kv[e], s[j][e]);
      if (WANT_OUT) acc = fmaf(s[j][e], qv[e], acc);
    }
    if (WANT_OUT) out[j] = row16_allreduce(acc);
  }
}

__device__ __forceinline__ float gate_decay(float a, float dt, float eA, float p0, float thr, int mode) {
  if (mode == PLA_GATE_LOG_DECAY) return __expf(a);
  const float x = a + dt;
  if (mode == PLA_GATE_LOWER_BOUND) return __expf(p0 * fast_sigmoid(eA * x));
  const float bx = p0 * x;
  const float sp = (bx <= thr) ? (1.0f / p0) * __logf(1.0f + __expf(bx)) : x;
  return __expf(-eA * sp);
}

template <typename act_t, bool IS_KDA, bool MTP, int RPW>
__global__ __launch_bounds__(256) void k_last_kernel(const KLastParams p) {
  constexpr int R = RPW / 4;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int grp = lane >> 4;
  const int c = lane & 15;
  const int i_n = blockIdx.x / p.HV;
  const int i_hv = blockIdx.x - i_n * p.HV;
  const int i_h = i_hv / (p.HV / p.H);
  const int row0 = (blockIdx.y * 4 + wave) * RPW + grp * R;

  int bos, T;
  if (p.cu_seqlens != nullptr) {
    bos = p.cu_seqlens[i_n];
    T = p.cu_seqlens[i_n + 1] - bos;
  } else {
    bos = i_n * p.T_max;
    T = p.T_max;
  }
  // Empty requests touch nothing (no slot / accepted load either).
  if (bos < 0 || T <= 0 || T > p.T_max) return;

  act_t* const o_base = reinterpret_cast<act_t*>(p.o) + ((int64_t)bos * p.HV + i_hv) * 128 + row0;
  int h0_idx = -1;
  if (p.h0_indices != nullptr) {
    if (p.stride_h0_indices_seq > 0) {
      const int accepted = (p.num_accepted != nullptr) ? p.num_accepted[i_n] : 1;
      const int col = accepted > 0 ? accepted - 1 : 0;
      h0_idx = p.h0_indices[(int64_t)i_n * p.stride_h0_indices_seq + col];
    } else {
      h0_idx = p.h0_indices[i_n];
    }
    if (p.is_sglang ? (h0_idx < 0) : (h0_idx <= 0)) {
      if (c == 0) {
        float z[R];
#pragma unroll
        for (int j = 0; j < R; ++j) z[j] = 0.f;
        for (int t = 0; t < T; ++t) store_rows<act_t, R>(o_base + (int64_t)t * p.HV * 128, z);
      }
      return;
    }
  }

  const bool have_state = p.h0 != nullptr && h0_idx >= 0;
  const int64_t tile_off = (int64_t)i_hv * 16384 + row0 * 128 + 4 * c;
  float* const h_rows = have_state ? p.h0 + (int64_t)h0_idx * p.h0_slot_stride + tile_off : nullptr;
  float s[R][8];
  if (have_state) {
    load_state<R>(h_rows, s);
  } else {
#pragma unroll
    for (int j = 0; j < R; ++j)
#pragma unroll
      for (int e = 0; e < 8; ++e) s[j][e] = 0.f;
  }

  int cidx = -1;
  if (MTP && p.cache != nullptr && p.cache_indices != nullptr) cidx = p.cache_indices[i_n];

  const float eA = (p.gate_mode == PLA_GATE_LOG_DECAY) ? 0.f : __expf(load_param(p.A_log, p.alog_dtype, i_hv));
  const act_t* const qp = reinterpret_cast<const act_t*>(p.q) + i_h * 128;
  const act_t* const kp = reinterpret_cast<const act_t*>(p.k) + i_h * 128;
  const act_t* const vp = reinterpret_cast<const act_t*>(p.v) + i_hv * 128 + row0;

  for (int t = 0; t < T; ++t) {
    const int64_t tok = (int64_t)bos + t;
    float qv[8], kv[8];
    load_k8(qp + tok * p.stride_q, c, qv);
    load_k8(kp + tok * p.stride_k, c, kv);
    float qn = p.scale, kn = 1.f;
    if (p.use_qk_l2norm) {
      float qs = 0.f, ks = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) { qs = fmaf(qv[e], qv[e], qs); ks = fmaf(kv[e], kv[e], ks); }
      qn = rsqrtf(row16_allreduce(qs) + 1e-6f) * p.scale;
      kn = rsqrtf(row16_allreduce(ks) + 1e-6f);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) { qv[e] *= qn; kv[e] *= kn; }

    // gate and beta
    float dec[8];
    float dec_scalar = 1.f;
    if constexpr (IS_KDA) {
      float av[8], dt[8];
      if (p.gate_mode == PLA_GATE_LOG_DECAY) {
        load_k8(reinterpret_cast<const float*>(p.a) + tok * p.stride_a + i_hv * 128, c, av);
#pragma unroll
        for (int e = 0; e < 8; ++e) dt[e] = 0.f;
      } else {
        load_k8(reinterpret_cast<const act_t*>(p.a) + tok * p.stride_a + i_hv * 128, c, av);
        if (p.dt_bias_is_f32) load_k8(reinterpret_cast<const float*>(p.dt_bias) + i_hv * 128, c, dt);
        else load_k8(reinterpret_cast<const act_t*>(p.dt_bias) + i_hv * 128, c, dt);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e)
        dec[e] = gate_decay(av[e], dt[e], eA, p.gate_p0, p.softplus_threshold, p.gate_mode);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) dec[e] = 1.f;
      float a_val, dt_val = 0.f;
      if (p.gate_mode == PLA_GATE_LOG_DECAY) {
        a_val = reinterpret_cast<const float*>(p.a)[tok * p.stride_a + i_hv];
      } else {
        a_val = to_float(reinterpret_cast<const act_t*>(p.a)[tok * p.stride_a + i_hv]);
        dt_val = p.dt_bias_is_f32 ? reinterpret_cast<const float*>(p.dt_bias)[i_hv]
                                  : to_float(reinterpret_cast<const act_t*>(p.dt_bias)[i_hv]);
      }
      dec_scalar = gate_decay(a_val, dt_val, eA, p.gate_p0, p.softplus_threshold, p.gate_mode);
    }
    float beta;
    if (p.beta_is_activated) beta = reinterpret_cast<const float*>(p.b)[tok * p.stride_b + i_hv];
    else beta = fast_sigmoid(to_float(reinterpret_cast<const act_t*>(p.b)[tok * p.stride_b + i_hv]));

    float vv[R];
    load_rows<act_t, R>(vp + tok * p.stride_v, vv);

    if constexpr (MTP) {
      // Eagle tree: continue from the snapshot of the parent step when it is not t-1.
      if (p.parents != nullptr && t != 0 && cidx >= 0) {
        const int64_t parent = p.parents[(int64_t)i_n * p.stride_parent_seq + (int64_t)t * p.stride_parent_token];
        if (parent >= 0 && parent < t && parent != t - 1) {
          __threadfence();   // the snapshot was written by these same lanes at step `parent`
          load_state<R>(p.cache + ((int64_t)cidx * p.cache_steps + parent) * p.HV * 16384 + tile_off, s);
        }
      }
    }

    float outv[R];
    delta_rows<R, IS_KDA, true>(s, dec, dec_scalar, kv, qv, vv, beta, outv);

    if constexpr (MTP) {
      float* snap = nullptr;
      if (p.is_sglang) {
        if (p.cache != nullptr && cidx >= 0)
          snap = p.cache + ((int64_t)cidx * p.cache_steps + t) * p.HV * 16384 + tile_off;
      } else if (p.stride_h0_indices_seq > 0 && p.h0_indices != nullptr && p.h0 != nullptr) {
        const int step_slot = p.h0_indices[(int64_t)i_n * p.stride_h0_indices_seq + t];
        if (step_slot > 0) snap = p.h0 + (int64_t)step_slot * p.h0_slot_stride + tile_off;
      }
      if (snap != nullptr) store_state<R>(snap, s);
    }
    if (c == 0) store_rows<act_t, R>(o_base + (int64_t)t * p.HV * 128, outv);
  }

  if (have_state && !p.disable_state_update) store_state<R>(h_rows, s);
}

struct FoldParams {
  float* h0; const void* rawv; const void* rawk; const float* gk; const float* beta;
  const int32_t* slot_idx; const int32_t* accept_lens;
  int64_t h0_slot_stride, rawv_slot_stride, rawk_slot_stride, gk_slot_stride, beta_slot_stride;
  int B, H, HV, L, null_block_id;
};

template <typename act_t, int RPW>
__global__ __launch_bounds__(256) void kda_fold_kernel(const FoldParams p) {
  constexpr int R = RPW / 4;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int grp = lane >> 4;
  const int c = lane & 15;
  const int i_n = blockIdx.x / p.HV;
  const int i_hv = blockIdx.x - i_n * p.HV;
  const int i_h = i_hv / (p.HV / p.H);
  const int row0 = (blockIdx.y * 4 + wave) * RPW + grp * R;

  const int slot = p.slot_idx[i_n];
  int n_acc = p.accept_lens[i_n];
  if (slot <= p.null_block_id || n_acc <= 0) return;
  if (n_acc > p.L) n_acc = p.L;

  float* const h_rows = p.h0 + (int64_t)slot * p.h0_slot_stride + (int64_t)i_hv * 16384 + row0 * 128 + 4 * c;
  float s[R][8];
  load_state<R>(h_rows, s);
  const act_t* const kp = reinterpret_cast<const act_t*>(p.rawk) + (int64_t)slot * p.rawk_slot_stride + (int64_t)i_h * p.L * 128;
  const act_t* const vp = reinterpret_cast<const act_t*>(p.rawv) + (int64_t)slot * p.rawv_slot_stride + (int64_t)i_hv * p.L * 128 + row0;
  const float* const gp = p.gk + (int64_t)slot * p.gk_slot_stride + (int64_t)i_hv * p.L * 128;
  const float* const bp = p.beta + (int64_t)slot * p.beta_slot_stride + (int64_t)i_hv * p.L;

  for (int t = 0; t < n_acc; ++t) {
    float kv[8], gv[8], dec[8], vv[R], unused[R];
    load_k8(kp + t * 128, c, kv);
    load_k8(gp + t * 128, c, gv);
    load_rows<act_t, R>(vp + t * 128, vv);
    float ks = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ks = fmaf(kv[e], kv[e], ks);
    const float kn = 1.0f / sqrtf(row16_allreduce(ks) + 1e-6f);
#pragma unroll
    for (int e = 0; e < 8; ++e) { kv[e] *= kn; dec[e] = __expf(gv[e]); }
    delta_rows<R, true, false>(s, dec, 1.f, kv, kv, vv, bp[t], unused);
  }
  store_state<R>(h_rows, s);
}

// ---- host side ---------------------------------------------------------------

// gfx950 tuning table: rows of the 128-row tile owned by one wavefront, chosen
// from the number of (request, value-head) tiles so that small batches still
// spread over all 256 CUs while large batches keep 64 state VGPRs in flight.
static int pick_rows_per_wave(int tiles, bool mtp) {
  (void)mtp;
  if (tiles >= 2048) return 32;
  if (tiles >= 512) return 16;
  return 8;
}

template <typename act_t, bool IS_KDA, bool MTP>
static int launch_rpw(const KLastParams& p, int rpw, hipStream_t stream) {
  const dim3 block(256);
  const unsigned tiles = (unsigned)p.B * (unsigned)p.HV;
  switch (rpw) {
    case 32: hipLaunchKernelGGL((k_last_kernel<act_t, IS_KDA, MTP, 32>), dim3(tiles, 1), block, 0, stream, p); break;
    case 16: hipLaunchKernelGGL((k_last_kernel<act_t, IS_KDA, MTP, 16>), dim3(tiles, 2), block, 0, stream, p); break;
    case 8:  hipLaunchKernelGGL((k_last_kernel<act_t, IS_KDA, MTP, 8>),  dim3(tiles, 4), block, 0, stream, p); break;
    default: return fail("rows_per_wave must be 0, 8, 16 or 32, got %d", rpw);
  }
  return check_launch("k_last_kernel launch");
}

template <typename act_t>
static int launch_flags(const KLastParams& p, bool is_kda, bool mtp, int rpw, hipStream_t stream) {
  if (is_kda) return mtp ? launch_rpw<act_t, true, true>(p, rpw, stream) : launch_rpw<act_t, true, false>(p, rpw, stream);
  return mtp ? launch_rpw<act_t, false, true>(p, rpw, stream) : launch_rpw<act_t, false, false>(p, rpw, stream);
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

static int run_k_last(const KLastParams& p, bool is_kda, bool mtp, int act_dtype, int rows_per_wave, void* stream) {
  const int rpw = rows_per_wave > 0 ? rows_per_wave : pick_rows_per_wave(p.B * p.HV, mtp);
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  if (act_dtype == PLA_BF16) return launch_flags<bf16_t>(p, is_kda, mtp, rpw, s);
  return launch_flags<f16_t>(p, is_kda, mtp, rpw, s);
}

}  // namespace pla

using namespace pla;

extern "C" int pla_k_last_packed_launch(
    const void* A_log, int alog_dtype, const void* a, const void* dt_bias,
    float softplus_beta, float softplus_threshold,
    const void* mixed_qkv, const void* b, void* o, float* h0,
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
  PLA_REQUIRE(aligned(h0, 16) && h0_slot_stride % 4 == 0, "state base and slot pitch require 16-byte alignment");
  PLA_REQUIRE(aligned(o, 16), "out requires 16-byte alignment");
  PLA_REQUIRE(h0_slot_stride >= (int64_t)HV * 16384, "state slot pitch must cover HV*V*K");
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
  return run_k_last(p, is_kda != 0, false, act_dtype, rows_per_wave, stream);
}

extern "C" int pla_k_last_launch(
    const void* A_log, int alog_dtype, const void* a, const void* dt_bias, int dt_bias_is_f32,
    float softplus_beta_or_lower_bound, float softplus_threshold, int gate_mode,
    const void* q, const void* k, const void* v, const void* b, int beta_is_activated,
    void* o, float* h0, const int32_t* cu_seqlens, float* cache,
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
  if (h0) PLA_REQUIRE(aligned(h0, 16) && h0_slot_stride % 4 == 0 && h0_slot_stride >= (int64_t)HV * 16384,
                      "state base and slot pitch require 16-byte alignment and must cover HV*V*K");
  if (cache) PLA_REQUIRE(aligned(cache, 16), "intermediate cache base requires 16-byte vector alignment");
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
  return run_k_last(p, is_kda != 0, mtp, act_dtype, rows_per_wave, stream);
}

extern "C" int pla_kda_fold_launch(
    float* h0, const void* rawv, const void* rawk, const float* gk, const float* beta,
    const int32_t* slot_idx, const int32_t* accept_lens,
    int64_t h0_slot_stride, int64_t rawv_slot_stride, int64_t rawk_slot_stride,
    int64_t gk_slot_stride, int64_t beta_slot_stride,
    int B, int H, int HV, int L, int null_block_id, int act_dtype, void* stream) {
  PLA_REQUIRE(h0 && rawv && rawk && gk && beta && slot_idx && accept_lens, "null tensor pointer");
  PLA_REQUIRE(B > 0 && L > 0, "fold requires B > 0 and L > 0");
  PLA_REQUIRE(H > 0 && HV >= H && HV % H == 0, "HV must be a positive multiple of H, got H=%d, HV=%d", H, HV);
  PLA_REQUIRE(act_dtype == PLA_BF16 || act_dtype == PLA_F16, "record dtype must be bf16 or fp16");
  PLA_REQUIRE(aligned(h0, 16) && h0_slot_stride % 4 == 0 && aligned(gk, 16) && gk_slot_stride % 4 == 0 &&
              aligned(rawk, 8) && rawk_slot_stride % 4 == 0 && aligned(rawv, 16) && rawv_slot_stride % 8 == 0,
              "state and record tensors require 16-byte alignment");
  FoldParams p{h0, rawv, rawk, gk, beta, slot_idx, accept_lens,
               h0_slot_stride, rawv_slot_stride, rawk_slot_stride, gk_slot_stride, beta_slot_stride,
               B, H, HV, L, null_block_id};
  const unsigned tiles = (unsigned)B * (unsigned)HV;
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  const int rpw = pick_rows_per_wave((int)tiles, true);
  const dim3 block(256);
  if (act_dtype == PLA_BF16) {
    if (rpw == 32) hipLaunchKernelGGL((kda_fold_kernel<bf16_t, 32>), dim3(tiles, 1), block, 0, s, p);
    else if (rpw == 16) hipLaunchKernelGGL((kda_fold_kernel<bf16_t, 16>), dim3(tiles, 2), block, 0, s, p);
    else hipLaunchKernelGGL((kda_fold_kernel<bf16_t, 8>), dim3(tiles, 4), block, 0, s, p);
  } else {
    if (rpw == 32) hipLaunchKernelGGL((kda_fold_kernel<f16_t, 32>), dim3(tiles, 1), block, 0, s, p);
    else if (rpw == 16) hipLaunchKernelGGL((kda_fold_kernel<f16_t, 16>), dim3(tiles, 2), block, 0, s, p);
    else hipLaunchKernelGGL((kda_fold_kernel<f16_t, 8>), dim3(tiles, 4), block, 0, s, p);
  }
  return check_launch("kda_fold_kernel launch");
}
