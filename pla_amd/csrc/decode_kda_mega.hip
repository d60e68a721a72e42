// Fused KDA decode step for gfx950: causal conv1d update (width 4) + SiLU, q/k L2 norm, per-channel
// gate, delta-rule recurrence on the indexed k-last FP32 state pool and the optional gated RMSNorm
// of the output, in one kernel (reference: src/decode/k-last/fused_kda_decode_mega_kernel.cuh:138-729,
// contract src/decode/k-last/fused_kda_decode_mega_host.cpp:77-300).
//
// One workgroup of four wavefronts per (request, head).  The 64 KiB state tile is requested first,
// so its sixteen 16-byte loads per lane are in flight while the workgroup runs the convolution:
// threads 0-127 own one q and one k channel each, threads 128-255 one v channel and that channel's
// decay.  A conv window belongs to exactly one thread, which reads its three taps, shifts them and
// appends the new sample in place.  The activated q, k (FP32), v (rounded to the activation type, as
// the reference does, :384) and the decays meet in LDS; after one barrier each wavefront runs the
// recurrence on its 32 V rows exactly as the plain decode kernel does (lanes 0-31 even rows, lanes
// 32-63 odd rows, four K channels per lane).  The output row is normalised over the head's 128
// values (sum of squares across the four wavefronts through LDS) and written by 128 threads.
// A request whose slot is negative writes zeros to its output row and touches neither pool
// (:214-232).

#include "decode_common.h"

namespace pla {

struct MegaParams {
  const float* a_log; const void* g; const float* dt_bias;
  const void* x_q; const void* x_k; const void* x_v; const void* beta;
  const float* w_q; const float* w_k; const float* w_v;
  const float* bias_q; const float* bias_k; const float* bias_v;
  void* cs_q; void* cs_k; void* cs_v;
  const void* g_out; const float* o_norm_weight; float norm_eps;
  float* state; const int32_t* state_indices; void* out;
  float scale, lower_bound;
  int H;
  int64_t x_row, beta_row, onorm_row, conv_slot, state_slot;
};

__device__ __forceinline__ float silu(float x) { return x * fast_sigmoid(x); }

// One channel of the width-4 causal convolution: taps are `tap_pitch` elements apart inside the
// slot's window (oldest first), the weights [4, dim] are width-major.  Shifts the window in place.
template <typename act_t>
__device__ __forceinline__ float conv_update(act_t* window, int64_t tap_pitch, act_t x_new, const float* w, int dim,
                                             const float* bias, int ch) {
  const act_t t0 = window[0], t1 = window[tap_pitch], t2 = window[2 * tap_pitch];
  float acc = bias != nullptr ? bias[ch] : 0.f;
  acc = fmaf(to_float(t0), w[ch], acc);
  acc = fmaf(to_float(t1), w[dim + ch], acc);
  acc = fmaf(to_float(t2), w[2 * dim + ch], acc);
  acc = fmaf(to_float(x_new), w[3 * dim + ch], acc);
  window[0] = t1;
  window[tap_pitch] = t2;
  window[2 * tap_pitch] = x_new;
  return acc;
}

template <typename act_t, bool USE_LOWER_BOUND, bool APPLY_ONORM>
__global__ __launch_bounds__(256) void kda_decode_mega_kernel(const MegaParams p) {
  constexpr int RPW = 32, R = RPW / 2;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, c = lane & 31;
  const int i_n = blockIdx.x / p.H;
  const int i_h = blockIdx.x - i_n * p.H;
  const int dim = p.H * 128;
  act_t* const o_row = reinterpret_cast<act_t*>(p.out) + (int64_t)i_n * dim + i_h * 128;

  const int slot = p.state_indices[i_n];
  if (slot < 0) {
    if (tid < 128) o_row[tid] = act_t{0};
    return;
  }

  __shared__ __align__(16) float sq[128], sk[128], sdec[128], sv[128], so[128];
  __shared__ float red[3][4];

  // state tile first: everything below overlaps its latency
  const int rowbase = wave * RPW;
  const int lane_off = ((rowbase + half) * 128 + 4 * c) * 4;
  const Tile<float> h_tile(p.state + (int64_t)slot * p.state_slot + (int64_t)i_h * 16384);
  float s[R][4];
  load_state<R>(h_tile, lane_off, s);

  const float eA = __expf(p.a_log[i_h]);
  const float beta = fast_sigmoid(to_float(reinterpret_cast<const act_t*>(p.beta)[(int64_t)i_n * p.beta_row + i_h]));
  const int64_t tap_pitch = 3 * (int64_t)dim;
  if (tid < 128) {
    const int ch = i_h * 128 + tid;
    const int64_t at = (int64_t)slot * p.conv_slot + ch;
    const act_t qx = reinterpret_cast<const act_t*>(p.x_q)[(int64_t)i_n * p.x_row + ch];
    const act_t kx = reinterpret_cast<const act_t*>(p.x_k)[(int64_t)i_n * p.x_row + ch];
    const float qa = silu(conv_update(reinterpret_cast<act_t*>(p.cs_q) + at, tap_pitch, qx, p.w_q, dim, p.bias_q, ch));
    const float ka = silu(conv_update(reinterpret_cast<act_t*>(p.cs_k) + at, tap_pitch, kx, p.w_k, dim, p.bias_k, ch));
    sq[tid] = qa;
    sk[tid] = ka;
    const float q2 = wave64_allreduce(qa * qa), k2 = wave64_allreduce(ka * ka);
    if (lane == 0) { red[0][wave] = q2; red[1][wave] = k2; }
  } else {
    const int t = tid - 128;
    const int ch = i_h * 128 + t;
    const int64_t at = (int64_t)slot * p.conv_slot + ch;
    const act_t vx = reinterpret_cast<const act_t*>(p.x_v)[(int64_t)i_n * p.x_row + ch];
    const float va = silu(conv_update(reinterpret_cast<act_t*>(p.cs_v) + at, tap_pitch, vx, p.w_v, dim, p.bias_v, ch));
    sv[t] = to_float(from_float<act_t>(va));
    const float graw = to_float(reinterpret_cast<const act_t*>(p.g)[(int64_t)i_n * dim + ch]);
    sdec[t] = gate_decay(graw, p.dt_bias[ch], eA, USE_LOWER_BOUND ? p.lower_bound : 1.0f, 20.0f,
                         USE_LOWER_BOUND ? PLA_GATE_LOWER_BOUND : PLA_GATE_SOFTPLUS);
  }
  __syncthreads();

  const float qn = fast_rsqrt(red[0][0] + red[0][1] + 1e-6f) * p.scale;
  const float kn = fast_rsqrt(red[1][0] + red[1][1] + 1e-6f);
  float qv[4], kv[4], dec[4];
  {
    const float4 q4 = *reinterpret_cast<const float4*>(&sq[4 * c]);
    const float4 k4 = *reinterpret_cast<const float4*>(&sk[4 * c]);
    const float4 d4 = *reinterpret_cast<const float4*>(&sdec[4 * c]);
    qv[0] = q4.x * qn; qv[1] = q4.y * qn; qv[2] = q4.z * qn; qv[3] = q4.w * qn;
    kv[0] = k4.x * kn; kv[1] = k4.y * kn; kv[2] = k4.z * kn; kv[3] = k4.w * kn;
    dec[0] = d4.x; dec[1] = d4.y; dec[2] = d4.z; dec[3] = d4.w;
  }
  float vv[R], outv[R];
#pragma unroll
  for (int j = 0; j < R; ++j) vv[j] = sv[rowbase + 2 * j + half];

  delta_rows<R, true, true>(s, dec, 1.f, kv, qv, vv, beta, outv);
  store_state<R>(h_tile, lane_off, s);

  // every lane of a half holds the half's sixteen outputs; lane j of the half publishes row 2j + half
  float o2 = 0.f;
#pragma unroll
  for (int j = 0; j < R; ++j) {
    o2 = fmaf(outv[j], outv[j], o2);
    if (c == j) so[rowbase + 2 * j + half] = outv[j];
  }
  if constexpr (APPLY_ONORM) {
    const LanePair both = swap_halves(o2);
    if (lane == 0) red[2][wave] = both.lo + both.hi;
  }
  __syncthreads();
  if (tid < 128) {
    float val = so[tid];
    if constexpr (APPLY_ONORM) {
      const float total = red[2][0] + red[2][1] + red[2][2] + red[2][3];
      const float rstd = fast_rsqrt(total * (1.0f / 128.0f) + p.norm_eps);
      const float gate = fast_sigmoid(to_float(
          reinterpret_cast<const act_t*>(p.g_out)[(int64_t)i_n * p.onorm_row + i_h * 128 + tid]));
      val = val * rstd * p.o_norm_weight[tid] * gate;
    }
    o_row[tid] = from_float<act_t>(val);
  }
}

template <typename act_t>
static int launch_mega(const MegaParams& p, int B, bool use_lb, bool onorm, hipStream_t stream) {
  const dim3 grid((unsigned)B * (unsigned)p.H), block(256);
  if (use_lb) {
    if (onorm) kda_decode_mega_kernel<act_t, true, true><<<grid, block, 0, stream>>>(p);
    else kda_decode_mega_kernel<act_t, true, false><<<grid, block, 0, stream>>>(p);
  } else {
    if (onorm) kda_decode_mega_kernel<act_t, false, true><<<grid, block, 0, stream>>>(p);
    else kda_decode_mega_kernel<act_t, false, false><<<grid, block, 0, stream>>>(p);
  }
  return check_launch("kda_decode_mega_kernel");
}

static bool aligned_to(const void* ptr, size_t a) { return (reinterpret_cast<uintptr_t>(ptr) % a) == 0; }

}  // namespace pla

extern "C" int pla_kda_decode_mega_launch(
    int act_dtype, int apply_onorm, int use_lower_bound,
    const float* a_log, const void* g, const float* dt_bias,
    const void* x_q, const void* x_k, const void* x_v, const void* beta,
    const float* w_q_t, const float* w_k_t, const float* w_v_t,
    const float* bias_q, const float* bias_k, const float* bias_v,
    void* cs_q, void* cs_k, void* cs_v,
    const void* g_out, const float* o_norm_weight, float norm_eps,
    float* state, const int32_t* state_indices, void* out,
    float scale, float lower_bound, int B, int H, int HV,
    int64_t x_row, int64_t beta_row, int64_t onorm_row,
    int64_t conv_slot, int64_t state_slot, void* stream) {
  using namespace pla;
  PLA_REQUIRE(act_dtype == PLA_BF16 || act_dtype == PLA_F16, "act_dtype must be PLA_BF16 or PLA_F16, got %d", act_dtype);
  PLA_REQUIRE(B > 0, "KDA decode fusion requires at least one row, got B=%d", B);
  PLA_REQUIRE(H > 0 && H == HV, "KDA decode fusion has one head count (H == HV), got H=%d HV=%d", H, HV);
  PLA_REQUIRE((int64_t)B * H <= 0x7fffffffLL, "B * H = %lld exceeds the grid limit", (long long)B * H);
  PLA_REQUIRE(a_log && g && dt_bias && x_q && x_k && x_v && beta && w_q_t && w_k_t && w_v_t && cs_q && cs_k && cs_v &&
              state && state_indices && out, "null tensor pointer");
  const bool onorm = apply_onorm != 0;
  PLA_REQUIRE(!onorm || (g_out != nullptr && o_norm_weight != nullptr),
              "output_gate and norm_weight must be provided together");
  PLA_REQUIRE(!onorm || norm_eps >= 0.f, "norm_eps must be non-negative");
  const int64_t dim = (int64_t)H * 128;
  PLA_REQUIRE(x_row >= 3 * dim, "x row pitch %lld is below 3 * H * 128", (long long)x_row);
  PLA_REQUIRE(beta_row >= H, "raw_beta row pitch %lld is below H", (long long)beta_row);
  PLA_REQUIRE(conv_slot >= 9 * dim, "conv_state slot pitch %lld is below 3 * H * 128 * 3", (long long)conv_slot);
  PLA_REQUIRE(state_slot >= dim * 128, "state slot pitch %lld is below H * 128 * 128", (long long)state_slot);
  PLA_REQUIRE(!onorm || onorm_row >= dim, "output_gate row pitch %lld is below H * 128", (long long)onorm_row);
  PLA_REQUIRE(aligned_to(state, 16) && state_slot % 4 == 0, "state base and slot pitch must be 16-byte aligned");

  MegaParams p;
  p.a_log = a_log; p.g = g; p.dt_bias = dt_bias;
  p.x_q = x_q; p.x_k = x_k; p.x_v = x_v; p.beta = beta;
  p.w_q = w_q_t; p.w_k = w_k_t; p.w_v = w_v_t;
  p.bias_q = bias_q; p.bias_k = bias_k; p.bias_v = bias_v;
  p.cs_q = cs_q; p.cs_k = cs_k; p.cs_v = cs_v;
  p.g_out = g_out; p.o_norm_weight = o_norm_weight; p.norm_eps = norm_eps;
  p.state = state; p.state_indices = state_indices; p.out = out;
  p.scale = scale; p.lower_bound = lower_bound;
  p.H = H;
  p.x_row = x_row; p.beta_row = beta_row; p.onorm_row = onorm_row; p.conv_slot = conv_slot; p.state_slot = state_slot;
  hipStream_t s = static_cast<hipStream_t>(stream);
  return act_dtype == PLA_BF16 ? launch_mega<bf16_t>(p, B, use_lower_bound != 0, onorm, s)
                               : launch_mega<f16_t>(p, B, use_lower_bound != 0, onorm, s);
}
