// pla.decode._C: the pybind11 extension module of the decode namespace, as the reference ships one
// (src/decode/k-last/fused_sigmoid_gating.cpp:160-259: plain pybind functions, argument names and positional
// order are API).  The functions validate their tensors, derive shapes, strides and the MTP mode exactly as the
// reference's host functions do (src/decode/k-last/fused_sigmoid_gating_cuda_k_last.cpp:239-435,
// src/decode/k-last/fused_sigmoid_gating_cuda_k_last_packed.cpp:82-204, shape rules
// src/decode/k-last/sanity_checks.h:60-112) and launch through the C ABI of libpla_gfx950.so on torch's
// current stream.  Torch is used for tensor metadata, the output allocation of the non-packed call and the
// stream; nothing here computes.  A failed check raises RuntimeError before any launch.

#include <torch/extension.h>
#include <c10/hip/HIPStream.h>

#include <c10/core/DeviceGuard.h>

#include <cmath>
#include <cstdlib>
#include <optional>
#include <string>
#include <variant>

#include "../../include/pla_gfx950.h"

namespace {

using torch::Tensor;
using OptTensor = std::optional<Tensor>;

int dtype_code(at::ScalarType t) {
  switch (t) {
    case at::kFloat: return PLA_F32;
    case at::kBFloat16: return PLA_BF16;
    case at::kHalf: return PLA_F16;
    default: TORCH_CHECK(false, "unsupported dtype ", t);
  }
}
const void* ptr(const OptTensor& t) { return t.has_value() ? t->data_ptr() : nullptr; }
void* stream_of(const Tensor& t) { return c10::hip::getCurrentHIPStream(t.get_device()).stream(); }
void launched(int rc) { TORCH_CHECK(rc == 0, pla_last_error()); }
bool bypass() {                                   // read once (reference: src/bypass_exec.h:44-50)
  static const bool on = [] { const char* v = std::getenv("PLA_BYPASS_EXEC"); return v && v[0] == '1' && v[1] == 0; }();
  return on;
}

// The reference's tile tuple (BV, WN, SN, HV_PER_CTA) is validated as it validates it
// (fused_sigmoid_gating_cuda_k_last_packed.cpp:268-271); on gfx950 only the number of state rows a wavefront
// owns is tunable: four wavefronts cover BV rows.
int rows_per_wave(const std::optional<std::array<int64_t, 4>>& tile, int64_t HV, int64_t H, int64_t V) {
  if (!tile) return 0;
  const auto [bv, wn, sn, hv_per_cta] = *tile;
  TORCH_CHECK(bv > 0 && wn > 0 && sn > 0 && V % bv == 0, "invalid k-last tile parameters");
  const int64_t hv_per_h = HV / H;
  TORCH_CHECK(hv_per_cta > 0 && hv_per_cta <= hv_per_h && hv_per_h % hv_per_cta == 0, "HV_PER_CTA must divide HV/H");
  return bv >= 128 ? 32 : bv >= 64 ? 16 : 8;
}

Tensor packed_impl(const Tensor& mixed_qkv, const Tensor& a, const Tensor& b, const Tensor& A_log, const Tensor& dt_bias,
                   double softplus_beta, double softplus_threshold, std::optional<double> scale,
                   const OptTensor& initial_state_source, const OptTensor& initial_state_indices, Tensor out,
                   bool use_qk_l2norm_in_kernel, const OptTensor& cu_seqlens, bool is_kda, std::optional<bool> is_sglang_opt,
                   const std::optional<std::array<int64_t, 4>>& tile) {
  if (bypass()) return out;
  const bool is_sglang = is_sglang_opt.value_or(true);
  TORCH_CHECK(initial_state_source.has_value(), "initial_state_source is required for k_last_packed");
  const Tensor& state = *initial_state_source;
  TORCH_CHECK(state.dim() == 4, "initial_state_source must have shape [slots, HV, V, K]");
  const int64_t HV = state.size(-3), V = state.size(-2), K = state.size(-1);
  TORCH_CHECK(K == 128 && V == 128, "fused_sigmoid_gating_delta_rule_forward_k_last_packed requires head_dim K == V == 128, got K=",
              K, ", V=", V);
  TORCH_CHECK(mixed_qkv.dim() == 2, "mixed_qkv must have shape [tokens, qkv_width]");
  const int64_t qk_width = mixed_qkv.size(1) - HV * V;
  TORCH_CHECK(qk_width > 0 && qk_width % (2 * K) == 0, "packed QKV width must equal 2*H*K + HV*V with H > 0");
  const int64_t H = qk_width / (2 * K);
  TORCH_CHECK(HV >= H && HV % H == 0, "HV must be a positive multiple of H, got H=", H, ", HV=", HV);
  const int64_t gate_width = HV * (is_kda ? K : 1);
  TORCH_CHECK(a.dim() >= 2 && a.size(-1) == gate_width, "a head dimensions must match HV and the gate type");
  TORCH_CHECK(b.dim() >= 2 && b.size(-1) == HV, "b head dimension must match HV");
  TORCH_CHECK(A_log.numel() == HV && dt_bias.numel() == gate_width, "A_log/dt_bias head dimensions must match HV and the gate type");
  TORCH_CHECK(out.dim() >= 3 && out.size(-2) == HV && out.size(-1) == V && out.numel() == mixed_qkv.size(0) * HV * V,
              "out must match the packed token count and [HV, V]");
  TORCH_CHECK(mixed_qkv.is_cuda(), "mixed_qkv must be a CUDA tensor");
  const auto act = mixed_qkv.scalar_type();
  TORCH_CHECK(act == at::kBFloat16 || act == at::kHalf, "mixed_qkv must be fp16 or bf16");
  TORCH_CHECK(a.scalar_type() == act && b.scalar_type() == act && dt_bias.scalar_type() == act && out.scalar_type() == act,
              "a, b, dt_bias and out must have mixed_qkv's dtype");
  TORCH_CHECK(state.scalar_type() == at::kFloat || state.scalar_type() == at::kBFloat16,
              "k-last state dtype must be float32 or bfloat16, got ", state.scalar_type());
  TORCH_CHECK(mixed_qkv.stride(1) == 1 && state.stride(-1) == 1 && state.stride(-2) == K && state.stride(-3) == V * K,
              "mixed_qkv rows and state slots must be dense");
  TORCH_CHECK(out.is_contiguous(), "out must be contiguous");
  const int64_t B = cu_seqlens.has_value() ? cu_seqlens->size(0) - 1 : mixed_qkv.size(0);
  if (cu_seqlens.has_value()) TORCH_CHECK(cu_seqlens->scalar_type() == at::kInt, "cu_seqlens's data type should be torch::kInt32");
  if (initial_state_indices.has_value())
    TORCH_CHECK(initial_state_indices->scalar_type() == at::kInt, "initial_state_indices's data type should be torch::kInt32");
  const int rpw = rows_per_wave(tile, HV, H, V);
  const float scale_val = scale.has_value() ? (float)*scale : 1.0f / std::sqrt((float)K);
  launched(pla_k_last_packed_launch(
      A_log.data_ptr(), dtype_code(A_log.scalar_type()), a.data_ptr(), dt_bias.data_ptr(), (float)softplus_beta,
      (float)softplus_threshold, mixed_qkv.data_ptr(), b.data_ptr(), out.data_ptr(), state.data_ptr(),
      dtype_code(state.scalar_type()), static_cast<const int32_t*>(ptr(cu_seqlens)),
      static_cast<const int32_t*>(ptr(initial_state_indices)), scale_val, 1, a.stride(a.dim() - 2), mixed_qkv.stride(0),
      b.stride(b.dim() - 2), state.stride(0), (int)B, (int)H, (int)HV, (int)K, (int)V, use_qk_l2norm_in_kernel ? 1 : 0,
      is_sglang ? 1 : 0, is_kda ? 1 : 0, dtype_code(act), rpw, stream_of(mixed_qkv)));
  return out;
}

// Shape of the state or the snapshot cache: [.., HV, V, K], or a flattened pool whose rows cover one slot.
void check_pool(const OptTensor& t, int64_t HV, int64_t V, int64_t K) {
  if (!t.has_value()) return;
  const bool physical = t->dim() >= 4 && t->size(-3) == HV && t->size(-2) == V && t->size(-1) == K;
  const bool flattened = t->dim() >= 2 && t->stride(-1) == 1 && t->stride(0) >= HV * V * K;
  TORCH_CHECK(physical || flattened,
              "state/cache head dimensions must match [HV, V, K], or be a flattened pool whose stride(0) covers HV*V*K "
              "with a unit-stride innermost dim");
}

int64_t packed_t_max(const Tensor& k, int64_t B, bool target_verify, int64_t cache_steps, int64_t slot_columns) {
  TORCH_CHECK(B > 0, "k-last requires at least one sequence");
  if (target_verify && slot_columns > 0) return slot_columns;
  if (k.size(0) == B) return k.size(1);
  if (!target_verify && k.size(0) == 1 && k.size(1) == B) return 1;
  if (target_verify) {
    if (cache_steps > 0) return cache_steps;
    TORCH_CHECK(k.size(1) % B == 0, "packed target-verify tokens must be divisible by batch size");
    return k.size(1) / B;
  }
  return k.size(1);
}

using StepsOrAccepted = std::optional<std::variant<Tensor, int64_t>>;

Tensor k_last_impl(const Tensor& A_log, const Tensor& a, const Tensor& dt_bias, double softplus_beta, double softplus_threshold,
                   const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& b, const OptTensor& initial_state_source,
                   const OptTensor& initial_state_indices, std::optional<double> scale, bool use_qk_l2norm_in_kernel,
                   const OptTensor& cu_seqlens, bool is_kda, bool disable_state_update,
                   const OptTensor& intermediate_states_buffer, const OptTensor& intermediate_state_indices,
                   const StepsOrAccepted& cache_steps_or_num_accept, const OptTensor& retrieve_parent_token,
                   std::optional<double> lower_bound, std::optional<bool> is_sglang_opt, const OptTensor& out,
                   const std::optional<std::array<int64_t, 4>>& tile) {
  if (bypass()) return out.has_value() ? *out : torch::zeros_like(v);
  const bool is_sglang = is_sglang_opt.value_or(true);
  TORCH_CHECK(!lower_bound.has_value() || is_kda, "lower_bound is only supported for KDA");

  int64_t cache_steps = 0;
  bool has_cache_steps = false;
  OptTensor num_accepted;
  if (cache_steps_or_num_accept.has_value()) {
    if (std::holds_alternative<Tensor>(*cache_steps_or_num_accept)) {
      num_accepted = std::get<Tensor>(*cache_steps_or_num_accept);
      TORCH_CHECK(num_accepted->scalar_type() == at::kInt, "num_accepted_tokens's data type should be torch::kInt32");
    } else {
      cache_steps = std::get<int64_t>(*cache_steps_or_num_accept);
      has_cache_steps = true;
    }
  }
  const OptTensor& idx = initial_state_indices;
  const int64_t stride_idx_seq = idx.has_value() && idx->dim() == 2 ? idx->stride(0) : 0;
  const bool vllm_spec = stride_idx_seq > 0;
  TORCH_CHECK(!vllm_spec || !is_sglang, "2D initial_state_indices is the vLLM spec-decode layout; pass is_sglang=False");
  TORCH_CHECK(!(vllm_spec && has_cache_steps),
              "vLLM spec decode expects num_accepted_tokens (a tensor) in cache_steps_or_num_accept, but received an int");

  const OptTensor& state = initial_state_source;
  const OptTensor& cache = intermediate_states_buffer;
  TORCH_CHECK(q.dim() == 4 && k.dim() == 4 && v.dim() == 4, "q, k, v must have shape [B, T, heads, dim]");
  const int64_t H = k.size(2), HV = v.size(2), K = k.size(3), V = v.size(3);
  TORCH_CHECK(H > 0 && HV >= H && HV % H == 0, "HV must be a positive multiple of H, got H=", H, ", HV=", HV);
  TORCH_CHECK(q.sizes() == k.sizes() && v.size(0) == k.size(0) && v.size(1) == k.size(1),
              "q/k shapes and q/k/v token dimensions must match");
  const int64_t gate_width = is_kda ? HV * K : HV;
  const bool a_tokens_heads_dim = is_kda && a.dim() == 3 && a.size(1) == HV && a.size(2) == K;
  TORCH_CHECK(a.dim() >= 2 && ((a.dim() == 4 && a.size(2) == HV && a.size(3) == (is_kda ? K : 1)) || a_tokens_heads_dim ||
                               (a.dim() != 4 && a.size(-1) == gate_width)),
              "a head dimensions must match HV and the gate type");
  TORCH_CHECK(b.dim() >= 2 && b.size(-1) == HV, "b head dimension must match HV");
  TORCH_CHECK(A_log.numel() == HV && dt_bias.numel() == gate_width, "A_log/dt_bias head dimensions must match HV and the gate type");
  check_pool(state, HV, V, K);
  check_pool(cache, HV, V, K);
  const auto state_dtype = state.has_value() ? state->scalar_type() : cache.has_value() ? cache->scalar_type() : at::kFloat;
  TORCH_CHECK(state_dtype == at::kFloat || state_dtype == at::kBFloat16, "k-last state dtype must be float32 or bfloat16, got ",
              state_dtype);
  TORCH_CHECK(!cache.has_value() || cache->scalar_type() == state_dtype,
              "initial_state_source and intermediate_states_buffer must have the same dtype");

  const int64_t B = cu_seqlens.has_value() ? cu_seqlens->size(0) - 1 : k.size(0);
  const bool target_verify = cache.has_value() || intermediate_state_indices.has_value() || retrieve_parent_token.has_value() ||
                             has_cache_steps || vllm_spec;
  const int64_t T_max = cu_seqlens.has_value() ? packed_t_max(k, B, target_verify, cache_steps, vllm_spec ? idx->size(1) : 0)
                                               : k.size(1);
  TORCH_CHECK(K == 128 && V == 128, "fused_sigmoid_gating_delta_rule_forward_k_last requires head_dim K == V == 128, got K=", K,
              ", V=", V);
  TORCH_CHECK(q.is_cuda(), "q must be a CUDA tensor");
  const auto act = q.scalar_type();
  TORCH_CHECK(act == at::kBFloat16 || act == at::kHalf, "q must be fp16 or bf16");
  TORCH_CHECK(k.scalar_type() == act && v.scalar_type() == act && a.scalar_type() == act && b.scalar_type() == act,
              "q, k, v, a, b must share one dtype");
  const float scale_val = scale.has_value() ? (float)*scale : 1.0f / std::sqrt((float)K);

  // the caller's `out`, or a new tensor shaped like v (fused_sigmoid_gating_cuda_k_last.cpp:146-159)
  Tensor o;
  if (out.has_value()) {
    o = *out;
    TORCH_CHECK(o.device() == v.device(), "out must be on the same device as v, got ", o.device(), " vs ", v.device());
    TORCH_CHECK(o.scalar_type() == act, "out dtype must match v (", act, "), got ", o.scalar_type());
    TORCH_CHECK(o.sizes() == v.sizes(), "out shape must match v ", v.sizes(), ", got ", o.sizes());
    TORCH_CHECK(o.is_contiguous(), "out must be contiguous");
  } else {
    o = torch::empty(v.sizes(), v.options());
  }

  // KDA gates come as [.., HV, K] or flattened [.., HV*K] (fused_sigmoid_gating_cuda_k_last.cpp:347-350)
  const int64_t stride_a = a.dim() == 4 ? a.stride(1) : a_tokens_heads_dim ? a.stride(0) : a.stride(a.dim() - 2);
  const bool mtp_verify = T_max > 1 || disable_state_update || target_verify;
  const auto want_dt = (is_kda && mtp_verify) ? at::kFloat : act;
  TORCH_CHECK(dt_bias.scalar_type() == want_dt, "dt_bias must be ", want_dt, " here (is_kda=", is_kda, ", mtp_verify=", mtp_verify,
              "): only KDA MTP verify reads it as float32, every other path reads it as q's dtype. Got ", dt_bias.scalar_type());
  if (cu_seqlens.has_value()) TORCH_CHECK(cu_seqlens->scalar_type() == at::kInt, "cu_seqlens's data type should be torch::kInt32");
  if (idx.has_value()) TORCH_CHECK(idx->scalar_type() == at::kInt, "initial_state_indices's data type should be torch::kInt32");
  if (intermediate_state_indices.has_value())
    TORCH_CHECK(intermediate_state_indices->scalar_type() == at::kInt && intermediate_state_indices->is_contiguous() &&
                    intermediate_state_indices->numel() >= B,
                "intermediate_state_indices must be contiguous int32 [B]");
  OptTensor parents = retrieve_parent_token;
  int64_t parent_seq_stride = 0, parent_token_stride = 0;
  if (parents.has_value()) {
    TORCH_CHECK(parents->scalar_type() == at::kLong || parents->scalar_type() == at::kInt,
                "retrieve_parent_token dtype should be int32 or int64");
    if (parents->scalar_type() != at::kLong) parents = parents->to(at::kLong);      // sglang's graph path allocates int32
    parent_seq_stride = parents->stride(0);
    parent_token_stride = parents->stride(1);
  }
  if (cache.has_value()) {
    TORCH_CHECK(cache->is_contiguous(), "intermediate_states_buffer must be contiguous");
    TORCH_CHECK(reinterpret_cast<uintptr_t>(cache->data_ptr()) % 16 == 0, "intermediate cache base requires 16-byte vector alignment");
  }
  // the request pitch of the cache is its allocated step dimension, not the number of draft tokens of this call
  // (fused_sigmoid_gating_cuda_k_last.cpp:407-413)
  const int64_t cache_steps_eff = cache.has_value() && cache->dim() >= 5 ? cache->size(1) : cache_steps;
  const int rpw = rows_per_wave(tile, HV, H, V);
  const auto token_stride = [](const Tensor& t) { return t.dim() == 4 ? t.stride(1) : t.stride(0); };
  launched(pla_k_last_launch(
      A_log.data_ptr(), dtype_code(A_log.scalar_type()), a.data_ptr(), dt_bias.data_ptr(), dt_bias.scalar_type() == at::kFloat ? 1 : 0,
      (float)(lower_bound.has_value() ? *lower_bound : softplus_beta), (float)softplus_threshold,
      lower_bound.has_value() ? PLA_GATE_LOWER_BOUND : PLA_GATE_SOFTPLUS, q.data_ptr(), k.data_ptr(), v.data_ptr(), b.data_ptr(), 0,
      o.data_ptr(), const_cast<void*>(ptr(state)), dtype_code(state_dtype), static_cast<const int32_t*>(ptr(cu_seqlens)),
      const_cast<void*>(ptr(cache)), static_cast<const int32_t*>(ptr(idx)),
      static_cast<const int32_t*>(ptr(intermediate_state_indices)), (int)cache_steps_eff,
      static_cast<const int64_t*>(ptr(parents)), parent_seq_stride, parent_token_stride, scale_val, (int)T_max, stride_a,
      token_stride(q), token_stride(k), token_stride(v), b.stride(b.dim() - 2), state.has_value() ? state->stride(0) : 0, (int)B,
      (int)H, (int)HV, (int)K, (int)V, use_qk_l2norm_in_kernel ? 1 : 0, disable_state_update ? 1 : 0,
      static_cast<const int32_t*>(ptr(num_accepted)), stride_idx_seq, is_sglang ? 1 : 0, is_kda ? 1 : 0, dtype_code(act), rpw,
      stream_of(q)));
  return o;
}

// Recurrent KDA decode from raw gate / beta projections (vLLM's fused_recurrent_kda plus a trailing is_sglang;
// reference wrapper src/decode/k-last/fused_recurrent_kda.cpp:146-314): argument problems raise ValueError or
// NotImplementedError as there, dt_bias is float32 and is narrowed to the activation dtype only for the pure-decode
// path, a 2-D per-token slot table sets disable_state_update.  Returns (out, initial_state).
std::pair<Tensor, Tensor> fused_recurrent_kda(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& raw_g,
                                              const Tensor& raw_beta, const Tensor& A_log, const OptTensor& dt_bias,
                                              std::optional<double> lower_bound, const Tensor& initial_state, const Tensor& cu_seqlens,
                                              const Tensor& ssm_state_indices, const OptTensor& num_accepted_tokens,
                                              const OptTensor& out, std::optional<bool> fuse_gate, bool is_sglang) {
  namespace py = pybind11;
  auto value_error = [](const std::string& m) { return py::value_error(m); };
  auto not_implemented = [](const std::string& m) { PyErr_SetString(PyExc_NotImplementedError, m.c_str()); return py::error_already_set(); };
  if (fuse_gate.has_value() && !*fuse_gate)
    throw not_implemented("pla.decode.kda.fused_recurrent_kda only implements the fused-gate path (fuse_gate=True): pass the raw "
                          "gate projection plus A_log/dt_bias and drop the separate _fused_kda_gate_beta call.");
  if (!dt_bias.has_value()) throw value_error("dt_bias is required by the fused-gate kernel path.");
  if (q.dim() != 4) throw value_error("q must be packed as [1, T, H, K], got " + std::to_string(q.dim()) + "D.");
  const int64_t B = q.size(0), T = q.size(1), H = q.size(2), K = q.size(3), V = v.size(-1);
  if (B != 1) throw value_error("q must be packed as [1, T, H, K], got batch " + std::to_string(B) + ".");
  if (K != 128 || V != 128)
    throw not_implemented("pla.decode.kda.fused_recurrent_kda requires head_dim K == V == 128, got K=" + std::to_string(K) +
                          ", V=" + std::to_string(V) + ".");
  auto torch_name = [](at::ScalarType t) { return std::string("torch.") + (t == at::kHalf ? "float16" : t == at::kBFloat16 ? "bfloat16" :
                                           t == at::kFloat ? "float32" : t == at::kDouble ? "float64" : c10::toString(t)); };
  if (initial_state.scalar_type() != at::kFloat) throw value_error("initial_state must be float32, got " + torch_name(initial_state.scalar_type()) + ".");
  if (ssm_state_indices.dim() != 1 && ssm_state_indices.dim() != 2)
    throw value_error("ssm_state_indices must be 1D or 2D, got " + std::to_string(ssm_state_indices.dim()) + "D");
  const bool per_token_slots = ssm_state_indices.dim() == 2;
  if (per_token_slots && is_sglang)
    throw value_error("a 2D ssm_state_indices is the vLLM spec-decode layout; sglang uses a 1D table plus its own "
                      "intermediate-state buffer.");
  if (dt_bias->scalar_type() != at::kFloat) throw value_error("dt_bias must be float32, got " + torch_name(dt_bias->scalar_type()) + ".");

  const at::ScalarType act = q.scalar_type();
  const Tensor a = raw_g.reshape({B * T, H * K}).to(act).contiguous();
  const Tensor b = raw_beta.reshape({B * T, H}).to(act).contiguous();
  const Tensor k_c = k.contiguous();
  const Tensor cu32 = cu_seqlens.to(at::kInt);
  const Tensor idx = ssm_state_indices.to(at::kInt).contiguous();
  Tensor dt = dt_bias->reshape({H, K});
  // whether the k-last call takes the MTP-verify path, which reads dt_bias as float32
  // (src/decode/k-last/fused_sigmoid_gating_cuda_k_last.cpp:225-236)
  const int64_t t_max = packed_t_max(k_c, cu32.size(0) - 1, per_token_slots, 0, per_token_slots ? idx.size(1) : 0);
  if (!(t_max > 1 || per_token_slots)) dt = dt.to(act);
  dt = dt.contiguous();
  StepsOrAccepted accepted;
  if (num_accepted_tokens.has_value()) accepted = std::variant<Tensor, int64_t>(num_accepted_tokens->to(at::kInt).contiguous());
  Tensor o = k_last_impl(A_log.reshape({-1}).contiguous(), a, dt, 1.0, 20.0, q.contiguous(), k_c, v.contiguous(), b, initial_state, idx,
                         1.0 / std::sqrt((double)K), true, cu32, true, per_token_slots, std::nullopt, std::nullopt, accepted,
                         std::nullopt, lower_bound, is_sglang, std::nullopt, std::nullopt);
  if (out.has_value()) {
    out->copy_(o);
    o = *out;
  }
  return {o, initial_state};
}

// Causal conv1d update + SiLU, gate, delta-rule recurrence and optional gated RMSNorm in one launch: the checks of
// the reference entry (src/decode/k-last/fused_kda_decode_mega_host.cpp:77-300), RuntimeError before anything is
// written; conv_state, state and out are updated in place.
void fused_kda_decode_mega_forward(const Tensor& x, const Tensor& weight, const OptTensor& bias, const Tensor& conv_state,
                                   const Tensor& raw_g, const Tensor& raw_beta, const Tensor& a_log, const Tensor& dt_bias,
                                   const Tensor& state_indices, const Tensor& state, const Tensor& out,
                                   std::optional<double> lower_bound, const OptTensor& output_gate, const OptTensor& norm_weight,
                                   double norm_eps) {
  if (bypass()) return;
  constexpr int64_t D = 128, W = 4;
  TORCH_CHECK(x.is_cuda(), "x must be a CUDA tensor");
  const at::ScalarType act = x.scalar_type();
  TORCH_CHECK(act == at::kBFloat16 || act == at::kHalf, "x must be a bfloat16 or float16 tensor");
  TORCH_CHECK(weight.is_cuda() && weight.scalar_type() == at::kFloat, "weight must be a CUDA float32 tensor");
  TORCH_CHECK(conv_state.is_cuda() && conv_state.scalar_type() == act, "conv_state must be a CUDA tensor with the same dtype as x");
  TORCH_CHECK(raw_g.is_cuda() && raw_g.scalar_type() == act, "raw_g must be a CUDA tensor with the same dtype as x");
  TORCH_CHECK(raw_beta.is_cuda() && raw_beta.scalar_type() == act, "raw_beta must be a CUDA tensor with the same dtype as x");
  TORCH_CHECK(a_log.is_cuda() && a_log.scalar_type() == at::kFloat, "A_log must be a CUDA float32 tensor");
  TORCH_CHECK(dt_bias.is_cuda() && dt_bias.scalar_type() == at::kFloat, "dt_bias must be a CUDA float32 tensor");
  TORCH_CHECK(state.is_cuda() && state.scalar_type() == at::kFloat, "state must be a CUDA float32 tensor");
  TORCH_CHECK(out.is_cuda() && out.scalar_type() == act, "out must be a CUDA tensor with the same dtype as x");
  TORCH_CHECK(state_indices.is_cuda() && state_indices.scalar_type() == at::kInt, "state_indices must be a CUDA int32 tensor");
  TORCH_CHECK(x.dim() == 2 && x.size(1) % (3 * D) == 0, "x must have shape [B, 3 * H * 128]");
  const int64_t B = x.size(0), H = x.size(1) / (3 * D);
  bool known = false;
  for (int64_t h : {4, 6, 8, 12, 16, 24, 48, 64, 96}) known = known || h == H;
  TORCH_CHECK(known, "H must be 4, 6, 8, 12, 16, 24, 48, 64, or 96, got ", H);
  TORCH_CHECK(B > 0, "KDA decode fusion requires at least one row");
  const int64_t dim = H * D;
  TORCH_CHECK(weight.dim() == 3 && weight.is_contiguous() && weight.size(0) == 3 && weight.size(1) == W && weight.size(2) == dim,
              "weight must have shape [3, 4, H * 128]");
  TORCH_CHECK(conv_state.dim() == 3 && conv_state.size(1) == 3 * dim && conv_state.size(2) == W - 1,
              "conv_state must have shape [slots, 3 * H * 128, 3]");
  TORCH_CHECK(raw_g.dim() == 4 && raw_g.size(0) == 1 && raw_g.size(1) == B && raw_g.size(2) == H && raw_g.size(3) == D,
              "raw_g must have shape [1, B, H, 128]");
  TORCH_CHECK(raw_beta.dim() == 3 && raw_beta.size(0) == 1 && raw_beta.size(1) == B && raw_beta.size(2) == H,
              "raw_beta must have shape [1, B, H]");
  TORCH_CHECK(a_log.is_contiguous() && a_log.numel() == H, "A_log must be contiguous with H elements");
  TORCH_CHECK(dt_bias.is_contiguous() && dt_bias.numel() == dim, "dt_bias must be contiguous with H * 128 elements");
  TORCH_CHECK(state_indices.is_contiguous() && state_indices.numel() == B, "state_indices must be contiguous with B elements");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D && state.size(3) == D,
              "state must have shape [slots, H, 128, 128]");
  TORCH_CHECK(out.dim() == 4 && out.size(0) == 1 && out.size(1) == B && out.size(2) == H && out.size(3) == D,
              "out must have shape [1, B, H, 128]");
  TORCH_CHECK(x.stride(1) == 1, "x must be contiguous in its channel dimension");
  TORCH_CHECK(conv_state.stride(0) >= 3 * dim * (W - 1) && conv_state.stride(1) == 1 && conv_state.stride(2) == 3 * dim,
              "conv_state must use the SD cache layout");
  TORCH_CHECK(state.stride(0) >= H * D * D && state.stride(1) == D * D && state.stride(2) == D && state.stride(3) == 1,
              "state must have contiguous [H, 128, 128] slot contents");
  TORCH_CHECK(raw_g.is_contiguous(), "raw_g must be contiguous");
  TORCH_CHECK(raw_beta.stride(2) == 1, "raw_beta must be contiguous in its head dimension");
  TORCH_CHECK(out.is_contiguous(), "out must be contiguous");
  const bool apply_onorm = output_gate.has_value();
  TORCH_CHECK(apply_onorm == norm_weight.has_value(), "output_gate and norm_weight must be provided together");
  int64_t onorm_row = 0;
  if (apply_onorm) {
    TORCH_CHECK(output_gate->is_cuda() && output_gate->scalar_type() == act, "output_gate must be a CUDA tensor with the same dtype as x");
    const bool gate_3d = output_gate->dim() == 3 && output_gate->size(0) == B && output_gate->size(1) == H && output_gate->size(2) == D;
    const bool gate_4d = output_gate->dim() == 4 && output_gate->size(0) == 1 && output_gate->size(1) == B && output_gate->size(2) == H &&
                         output_gate->size(3) == D;
    TORCH_CHECK(gate_3d || gate_4d, "output_gate must have shape [B, H, 128] or [1, B, H, 128]");
    const int row_dim = gate_3d ? 0 : 1;
    TORCH_CHECK(output_gate->stride(-1) == 1, "output_gate must be contiguous in its last dimension");
    TORCH_CHECK(output_gate->stride(row_dim + 1) == D, "output_gate must have contiguous head rows");
    TORCH_CHECK(norm_weight->is_cuda() && norm_weight->scalar_type() == at::kFloat, "norm_weight must be a CUDA float32 tensor");
    TORCH_CHECK(norm_weight->is_contiguous() && norm_weight->numel() == D, "norm_weight must be contiguous with 128 elements");
    TORCH_CHECK(norm_eps >= 0.0, "norm_eps must be non-negative");
    onorm_row = output_gate->stride(row_dim);
  }
  if (bias.has_value()) {
    TORCH_CHECK(bias->is_cuda() && bias->scalar_type() == at::kFloat, "bias must be a CUDA float32 tensor");
    TORCH_CHECK(bias->is_contiguous() && bias->numel() == 3 * dim, "bias must be contiguous with 3 * H * 128 elements");
  }
  const int64_t eb = x.element_size();
  const char* xp = static_cast<const char*>(x.data_ptr());
  const char* wp = static_cast<const char*>(weight.data_ptr());
  char* cp = static_cast<char*>(conv_state.data_ptr());
  const int64_t seg_b = dim * eb, wseg_b = dim * W * 4, cseg_b = dim * conv_state.stride(1) * eb;
  const char* bp = bias.has_value() ? static_cast<const char*>(bias->data_ptr()) : nullptr;
  const c10::DeviceGuard guard(x.device());
  launched(pla_kda_decode_mega_launch(
      dtype_code(act), apply_onorm ? 1 : 0, lower_bound.has_value() ? 1 : 0, a_log.data_ptr<float>(), raw_g.data_ptr(),
      dt_bias.data_ptr<float>(), xp, xp + seg_b, xp + 2 * seg_b, raw_beta.data_ptr(),
      reinterpret_cast<const float*>(wp), reinterpret_cast<const float*>(wp + wseg_b), reinterpret_cast<const float*>(wp + 2 * wseg_b),
      reinterpret_cast<const float*>(bp), bp ? reinterpret_cast<const float*>(bp + dim * 4) : nullptr,
      bp ? reinterpret_cast<const float*>(bp + 2 * dim * 4) : nullptr, cp, cp + cseg_b, cp + 2 * cseg_b, ptr(output_gate),
      static_cast<const float*>(ptr(norm_weight)), (float)norm_eps, state.data_ptr<float>(), state_indices.data_ptr<int32_t>(),
      out.data_ptr(), 1.0f / std::sqrt((float)D), lower_bound.has_value() ? (float)*lower_bound : 0.f, (int)B, (int)H, (int)H,
      x.stride(0), raw_beta.stride(1), onorm_row, conv_state.stride(0), state.stride(0), stream_of(x)));
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  namespace py = pybind11;
  m.def("fused_kda_decode_mega_forward", &fused_kda_decode_mega_forward,
        "KDA decode step fused on gfx950: conv1d update + SiLU, gate, recurrence, optional gated RMSNorm (vLLM contract)",
        py::arg("x"), py::arg("weight"), py::arg("bias") = py::none(), py::arg("conv_state"), py::arg("raw_g"), py::arg("raw_beta"),
        py::arg("a_log"), py::arg("dt_bias"), py::arg("state_indices"), py::arg("state"), py::arg("out"),
        py::arg("lower_bound") = py::none(), py::arg("output_gate") = py::none(), py::arg("norm_weight") = py::none(),
        py::arg("norm_eps") = 1e-5);
  m.def("fused_recurrent_kda", &fused_recurrent_kda,
        "Recurrent KDA decode from raw gate / beta (vLLM fused_recurrent_kda contract; is_sglang selects the sglang pad-slot "
        "convention).  Returns (out, initial_state); the state pool is updated in place.",
        py::arg("q"), py::arg("k"), py::arg("v"), py::arg("raw_g"), py::arg("raw_beta"), py::arg("A_log"), py::arg("dt_bias"),
        py::arg("lower_bound"), py::arg("initial_state"), py::arg("cu_seqlens"), py::arg("ssm_state_indices"),
        py::arg("num_accepted_tokens") = py::none(), py::arg("out") = py::none(), py::arg("fuse_gate") = py::none(),
        py::arg("is_sglang") = false);
  m.doc() = "pla.decode._C for MI355X: k-last gated delta-rule decode and MTP verify over libpla_gfx950.so";
  m.def(
      "fused_sigmoid_gating_delta_rule_forward_k_last",
      [](const Tensor& A_log, const Tensor& a, const Tensor& dt_bias, double softplus_beta, double softplus_threshold,
         const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& b, const OptTensor& initial_state_source,
         const OptTensor& initial_state_indices, std::optional<double> scale, bool use_qk_l2norm_in_kernel,
         const OptTensor& cu_seqlens, bool is_kda, bool disable_state_update, const OptTensor& intermediate_states_buffer,
         const OptTensor& intermediate_state_indices, const StepsOrAccepted& cache_steps_or_num_accept,
         const OptTensor& retrieve_parent_token, std::optional<double> lower_bound, std::optional<bool> is_sglang,
         const OptTensor& out) {
        return k_last_impl(A_log, a, dt_bias, softplus_beta, softplus_threshold, q, k, v, b, initial_state_source,
                           initial_state_indices, scale, use_qk_l2norm_in_kernel, cu_seqlens, is_kda, disable_state_update,
                           intermediate_states_buffer, intermediate_state_indices, cache_steps_or_num_accept,
                           retrieve_parent_token, lower_bound, is_sglang, out, std::nullopt);
      },
      py::arg("A_log"), py::arg("a"), py::arg("dt_bias"), py::arg("softplus_beta"), py::arg("softplus_threshold"), py::arg("q"),
      py::arg("k"), py::arg("v"), py::arg("b"), py::arg("initial_state_source"), py::arg("initial_state_indices"),
      py::arg("scale"), py::arg("use_qk_l2norm_in_kernel"), py::arg("cu_seqlens"), py::arg("is_kda"),
      py::arg("disable_state_update"), py::arg("intermediate_states_buffer"), py::arg("intermediate_state_indices"),
      py::arg("cache_steps_or_num_accept"), py::arg("retrieve_parent_token"), py::arg("lower_bound") = py::none(),
      py::arg("is_sglang") = py::none(), py::arg("out") = py::none());
  m.def(
      "fused_sigmoid_gating_delta_rule_forward_k_last_packed",
      [](const Tensor& mixed_qkv, const Tensor& a, const Tensor& b, const Tensor& A_log, const Tensor& dt_bias,
         double softplus_beta, double softplus_threshold, std::optional<double> scale, const OptTensor& initial_state_source,
         const OptTensor& initial_state_indices, Tensor out, bool use_qk_l2norm_in_kernel, const OptTensor& cu_seqlens,
         bool is_kda, std::optional<bool> is_sglang) {
        return packed_impl(mixed_qkv, a, b, A_log, dt_bias, softplus_beta, softplus_threshold, scale, initial_state_source,
                           initial_state_indices, out, use_qk_l2norm_in_kernel, cu_seqlens, is_kda, is_sglang, std::nullopt);
      },
      py::arg("mixed_qkv"), py::arg("a"), py::arg("b"), py::arg("A_log"), py::arg("dt_bias"), py::arg("softplus_beta"),
      py::arg("softplus_threshold"), py::arg("scale"), py::arg("initial_state_source"), py::arg("initial_state_indices"),
      py::arg("out"), py::arg("use_qk_l2norm_in_kernel"), py::arg("cu_seqlens"), py::arg("is_kda"),
      py::arg("is_sglang") = py::none());
  m.def(
      "fused_sigmoid_gating_delta_rule_forward_k_last_tunable",
      [](const Tensor& A_log, const Tensor& a, const Tensor& dt_bias, double softplus_beta, double softplus_threshold,
         const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& b, const OptTensor& initial_state_source,
         const OptTensor& initial_state_indices, std::optional<double> scale, bool use_qk_l2norm_in_kernel,
         const OptTensor& cu_seqlens, bool is_kda, bool disable_state_update, const OptTensor& intermediate_states_buffer,
         const OptTensor& intermediate_state_indices, const StepsOrAccepted& cache_steps_or_num_accept,
         const OptTensor& retrieve_parent_token, int64_t bv, int64_t wn, int64_t sn, int64_t hv_per_cta,
         std::optional<bool> is_sglang, std::optional<double> lower_bound, const OptTensor& out) {
        return k_last_impl(A_log, a, dt_bias, softplus_beta, softplus_threshold, q, k, v, b, initial_state_source,
                           initial_state_indices, scale, use_qk_l2norm_in_kernel, cu_seqlens, is_kda, disable_state_update,
                           intermediate_states_buffer, intermediate_state_indices, cache_steps_or_num_accept,
                           retrieve_parent_token, lower_bound, is_sglang, out, std::array<int64_t, 4>{bv, wn, sn, hv_per_cta});
      },
      py::arg("A_log"), py::arg("a"), py::arg("dt_bias"), py::arg("softplus_beta"), py::arg("softplus_threshold"), py::arg("q"),
      py::arg("k"), py::arg("v"), py::arg("b"), py::arg("initial_state_source"), py::arg("initial_state_indices"),
      py::arg("scale"), py::arg("use_qk_l2norm_in_kernel"), py::arg("cu_seqlens"), py::arg("is_kda"),
      py::arg("disable_state_update"), py::arg("intermediate_states_buffer"), py::arg("intermediate_state_indices"),
      py::arg("cache_steps_or_num_accept"), py::arg("retrieve_parent_token"), py::arg("bv"), py::arg("wn"), py::arg("sn"),
      py::arg("hv_per_cta"), py::arg("is_sglang") = py::none(), py::arg("lower_bound") = py::none(), py::arg("out") = py::none());
  m.def(
      "fused_sigmoid_gating_delta_rule_forward_k_last_packed_tunable",
      [](const Tensor& mixed_qkv, const Tensor& a, const Tensor& b, const Tensor& A_log, const Tensor& dt_bias,
         double softplus_beta, double softplus_threshold, std::optional<double> scale, const OptTensor& initial_state_source,
         const OptTensor& initial_state_indices, Tensor out, bool use_qk_l2norm_in_kernel, const OptTensor& cu_seqlens,
         bool is_kda, int64_t bv, int64_t wn, int64_t sn, int64_t hv_per_cta, std::optional<bool> is_sglang) {
        return packed_impl(mixed_qkv, a, b, A_log, dt_bias, softplus_beta, softplus_threshold, scale, initial_state_source,
                           initial_state_indices, out, use_qk_l2norm_in_kernel, cu_seqlens, is_kda, is_sglang,
                           std::array<int64_t, 4>{bv, wn, sn, hv_per_cta});
      },
      py::arg("mixed_qkv"), py::arg("a"), py::arg("b"), py::arg("A_log"), py::arg("dt_bias"), py::arg("softplus_beta"),
      py::arg("softplus_threshold"), py::arg("scale"), py::arg("initial_state_source"), py::arg("initial_state_indices"),
      py::arg("out"), py::arg("use_qk_l2norm_in_kernel"), py::arg("cu_seqlens"), py::arg("is_kda"), py::arg("bv"), py::arg("wn"),
      py::arg("sn"), py::arg("hv_per_cta"), py::arg("is_sglang") = py::none());
}
