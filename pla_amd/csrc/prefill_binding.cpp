// pla.prefill.flashqla._C and pla.prefill.flashkdapro._C: the compiled host layer of the two prefill namespaces, as
// the reference ships one extension module per namespace (setup.py:560,608; the FlashKDAPro facade calls
// _C.flashkda_fwd with 15 positional arguments, pla/prefill/flashkdapro/ops.py:215-219; the FlashQLA module binds
// its stage launchers, src/prefill/flashqla/host/torch_extension_cute.cc:1361-1427).  This file is compiled twice,
// once per module (PLA_BIND_FLASHQLA / PLA_BIND_FLASHKDAPRO).
//
// Division of work with the Python facades (pla_amd/prefill/*/ops.py): a facade hands every call to its module's
// try_* function first.  That function takes the call only if it is in the plain form a serving framework passes:
// tensors on one GPU, dense rows at the alignments the kernels read, FP32 k-last states, int32 metadata.  It then
// allocates the outputs and the workspace from torch's allocator and launches through the C ABI of
// libpla_gfx950.so on torch's current stream: no Python between the argument check and the launch.  For any other
// form it returns None and launches nothing; the facade then runs its own path, which holds the conversions
// (bf16 or strided states, int64 offsets), the diagnostics of PLA_SANITY_CHECK and every error message.  So a call
// is refused in one place only, and the compiled path never accepts what the facade would refuse: each predicate
// below is the facade's own check or stricter.

#include <torch/extension.h>
#include <c10/hip/HIPStream.h>

#include <cmath>
#include <cstdlib>
#include <optional>
#include <vector>

#include "../../include/pla_gfx950.h"

namespace {

using torch::Tensor;
using OptTensor = std::optional<Tensor>;

void* stream_of(const Tensor& t) { return c10::hip::getCurrentHIPStream(t.get_device()).stream(); }
void launched(int rc) { TORCH_CHECK(rc == 0, pla_last_error()); }
bool sanity_mode() {                      // read on every call, as the facades read it
  const char* v = std::getenv("PLA_SANITY_CHECK");
  return v && v[0] == '1' && v[1] == 0;
}
bool aligned(const Tensor& t, int bytes) { return reinterpret_cast<uintptr_t>(t.data_ptr()) % bytes == 0; }
bool same_gpu(const Tensor& t, const Tensor& ref) { return t.is_cuda() && t.device() == ref.device(); }
// [tokens, heads, 128] rows (the leading dims may be [1, tokens]): heads and features dense
bool token_rows(const Tensor& t, int64_t tokens, int64_t heads, int lead) {
  return t.dim() == lead + 3 && (lead == 0 || t.size(0) == 1) && t.size(lead) == tokens && t.size(lead + 1) == heads &&
         t.size(lead + 2) == 128 && t.stride(lead + 2) == 1 && t.stride(lead + 1) == 128;
}
bool plain_offsets(const OptTensor& cu, const Tensor& ref) {
  return cu.has_value() && same_gpu(*cu, ref) && cu->scalar_type() == at::kInt && cu->dim() == 1 && cu->numel() >= 2 &&
         cu->is_contiguous();
}
// host offsets, when given, must describe the same packed batch (the facade's rule); None is fine
bool plain_raw_offsets(const py::object& raw, int64_t batch, int64_t tokens, std::vector<int32_t>* values = nullptr) {
  if (raw.is_none()) return true;
  if (!py::isinstance<py::tuple>(raw) && !py::isinstance<py::list>(raw)) return false;
  const py::sequence seq = py::reinterpret_borrow<py::sequence>(raw);
  if ((int64_t)py::len(seq) != batch + 1) return false;
  if (values) values->reserve(batch + 1);
  int64_t before = 0;
  for (int64_t i = 0; i <= batch; ++i) {
    if (!py::isinstance<py::int_>(seq[i])) return false;
    const int64_t x = seq[i].cast<int64_t>();
    if ((i == 0 && x != 0) || x < before || x > tokens) return false;
    before = x;
    if (values) values->push_back((int32_t)x);
  }
  return true;
}
// FP32 k-last states [slots, heads, 128, 128] the kernels can address: a dense tile per (slot, head), slot pitch and
// base at 16 bytes
bool plain_states(const Tensor& t, const Tensor& ref, int64_t heads) {
  return same_gpu(t, ref) && t.scalar_type() == at::kFloat && t.dim() == 4 && t.size(1) == heads && t.size(2) == 128 &&
         t.size(3) == 128 && t.stride(3) == 1 && t.stride(2) == 128 && t.stride(1) == 128 * 128 && t.stride(0) % 4 == 0 &&
         aligned(t, 16);
}
bool plain_indices(const Tensor& t, const Tensor& ref, int64_t batch) {
  return same_gpu(t, ref) && t.scalar_type() == at::kInt && t.dim() == 1 && t.numel() == batch && t.is_contiguous();
}

#ifdef PLA_BIND_FLASHQLA
// ---------------------------------------------------------------------------------------------------------------
// GDN chunk-64 prefill: chunk_gated_delta_rule_fwd and gdn_prefill_packed_qkv_fwd (pla/prefill/flashqla/ops.py:225-248,
// 651-738 of the reference).  Returns (g_cum, workspace, o, None, final_state) or None.
struct GdnCall {
  const void* q; const void* k; const void* v;
  int64_t stride_q, stride_k, stride_v, tokens, Hg, H;
  at::ScalarType act;
  Tensor ref;                       // a tensor of the call (device, options)
};

py::object gdn_launch(const GdnCall& c, const OptTensor& g, const OptTensor& beta, const OptTensor& raw_gate_a,
                      const OptTensor& raw_beta_b, const OptTensor& A_log, const OptTensor& dt_bias, const Tensor& cu,
                      double scale, bool normalize_qk, const OptTensor& initial_state, const OptTensor& indices,
                      bool output_final_state, const std::vector<int32_t>& host_offsets) {
  const int64_t T = c.tokens, H = c.H, batch = cu.numel() - 1;
  const bool raw = raw_gate_a.has_value();
  if (raw) {
    if (!raw_beta_b || !A_log || !dt_bias || g || beta || !normalize_qk) return py::none();
    for (const Tensor* t : {&*raw_gate_a, &*raw_beta_b})
      if (!same_gpu(*t, c.ref) || t->scalar_type() != c.act || t->dim() != 2 || t->size(0) != T || t->size(1) != H || t->stride(1) != 1)
        return py::none();
    for (const Tensor* t : {&*A_log, &*dt_bias})
      if (!same_gpu(*t, c.ref) || t->scalar_type() != at::kFloat || t->numel() != H || !t->is_contiguous()) return py::none();
  } else {
    if (!g || !beta || raw_beta_b || A_log || dt_bias) return py::none();
    for (const Tensor* t : {&*g, &*beta})
      if (!same_gpu(*t, c.ref) || t->scalar_type() != at::kFloat || t->numel() != T * H || !t->is_contiguous() ||
          t->dim() != 3 || t->size(0) != 1 || t->size(1) != T)
        return py::none();
  }
  const bool indexed = indices.has_value();
  if (initial_state) {
    if (!plain_states(*initial_state, c.ref, H) || !initial_state->is_contiguous()) return py::none();
    if (!indexed && initial_state->size(0) < batch) return py::none();
  }
  if (indexed && (!initial_state || !plain_indices(*indices, c.ref, batch))) return py::none();

  const auto dev = c.ref.options();
  Tensor o = at::empty({1, T, H, 128}, dev.dtype(c.act));
  Tensor g_cum = at::empty({1, T, H}, dev.dtype(at::kFloat));
  const int64_t ws_bytes = pla_gdn_prefill_workspace_bytes((int)T, (int)batch, (int)c.Hg, (int)H);
  Tensor ws = at::empty({ws_bytes}, dev.dtype(at::kByte));
  const float* h0 = initial_state ? initial_state->data_ptr<float>() : nullptr;
  const int64_t h0_stride = initial_state ? initial_state->stride(0) : 0;
  float* ht = nullptr;
  int64_t ht_stride = 0;
  const int32_t* idx = indexed ? indices->data_ptr<int32_t>() : nullptr;
  Tensor final_state;
  if (indexed) {                                  // the pool is updated in place
    ht = initial_state->data_ptr<float>();
    ht_stride = h0_stride;
  } else if (output_final_state) {
    final_state = at::empty({batch, H, 128, 128}, dev.dtype(at::kFloat));
    // sequences of length zero keep their incoming state
    if (initial_state) final_state.copy_(initial_state->narrow(0, 0, batch));
    else final_state.zero_();
    ht = final_state.data_ptr<float>();
    ht_stride = final_state.stride(0);
  }
  launched(pla_gdn_prefill_launch_raw(
      c.q, c.k, c.v, c.stride_q, c.stride_k, c.stride_v,
      raw ? raw_gate_a->data_ptr() : nullptr, raw ? raw_beta_b->data_ptr() : nullptr, raw ? raw_gate_a->stride(0) : 0,
      raw ? raw_beta_b->stride(0) : 0, raw ? A_log->data_ptr<float>() : nullptr, raw ? dt_bias->data_ptr<float>() : nullptr,
      raw ? nullptr : g->data_ptr<float>(), raw ? nullptr : beta->data_ptr<float>(),
      cu.data_ptr<int32_t>(), (int)batch, (int)T, (float)scale, normalize_qk ? 1 : 0,
      h0, idx, h0_stride, ht, idx, ht_stride, o.data_ptr(), ws.data_ptr(), ws_bytes, g_cum.data_ptr<float>(),
      nullptr, (int)c.Hg, (int)H, 128, 128, c.act == at::kHalf ? PLA_F16 : PLA_BF16, stream_of(c.ref),
      host_offsets.empty() ? nullptr : host_offsets.data()));
  py::object final_obj = py::none();
  if (output_final_state) {
    if (indexed) final_obj = py::cast(initial_state->index_select(0, indices->to(at::kLong)));
    else final_obj = py::cast(final_state);
  }
  return py::make_tuple(g_cum, ws, o, py::none(), final_obj);
}

py::object try_chunk_gated_delta_rule_fwd(
    const Tensor& q, const Tensor& k, const Tensor& v, const OptTensor& g, const OptTensor& beta, std::optional<double> scale,
    const OptTensor& initial_state, const OptTensor& initial_state_indices, const OptTensor& cu_seqlens,
    bool output_final_state, const py::object& overlap_warmup_threshold, bool normalize_qk, const py::object& raw_cu_seqlens,
    const OptTensor& raw_gate_a, const OptTensor& raw_beta_b, const OptTensor& A_log, const OptTensor& dt_bias,
    const py::object& final_state_dtype) {
  if (sanity_mode() || !q.is_cuda()) return py::none();
  const at::ScalarType act = q.scalar_type();
  if ((act != at::kBFloat16 && act != at::kHalf) || k.scalar_type() != act || v.scalar_type() != act) return py::none();
  if (q.dim() != 4 || q.size(0) != 1 || q.size(1) == 0) return py::none();
  const int64_t T = q.size(1), Hg = q.size(2);
  if (v.dim() != 4 || Hg <= 0) return py::none();
  const int64_t H = v.size(2);
  if (H <= 0 || H % Hg != 0 || !token_rows(q, T, Hg, 1) || !token_rows(k, T, Hg, 1) || !token_rows(v, T, H, 1)) return py::none();
  if (!same_gpu(k, q) || !same_gpu(v, q)) return py::none();
  // q / k rows must start on 4-byte boundaries, v rows on 16-byte ones (the facade materialises other views)
  if (!aligned(q, 4) || q.stride(1) % 2 || !aligned(k, 4) || k.stride(1) % 2 || !aligned(v, 16) || v.stride(1) % 8) return py::none();
  if (!overlap_warmup_threshold.is_none()) {
    if (!py::isinstance<py::float_>(overlap_warmup_threshold) && !py::isinstance<py::int_>(overlap_warmup_threshold)) return py::none();
    if (!std::isfinite(overlap_warmup_threshold.cast<double>())) return py::none();
  }
  if (!plain_offsets(cu_seqlens, q)) return py::none();
  const int64_t batch = cu_seqlens->numel() - 1;
  std::vector<int32_t> host_offsets;
  if (!plain_raw_offsets(raw_cu_seqlens, batch, T, &host_offsets)) return py::none();
  if (!final_state_dtype.is_none()) {             // only the FP32 form is taken here
    const auto torch_mod = py::module_::import("torch");
    if (!final_state_dtype.is(torch_mod.attr("float32"))) return py::none();
  }
  GdnCall c{q.data_ptr(), k.data_ptr(), v.data_ptr(), q.stride(1), k.stride(1), v.stride(1), T, Hg, H, act, q};
  return gdn_launch(c, g, beta, raw_gate_a, raw_beta_b, A_log, dt_bias, *cu_seqlens, scale.value_or(1.0 / std::sqrt(128.0)),
                    normalize_qk, initial_state, initial_state_indices, output_final_state, host_offsets);
}

py::object try_gdn_prefill_packed_qkv_fwd(
    const Tensor& packed_qkv, const OptTensor& raw_gate_a, const OptTensor& raw_beta_b, const OptTensor& A_log,
    const OptTensor& dt_bias, const OptTensor& cu_seqlens, int64_t num_qk_heads, int64_t num_v_heads,
    std::optional<double> scale, const OptTensor& initial_state, const OptTensor& initial_state_indices,
    bool output_final_state, const py::object& overlap_warmup_threshold, const py::object& raw_cu_seqlens,
    const py::object& final_state_dtype) {
  if (sanity_mode() || !packed_qkv.is_cuda() || packed_qkv.dim() != 2 || packed_qkv.stride(1) != 1) return py::none();
  const at::ScalarType act = packed_qkv.scalar_type();
  if (act != at::kBFloat16 && act != at::kHalf) return py::none();
  const int64_t T = packed_qkv.size(0), Hg = num_qk_heads, H = num_v_heads;
  if (T == 0 || Hg <= 0 || H <= 0 || H % Hg != 0 || packed_qkv.size(1) != 2 * Hg * 128 + H * 128) return py::none();
  const int64_t pitch = packed_qkv.stride(0);
  if (pitch < packed_qkv.size(1) || pitch % 8 != 0 || !aligned(packed_qkv, 16)) return py::none();
  if (!raw_gate_a || !raw_beta_b || !A_log || !dt_bias) return py::none();
  if (!overlap_warmup_threshold.is_none()) {
    if (!py::isinstance<py::float_>(overlap_warmup_threshold) && !py::isinstance<py::int_>(overlap_warmup_threshold)) return py::none();
    if (!std::isfinite(overlap_warmup_threshold.cast<double>())) return py::none();
  }
  if (!plain_offsets(cu_seqlens, packed_qkv)) return py::none();
  std::vector<int32_t> host_offsets;
  if (!plain_raw_offsets(raw_cu_seqlens, cu_seqlens->numel() - 1, T, &host_offsets)) return py::none();
  if (!final_state_dtype.is_none()) {
    const auto torch_mod = py::module_::import("torch");
    if (!final_state_dtype.is(torch_mod.attr("float32"))) return py::none();
  }
  const char* base = static_cast<const char*>(packed_qkv.data_ptr());
  GdnCall c{base, base + Hg * 128 * 2, base + 2 * Hg * 128 * 2, pitch, pitch, pitch, T, Hg, H, act, packed_qkv};
  return gdn_launch(c, std::nullopt, std::nullopt, raw_gate_a, raw_beta_b, A_log, dt_bias, *cu_seqlens,
                    scale.value_or(1.0 / std::sqrt(128.0)), true, initial_state, initial_state_indices, output_final_state,
                    host_offsets);
}
#endif  // PLA_BIND_FLASHQLA

#ifdef PLA_BIND_FLASHKDAPRO
// ---------------------------------------------------------------------------------------------------------------
// KDA chunk-64 prefill: flashkda_fwd with the 15 positional arguments of the reference's _C.flashkda_fwd
// (pla/prefill/flashkdapro/ops.py:215-219).  True: launched; False: not in the plain form, nothing launched.
bool try_flashkda_fwd(const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& g, const Tensor& beta, const Tensor& A_log,
                      const Tensor& dt_bias, const Tensor& out, double scale, double lower_bound, const OptTensor& initial_state,
                      const OptTensor& final_state, const OptTensor& cu_seqlens, const OptTensor& state_indices,
                      const py::object& raw_cu_seqlens) {
  if (sanity_mode() || !q.is_cuda() || q.dim() != 3 || q.size(0) == 0) return false;
  const int64_t T = q.size(0), H = q.size(1);
  for (const Tensor* t : {&q, &k, &v, &g})
    if (!same_gpu(*t, q) || t->scalar_type() != at::kBFloat16 || !token_rows(*t, T, H, 0) || !aligned(*t, 16) || t->stride(0) % 8 != 0)
      return false;
  if (!same_gpu(beta, q) || beta.scalar_type() != at::kBFloat16 || beta.dim() != 2 || beta.size(0) != T || beta.size(1) != H ||
      beta.stride(1) != 1)
    return false;
  if (!same_gpu(A_log, q) || A_log.scalar_type() != at::kFloat || A_log.numel() != H || !A_log.is_contiguous()) return false;
  if (!same_gpu(dt_bias, q) || dt_bias.scalar_type() != at::kFloat || dt_bias.numel() != H * 128 || !dt_bias.is_contiguous()) return false;
  if (!same_gpu(out, q) || out.scalar_type() != at::kBFloat16 || out.dim() != 3 || out.size(0) != T || out.size(1) != H ||
      out.size(2) != 128 || !out.is_contiguous() || !aligned(out, 16))
    return false;
  if (!(lower_bound >= -5.0 && lower_bound <= 0.0)) return false;
  if (!plain_offsets(cu_seqlens, q)) return false;
  const int64_t N = cu_seqlens->numel() - 1;
  std::vector<int32_t> host_offsets;
  if (!plain_raw_offsets(raw_cu_seqlens, N, T, &host_offsets)) return false;
  const bool indexed = state_indices.has_value();
  if (indexed && (!plain_indices(*state_indices, q, N) || (!initial_state && !final_state))) return false;
  for (const OptTensor* t : {&initial_state, &final_state})
    if (t->has_value() && (!plain_states(**t, q, H) || (!indexed && (*t)->size(0) < N))) return false;
  if (final_state && final_state->data_ptr() == out.data_ptr()) return false;

  const int64_t ws_bytes = pla_kda_prefill_workspace_bytes((int)T, (int)N, (int)H);
  Tensor ws = at::empty({ws_bytes}, q.options().dtype(at::kByte));
  if (final_state && !(initial_state && final_state->data_ptr() == initial_state->data_ptr())) {
    // sequences of length zero keep their incoming (or zero) state
    if (indexed) {
      const Tensor rows = state_indices->to(at::kLong);
      if (initial_state) final_state->index_copy_(0, rows, initial_state->index_select(0, rows));
      else final_state->index_fill_(0, rows, 0);
    } else if (initial_state) {
      final_state->narrow(0, 0, N).copy_(initial_state->narrow(0, 0, N));
    } else {
      final_state->narrow(0, 0, N).zero_();
    }
  }
  const int32_t* idx = indexed ? state_indices->data_ptr<int32_t>() : nullptr;
  launched(pla_kda_prefill_launch_raw(
      q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), beta.data_ptr(), q.stride(0), k.stride(0), v.stride(0), g.stride(0),
      beta.stride(0), A_log.data_ptr<float>(), dt_bias.data_ptr<float>(), (float)lower_bound, (float)scale,
      cu_seqlens->data_ptr<int32_t>(), (int)N, (int)T,
      initial_state ? initial_state->data_ptr<float>() : nullptr, idx, initial_state ? initial_state->stride(0) : 0,
      final_state ? final_state->data_ptr<float>() : nullptr, idx, final_state ? final_state->stride(0) : 0,
      out.data_ptr(), ws.data_ptr(), ws_bytes, (int)H, 128, 128, PLA_BF16, stream_of(q),
      host_offsets.empty() ? nullptr : host_offsets.data()));
  return true;
}
#endif  // PLA_BIND_FLASHKDAPRO

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
#ifdef PLA_BIND_FLASHQLA
  m.doc() = "Compiled host layer of pla.prefill.flashqla (GDN chunk-64 prefill on gfx950)";
  m.def("try_chunk_gated_delta_rule_fwd", &try_chunk_gated_delta_rule_fwd,
        "chunk_gated_delta_rule_fwd for calls in the plain form; None (nothing launched) for any other",
        py::arg("q"), py::arg("k"), py::arg("v"), py::arg("g"), py::arg("beta"), py::arg("scale"), py::arg("initial_state"),
        py::arg("initial_state_indices"), py::arg("cu_seqlens"), py::arg("output_final_state"),
        py::arg("overlap_warmup_threshold"), py::arg("normalize_qk"), py::arg("raw_cu_seqlens"), py::arg("raw_gate_a"),
        py::arg("raw_beta_b"), py::arg("A_log"), py::arg("dt_bias"), py::arg("final_state_dtype"));
  m.def("try_gdn_prefill_packed_qkv_fwd", &try_gdn_prefill_packed_qkv_fwd,
        "gdn_prefill_packed_qkv_fwd for calls in the plain form; None (nothing launched) for any other",
        py::arg("packed_qkv"), py::arg("raw_gate_a"), py::arg("raw_beta_b"), py::arg("A_log"), py::arg("dt_bias"),
        py::arg("cu_seqlens"), py::arg("num_qk_heads"), py::arg("num_v_heads"), py::arg("scale"), py::arg("initial_state"),
        py::arg("initial_state_indices"), py::arg("output_final_state"), py::arg("overlap_warmup_threshold"),
        py::arg("raw_cu_seqlens"), py::arg("final_state_dtype"));
#endif
#ifdef PLA_BIND_FLASHKDAPRO
  m.doc() = "Compiled host layer of pla.prefill.flashkdapro (KDA chunk-64 prefill on gfx950)";
  m.def("try_flashkda_fwd", &try_flashkda_fwd,
        "flashkda_fwd for calls in the plain form: True when launched, False (nothing launched) for any other form",
        py::arg("q"), py::arg("k"), py::arg("v"), py::arg("g"), py::arg("beta"), py::arg("A_log"), py::arg("dt_bias"),
        py::arg("out"), py::arg("scale"), py::arg("lower_bound"), py::arg("initial_state"), py::arg("final_state"),
        py::arg("cu_seqlens"), py::arg("state_indices"), py::arg("raw_cu_seqlens"));
  // the reference's entry point: same 15 positional arguments, raises where it cannot take the call
  m.def("flashkda_fwd",
        [](const Tensor& q, const Tensor& k, const Tensor& v, const Tensor& g, const Tensor& beta, const Tensor& A_log,
           const Tensor& dt_bias, const Tensor& out, double scale, double lower_bound, const OptTensor& initial_state,
           const OptTensor& final_state, const OptTensor& cu_seqlens, const OptTensor& state_indices,
           const py::object& raw_cu_seqlens) {
          if (!try_flashkda_fwd(q, k, v, g, beta, A_log, dt_bias, out, scale, lower_bound, initial_state, final_state, cu_seqlens,
                                state_indices, raw_cu_seqlens))
            throw py::value_error("flashkda_fwd: the compiled entry point takes bf16 rows at 16-byte alignment, FP32 k-last "
                                  "states and int32 offsets on one GPU; pla.prefill.flashkdapro.flashkda_fwd converts other forms");
        },
        py::arg("q"), py::arg("k"), py::arg("v"), py::arg("g"), py::arg("beta"), py::arg("A_log"), py::arg("dt_bias"),
        py::arg("out"), py::arg("scale"), py::arg("lower_bound"), py::arg("initial_state"), py::arg("final_state"),
        py::arg("cu_seqlens"), py::arg("state_indices"), py::arg("raw_cu_seqlens"));
#endif
}
