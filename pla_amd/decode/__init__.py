"""k-last gated delta-rule decode and MTP verify on MI355X (``pla.decode`` drop-in).

Same function names, positional argument order, tensor contracts, ownership and
error behaviour as the reference's ``pla.decode`` extension
(src/decode/k-last/fused_sigmoid_gating.cpp:167-235; host logic
src/decode/k-last/fused_sigmoid_gating_cuda_k_last.cpp:239-435 and
src/decode/k-last/fused_sigmoid_gating_cuda_k_last_packed.cpp:82-204).
The work is done by hand-written gfx950 kernels behind the C ABI of
``libpla_gfx950.so``; the host side here only validates, derives shapes and
strides and launches on the current stream.  No allocation (except ``out`` of
the non-packed call when the caller passes none), no device-to-host copy, so
every call is graph-capturable.
"""

import os

import torch

from .. import _lib

__all__ = [
    "fused_sigmoid_gating_delta_rule_forward_k_last",
    "fused_sigmoid_gating_delta_rule_forward_k_last_packed",
]

_BYPASS = os.environ.get("PLA_BYPASS_EXEC", "0") == "1"   # read once, like src/bypass_exec.h:44-50

# The compiled host layer (pybind11 over the same C ABI; pla_amd/csrc/decode_binding.cpp): the two public entry
# points go through it, as the reference's facade goes through pla.decode._C.  It is imported on first use.  The
# Python implementations below are the same checks and the same launches through ctypes; they serve the
# PLA_SANITY_CHECK diagnostics (value checks that read tensors back), the tunable entry points' callers that
# pass a tile, and a tree in which only the library has been built (`python -m pla_amd.build` builds both).
_native = None


def _compiled():
    global _native
    if _native is None:
        try:
            # importlib, not `from . import _C`: the latter falls back to this module's __getattr__ when the
            # import fails and would recurse
            import importlib
            module = importlib.import_module("._C", __name__)
        except ModuleNotFoundError as exc:
            if exc.name is None or not exc.name.endswith("_C"):
                raise
            module = False
        _native = module
    return _native


def __getattr__(name):
    if name == "_C":
        module = _compiled()
        if module is False:
            raise ImportError("pla.decode._C is not built: run `python -m pla_amd.build`")
        return module
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


# Messages name dtypes and shapes the way the compiled host layer (and the reference's C++) prints them: the scalar
# type's name ("Half", "Float", "BFloat16") and sizes in brackets.
_CPP_DTYPE = {torch.float16: "Half", torch.bfloat16: "BFloat16", torch.float32: "Float", torch.float64: "Double",
              torch.int32: "Int", torch.int64: "Long", torch.int16: "Short", torch.int8: "Char", torch.uint8: "Byte",
              torch.bool: "Bool"}


def _dt(dtype):
    return _CPP_DTYPE.get(dtype, str(dtype))


def _sizes(shape):
    return "[" + ", ".join(str(int(n)) for n in shape) + "]"


def _sanity_enabled():
    # Read on every call (src/sanity_check.h:50-53).
    return os.environ.get("PLA_SANITY_CHECK", "0") == "1"


def _rows_per_wave_from_tile(bv, wn, sn, hv_per_cta, HV, H, V):
    """Map the reference's tunable tile tuple onto the one gfx950 tunable.

    The reference exposes (BV, WN, SN, HV_PER_CTA); on gfx950 the only tile
    parameter is the number of V-rows a wavefront owns.  A workgroup of four
    wavefronts covers ``bv`` rows, so rows_per_wave = bv / 4 clamped to {8,16,32}.
    The tuple is validated exactly like the reference does
    (fused_sigmoid_gating_cuda_k_last_packed.cpp:268-271).
    """
    _check(bv > 0 and wn > 0 and sn > 0 and V % bv == 0, "invalid k-last tile parameters")
    hv_per_h = HV // H
    _check(hv_per_cta > 0 and hv_per_cta <= hv_per_h and hv_per_h % hv_per_cta == 0,
           "HV_PER_CTA must divide HV/H")
    return 32 if bv >= 128 else 16 if bv >= 64 else 8


def _packed_heads(mixed_qkv, a, b, A_log, dt_bias, out, HV, K, V, is_kda):
    # src/decode/k-last/sanity_checks.h:60-82
    _check(mixed_qkv.dim() == 2, "mixed_qkv must have shape [tokens, qkv_width]")
    qk_width = mixed_qkv.size(1) - HV * V
    _check(qk_width > 0 and qk_width % (2 * K) == 0,
           "packed QKV width must equal 2*H*K + HV*V with H > 0")
    H = qk_width // (2 * K)
    _check(HV >= H and HV % H == 0, f"HV must be a positive multiple of H, got H={H}, HV={HV}")
    gate_width = HV * (K if is_kda else 1)
    _check(a.dim() >= 2 and a.size(-1) == gate_width, "a head dimensions must match HV and the gate type")
    _check(b.dim() >= 2 and b.size(-1) == HV, "b head dimension must match HV")
    _check(A_log.numel() == HV and dt_bias.numel() == gate_width,
           "A_log/dt_bias head dimensions must match HV and the gate type")
    _check(out.dim() >= 3 and out.size(-2) == HV and out.size(-1) == V
           and out.numel() == mixed_qkv.size(0) * HV * V,
           "out must match the packed token count and [HV, V]")
    return H


def _packed_impl(mixed_qkv, a, b, A_log, dt_bias, softplus_beta, softplus_threshold, scale,
                 initial_state_source, initial_state_indices, out, use_qk_l2norm_in_kernel,
                 cu_seqlens, is_kda, is_sglang, tile):
    if _BYPASS:
        return out
    is_sglang = True if is_sglang is None else bool(is_sglang)
    _check(initial_state_source is not None, "initial_state_source is required for k_last_packed")
    state = initial_state_source
    _check(state.dim() == 4, "initial_state_source must have shape [slots, HV, V, K]")
    HV, V, K = state.size(-3), state.size(-2), state.size(-1)
    _check(K == 128 and V == 128,
           "fused_sigmoid_gating_delta_rule_forward_k_last_packed requires "
           f"head_dim K == V == 128, got K={K}, V={V}")
    H = _packed_heads(mixed_qkv, a, b, A_log, dt_bias, out, HV, K, V, is_kda)
    _check(mixed_qkv.is_cuda, "mixed_qkv must be a CUDA tensor")
    _check(mixed_qkv.dtype in (torch.bfloat16, torch.float16), "mixed_qkv must be fp16 or bf16")
    _check(a.dtype == mixed_qkv.dtype and b.dtype == mixed_qkv.dtype and dt_bias.dtype == mixed_qkv.dtype
           and out.dtype == mixed_qkv.dtype, "a, b, dt_bias and out must have mixed_qkv's dtype")
    _check(state.dtype in (torch.float32, torch.bfloat16),
           f"k-last state dtype must be float32 or bfloat16, got {_dt(state.dtype)}")
    _check(mixed_qkv.stride(1) == 1 and state.stride(-1) == 1 and state.stride(-2) == K
           and state.stride(-3) == V * K, "mixed_qkv rows and state slots must be dense")
    _check(out.is_contiguous(), "out must be contiguous")
    B = cu_seqlens.size(0) - 1 if cu_seqlens is not None else mixed_qkv.size(0)
    if cu_seqlens is not None:
        _check(cu_seqlens.dtype == torch.int32, "cu_seqlens's data type should be torch::kInt32")
    if initial_state_indices is not None:
        _check(initial_state_indices.dtype == torch.int32,
               "initial_state_indices's data type should be torch::kInt32")
    if _sanity_enabled():
        from .._sanity import sanity_packed
        sanity_packed(mixed_qkv, a, b, A_log, dt_bias, state, initial_state_indices, out,
                      cu_seqlens, is_kda, is_sglang, B, H, HV)
    rpw = 0 if tile is None else _rows_per_wave_from_tile(*tile, HV, H, V)
    scale_val = float(scale) if scale is not None else K ** -0.5
    _lib.call(
        "pla_k_last_packed_launch",
        A_log.data_ptr(), _lib.dtype_code(A_log.dtype), a.data_ptr(), dt_bias.data_ptr(),
        float(softplus_beta), float(softplus_threshold),
        mixed_qkv.data_ptr(), b.data_ptr(), out.data_ptr(), state.data_ptr(), _lib.dtype_code(state.dtype),
        _lib.ptr(cu_seqlens), _lib.ptr(initial_state_indices),
        scale_val, 1,
        a.stride(a.dim() - 2), mixed_qkv.stride(0), b.stride(b.dim() - 2), state.stride(0),
        B, H, HV, K, V,
        int(bool(use_qk_l2norm_in_kernel)), int(is_sglang), int(bool(is_kda)),
        _lib.dtype_code(mixed_qkv.dtype), rpw, _lib.current_stream(mixed_qkv.device))
    return out


def fused_sigmoid_gating_delta_rule_forward_k_last_packed(
        mixed_qkv, a, b, A_log, dt_bias, softplus_beta, softplus_threshold, scale,
        initial_state_source, initial_state_indices, out, use_qk_l2norm_in_kernel,
        cu_seqlens, is_kda, is_sglang=None):
    """One-token GDN/KDA decode straight from ``mixed_qkv [tokens, 2*H*128 + HV*128]``.

    Updates ``initial_state_source[initial_state_indices[n]]`` in place, writes the
    caller's ``out`` and returns it.  A padded slot (``< 0`` for sglang, ``<= 0``
    otherwise) yields zeros and touches no state; a request of length zero
    touches nothing.
    """
    native = _compiled()
    if native and not _sanity_enabled():
        return native.fused_sigmoid_gating_delta_rule_forward_k_last_packed(
            mixed_qkv, a, b, A_log, dt_bias, softplus_beta, softplus_threshold, scale, initial_state_source,
            initial_state_indices, out, use_qk_l2norm_in_kernel, cu_seqlens, is_kda, is_sglang)
    return _packed_impl(mixed_qkv, a, b, A_log, dt_bias, softplus_beta, softplus_threshold, scale,
                        initial_state_source, initial_state_indices, out, use_qk_l2norm_in_kernel,
                        cu_seqlens, is_kda, is_sglang, None)


def _k_last_heads(q, k, v, a, b, A_log, dt_bias, state, cache, is_kda):
    # src/decode/k-last/fused_sigmoid_gating_cuda_k_last.cpp:57-97
    _check(q.dim() == 4 and k.dim() == 4 and v.dim() == 4, "q, k, v must have shape [B, T, heads, dim]")
    H, HV, K, V = k.size(2), v.size(2), k.size(3), v.size(3)
    _check(H > 0 and HV >= H and HV % H == 0, f"HV must be a positive multiple of H, got H={H}, HV={HV}")
    _check(q.shape == k.shape and v.size(0) == k.size(0) and v.size(1) == k.size(1),
           "q/k shapes and q/k/v token dimensions must match")
    gate_width = HV * K if is_kda else HV
    _check(a.dim() >= 2 and ((a.dim() == 4 and a.size(2) == HV and a.size(3) == (K if is_kda else 1))
                             or (is_kda and a.dim() == 3 and a.size(1) == HV and a.size(2) == K)
                             or (a.dim() != 4 and a.size(-1) == gate_width)),
           "a head dimensions must match HV and the gate type")
    _check(b.dim() >= 2 and b.size(-1) == HV, "b head dimension must match HV")
    _check(A_log.numel() == HV and dt_bias.numel() == gate_width,
           "A_log/dt_bias head dimensions must match HV and the gate type")
    for t in (state, cache):
        if t is not None:
            physical = t.dim() >= 4 and t.size(-3) == HV and t.size(-2) == V and t.size(-1) == K
            flattened = t.dim() >= 2 and t.stride(-1) == 1 and t.stride(0) >= HV * V * K
            _check(physical or flattened,
                   "state/cache head dimensions must match [HV, V, K], or be a flattened pool whose "
                   "stride(0) covers HV*V*K with a unit-stride innermost dim")
    return H, HV, K, V


def _packed_t_max(k, B, target_verify, cache_steps, logical_slot_columns):
    # src/decode/k-last/sanity_checks.h:84-112
    _check(B > 0, "k-last requires at least one sequence")
    if target_verify and logical_slot_columns > 0:
        return logical_slot_columns
    if k.size(0) == B:
        return k.size(1)
    if not target_verify and k.size(0) == 1 and k.size(1) == B:
        return 1
    if target_verify:
        if cache_steps > 0:
            return cache_steps
        _check(k.size(1) % B == 0, "packed target-verify tokens must be divisible by batch size")
        return k.size(1) // B
    return k.size(1)


def _resolve_out(out, v):
    # src/decode/k-last/fused_sigmoid_gating_cuda_k_last.cpp:146-159
    if out is None:
        return torch.empty(v.shape, dtype=v.dtype, device=v.device)
    _check(out.device == v.device, f"out must be on the same device as v, got {out.device} vs {v.device}")
    _check(out.dtype == v.dtype, f"out dtype must match v ({_dt(v.dtype)}), got {_dt(out.dtype)}")
    _check(out.shape == v.shape, f"out shape must match v {_sizes(v.shape)}, got {_sizes(out.shape)}")
    _check(out.is_contiguous(), "out must be contiguous")
    return out


def _token_stride(t):
    return t.stride(1) if t.dim() == 4 else t.stride(0)


def _k_last_impl(A_log, a, dt_bias, softplus_beta, softplus_threshold, q, k, v, b,
                 initial_state_source, initial_state_indices, scale, use_qk_l2norm_in_kernel,
                 cu_seqlens, is_kda, disable_state_update, intermediate_states_buffer,
                 intermediate_state_indices, cache_steps_or_num_accept, retrieve_parent_token,
                 lower_bound, is_sglang, out, tile):
    if _BYPASS:
        return out if out is not None else torch.zeros(v.shape, dtype=v.dtype, device=v.device)
    is_sglang = True if is_sglang is None else bool(is_sglang)
    _check(lower_bound is None or is_kda, "lower_bound is only supported for KDA")

    cache_steps, num_accepted, has_cache_steps = 0, None, False
    if cache_steps_or_num_accept is not None:
        if isinstance(cache_steps_or_num_accept, torch.Tensor):
            num_accepted = cache_steps_or_num_accept
            _check(num_accepted.dtype == torch.int32, "num_accepted_tokens's data type should be torch::kInt32")
        else:
            cache_steps, has_cache_steps = int(cache_steps_or_num_accept), True

    idx = initial_state_indices
    stride_idx_seq = idx.stride(0) if (idx is not None and idx.dim() == 2) else 0
    vllm_spec = stride_idx_seq > 0
    _check(not vllm_spec or not is_sglang,
           "2D initial_state_indices is the vLLM spec-decode layout; pass is_sglang=False")
    _check(not (vllm_spec and has_cache_steps),
           "vLLM spec decode expects num_accepted_tokens (a tensor) in "
           "cache_steps_or_num_accept, but received an int")

    state, cache = initial_state_source, intermediate_states_buffer
    H, HV, K, V = _k_last_heads(q, k, v, a, b, A_log, dt_bias, state, cache, is_kda)
    state_dtype = state.dtype if state is not None else (cache.dtype if cache is not None else torch.float32)
    _check(state_dtype in (torch.float32, torch.bfloat16),
           f"k-last state dtype must be float32 or bfloat16, got {_dt(state_dtype)}")
    _check(cache is None or cache.dtype == state_dtype,
           "initial_state_source and intermediate_states_buffer must have the same dtype")

    B = cu_seqlens.size(0) - 1 if cu_seqlens is not None else k.size(0)
    target_verify = (cache is not None or intermediate_state_indices is not None
                     or retrieve_parent_token is not None or has_cache_steps or vllm_spec)
    if cu_seqlens is not None:
        T_max = _packed_t_max(k, B, target_verify, cache_steps, idx.size(1) if vllm_spec else 0)
    else:
        T_max = k.size(1)
    _check(K == 128 and V == 128,
           "fused_sigmoid_gating_delta_rule_forward_k_last requires "
           f"head_dim K == V == 128, got K={K}, V={V}")
    _check(q.is_cuda, "q must be a CUDA tensor")
    _check(q.dtype in (torch.bfloat16, torch.float16), "q must be fp16 or bf16")
    _check(k.dtype == q.dtype and v.dtype == q.dtype and a.dtype == q.dtype and b.dtype == q.dtype,
           "q, k, v, a, b must share one dtype")
    scale_val = float(scale) if scale is not None else K ** -0.5
    o = _resolve_out(out, v)

    # KDA accepts [tokens, HV, K] and the flattened [tokens, HV*K]
    # (fused_sigmoid_gating_cuda_k_last.cpp:347-350).
    if a.dim() == 4:
        stride_a = a.stride(1)
    elif is_kda and a.dim() == 3 and a.size(1) == HV and a.size(2) == K:
        stride_a = a.stride(0)
    else:
        stride_a = a.stride(a.dim() - 2)

    mtp_verify = T_max > 1 or bool(disable_state_update) or target_verify
    want = torch.float32 if (is_kda and mtp_verify) else q.dtype
    _check(dt_bias.dtype == want,
           f"dt_bias must be {_dt(want)} here (is_kda={int(bool(is_kda))}, mtp_verify={int(bool(mtp_verify))}): only KDA MTP "
           f"verify reads it as float32, every other path reads it as q's dtype. Got {_dt(dt_bias.dtype)}")

    for name, t in (("cu_seqlens", cu_seqlens), ("initial_state_indices", idx)):
        if t is not None:
            _check(t.dtype == torch.int32, f"{name}'s data type should be torch::kInt32")
    if intermediate_state_indices is not None:
        _check(intermediate_state_indices.dtype == torch.int32 and intermediate_state_indices.is_contiguous()
               and intermediate_state_indices.numel() >= B,
               "intermediate_state_indices must be contiguous int32 [B]")
    parents = retrieve_parent_token
    sps = spt = 0
    if parents is not None:
        _check(parents.dtype in (torch.int64, torch.int32), "retrieve_parent_token dtype should be int32 or int64")
        if parents.dtype != torch.int64:
            parents = parents.to(torch.int64)      # sglang's graph path allocates int32
        sps, spt = parents.stride(0), parents.stride(1)
    if cache is not None:
        _check(cache.is_contiguous(), "intermediate_states_buffer must be contiguous")
        _check(cache.data_ptr() % 16 == 0, "intermediate cache base requires 16-byte vector alignment")
    # The request pitch of the cache is its allocated step dim, not the runtime
    # draft-token count (fused_sigmoid_gating_cuda_k_last.cpp:407-413).
    cache_steps_eff = cache.size(1) if (cache is not None and cache.dim() >= 5) else cache_steps

    if _sanity_enabled():
        from .._sanity import sanity_k_last
        sanity_k_last(q, k, v, a, b, A_log, dt_bias, state, idx, cu_seqlens, is_kda, cache,
                      intermediate_state_indices, num_accepted, parents, is_sglang, B, T_max, H, HV)

    rpw = 0 if tile is None else _rows_per_wave_from_tile(*tile, HV, H, V)
    if lower_bound is not None:
        gate_mode, p0 = _lib.GATE_LOWER_BOUND, float(lower_bound)
    else:
        gate_mode, p0 = _lib.GATE_SOFTPLUS, float(softplus_beta)
    _lib.call(
        "pla_k_last_launch",
        A_log.data_ptr(), _lib.dtype_code(A_log.dtype), a.data_ptr(), dt_bias.data_ptr(),
        int(dt_bias.dtype == torch.float32), p0, float(softplus_threshold), gate_mode,
        q.data_ptr(), k.data_ptr(), v.data_ptr(), b.data_ptr(), 0,
        o.data_ptr(), _lib.ptr(state), _lib.dtype_code(state_dtype), _lib.ptr(cu_seqlens), _lib.ptr(cache),
        _lib.ptr(idx), _lib.ptr(intermediate_state_indices), int(cache_steps_eff),
        _lib.ptr(parents), sps, spt, scale_val, int(T_max),
        stride_a, _token_stride(q), _token_stride(k), _token_stride(v), b.stride(b.dim() - 2),
        state.stride(0) if state is not None else 0,
        B, H, HV, K, V, int(bool(use_qk_l2norm_in_kernel)), int(bool(disable_state_update)),
        _lib.ptr(num_accepted), stride_idx_seq, int(is_sglang), int(bool(is_kda)),
        _lib.dtype_code(q.dtype), rpw, _lib.current_stream(q.device))
    return o


def fused_sigmoid_gating_delta_rule_forward_k_last(
        A_log, a, dt_bias, softplus_beta, softplus_threshold, q, k, v, b,
        initial_state_source, initial_state_indices, scale, use_qk_l2norm_in_kernel,
        cu_seqlens, is_kda, disable_state_update, intermediate_states_buffer,
        intermediate_state_indices, cache_steps_or_num_accept, retrieve_parent_token,
        lower_bound=None, is_sglang=None, out=None):
    """Non-packed GDN/KDA decode and MTP verify (chain, eagle tree, vLLM slot table).

    Modes are resolved exactly as the reference host does: a 2-D
    ``initial_state_indices`` selects vLLM spec decode (start slot = column
    ``max(num_accepted-1, 0)``, step ``t`` snapshot to slot ``table[n, t]`` when
    positive); an intermediate buffer with indices and an int ``cache_steps``
    selects SGLang verify (snapshot to ``cache[cache_idx, t]``);
    ``retrieve_parent_token`` adds the eagle-tree parent reload;
    ``disable_state_update`` suppresses the final write-back.
    """
    native = _compiled()
    if native and not _sanity_enabled():
        return native.fused_sigmoid_gating_delta_rule_forward_k_last(
            A_log, a, dt_bias, softplus_beta, softplus_threshold, q, k, v, b, initial_state_source,
            initial_state_indices, scale, use_qk_l2norm_in_kernel, cu_seqlens, is_kda, disable_state_update,
            intermediate_states_buffer, intermediate_state_indices, cache_steps_or_num_accept, retrieve_parent_token,
            lower_bound, is_sglang, out)
    return _k_last_impl(A_log, a, dt_bias, softplus_beta, softplus_threshold, q, k, v, b,
                        initial_state_source, initial_state_indices, scale, use_qk_l2norm_in_kernel,
                        cu_seqlens, is_kda, disable_state_update, intermediate_states_buffer,
                        intermediate_state_indices, cache_steps_or_num_accept, retrieve_parent_token,
                        lower_bound, is_sglang, out, None)
