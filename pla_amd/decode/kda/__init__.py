"""``pla.decode.kda`` drop-in: recurrent KDA decode from raw gate / beta projections, and the
fused conv + gate + recurrence + norm decode step.

``fused_recurrent_kda`` mirrors the reference wrapper src/decode/k-last/fused_recurrent_kda.cpp:146-314
(vLLM's ``fused_recurrent_kda`` signature plus a trailing ``is_sglang``): raises
``ValueError`` / ``NotImplementedError`` for the same argument problems, requires a
float32 ``dt_bias`` and narrows it to the activation dtype only for the pure-decode
path, and forwards to the k-last entry point with ``disable_state_update`` set when a
2-D per-token slot table is given.
"""

import os

import torch

from ... import _lib
from .. import fused_sigmoid_gating_delta_rule_forward_k_last, _packed_t_max

__all__ = ["fused_recurrent_kda", "fused_kda_decode_mega_forward"]

_BYPASS = os.environ.get("PLA_BYPASS_EXEC", "0") == "1"   # read once, like src/bypass_exec.h:44-50
_MEGA_HEADS = (4, 6, 8, 12, 16, 24, 48, 64, 96)

_SOFTPLUS_BETA = 1.0
_SOFTPLUS_THRESHOLD = 20.0


def _takes_mtp_path(k, cu_seqlens, state_indices, disable_state_update):
    # src/decode/k-last/fused_sigmoid_gating_cuda_k_last.cpp:225-236
    target_verify = state_indices.dim() == 2
    cols = state_indices.size(1) if target_verify else 0
    B = cu_seqlens.size(0) - 1
    t_max = _packed_t_max(k, B, target_verify, 0, cols)
    return t_max > 1 or disable_state_update or target_verify


def _native():
    """pla.decode._C when it is built and the PLA_SANITY_CHECK diagnostics are off (they live in the Python path)."""
    from .. import _compiled, _sanity_enabled
    module = _compiled()
    return module if module and not _sanity_enabled() else None


def fused_recurrent_kda(q, k, v, raw_g, raw_beta, A_log, dt_bias, lower_bound, initial_state,
                        cu_seqlens, ssm_state_indices, num_accepted_tokens=None, out=None,
                        fuse_gate=None, is_sglang=False):
    """Returns ``(out, initial_state)``; the state pool is updated in place."""
    native = _native()
    if native:
        return native.fused_recurrent_kda(q, k, v, raw_g, raw_beta, A_log, dt_bias, lower_bound, initial_state, cu_seqlens,
                                          ssm_state_indices, num_accepted_tokens, out, fuse_gate, is_sglang)
    return _fused_recurrent_kda_impl(q, k, v, raw_g, raw_beta, A_log, dt_bias, lower_bound, initial_state, cu_seqlens,
                                     ssm_state_indices, num_accepted_tokens, out, fuse_gate, is_sglang)


def _fused_recurrent_kda_impl(q, k, v, raw_g, raw_beta, A_log, dt_bias, lower_bound, initial_state,
                              cu_seqlens, ssm_state_indices, num_accepted_tokens, out, fuse_gate, is_sglang):
    if fuse_gate is not None and not fuse_gate:
        raise NotImplementedError(
            "pla.decode.kda.fused_recurrent_kda only implements the fused-gate path (fuse_gate=True): "
            "pass the raw gate projection plus A_log/dt_bias and drop the separate _fused_kda_gate_beta call.")
    if dt_bias is None:
        raise ValueError("dt_bias is required by the fused-gate kernel path.")
    if q.dim() != 4:
        raise ValueError(f"q must be packed as [1, T, H, K], got {q.dim()}D.")
    B, T, H, K = q.shape
    V = v.size(-1)
    if B != 1:
        raise ValueError(f"q must be packed as [1, T, H, K], got batch {B}.")
    if K != 128 or V != 128:
        raise NotImplementedError(
            f"pla.decode.kda.fused_recurrent_kda requires head_dim K == V == 128, got K={K}, V={V}.")
    if initial_state.dtype != torch.float32:
        raise ValueError(f"initial_state must be float32, got {initial_state.dtype}.")
    if ssm_state_indices.dim() not in (1, 2):
        raise ValueError(f"ssm_state_indices must be 1D or 2D, got {ssm_state_indices.dim()}D")
    per_token_slots = ssm_state_indices.dim() == 2
    if per_token_slots and is_sglang:
        raise ValueError("a 2D ssm_state_indices is the vLLM spec-decode layout; sglang uses a 1D table "
                         "plus its own intermediate-state buffer.")
    if dt_bias.dtype != torch.float32:
        raise ValueError(f"dt_bias must be float32, got {dt_bias.dtype}.")

    act = q.dtype
    a = raw_g.reshape(B * T, H * K).to(act).contiguous()
    b = raw_beta.reshape(B * T, H).to(act).contiguous()
    k_c = k.contiguous()
    cu32 = cu_seqlens.to(torch.int32)
    idx = ssm_state_indices.to(torch.int32).contiguous()
    dt = dt_bias.reshape(H, K)
    if not _takes_mtp_path(k_c, cu32, idx, per_token_slots):
        dt = dt.to(act)
    dt = dt.contiguous()
    num_accepted = None if num_accepted_tokens is None else num_accepted_tokens.to(torch.int32).contiguous()
    o = fused_sigmoid_gating_delta_rule_forward_k_last(
        A_log.reshape(-1).contiguous(), a, dt, _SOFTPLUS_BETA, _SOFTPLUS_THRESHOLD,
        q.contiguous(), k_c, v.contiguous(), b, initial_state, idx, float(K) ** -0.5, True,
        cu32, True, per_token_slots, None, None, num_accepted, None,
        None if lower_bound is None else float(lower_bound), is_sglang, None)
    if out is not None:
        out.copy_(o)
        o = out
    return o, initial_state


def _require(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def fused_kda_decode_mega_forward(x, weight, bias=None, conv_state=None, raw_g=None, raw_beta=None, a_log=None,
                                  dt_bias=None, state_indices=None, state=None, out=None, lower_bound=None,
                                  output_gate=None, norm_weight=None, norm_eps=1e-5):
    """Causal conv1d update + SiLU, gate, delta-rule recurrence and optional gated RMSNorm in one launch.

    Same arguments, layouts and checks as the reference entry
    (src/decode/k-last/fused_kda_decode_mega_host.cpp:77-300, pybind
    src/decode/k-last/fused_sigmoid_gating.cpp:236-245): ``conv_state``, ``state`` and ``out`` are
    updated in place, the return value is ``None``, rejected arguments raise ``RuntimeError`` before
    anything is written.  A request whose ``state_indices`` entry is negative gets a zero output row
    and touches neither pool; slot 0 is an ordinary slot.
    """
    native = _native()
    if native:
        return native.fused_kda_decode_mega_forward(x, weight, bias, conv_state, raw_g, raw_beta, a_log, dt_bias,
                                                    state_indices, state, out, lower_bound, output_gate, norm_weight,
                                                    norm_eps)
    return _mega_impl(x, weight, bias, conv_state, raw_g, raw_beta, a_log, dt_bias, state_indices, state, out,
                      lower_bound, output_gate, norm_weight, norm_eps)


def _mega_impl(x, weight, bias, conv_state, raw_g, raw_beta, a_log, dt_bias, state_indices, state, out, lower_bound,
               output_gate, norm_weight, norm_eps):
    if _BYPASS:
        return None
    D, W = 128, 4
    _require(x.is_cuda, "x must be a CUDA tensor")
    act = x.dtype
    _require(act in (torch.bfloat16, torch.float16), "x must be a bfloat16 or float16 tensor")
    _require(weight.is_cuda and weight.dtype == torch.float32, "weight must be a CUDA float32 tensor")
    _require(conv_state.is_cuda and conv_state.dtype == act, "conv_state must be a CUDA tensor with the same dtype as x")
    _require(raw_g.is_cuda and raw_g.dtype == act, "raw_g must be a CUDA tensor with the same dtype as x")
    _require(raw_beta.is_cuda and raw_beta.dtype == act, "raw_beta must be a CUDA tensor with the same dtype as x")
    _require(a_log.is_cuda and a_log.dtype == torch.float32, "A_log must be a CUDA float32 tensor")
    _require(dt_bias.is_cuda and dt_bias.dtype == torch.float32, "dt_bias must be a CUDA float32 tensor")
    _require(state.is_cuda and state.dtype == torch.float32, "state must be a CUDA float32 tensor")
    _require(out.is_cuda and out.dtype == act, "out must be a CUDA tensor with the same dtype as x")
    _require(state_indices.is_cuda and state_indices.dtype == torch.int32, "state_indices must be a CUDA int32 tensor")

    _require(x.dim() == 2 and x.size(1) % (3 * D) == 0, "x must have shape [B, 3 * H * 128]")
    B = x.size(0)
    H = x.size(1) // (3 * D)
    _require(H in _MEGA_HEADS, f"H must be 4, 6, 8, 12, 16, 24, 48, 64, or 96, got {H}")
    _require(B > 0, "KDA decode fusion requires at least one row")
    dim = H * D
    _require(weight.dim() == 3 and weight.is_contiguous() and tuple(weight.shape) == (3, W, dim),
             "weight must have shape [3, 4, H * 128]")
    _require(conv_state.dim() == 3 and conv_state.size(1) == 3 * dim and conv_state.size(2) == W - 1,
             "conv_state must have shape [slots, 3 * H * 128, 3]")
    _require(tuple(raw_g.shape) == (1, B, H, D), "raw_g must have shape [1, B, H, 128]")
    _require(tuple(raw_beta.shape) == (1, B, H), "raw_beta must have shape [1, B, H]")
    _require(a_log.is_contiguous() and a_log.numel() == H, "A_log must be contiguous with H elements")
    _require(dt_bias.is_contiguous() and dt_bias.numel() == dim, "dt_bias must be contiguous with H * 128 elements")
    _require(state_indices.is_contiguous() and state_indices.numel() == B,
             "state_indices must be contiguous with B elements")
    _require(state.dim() == 4 and tuple(state.shape[1:]) == (H, D, D), "state must have shape [slots, H, 128, 128]")
    _require(tuple(out.shape) == (1, B, H, D), "out must have shape [1, B, H, 128]")
    _require(x.stride(1) == 1, "x must be contiguous in its channel dimension")
    _require(conv_state.stride(0) >= 3 * dim * (W - 1) and conv_state.stride(1) == 1 and conv_state.stride(2) == 3 * dim,
             "conv_state must use the SD cache layout")
    _require(state.stride(0) >= H * D * D and state.stride(1) == D * D and state.stride(2) == D and state.stride(3) == 1,
             "state must have contiguous [H, 128, 128] slot contents")
    _require(raw_g.is_contiguous(), "raw_g must be contiguous")
    _require(raw_beta.stride(2) == 1, "raw_beta must be contiguous in its head dimension")
    _require(out.is_contiguous(), "out must be contiguous")

    apply_onorm = output_gate is not None
    _require(apply_onorm == (norm_weight is not None), "output_gate and norm_weight must be provided together")
    onorm_row = 0
    if apply_onorm:
        _require(output_gate.is_cuda and output_gate.dtype == act,
                 "output_gate must be a CUDA tensor with the same dtype as x")
        gate_3d = tuple(output_gate.shape) == (B, H, D)
        gate_4d = tuple(output_gate.shape) == (1, B, H, D)
        _require(gate_3d or gate_4d, "output_gate must have shape [B, H, 128] or [1, B, H, 128]")
        row_dim = 0 if gate_3d else 1
        _require(output_gate.stride(-1) == 1, "output_gate must be contiguous in its last dimension")
        _require(output_gate.stride(row_dim + 1) == D, "output_gate must have contiguous head rows")
        _require(norm_weight.is_cuda and norm_weight.dtype == torch.float32, "norm_weight must be a CUDA float32 tensor")
        _require(norm_weight.is_contiguous() and norm_weight.numel() == D,
                 "norm_weight must be contiguous with 128 elements")
        _require(norm_eps >= 0.0, "norm_eps must be non-negative")
        onorm_row = output_gate.stride(row_dim)
    if bias is not None:
        _require(bias.is_cuda and bias.dtype == torch.float32, "bias must be a CUDA float32 tensor")
        _require(bias.is_contiguous() and bias.numel() == 3 * dim, "bias must be contiguous with 3 * H * 128 elements")

    if os.environ.get("PLA_SANITY_CHECK", "0") == "1":           # read on every call, like src/sanity_check.h
        from ..._sanity import sanity_kda_decode_mega
        sanity_kda_decode_mega(x, weight, bias, conv_state, state_indices, state, lower_bound, output_gate,
                               norm_weight, norm_eps)

    eb = x.element_size()
    xp, wp, cp = x.data_ptr(), weight.data_ptr(), conv_state.data_ptr()
    seg_b, wseg_b, cseg_b = dim * eb, dim * W * 4, dim * conv_state.stride(1) * eb
    bp = None if bias is None else bias.data_ptr()
    with torch.cuda.device(x.device):
        _lib.call(
            "pla_kda_decode_mega_launch", _lib.dtype_code(act), int(apply_onorm), int(lower_bound is not None),
            a_log.data_ptr(), raw_g.data_ptr(), dt_bias.data_ptr(),
            xp, xp + seg_b, xp + 2 * seg_b, raw_beta.data_ptr(),
            wp, wp + wseg_b, wp + 2 * wseg_b,
            bp, None if bp is None else bp + dim * 4, None if bp is None else bp + 2 * dim * 4,
            cp, cp + cseg_b, cp + 2 * cseg_b,
            _lib.ptr(output_gate), _lib.ptr(norm_weight), float(norm_eps),
            state.data_ptr(), state_indices.data_ptr(), out.data_ptr(),
            float(D) ** -0.5, 0.0 if lower_bound is None else float(lower_bound), B, H, H,
            x.stride(0), raw_beta.stride(1), onorm_row, conv_state.stride(0), state.stride(0),
            _lib.current_stream(x.device))
    return None
