"""``pla.decode.kda`` drop-in: recurrent KDA decode from raw gate / beta projections.

Mirrors the reference wrapper src/decode/k-last/fused_recurrent_kda.cpp:146-314
(vLLM's ``fused_recurrent_kda`` signature plus a trailing ``is_sglang``): raises
``ValueError`` / ``NotImplementedError`` for the same argument problems, requires a
float32 ``dt_bias`` and narrows it to the activation dtype only for the pure-decode
path, and forwards to the k-last entry point with ``disable_state_update`` set when a
2-D per-token slot table is given.
"""

import torch

from .. import fused_sigmoid_gating_delta_rule_forward_k_last, _packed_t_max

__all__ = ["fused_recurrent_kda"]

_SOFTPLUS_BETA = 1.0
_SOFTPLUS_THRESHOLD = 20.0


def _takes_mtp_path(k, cu_seqlens, state_indices, disable_state_update):
    # src/decode/k-last/fused_sigmoid_gating_cuda_k_last.cpp:225-236
    target_verify = state_indices.dim() == 2
    cols = state_indices.size(1) if target_verify else 0
    B = cu_seqlens.size(0) - 1
    t_max = _packed_t_max(k, B, target_verify, 0, cols)
    return t_max > 1 or disable_state_update or target_verify


def fused_recurrent_kda(q, k, v, raw_g, raw_beta, A_log, dt_bias, lower_bound, initial_state,
                        cu_seqlens, ssm_state_indices, num_accepted_tokens=None, out=None,
                        fuse_gate=None, is_sglang=False):
    """Returns ``(out, initial_state)``; the state pool is updated in place."""
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
