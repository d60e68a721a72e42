"""Tunable k-last entry points (``pla.decode.private`` drop-in).

Same signatures as the reference's auto-tune hooks
(src/decode/k-last/fused_sigmoid_gating.cpp:204-235): the ordinary arguments
followed by the tile tuple ``(bv, wn, sn, hv_per_cta)``.  On gfx950 the tuple is
validated like the reference validates it and ``bv`` selects how many V-rows a
wavefront owns (bv/4 clamped to 8, 16 or 32); ``wn``, ``sn`` and ``hv_per_cta``
have no gfx950 counterpart because the kernel stages nothing through LDS.
"""

from .. import _k_last_impl, _packed_impl

__all__ = [
    "fused_sigmoid_gating_delta_rule_forward_k_last_tunable",
    "fused_sigmoid_gating_delta_rule_forward_k_last_packed_tunable",
]


def fused_sigmoid_gating_delta_rule_forward_k_last_tunable(
        A_log, a, dt_bias, softplus_beta, softplus_threshold, q, k, v, b,
        initial_state_source, initial_state_indices, scale, use_qk_l2norm_in_kernel,
        cu_seqlens, is_kda, disable_state_update, intermediate_states_buffer,
        intermediate_state_indices, cache_steps_or_num_accept, retrieve_parent_token,
        bv, wn, sn, hv_per_cta, is_sglang=None, lower_bound=None, out=None):
    return _k_last_impl(A_log, a, dt_bias, softplus_beta, softplus_threshold, q, k, v, b,
                        initial_state_source, initial_state_indices, scale, use_qk_l2norm_in_kernel,
                        cu_seqlens, is_kda, disable_state_update, intermediate_states_buffer,
                        intermediate_state_indices, cache_steps_or_num_accept, retrieve_parent_token,
                        lower_bound, is_sglang, out, (bv, wn, sn, hv_per_cta))


def fused_sigmoid_gating_delta_rule_forward_k_last_packed_tunable(
        mixed_qkv, a, b, A_log, dt_bias, softplus_beta, softplus_threshold, scale,
        initial_state_source, initial_state_indices, out, use_qk_l2norm_in_kernel,
        cu_seqlens, is_kda, bv, wn, sn, hv_per_cta, is_sglang=None):
    return _packed_impl(mixed_qkv, a, b, A_log, dt_bias, softplus_beta, softplus_threshold, scale,
                        initial_state_source, initial_state_indices, out, use_qk_l2norm_in_kernel,
                        cu_seqlens, is_kda, is_sglang, (bv, wn, sn, hv_per_cta))
