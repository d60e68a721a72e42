"""Accepted-prefix commit of KDA speculative decoding (``pla.decode.kda_replayssm_sglang``).

Covers the recurrence half of the reference's
``commit_kda_replayssm_after_verify`` (pla/decode/kda_replayssm_sglang/__init__.py:162-215):
for every layer, each request's accepted prefix of recorded tokens (raw k, raw v, per-channel
log-decay, beta) is replayed into the FP32 checkpoint ``temporal`` in place.  A request whose
slot is ``<= null_block_id`` or whose accepted length is ``<= 0`` leaves its checkpoint
bit-identical (src/decode/kda_replayssm/kda_mtp_fold.cu:306).  The convolution-window
rollback and the ring writers of the verify kernel belong to the conv front end and are not
part of this package.
"""

import torch

from ... import _lib

__all__ = ["fold_accepted_prefix", "commit_kda_replayssm_after_verify", "kda_mtp_verify"]


def fold_accepted_prefix(temporal, rawv, rawk, gk, beta, state_batch_indices, accept_lens,
                         null_block_id=-1):
    """Replay ``accept_lens[n]`` recorded tokens into ``temporal[:, state_batch_indices[n]]``.

    temporal [layers, slots, HV, 128, 128] float32; rawv [layers, slots, HV, L, 128] and
    rawk [layers, slots, H, L, 128] in bf16/fp16; gk [layers, slots, HV, L, 128] float32
    log-decay; beta [layers, slots, HV, L] float32; indices / lengths int32 [B].
    One launch per layer on the current stream.
    """
    if temporal.dim() != 5 or temporal.dtype != torch.float32:
        raise RuntimeError("temporal must be float32 [layers, slots, HV, V, K]")
    layers, slots, HV, V, K = temporal.shape
    if V != 128 or K != 128:
        raise RuntimeError(f"fold requires head_dim K == V == 128, got K={K}, V={V}")
    H, L = rawk.shape[2], rawk.shape[3]
    for name, t, shape in (("rawv", rawv, (layers, slots, HV, L, 128)), ("rawk", rawk, (layers, slots, H, L, 128)),
                           ("gk", gk, (layers, slots, HV, L, 128)), ("beta", beta, (layers, slots, HV, L))):
        if tuple(t.shape) != shape or not t[0, 0].is_contiguous():
            raise RuntimeError(f"{name} must be {shape} with contiguous slots, got {tuple(t.shape)}")
    if rawv.dtype != rawk.dtype or rawk.dtype not in (torch.bfloat16, torch.float16):
        raise RuntimeError("rawk / rawv must share bf16 or fp16")
    if gk.dtype != torch.float32 or beta.dtype != torch.float32:
        raise RuntimeError("gk and beta records must be float32")
    if state_batch_indices.dtype != torch.int32 or accept_lens.dtype != torch.int32:
        raise RuntimeError("state_batch_indices and accept_lens must be int32")
    B = state_batch_indices.numel()
    if accept_lens.numel() != B:
        raise RuntimeError("accept_lens must have one entry per request")
    if not temporal[0, 0].is_contiguous():
        raise RuntimeError("temporal slots must be dense [HV, V, K]")
    stream = _lib.current_stream(temporal.device)
    act = _lib.dtype_code(rawk.dtype)
    for layer in range(layers):
        _lib.call("pla_kda_fold_launch", temporal[layer].data_ptr(), rawv[layer].data_ptr(), rawk[layer].data_ptr(),
                  gk[layer].data_ptr(), beta[layer].data_ptr(), state_batch_indices.data_ptr(),
                  accept_lens.data_ptr(), temporal.stride(1), rawv.stride(1), rawk.stride(1), gk.stride(1),
                  beta.stride(1), B, H, HV, L, int(null_block_id), act, stream)


def commit_kda_replayssm_after_verify(*, spec_state, state_batch_indices, accept_lens,
                                      last_correct_step_indices=None, mamba_track_indices=None,
                                      mamba_steps_to_track=None, null_block_id=-1,
                                      conv_state_layout="dim_width"):
    """Keyword-only entry with the reference's name: folds every layer's accepted window into
    ``spec_state.temporal``.  Only the recurrent state is committed here; boundary / track
    snapshots and the conv-window rollback are rejected rather than silently skipped."""
    if mamba_track_indices is not None or mamba_steps_to_track is not None:
        raise NotImplementedError("track snapshots are not part of the gfx950 commit path")
    fold_accepted_prefix(spec_state.temporal, spec_state.replayssm_rawv, spec_state.replayssm_rawk,
                         spec_state.replayssm_g, spec_state.replayssm_beta,
                         state_batch_indices, accept_lens, null_block_id)


def kda_mtp_verify(q, k, v, g, beta, recurrent_state, ssm_state_indices, cu_seqlens, scale=None,
                   out=None, use_qk_l2norm=True, max_tokens=None):
    """Speculative verify from an already evaluated gate: T draft tokens per request are run
    through the recurrence starting from ``recurrent_state[ssm_state_indices[n]]``, which is
    read once and never written (the read-once verify of
    src/decode/kda_replayssm/kda_mtp_verify.cu:630-700 without its conv front end).

    q, k [1, tokens, H, 128], v [1, tokens, HV, 128] bf16/fp16; g [tokens, HV, 128] float32
    per-channel log-decay; beta [tokens, HV] float32 (activated); slots < 0 are padding.
    Returns ``out`` [1, tokens, HV, 128].
    """
    if q.dim() != 4 or q.size(0) != 1:
        raise ValueError("q must be packed as [1, tokens, H, 128]")
    tokens, H, K = q.size(1), q.size(2), q.size(3)
    HV, V = v.size(2), v.size(3)
    if K != 128 or V != 128:
        raise NotImplementedError(f"kda_mtp_verify requires head_dim K == V == 128, got K={K}, V={V}")
    if g.dtype != torch.float32 or beta.dtype != torch.float32:
        raise ValueError("g (log-decay) and beta must be float32")
    if tuple(g.shape) != (tokens, HV, 128) or tuple(beta.shape) != (tokens, HV):
        raise ValueError("g must be [tokens, HV, 128] and beta [tokens, HV]")
    if not (g.is_contiguous() and beta.is_contiguous()):
        raise ValueError("g and beta must be contiguous")
    if recurrent_state.dtype != torch.float32:
        raise ValueError("recurrent_state must be float32")
    B = cu_seqlens.numel() - 1
    if max_tokens is None:
        if tokens % B:
            raise ValueError("pass max_tokens for ragged requests")
        max_tokens = tokens // B
    if out is None:
        out = torch.empty_like(v, memory_format=torch.contiguous_format)
    _lib.call(
        "pla_k_last_launch",
        None, _lib.F32, g.data_ptr(), None, 0, 0.0, 20.0, _lib.GATE_LOG_DECAY,
        q.data_ptr(), k.data_ptr(), v.data_ptr(), beta.data_ptr(), 1,
        out.data_ptr(), recurrent_state.data_ptr(), _lib.F32, cu_seqlens.data_ptr(), None,
        ssm_state_indices.data_ptr(), None, 0, None, 0, 0,
        float(scale) if scale is not None else K ** -0.5, int(max_tokens),
        HV * 128, q.stride(1), k.stride(1), v.stride(1), HV, recurrent_state.stride(0),
        B, H, HV, K, V, int(bool(use_qk_l2norm)), 1, None, 0, 1, 1,
        _lib.dtype_code(q.dtype), 0, _lib.current_stream(q.device))
    return out
