"""KDA speculative decoding with replay records (``pla.decode.kda_replayssm_sglang``).

``fused_kda_decode_mtp_dspark`` (reference pla/decode/kda_replayssm_sglang/__init__.py:74-159): verify of the
draft tokens in ring mode.  Conv front end, gate and recurrence in one launch; the persistent
recurrent and conv states are read-only, the per-token records go to the four rings and the conv
window after every token to the scratch rows.

``commit_kda_replayssm_after_verify`` (same file :162-211): for every layer, each request's accepted
prefix of recorded tokens (raw k, raw v, per-channel log-decay, beta) is replayed into the FP32
checkpoint ``temporal`` in place, and the conv state is rolled back to the window of the last
accepted step.  A request whose slot is ``<= null_block_id`` or whose accepted length is ``<= 0``
leaves its checkpoint bit-identical (src/decode/kda_replayssm/kda_mtp_fold.cu:306).  Track
snapshots (``mamba_track_indices`` / ``mamba_steps_to_track``) store the state after the tracked step
and the conv window of that step to the tracked slot.
"""

import ctypes
import os

import torch

from ... import _lib

__all__ = ["fused_kda_decode_mtp_dspark", "commit_kda_replayssm_after_verify", "conv_window_scatter",
           "fold_accepted_prefix", "kda_mtp_verify"]

_BYPASS = os.environ.get("PLA_BYPASS_EXEC", "0") == "1"   # read once, like src/bypass_exec.h:44-50


def fold_accepted_prefix(temporal, rawv, rawk, gk, beta, state_batch_indices, accept_lens,
                         null_block_id=-1, track_indices=None, track_steps=None):
    """Replay ``accept_lens[n]`` recorded tokens into ``temporal[:, state_batch_indices[n]]``.
    With ``track_indices`` / ``track_steps`` (int32 [B]) the state after step ``track_steps[n]`` is also
    stored to slot ``track_indices[n]`` when that slot is ``> null_block_id``
    (src/decode/kda_replayssm/kda_mtp_fold.cu:462-478).

    temporal [layers, slots, HV, 128, 128] float32; rawv [layers, slots, HV, L, 128] and
    rawk [layers, slots, H, L, 128] in bf16/fp16; gk [layers, slots, HV, L, 128] float32
    log-decay; beta [layers, slots, HV, L] float32; indices / lengths int32 [B].
    One launch for all layers on the current stream.
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
    if (track_indices is None) != (track_steps is None):
        raise RuntimeError("track indices and steps must be given together")
    if track_indices is not None:
        track_indices = track_indices.to(torch.int32).contiguous()
        track_steps = track_steps.to(torch.int32).contiguous()
        if track_indices.numel() != B or track_steps.numel() != B:
            raise RuntimeError("track indices and steps must have one entry per request")
    if not temporal[0, 0].is_contiguous():
        raise RuntimeError("temporal slots must be dense [HV, V, K]")
    stream = _lib.current_stream(temporal.device)
    act = _lib.dtype_code(rawk.dtype)
    if layers == 0 or B == 0:
        return
    _lib.call("pla_kda_fold_launch", temporal.data_ptr(), rawv.data_ptr(), rawk.data_ptr(), gk.data_ptr(), beta.data_ptr(),
              state_batch_indices.data_ptr(), accept_lens.data_ptr(), _lib.ptr(track_indices), _lib.ptr(track_steps),
              temporal.stride(1), rawv.stride(1), rawk.stride(1), gk.stride(1), beta.stride(1),
              layers, temporal.stride(0), rawv.stride(0), rawk.stride(0), gk.stride(0), beta.stride(0),
              B, H, HV, L, int(null_block_id), act, stream)


def _index(t):
    if t.dim() != 1 or t.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("indices must be int32/int64 vectors")
    t = t.contiguous()
    return t, int(t.dtype == torch.int64)


def conv_window_scatter(dst, src, dst_idx, step_idx):
    """``dst[layer, dst_idx[r]] = src[layer, r, step_idx[r]]`` for every request ``r`` with a non-negative
    step and destination (reference binding src/decode/kda_replayssm_sglang/kda_mtp_fold_host.cpp:152-224).
    dst [layers, slots, dim, width-1] (or its ``width_dim`` transpose view), src [layers, rows, steps, dim,
    width-1], bf16 or float32; out-of-range requests are skipped."""
    if _BYPASS:
        return
    if dst.dim() != 4 or src.dim() != 5:
        raise RuntimeError("ranks: dst 4, src 5")
    if not (dst.is_cuda and src.device == dst.device and dst.dtype == src.dtype):
        raise RuntimeError("conv source and destination must have the same CUDA device and dtype")
    if not (src.size(0) == dst.size(0) and src.size(3) == dst.size(2) and src.size(4) == dst.size(3)):
        raise RuntimeError("conv source/destination shape mismatch")
    if not (dst.is_contiguous() or dst.transpose(-1, -2).is_contiguous()):
        raise RuntimeError("conv destination must be contiguous in dim_width or width_dim layout")
    if dst_idx.numel() != step_idx.numel() or dst_idx.device != dst.device or step_idx.device != dst.device:
        raise RuntimeError("invalid conv scatter indices")
    di, di_wide = _index(dst_idx)
    st, st_wide = _index(step_idx)
    if dst.dtype not in (torch.bfloat16, torch.float32):
        raise RuntimeError(f"conv scatter: unsupported dtype {dst.dtype}")
    km1 = dst.size(3)
    if not 1 <= km1 <= 4:
        raise RuntimeError(f"conv scatter: unsupported conv window {km1}")
    if st.numel() == 0:
        return
    with torch.cuda.device(dst.device):
        _lib.call("pla_conv_window_scatter_launch", dst.element_size(), km1, src.data_ptr(), dst.data_ptr(),
                  di.data_ptr(), di_wide, st.data_ptr(), st_wide, dst.size(0), dst.size(2), st.numel(),
                  *src.stride(), *dst.stride(), src.size(1), src.size(2), dst.size(1),
                  _lib.current_stream(dst.device))


def commit_kda_replayssm_after_verify(*, spec_state, state_batch_indices, accept_lens,
                                      last_correct_step_indices=None, mamba_track_indices=None,
                                      mamba_steps_to_track=None, null_block_id=-1,
                                      conv_state_layout="dim_width"):
    """Keyword-only entry with the reference's name: folds every layer's accepted window into
    ``spec_state.temporal`` and rolls the conv states back to the window of the last accepted step.
    ``spec_state`` carries ``temporal``, ``replayssm_rawv/rawk/g/beta`` and, for the rollback, the lists
    ``conv`` ([layers, slots, dim, width-1] each) and ``intermediate_conv_window``
    ([layers, rows, steps, dim, width-1] each); ``conv_state_layout="width_dim"`` takes the transposed
    pools."""
    assert conv_state_layout in ("dim_width", "width_dim")
    if (mamba_track_indices is None) != (mamba_steps_to_track is None):
        raise ValueError("mamba_track_indices and mamba_steps_to_track must be given together")
    fold_accepted_prefix(spec_state.temporal, spec_state.replayssm_rawv, spec_state.replayssm_rawk,
                         spec_state.replayssm_g, spec_state.replayssm_beta,
                         state_batch_indices, accept_lens, null_block_id,
                         mamba_track_indices, mamba_steps_to_track)
    conv = getattr(spec_state, "conv", None)
    windows = getattr(spec_state, "intermediate_conv_window", None)
    if conv is None or windows is None:
        return
    if last_correct_step_indices is None:
        raise ValueError("the conv rollback needs last_correct_step_indices")
    assert len(conv) == len(windows)
    for conv_states, interm_conv in zip(conv, windows):
        if conv_state_layout == "width_dim":
            conv_states = conv_states.transpose(-1, -2)
            interm_conv = interm_conv.transpose(-1, -2)
        conv_window_scatter(conv_states, interm_conv, state_batch_indices, last_correct_step_indices)
        if mamba_track_indices is not None and mamba_steps_to_track is not None:
            conv_window_scatter(conv_states, interm_conv, mamba_track_indices, mamba_steps_to_track)


def fused_kda_decode_mtp_dspark(*, x_q, x_k, x_v, w_q, w_k, w_v, cs_q, cs_k, cs_v, g, beta, A_log, dt_bias,
                                recurrent_state, intermediate_ssm=None, intermediate_state_indices,
                                intermediate_conv_q, intermediate_conv_k, intermediate_conv_v,
                                ssm_state_indices, cu_seqlens, lower_bound, scale=None,
                                replayssm_rawv=None, replayssm_rawk=None, replayssm_g=None, replayssm_beta=None,
                                onorm_gate=None, onorm_weight=None, onorm_eps=None, out=None):
    """KDA verify of the draft tokens in ring mode (all four ``replayssm_*`` rings are required;
    ``intermediate_ssm`` snapshots are not written).  Returns ``out`` [1, T, H, 128].

    Shapes and layouts as the reference binding checks them
    (src/decode/kda_replayssm_sglang/kda_mtp_verify_host.cpp:108-222): q/k/v/g bf16 [1, T, H, 128] with an
    optional token stride, beta bf16 [1, T, H]; conv weights float32 [H*128, 4]; conv states bf16
    [slots, H*128, 3] and windows bf16 [rows, steps, H*128, 3] with any positive strides; state float32
    [slots, H, 128, 128], rings [slots, H, L, 128] (bf16 rawv / rawk, float32 g) and [slots, H, L] (float32
    beta), ``out`` bf16, all contiguous; index tensors int32 or int64.  ``T`` must be ``N`` times the draft
    window (at most 32 tokens, as in the reference).
    """
    rings = (replayssm_rawv, replayssm_rawk, replayssm_g, replayssm_beta)
    if any(r is None for r in rings):
        raise ValueError("pla.decode.kda_mtp_sglang.fused_kda_decode_mtp_dspark implements CACHE_RING only; "
                         "pass all four replayssm_* rings.")
    onorm_args = (onorm_gate, onorm_weight, onorm_eps)
    apply_onorm = all(v is not None for v in onorm_args)
    if any(v is not None for v in onorm_args) and not apply_onorm:
        raise ValueError("fused output norm requires onorm_gate, onorm_weight, and onorm_eps")
    if scale is None:
        scale = 128 ** -0.5
    if out is None:
        out = torch.empty_like(x_v, memory_format=torch.contiguous_format)
    if _BYPASS:
        return out

    def need(cond, msg):
        if not cond:
            raise RuntimeError(msg)

    D, W = 128, 4
    need(x_q.dim() == 4 and x_q.size(0) == 1, "x_q must be [1, T, H, 128]")
    need(x_q.is_cuda, "verify requires CUDA tensors")
    T, H = x_q.size(1), x_q.size(2)
    need(x_q.size(3) == D, "specialised for head_dim 128")
    N = cu_seqlens.numel() - 1
    need(N > 0 and T > 0 and H > 0 and T % N == 0, "dense 1 + num_spec tokens per request")
    t_loop = T // N
    need(replayssm_rawv.dim() == 4, "rawv ring must be [slot, H, L, 128]")
    L, slots = replayssm_rawv.size(2), replayssm_rawv.size(0)
    need(L >= t_loop, "ring shorter than the draft window")
    need(recurrent_state.dtype == torch.float32, "recurrent state must be fp32")
    need(x_q.dtype == torch.bfloat16, "inputs must be bf16")
    need(tuple(recurrent_state.shape) == (slots, H, D, D), "state must be [slot, H, 128, 128]")
    everything = [x_k, x_v, g, beta, w_q, w_k, w_v, cs_q, cs_k, cs_v, A_log, dt_bias, recurrent_state, out,
                  intermediate_conv_q, intermediate_conv_k, intermediate_conv_v, *rings, ssm_state_indices,
                  intermediate_state_indices, cu_seqlens]
    need(all(t.device == x_q.device for t in everything), "verify tensors must share one device")
    need(all(tuple(t.shape) == (slots, H, L, D) for t in rings[:3]), "invalid verify ring shape")
    need(tuple(replayssm_beta.shape) == (slots, H, L) and replayssm_rawv.dtype == torch.bfloat16
         and replayssm_rawk.dtype == torch.bfloat16 and replayssm_g.dtype == torch.float32
         and replayssm_beta.dtype == torch.float32, "invalid verify ring dtype/shape")
    w_q, w_k, w_v = w_q.contiguous(), w_k.contiguous(), w_v.contiguous()
    need(all(tuple(t.shape) == (H * D, W) and t.dtype == torch.float32 for t in (w_q, w_k, w_v)),
         "conv weights must be contiguous fp32 [H*128, 4]")
    A_log, dt_bias = A_log.contiguous(), dt_bias.contiguous()
    need(A_log.numel() == H and dt_bias.numel() == H * D and A_log.dtype == torch.float32
         and dt_bias.dtype == torch.float32, "invalid gate weights")
    need(recurrent_state.storage_offset() % 4 == 0, "recurrent state must be 16-byte aligned for float4 loads")
    need(ssm_state_indices.numel() == N and intermediate_state_indices.numel() >= N, "verify index count mismatch")

    def input_stride(x):
        need(x.shape == x_q.shape and x.dtype == torch.bfloat16, "Q/K/V and g must be bf16 [1, T, H, 128]")
        need(x.stride(3) == 1 and x.stride(2) == D and x.stride(1) >= H * D,
             "Q/K/V and g must have contiguous head/channel dimensions")
        return [x.stride(1)]

    def conv_strides(x):
        need(x.dim() == 3 and x.size(0) == slots and x.size(1) == H * D and x.size(2) == W - 1
             and x.dtype == torch.bfloat16, "conv states must be bf16 [slot, H*128, 3]")
        need(all(st > 0 for st in x.stride()), "conv state strides must be positive")
        return list(x.stride())

    def window_strides(x):
        need(x.dim() == 4 and x.size(1) >= t_loop and x.size(2) == H * D and x.size(3) == W - 1
             and x.dtype == torch.bfloat16, "conv windows must be bf16 [scratch, step, H*128, 3]")
        need(all(st > 0 for st in x.stride()), "conv window strides must be positive")
        return list(x.stride())

    need(beta.dim() == 3 and beta.size(0) == 1 and beta.size(1) == T and beta.size(2) == H
         and beta.dtype == torch.bfloat16 and beta.stride(2) == 1 and beta.stride(1) >= H,
         "beta must be bf16 [1, T, H] with contiguous heads")
    need(out.shape == x_q.shape and out.is_contiguous() and out.dtype == torch.bfloat16
         and recurrent_state.is_contiguous() and all(r.is_contiguous() for r in rings),
         "output, recurrent state and rings must be contiguous")
    strides = (input_stride(x_q) + input_stride(x_k) + input_stride(x_v) + input_stride(g) + [beta.stride(1)]
               + conv_strides(cs_q) + conv_strides(cs_k) + conv_strides(cs_v)
               + window_strides(intermediate_conv_q) + window_strides(intermediate_conv_k)
               + window_strides(intermediate_conv_v))
    gate_stride = 0
    if apply_onorm:
        need(onorm_gate.device == x_q.device and onorm_weight.device == x_q.device,
             "output-norm tensors must share the verify device")
        need(onorm_gate.shape == x_q.shape and onorm_gate.dtype == torch.bfloat16 and onorm_gate.stride(3) == 1
             and onorm_gate.stride(2) == D and onorm_gate.stride(1) >= H * D,
             "output-norm gate must be bf16 [1, T, H, 128] with contiguous head/channel dimensions")
        need(onorm_weight.dim() == 1 and onorm_weight.size(0) == D and onorm_weight.is_contiguous()
             and onorm_weight.dtype == torch.float32, "output-norm weight must be contiguous fp32 [128]")
        need(onorm_eps == onorm_eps and abs(onorm_eps) != float("inf") and onorm_eps >= 0.0,
             "output-norm eps must be finite and non-negative")
        gate_stride = onorm_gate.stride(1)
    si, si_wide = _index(ssm_state_indices)
    sc, sc_wide = _index(intermediate_state_indices)
    cu, cu_wide = _index(cu_seqlens)
    if os.environ.get("PLA_SANITY_CHECK", "0") == "1":            # read on every call, like src/sanity_check.h
        from ..._sanity import sanity_verify_dspark
        sanity_verify_dspark(x_q, x_k, x_v, w_q, w_k, w_v, cs_q, cs_k, cs_v, recurrent_state, intermediate_conv_q,
                             si, sc, cu, N, T, t_loop, slots, float(scale), float(lower_bound),
                             onorm_weight if apply_onorm else None, onorm_eps if apply_onorm else None)
    c_strides = (ctypes.c_int64 * 26)(*strides)
    with torch.cuda.device(x_q.device):
        _lib.call(
            "pla_kda_verify_dspark_launch", x_q.data_ptr(), x_k.data_ptr(), x_v.data_ptr(), g.data_ptr(),
            beta.data_ptr(), w_q.data_ptr(), w_k.data_ptr(), w_v.data_ptr(), cs_q.data_ptr(), cs_k.data_ptr(),
            cs_v.data_ptr(), A_log.data_ptr(), dt_bias.data_ptr(), recurrent_state.data_ptr(), out.data_ptr(),
            intermediate_conv_q.data_ptr(), intermediate_conv_k.data_ptr(), intermediate_conv_v.data_ptr(),
            replayssm_rawv.data_ptr(), replayssm_rawk.data_ptr(), replayssm_g.data_ptr(), replayssm_beta.data_ptr(),
            si.data_ptr(), si_wide, sc.data_ptr(), sc_wide, cu.data_ptr(), cu_wide,
            H, N, t_loop, L, float(scale), float(lower_bound), ctypes.cast(c_strides, ctypes.c_void_p),
            _lib.ptr(onorm_gate) if apply_onorm else None, _lib.ptr(onorm_weight) if apply_onorm else None,
            gate_stride, float(onorm_eps) if apply_onorm else 0.0, _lib.current_stream(x_q.device))
    return out


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
