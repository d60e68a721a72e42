"""Diagnostic input checks enabled by ``PLA_SANITY_CHECK=1``.

Mirrors what the reference rejects in diagnostic mode
(src/decode/k-last/sanity_checks.h:140-440): every rejection raises
``RuntimeError("PLA_SANITY_CHECK [op]: ...")`` before anything is launched, so
no state is written.  Value checks (offsets, slots, finiteness) read device
memory and are therefore skipped while a stream is being captured
(src/sanity_check.h:60-72).
"""

import torch


def _fail(op, msg):
    raise RuntimeError(f"PLA_SANITY_CHECK [{op}]: {msg}")


def _capturing():
    return torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()


def _token_rows(op, t, name, token_axis, width):
    expected = 1
    for d in range(t.dim() - 1, token_axis, -1):
        if t.size(d) > 1 and t.stride(d) != expected:
            _fail(op, f"{name} head/feature axes must be contiguous")
        expected *= t.size(d)
    if expected != width or t.stride(token_axis) < width:
        _fail(op, f"{name} token stride must cover its complete head/feature row")
    if t.stride(token_axis) > 2 ** 31 - 1:
        _fail(op, f"{name} addressing exceeds the kernel's int32 offset domain")


def _check_offsets(op, cu, B, T_max, ntok):
    vals = cu.tolist()
    if len(vals) != B + 1 or vals[0] != 0:
        _fail(op, "cu_seqlens must start at 0 and have B+1 entries")
    for lo, hi in zip(vals, vals[1:]):
        if hi < lo:
            _fail(op, "cu_seqlens must be non-decreasing")
        if hi - lo > T_max:
            _fail(op, "a request is longer than the kernel's token capacity")
    if vals[-1] > ntok:
        _fail(op, "cu_seqlens exceeds the token dimension")
    return vals


def _check_slots(op, slots, lengths, nslots, is_sglang):
    seen = set()
    for slot, length in zip(slots, lengths):
        if length == 0:
            continue                       # empty requests consume no slot
        if slot < 0 or (not is_sglang and slot == 0):
            continue                       # padding
        if slot >= nslots:
            _fail(op, f"state slot {slot} out of range [0, {nslots})")
        if slot in seen:
            _fail(op, f"two active requests alias state slot {slot}")
        seen.add(slot)


def sanity_packed(mixed_qkv, a, b, A_log, dt_bias, state, indices, out, cu, is_kda, is_sglang, B, H, HV):
    op = "k_last_packed"
    if mixed_qkv.device != state.device or mixed_qkv.device.index != torch.cuda.current_device():
        _fail(op, "tensors must live on the current device")
    if mixed_qkv.data_ptr() % 16 or (mixed_qkv.stride(0) * mixed_qkv.element_size()) % 16:
        _fail(op, "mixed_qkv base and token stride must be 16-byte aligned")
    if state.data_ptr() % 16 or (state.stride(0) * state.element_size()) % 16:
        _fail(op, "state base and slot pitch must be 16-byte aligned")
    if A_log.dtype not in (torch.float32, torch.float16, torch.bfloat16):
        _fail(op, "A_log must be fp32, fp16 or bf16")
    if indices is not None and (indices.dim() != 1 or indices.numel() < B):
        _fail(op, "initial_state_indices must be int32 [B]")
    if _capturing():
        return
    ntok = mixed_qkv.size(0)
    if cu is not None:
        vals = _check_offsets(op, cu, B, 1, ntok)
        lengths = [hi - lo for lo, hi in zip(vals, vals[1:])]
    else:
        lengths = [1] * B
    if indices is not None:
        _check_slots(op, indices.tolist()[:B], lengths, state.size(0), is_sglang)
    if not torch.isfinite(mixed_qkv.float()).all():
        _fail(op, "mixed_qkv contains non-finite values")


def sanity_k_last(q, k, v, a, b, A_log, dt_bias, state, indices, cu, is_kda, cache, cache_indices,
                  num_accepted, parents, is_sglang, B, T_max, H, HV):
    op = "k_last"
    if q.device.index != torch.cuda.current_device():
        _fail(op, "tensors must live on the current device")
    for name, t, width in (("q", q, H * 128), ("k", k, H * 128), ("v", v, HV * 128)):
        _token_rows(op, t, name, 1, width)
        if t.data_ptr() % 16 or (t.stride(1) * t.element_size()) % 16:
            _fail(op, f"{name} base and token stride must be 16-byte aligned")
    if state is not None and (state.data_ptr() % 16 or (state.stride(0) * state.element_size()) % 16):
        _fail(op, "state base and slot pitch must be 16-byte aligned")
    if indices is not None:
        if indices.dim() == 2 and is_sglang:
            _fail(op, "a 2-D slot table requires is_sglang=False")
        if indices.dim() == 2 and indices.stride(1) != 1:
            _fail(op, "slot-table columns must be contiguous")
    if num_accepted is not None and (indices is None or indices.dim() != 2):
        _fail(op, "num_accepted_tokens requires a 2-D slot table")
    if parents is not None and (cache is None or cache_indices is None):
        _fail(op, "retrieve_parent_token requires the intermediate cache and its indices")
    if _capturing():
        return
    ntok = q.size(0) * q.size(1)
    if cu is not None:
        vals = _check_offsets(op, cu, B, T_max, ntok)
        lengths = [hi - lo for lo, hi in zip(vals, vals[1:])]
    else:
        lengths = [T_max] * B
    if indices is not None and state is not None:
        if indices.dim() == 1:
            _check_slots(op, indices.tolist()[:B], lengths, state.size(0), is_sglang)
        else:
            table = indices.tolist()
            acc = num_accepted.tolist() if num_accepted is not None else [1] * B
            start = [row[max(n - 1, 0) if n > 0 else 0] for row, n in zip(table, acc)]
            _check_slots(op, start, lengths, state.size(0), is_sglang)
    if parents is not None:
        for n, length in enumerate(lengths):
            row = parents[n].tolist()
            for t in range(1, length):
                if row[t] >= t:
                    _fail(op, "a parent step must precede its token")


def sanity_kda_decode_mega(x, weight, bias, conv_state, state_indices, state, lower_bound, output_gate,
                           norm_weight, norm_eps):
    """Diagnostic checks of the fused KDA decode step
    (src/decode/k-last/kda_decode_sanity.h:44-109): slot pitch alignment, finite negative
    ``lower_bound``, finite ``norm_eps``; value checks (skipped during capture): active slots inside
    both pools, no two requests on one non-zero slot, finite selected inputs and pool rows."""
    import math
    op = "fused_kda_decode"
    if state_indices.dim() != 1:
        _fail(op, "state_indices must be a vector")
    if state.storage_offset() % 4 != 0 or state.stride(0) % 4 != 0:
        _fail(op, "state slots must be 16-byte aligned for float4 access")
    if lower_bound is not None and not (math.isfinite(lower_bound) and lower_bound < 0.0):
        _fail(op, "lower_bound must be a finite negative float32 value")
    if output_gate is not None and not (math.isfinite(norm_eps) and norm_eps >= 0.0):
        _fail(op, "norm_eps must be a finite non-negative float32 value")
    if _capturing():
        return
    seen = set()
    active = False
    for n, slot in enumerate(state_indices.tolist()):
        if slot < 0:
            continue
        if slot >= state.size(0) or slot >= conv_state.size(0):
            _fail(op, f"state index {slot} exceeds recurrent/conv pool capacity")
        if slot != 0:
            if slot in seen:
                _fail(op, f"requests must not concurrently update the same state slot: {slot}")
            seen.add(slot)
        else:
            continue
        active = True
        for name, t in (("selected x", x[n]), ("selected state", state[slot]),
                        ("selected conv_state", conv_state[slot])):
            if not bool(torch.isfinite(t).all()):
                _fail(op, f"{name} must be finite")
        if output_gate is not None:
            gate = output_gate[n] if output_gate.dim() == 3 else output_gate[0, n]
            if not bool(torch.isfinite(gate).all()):
                _fail(op, "selected output_gate must be finite")
    if active:
        for name, t in (("weight", weight), ("bias", bias), ("norm_weight", norm_weight)):
            if t is not None and not bool(torch.isfinite(t).all()):
                _fail(op, f"{name} must be finite")


def sanity_verify_dspark(x_q, x_k, x_v, w_q, w_k, w_v, cs_q, cs_k, cs_v, h0, ic_q, slot_idx, scratch_idx, cu_seqlens,
                         N, T, t_loop, slots, scale, lower_bound, onorm_weight, onorm_eps):
    """Diagnostic checks of the KDA verify with replay records
    (src/decode/kda_replayssm_sglang/sanity_checks.h:90-160): finite float32 scalars; value checks
    (skipped during capture): dense offsets of ``t_loop`` tokens per request, active slots and scratch
    rows in range, no two requests writing one slot's rings or one scratch row, finite selected inputs."""
    import math
    op = "kda_verify_dspark"
    if not math.isfinite(scale):
        _fail(op, "scale must be representable as a finite float32 value")
    if not (math.isfinite(lower_bound) and lower_bound < 0.0):
        _fail(op, "lower_bound must be a finite negative float32 value")
    if onorm_eps is not None and not (math.isfinite(onorm_eps) and onorm_eps >= 0.0):
        _fail(op, "onorm_eps must be a finite non-negative float32 value")
    if _capturing():
        return
    offsets = cu_seqlens.tolist()
    if offsets[0] != 0 or offsets[-1] != T:
        _fail(op, "cu_seqlens must cover exactly the packed tokens")
    ring_writers, window_writers = set(), set()
    active = False
    for n, (slot, row) in enumerate(zip(slot_idx.tolist(), scratch_idx.tolist()[:N])):
        if offsets[n + 1] - offsets[n] != t_loop:
            _fail(op, f"every request must own exactly {t_loop} tokens (request {n})")
        if slot < 0:
            continue
        if slot >= slots:
            _fail(op, f"state/ring slot is out of bounds at request {n}")
        if not 0 <= row < ic_q.size(0):
            _fail(op, f"scratch row is out of bounds at request {n}")
        if slot in ring_writers:
            _fail(op, f"two requests write the rings of slot {slot}")
        if row in window_writers:
            _fail(op, f"two requests write scratch row {row}")
        ring_writers.add(slot)
        window_writers.add(row)
        active = True
        for name, t in (("selected h0", h0[slot]), ("selected cs_q", cs_q[slot]), ("selected cs_k", cs_k[slot]),
                        ("selected cs_v", cs_v[slot]), ("selected x_q", x_q[:, offsets[n]:offsets[n + 1]]),
                        ("selected x_k", x_k[:, offsets[n]:offsets[n + 1]]),
                        ("selected x_v", x_v[:, offsets[n]:offsets[n + 1]])):
            if not bool(torch.isfinite(t).all()):
                _fail(op, f"{name} must be finite")
    if active:
        for name, t in (("w_q", w_q), ("w_k", w_k), ("w_v", w_v), ("onorm_weight", onorm_weight)):
            if t is not None and not bool(torch.isfinite(t).all()):
                _fail(op, f"{name} must be finite")
