"""GDN chunked prefill on MI355X behind FlashQLA's Python interface.

Same functions, argument names and return contract as the reference
(pla/prefill/flashqla/ops.py:225-248, 651-738): ``chunk_gated_delta_rule_fwd`` returns
``(g_cum, A, o, None, final_state)`` and updates an indexed k-last pool in place even when
``output_final_state`` is false; ``gdn_prefill_packed_qkv_fwd`` takes the post-convolution
``[T, Q|K|V]`` buffer plus raw gate / beta logits and consumes zero-copy strided views.

Differences that follow from the gfx950 design: the chunk size is 64 (the reference's
kernels use 32), so the staging tensors ``g_cum`` and ``A`` have chunk-64 meaning (``A`` is
the bf16 high part of ``L^-1 diag(beta)`` per chunk, ``[chunks, H, 64, 64]``); the planner
arguments ``auto_cp``, ``overlap_warmup_threshold`` and ``force_tc01_cp_candidate`` are accepted
and have no effect because every sequence keeps its full history in one pass; chunk metadata is
built on the device, so no call ever reads ``cu_seqlens`` back to the host (``raw_cu_seqlens`` is
validated and used for two host-side decisions that change no bit of the results:
``pla_gdn_prefill_launch_raw``).  States are FP32 and k-last ``[slots, H, DV, DK]``; the legacy
k-first ``[N, H, DK, DV]`` state form is not provided.
"""

import ctypes
import math
from typing import Optional, Sequence, Tuple, Union

import torch

from ... import _lib
from .. import _sanity

CHUNK_SIZE = 64
DK = 128
DV = 128


# The compiled host layer (pla_amd/csrc/prefill_binding.cpp, `python -m pla_amd.build`): every call is offered to it
# first.  It takes calls in the plain serving form (dense rows on one GPU, FP32 k-last states, int32 offsets),
# allocates and launches without Python in between, and returns None for any other form, which then runs below
# with its conversions, diagnostics and error messages.  A tree without the module runs everything below.
_native = None


def _compiled():
    global _native
    if _native is None:
        try:
            import importlib
            _native = importlib.import_module("._C", __package__)
        except ModuleNotFoundError as exc:
            if exc.name is None or not exc.name.endswith("_C"):
                raise
            _native = False
    return _native


def _workspace(T, N, Hg, H, device):
    nbytes = _lib.load().pla_gdn_prefill_workspace_bytes(T, N, Hg, H)
    return torch.empty(nbytes, dtype=torch.uint8, device=device), nbytes


def chunk_gated_delta_rule_fwd(
    q: torch.Tensor,                       # [1, T, Hg, DK] bf16
    k: torch.Tensor,                       # [1, T, Hg, DK] bf16
    v: torch.Tensor,                       # [1, T, H, DV] bf16
    g: Optional[torch.Tensor],             # [1, T, H] fp32 log gate
    beta: Optional[torch.Tensor],          # [1, T, H] fp32 activated beta
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,          # [slots, H, DV, DK] fp32 (k-last)
    initial_state_indices: Optional[torch.Tensor] = None,  # [batch] int32 slots
    cu_seqlens: Optional[torch.Tensor] = None,             # [batch+1] int32
    output_final_state: bool = True,
    auto_cp: bool = True,
    overlap_warmup_threshold: Optional[float] = None,
    force_tc01_cp_candidate: bool = False,
    normalize_qk: bool = False,
    raw_cu_seqlens: Optional[Union[Sequence[int], torch.Tensor]] = None,
    raw_gate_a: Optional[torch.Tensor] = None,   # [T, H] bf16
    raw_beta_b: Optional[torch.Tensor] = None,   # [T, H] bf16
    A_log: Optional[torch.Tensor] = None,        # [H] fp32
    dt_bias: Optional[torch.Tensor] = None,      # [H] fp32
    final_state_dtype: Optional[torch.dtype] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, None, Optional[torch.Tensor]]:
    """Returns ``(g_cum_32, A, O, None, final_state)``.

    With ``initial_state_indices`` the state is an indexed pool updated in place (also when
    ``output_final_state`` is false) and ``final_state`` is the gathered copy ``pool[indices]``.
    Without indices ``initial_state`` is ``[batch, H, DV, DK]`` (read only) and a new
    ``final_state`` of the same shape is returned.  ``cu_seqlens`` may end before the physical
    token count; the padded suffix of ``O`` is zero and never touches a state.
    """
    native = _compiled()
    if native:
        try:
            taken = native.try_chunk_gated_delta_rule_fwd(
                q, k, v, g, beta, scale, initial_state, initial_state_indices, cu_seqlens, bool(output_final_state),
                overlap_warmup_threshold, bool(normalize_qk), raw_cu_seqlens, raw_gate_a, raw_beta_b, A_log, dt_bias,
                final_state_dtype)
        except TypeError:
            taken = None              # an argument of another type than the compiled signature: the checks below name it
        if taken is not None:
            return taken
    if not q.is_cuda:
        raise ValueError("q must be a CUDA tensor")
    raw_gate_args = (raw_gate_a, raw_beta_b, A_log, dt_bias)
    use_raw_gating = any(t is not None for t in raw_gate_args)
    if use_raw_gating and any(t is None for t in raw_gate_args):
        raise ValueError("raw gating requires raw_gate_a, raw_beta_b, A_log and dt_bias together")
    if use_raw_gating and (g is not None or beta is not None):
        raise ValueError("pass either g/beta or the raw gating tensors, not both")
    if not use_raw_gating and (g is None or beta is None):
        raise ValueError("g and beta are required without raw gating")
    if use_raw_gating and not normalize_qk:
        raise ValueError("raw gating is fused with q/k normalisation: pass normalize_qk=True")
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4 or q.size(0) != 1:
        raise ValueError("q, k, v must be packed as [1, T, heads, dim]")
    if q.dtype not in (torch.bfloat16, torch.float16) or k.dtype != q.dtype or v.dtype != q.dtype:
        raise ValueError("q, k, v must share bf16 or fp16")
    num_tokens, Hg, H = q.size(1), k.size(2), v.size(2)
    if q.shape != k.shape or v.size(1) != num_tokens:
        raise ValueError("q/k shapes and q/k/v token dimensions must match")
    if q.size(3) != DK or v.size(3) != DV:
        raise ValueError("head_dim must be 128")
    if Hg <= 0 or H % Hg != 0:
        raise ValueError(f"H must be a positive multiple of Hg, got H={H}, Hg={Hg}")
    for name, t in (("q", q), ("k", k), ("v", v)):
        if t.stride(3) != 1 or t.stride(2) != 128:
            raise ValueError(f"{name} head/feature axes must be contiguous")
    # q / k rows must start on 4-byte boundaries (the library copies rows that are not 16-byte aligned itself), v rows
    # are copied to LDS in 16-byte pieces: a view that breaks those alignments is materialised once
    if q.data_ptr() % 4 or q.stride(1) % 2:
        q = q.contiguous()
    if k.data_ptr() % 4 or k.stride(1) % 2:
        k = k.contiguous()
    if v.data_ptr() % 16 or v.stride(1) % 8:
        v = v.contiguous()
    if overlap_warmup_threshold is not None and (not math.isfinite(overlap_warmup_threshold)):
        raise ValueError("overlap_warmup_threshold must be finite")
    if scale is None:
        scale = q.size(-1) ** -0.5

    _sanity.offsets(cu_seqlens, num_tokens,
                    raw_cu_seqlens.tolist() if isinstance(raw_cu_seqlens, torch.Tensor) else raw_cu_seqlens, reference=q)
    _sanity.operand_range(q, v=v, initial_state=initial_state)
    if cu_seqlens is None:
        cu_seqlens = torch.tensor([0, num_tokens], dtype=torch.int32, device=q.device)
    cu32 = cu_seqlens.to(device=q.device, dtype=torch.int32).contiguous()
    if cu32.ndim != 1:
        raise ValueError("cu_seqlens must be a rank-1 tensor")
    batch = cu32.numel() - 1
    if batch <= 0:
        raise ValueError("cu_seqlens must describe at least one sequence")
    raw = None
    if raw_cu_seqlens is not None:
        if isinstance(raw_cu_seqlens, torch.Tensor):
            if (raw_cu_seqlens.device.type != "cpu" or raw_cu_seqlens.ndim != 1
                    or raw_cu_seqlens.dtype not in (torch.int32, torch.int64)):
                raise ValueError("raw_cu_seqlens must be a 1-D CPU int32 or int64 tensor")
            raw_cu_seqlens = raw_cu_seqlens.tolist()
        raw = tuple(raw_cu_seqlens)
        if len(raw) != batch + 1 or raw[0] != 0 or any(b < a for a, b in zip(raw, raw[1:])) \
                or raw[-1] > num_tokens:
            raise ValueError("raw_cu_seqlens must be monotone offsets matching cu_seqlens")

    indexed = initial_state_indices is not None
    # One dtype covers the incoming state, the indexed pool and the returned state (reference rule,
    # pla/prefill/flashqla/ops.py:440-451): final_state_dtype selects it, must agree with initial_state when
    # one is given, and defaults to that dtype, or to fp32 without an incoming state.
    if final_state_dtype is None:
        state_dtype = initial_state.dtype if initial_state is not None else torch.float32
    else:
        if final_state_dtype not in (torch.float32, torch.bfloat16):
            raise ValueError("final_state_dtype must be fp32 or bf16")
        if initial_state is not None and final_state_dtype != initial_state.dtype:
            raise ValueError("final_state_dtype must match the initial_state dtype")
        state_dtype = final_state_dtype
    if state_dtype == torch.bfloat16:
        # The kernels keep FP32 states: bf16 states are widened before the first kernel (exactly) and rounded
        # once after the last one; an indexed bf16 pool is updated in place at its indexed slots.
        if initial_state is not None and (initial_state.ndim != 4 or initial_state.size(1) != H
                                          or initial_state.size(2) != DV or initial_state.size(3) != DK):
            raise ValueError("initial_state must be [num_states,H,DV,DK] (k-last)")
        if indexed:
            idx = initial_state_indices
            if initial_state is None:
                raise ValueError("indexed initial_state must be given")
            if (idx.device != q.device or idx.dtype != torch.int32 or not idx.is_contiguous()
                    or idx.ndim != 1 or idx.numel() != batch):
                raise ValueError("initial_state_indices must be contiguous int32 [batch] on q.device")
            init32 = initial_state[idx.long()].to(torch.float32)
        else:
            if initial_state is not None and initial_state.size(0) < batch:
                raise ValueError("initial_state must be [num_states>=batch,H,DV,DK] (k-last)")
            init32 = None if initial_state is None else initial_state[:batch].to(torch.float32).contiguous()
        g_cum, ws, o, _, final32 = chunk_gated_delta_rule_fwd(
            q, k, v, g, beta, scale=scale, initial_state=init32, initial_state_indices=None, cu_seqlens=cu_seqlens,
            output_final_state=output_final_state or indexed, auto_cp=auto_cp,
            overlap_warmup_threshold=overlap_warmup_threshold, force_tc01_cp_candidate=force_tc01_cp_candidate,
            normalize_qk=normalize_qk, raw_cu_seqlens=raw_cu_seqlens, raw_gate_a=raw_gate_a, raw_beta_b=raw_beta_b,
            A_log=A_log, dt_bias=dt_bias, final_state_dtype=None)
        final = None if final32 is None else final32.to(torch.bfloat16)
        if indexed:
            initial_state[idx.long()] = final
        return g_cum, ws, o, None, (final if output_final_state else None)
    if indexed:
        if initial_state is None or initial_state.dtype != torch.float32 or not initial_state.is_contiguous():
            raise ValueError("indexed initial_state must be contiguous fp32")
        if (initial_state.ndim != 4 or initial_state.size(1) != H or initial_state.size(2) != DV
                or initial_state.size(3) != DK):
            raise ValueError("indexed initial_state must be [num_slots,H,DV,DK]")
        idx = initial_state_indices
        if (idx.device != q.device or idx.dtype != torch.int32 or not idx.is_contiguous()
                or idx.ndim != 1 or idx.numel() != batch):
            raise ValueError("initial_state_indices must be contiguous int32 [batch] on q.device")
    elif initial_state is not None:
        if initial_state.dtype != torch.float32 or not initial_state.is_contiguous():
            raise ValueError("initial_state must be contiguous fp32")
        if (initial_state.ndim != 4 or initial_state.size(0) < batch or initial_state.size(1) != H
                or initial_state.size(2) != DV or initial_state.size(3) != DK):
            raise ValueError("initial_state must be [num_states>=batch,H,DV,DK] (k-last)")

    dev = q.device
    o = torch.empty(1, num_tokens, H, DV, dtype=q.dtype, device=dev)
    g_cum = torch.empty(1, num_tokens, H, dtype=torch.float32, device=dev)
    ws, ws_bytes = _workspace(num_tokens, batch, Hg, H, dev)

    if indexed:
        h0, h0_idx, ht, ht_idx = initial_state, initial_state_indices, initial_state, initial_state_indices
        final = None
    else:
        h0, h0_idx = initial_state, None
        final = torch.empty(batch, H, DV, DK, dtype=torch.float32, device=dev) if output_final_state else None
        ht, ht_idx = final, None
        if final is not None:
            # sequences of length zero keep their incoming state
            if initial_state is not None:
                final.copy_(initial_state[:batch])
            else:
                final.zero_()

    if use_raw_gating:
        for name, t in (("raw_gate_a", raw_gate_a), ("raw_beta_b", raw_beta_b)):
            if t.dtype != q.dtype or t.dim() != 2 or t.size(0) != num_tokens or t.size(1) != H or t.stride(1) != 1:
                raise ValueError(f"{name} must be [T,H] in q's dtype with contiguous heads")
        for name, t in (("A_log", A_log), ("dt_bias", dt_bias)):
            if t.dtype != torch.float32 or t.numel() != H or not t.is_contiguous():
                raise ValueError(f"{name} must be contiguous fp32 [H]")
        a_ptr, b_ptr, sa, sb = raw_gate_a.data_ptr(), raw_beta_b.data_ptr(), raw_gate_a.stride(0), raw_beta_b.stride(0)
        al_ptr, dt_ptr, g_ptr, bt_ptr = A_log.data_ptr(), dt_bias.data_ptr(), None, None
    else:
        g32 = g.reshape(num_tokens, H)
        b32 = beta.reshape(num_tokens, H)
        if g32.dtype != torch.float32 or b32.dtype != torch.float32 or not g32.is_contiguous() or not b32.is_contiguous():
            raise ValueError("g and beta must be contiguous fp32 [1,T,H]")
        a_ptr = b_ptr = al_ptr = dt_ptr = None
        sa = sb = 0
        g_ptr, bt_ptr = g32.data_ptr(), b32.data_ptr()

    # host offsets, when the caller has them, go along (one decision is taken from them: see pla_gdn_prefill_launch_raw)
    raw_host = (ctypes.c_int32 * (batch + 1))(*raw) if raw is not None else None
    _lib.call(
        "pla_gdn_prefill_launch_raw",
        q.data_ptr(), k.data_ptr(), v.data_ptr(), q.stride(1), k.stride(1), v.stride(1),
        a_ptr, b_ptr, sa, sb, al_ptr, dt_ptr, g_ptr, bt_ptr,
        cu32.data_ptr(), batch, num_tokens, float(scale), int(bool(normalize_qk)),
        _lib.ptr(h0), _lib.ptr(h0_idx), h0.stride(0) if h0 is not None else 0,
        _lib.ptr(ht), _lib.ptr(ht_idx), ht.stride(0) if ht is not None else 0,
        o.data_ptr(), ws.data_ptr(), ws_bytes, g_cum.data_ptr(), None,
        Hg, H, DK, DV, _lib.dtype_code(q.dtype), _lib.current_stream(dev),
        ctypes.cast(raw_host, ctypes.c_void_p) if raw_host is not None else None)

    if output_final_state:
        final = initial_state[initial_state_indices.long()] if indexed else final
    else:
        final = None
    return g_cum, ws, o, None, final


def gdn_prefill_packed_qkv_fwd(
    packed_qkv: torch.Tensor,                # [T, 2*Hg*DK + H*DV] bf16
    raw_gate_a: torch.Tensor,                # [T,H] bf16
    raw_beta_b: torch.Tensor,                # [T,H] bf16
    A_log: torch.Tensor,                     # [H] fp32
    dt_bias: torch.Tensor,                   # [H] fp32
    cu_seqlens: torch.Tensor,                # [batch+1] int32
    *,
    num_qk_heads: int,
    num_v_heads: int,
    scale: Optional[float] = None,
    initial_state: Optional[torch.Tensor] = None,
    initial_state_indices: Optional[torch.Tensor] = None,
    output_final_state: bool = True,
    auto_cp: bool = True,
    overlap_warmup_threshold: Optional[float] = None,
    force_tc01_cp_candidate: bool = False,
    raw_cu_seqlens: Optional[Union[Sequence[int], torch.Tensor]] = None,
    final_state_dtype: Optional[torch.dtype] = None,
):
    """GDN prefill directly on a post-convolution ``Q|K|V`` buffer (token stride may exceed the
    row width; features inside a token contiguous).  Q/K/V are aliases of ``packed_qkv``."""
    native = _compiled()
    if native:
        try:
            taken = native.try_gdn_prefill_packed_qkv_fwd(
                packed_qkv, raw_gate_a, raw_beta_b, A_log, dt_bias, cu_seqlens, num_qk_heads, num_v_heads, scale,
                initial_state, initial_state_indices, bool(output_final_state), overlap_warmup_threshold, raw_cu_seqlens,
                final_state_dtype)
        except TypeError:
            taken = None
        if taken is not None:
            return taken
    if not packed_qkv.is_cuda:
        raise ValueError("packed_qkv must be a CUDA tensor")
    if packed_qkv.ndim != 2:
        raise ValueError("packed_qkv must be rank-2 [T,QKV]")
    if packed_qkv.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError("packed_qkv must be fp16 or bf16")
    if packed_qkv.stride(1) != 1:
        raise ValueError("packed_qkv features must be contiguous")
    if num_qk_heads <= 0 or num_v_heads <= 0:
        raise ValueError("num_qk_heads and num_v_heads must be positive")
    T = packed_qkv.size(0)
    if T == 0:
        raise ValueError("GDN packed prefill does not support an empty token dimension")
    Hg, H = int(num_qk_heads), int(num_v_heads)
    qk_width = Hg * DK
    packed_width = 2 * qk_width + H * DV
    if packed_qkv.size(1) != packed_width:
        raise ValueError(f"packed_qkv width must be {packed_width} for H={H}, Hg={Hg}, got {packed_qkv.size(1)}")
    token_stride = packed_qkv.stride(0)
    if token_stride < packed_width:
        raise ValueError("packed_qkv token stride must cover the complete Q|K|V row")
    off = packed_qkv.storage_offset()
    batch_stride = max(T, 1) * token_stride
    q = packed_qkv.as_strided((1, T, Hg, DK), (batch_stride, token_stride, DK, 1), storage_offset=off)
    k = packed_qkv.as_strided((1, T, Hg, DK), (batch_stride, token_stride, DK, 1), storage_offset=off + qk_width)
    v = packed_qkv.as_strided((1, T, H, DV), (batch_stride, token_stride, DV, 1), storage_offset=off + 2 * qk_width)
    return chunk_gated_delta_rule_fwd(
        q, k, v, None, None, scale=scale, initial_state=initial_state,
        initial_state_indices=initial_state_indices, cu_seqlens=cu_seqlens,
        output_final_state=output_final_state, auto_cp=auto_cp,
        overlap_warmup_threshold=overlap_warmup_threshold,
        force_tc01_cp_candidate=force_tc01_cp_candidate, normalize_qk=True,
        raw_cu_seqlens=raw_cu_seqlens, raw_gate_a=raw_gate_a, raw_beta_b=raw_beta_b,
        A_log=A_log, dt_bias=dt_bias, final_state_dtype=final_state_dtype)
