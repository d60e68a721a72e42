"""KDA chunked prefill on MI355X behind FlashKDAPro's Python interface.

``flashkda_fwd`` keeps the reference's signature, ownership and error behaviour
(pla/prefill/flashkdapro/ops.py:68-219): the caller owns ``out`` and ``final_state``; the function
returns ``None``; ``g`` is the raw gate (the lower-bound gate is applied inside), ``beta`` raw
logits; ``state_pool`` + ``state_indices`` update an indexed pool in place.

Differences that follow from the gfx950 design: chunk size 64; states are FP32 only and are NOT
rounded to bf16 at the read / publish boundary (the reference's tc01 backend rounds them); chunk
metadata is built on the device, and ``raw_cu_seqlens`` is validated and used for one host-side
decision that changes no bit of the results (``pla_kda_prefill_launch_raw``); there is
one backend, so the ``PLA_FLASHKDA_*`` routing variables have no effect.
"""

import ctypes
from typing import Optional, Tuple

import torch

from ... import _lib
from .. import _sanity

CHUNK_SIZE = 64
DK = 128
DV = 128


def _token_rows(name, t, H, width):
    """[T, H, width] with contiguous heads/channels; returns the token pitch or None if a copy is needed."""
    if t.dim() != 3 or t.size(1) != H or t.size(2) != width:
        raise ValueError(f"{name} must be [total_tokens, H, {width}], got {tuple(t.shape)}")
    if t.stride(2) == 1 and t.stride(1) == width and t.stride(0) % 8 == 0 and t.data_ptr() % 16 == 0:
        return t, t.stride(0)
    t = t.contiguous()
    return t, t.stride(0)


# The compiled host layer (pla_amd/csrc/prefill_binding.cpp): see pla_amd/prefill/flashqla/ops.py.
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


def _workspace(T, N, H, device):
    nbytes = _lib.load().pla_kda_prefill_workspace_bytes(T, N, H)
    return torch.empty(nbytes, dtype=torch.uint8, device=device), nbytes


def flashkda_fwd(
    q: torch.Tensor,                       # [total_tokens, H, DK] bf16
    k: torch.Tensor,                       # [total_tokens, H, DK] bf16
    v: torch.Tensor,                       # [total_tokens, H, DV] bf16
    g: torch.Tensor,                       # [total_tokens, H, DK] bf16 (raw gate)
    beta: torch.Tensor,                    # [total_tokens, H] bf16 (raw logits)
    A_log: torch.Tensor,                   # [H] fp32
    dt_bias: torch.Tensor,                 # [H, DK] fp32
    out: torch.Tensor,                     # [total_tokens, H, DV] bf16   (written)
    scale: Optional[float] = None,
    lower_bound: float = -5.0,
    initial_state: Optional[torch.Tensor] = None,   # [N, H, DV, DK] fp32
    final_state: Optional[torch.Tensor] = None,     # [N, H, DV, DK] fp32 (written)
    cu_seqlens: Optional[torch.Tensor] = None,      # [N+1] int32 (int64 accepted)
    state_pool: Optional[torch.Tensor] = None,      # [slots,H,DV,DK] fp32 (in-place)
    state_indices: Optional[torch.Tensor] = None,   # [N] int32 cache slots
    raw_cu_seqlens: Optional[Tuple[int, ...]] = None,
) -> None:
    """FlashKDA prefill forward. Writes ``out`` (and ``final_state`` / ``state_pool``)."""
    native = _compiled()
    if native and (state_pool is None or (initial_state is None and final_state is None and state_indices is not None)):
        first, last = (state_pool, state_pool) if state_pool is not None else (initial_state, final_state)
        try:
            if native.try_flashkda_fwd(q, k, v, g, beta, A_log, dt_bias, out, 128 ** -0.5 if scale is None else float(scale),
                                       float(lower_bound), first, last, cu_seqlens, state_indices, raw_cu_seqlens):
                return None
        except TypeError:
            pass                      # an argument of another type than the compiled signature: the checks below name it
    if not q.is_cuda:
        raise ValueError("q must be a CUDA tensor")
    for name, t in (("k", k), ("v", v), ("g", g), ("beta", beta), ("A_log", A_log), ("dt_bias", dt_bias), ("out", out)):
        if t.device != q.device:
            raise ValueError(f"{name} must be on {q.device}, got {t.device}")
    for name, t in (("initial_state", initial_state), ("final_state", final_state), ("cu_seqlens", cu_seqlens),
                    ("state_pool", state_pool), ("state_indices", state_indices)):
        if t is not None and t.device != q.device:
            raise ValueError(f"{name} must be on {q.device}, got {t.device}")
    if state_pool is not None:
        if initial_state is not None or final_state is not None:
            raise ValueError("state_pool is mutually exclusive with initial_state/final_state")
        if state_indices is None:
            raise ValueError("state_pool requires state_indices")
        initial_state = state_pool
        final_state = state_pool
    elif state_indices is not None and initial_state is None and final_state is None:
        raise ValueError("state_indices requires state_pool, initial_state, or final_state")
    if q.dim() != 3 or q.size(2) != DK:
        raise ValueError("q must be [total_tokens, H, 128]")
    T, H = q.size(0), q.size(1)
    if T == 0:
        raise ValueError("flashkda_fwd does not support an empty token dimension")
    for name, t in (("q", q), ("k", k), ("v", v), ("g", g), ("beta", beta), ("out", out)):
        if t.dtype != torch.bfloat16:
            raise ValueError(f"{name} must be bf16")
    if scale is None:
        scale = q.size(-1) ** -0.5
    if not (-5.0 <= float(lower_bound) <= 0.0):
        raise ValueError("lower_bound is expected in [-5, 0]")
    if tuple(out.shape) != (T, H, DV) or not out.is_contiguous():
        raise ValueError("out must be contiguous [total_tokens, H, DV]")
    q, sq = _token_rows("q", q, H, DK)
    k, sk = _token_rows("k", k, H, DK)
    v, sv = _token_rows("v", v, H, DV)
    g, sg = _token_rows("g", g, H, DK)
    if beta.dim() != 2 or beta.size(0) != T or beta.size(1) != H:
        raise ValueError("beta must be [total_tokens, H]")
    if beta.stride(1) != 1:
        beta = beta.contiguous()
    A_log = A_log.to(torch.float32).contiguous()
    dt_bias = dt_bias.to(torch.float32).reshape(H, DK).contiguous()
    if A_log.numel() != H:
        raise ValueError("A_log must be [H]")

    _sanity.offsets(cu_seqlens, T, raw_cu_seqlens, reference=q)
    _sanity.operand_range(q, v=v, initial_state=initial_state)
    if cu_seqlens is None:
        cu32 = torch.tensor([0, T], dtype=torch.int32, device=q.device)
    else:
        if cu_seqlens.dtype not in (torch.int32, torch.int64):
            raise ValueError("cu_seqlens must be int32 or int64")
        cu32 = cu_seqlens.to(torch.int32).contiguous()
    N = cu32.numel() - 1
    if N <= 0:
        raise ValueError("cu_seqlens must describe at least one sequence")
    raw_host = None
    if raw_cu_seqlens is not None:
        raw = tuple(int(x) for x in raw_cu_seqlens)
        if len(raw) != N + 1 or raw[0] != 0 or any(b < a for a, b in zip(raw, raw[1:])) or raw[-1] > T:
            raise ValueError("raw_cu_seqlens must be N+1 monotone offsets describing the same packed batch")
        # host offsets, when the caller has them, go along (one decision is taken from them: see pla_kda_prefill_launch_raw)
        raw_host = (ctypes.c_int32 * (N + 1))(*raw)

    indexed = state_indices is not None
    if indexed and (state_indices.dtype != torch.int32 or state_indices.dim() != 1 or state_indices.numel() != N
                    or not state_indices.is_contiguous()):
        raise ValueError("state_indices must be contiguous int32 [N]")
    staged = False
    for name, t in (("initial_state", initial_state), ("final_state", final_state)):
        if t is None:
            continue
        if t.dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"{name} must be fp32 or bf16")
        if t.dim() != 4 or t.size(1) != H or t.size(2) != DV or t.size(3) != DK:
            raise ValueError(f"{name} must be [N, H, DV, DK]")
        if not indexed and t.size(0) < N:
            raise ValueError(f"{name} must hold at least N states")
        # the kernels read and write dense FP32 slots; anything else goes through a dense FP32 copy
        staged = staged or t.dtype != torch.float32 or not t[0].is_contiguous() or t.stride(0) % 4 != 0 or t.data_ptr() % 16 != 0
    if initial_state is not None and final_state is not None and initial_state.dtype != final_state.dtype:
        raise ValueError("initial_state and final_state must have the same dtype")
    if final_state is not None and final_state.data_ptr() == out.data_ptr():
        raise ValueError("final_state must not share storage with out")
    if staged:
        # As the reference does for layouts its kernels do not consume in place: the states are materialised
        # once before the first kernel (exactly: bf16 widens to FP32) and written back after the last one
        # (bf16 states are rounded once, at the end).  Sequences of length zero publish their incoming state.
        rows = state_indices.long() if indexed else slice(0, N)
        init32 = None if initial_state is None else initial_state[rows].to(torch.float32).contiguous()
        fin32 = None
        if final_state is not None:
            fin32 = torch.empty(N, H, DV, DK, dtype=torch.float32, device=q.device)
        flashkda_fwd(q, k, v, g, beta, A_log, dt_bias, out, scale=scale, lower_bound=lower_bound, initial_state=init32,
                     final_state=fin32, cu_seqlens=cu_seqlens, raw_cu_seqlens=raw_cu_seqlens)
        if final_state is not None:
            final_state[rows] = fin32.to(final_state.dtype)
        return None

    ws, nbytes = _workspace(T, N, H, q.device)
    if final_state is not None and not (initial_state is not None and final_state.data_ptr() == initial_state.data_ptr()):
        # sequences of length zero keep their incoming (or zero) state
        if initial_state is not None:
            if indexed:
                final_state[state_indices.long()] = initial_state[state_indices.long()]
            else:
                final_state[:N].copy_(initial_state[:N])
        else:
            if indexed:
                final_state[state_indices.long()] = 0
            else:
                final_state[:N].zero_()
    idx_ptr = _lib.ptr(state_indices) if indexed else None
    _lib.call(
        "pla_kda_prefill_launch_raw",
        q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), beta.data_ptr(),
        sq, sk, sv, sg, beta.stride(0),
        A_log.data_ptr(), dt_bias.data_ptr(), float(lower_bound), float(scale),
        cu32.data_ptr(), N, T,
        _lib.ptr(initial_state), idx_ptr, initial_state.stride(0) if initial_state is not None else 0,
        _lib.ptr(final_state), idx_ptr, final_state.stride(0) if final_state is not None else 0,
        out.data_ptr(), ws.data_ptr(), nbytes, H, DK, DV, _lib.BF16, _lib.current_stream(q.device), raw_host)
    return None
