"""Diagnostic checks of prefill metadata, enabled by ``PLA_SANITY_CHECK=1`` (read on every call).

Mirrors the reference helper pla/prefill/_sanity.py:46-110: a violation raises
``AssertionError("PLA_SANITY_CHECK [prefill]: ...")`` before anything is launched.  The offsets are
checked before they are narrowed to int32; device values are compared with ``raw_cu_seqlens`` only
outside stream capture (they would need a device-to-host copy).
"""

import numbers
import os

import torch

_INT32_MAX = 2 ** 31 - 1


def enabled():
    return os.environ.get("PLA_SANITY_CHECK") == "1"


def check(condition, message):
    if not condition:
        raise AssertionError(f"PLA_SANITY_CHECK [prefill]: {message}")


def _capturing(reference):
    if not reference.is_cuda:
        return False
    with torch.cuda.device(reference.device):
        return torch.cuda.is_current_stream_capturing()


def _offset_values(values, capacity, count=None):
    values = tuple(values)
    check(len(values) >= 2 and (count is None or len(values) == count), "offsets must have batch+1 entries")
    check(all(isinstance(v, numbers.Integral) for v in values), "offsets must contain integers")
    check(values[0] == 0, "offsets must start at zero")
    check(all(0 <= a <= b <= min(capacity, _INT32_MAX) for a, b in zip(values, values[1:])),
          "offsets must be monotonic and within token capacity/int32 range")
    return values


def offsets(cu, capacity, raw=None, *, reference=None):
    """Checks ``cu`` (device or host offsets, None for one fixed-length sequence) and ``raw`` (host
    offsets) against the token capacity and against each other.  No-op unless the mode is on."""
    if not enabled():
        return
    check(isinstance(capacity, numbers.Integral) and 0 <= capacity <= _INT32_MAX, "token capacity must fit int32")
    if cu is None:
        if raw is not None:
            check(_offset_values(raw, capacity, 2) == (0, capacity), "fixed-length host offsets must be [0,T]")
        return
    check(isinstance(cu, torch.Tensor) and cu.layout == torch.strided, "cu_seqlens must be a strided tensor")
    check(cu.ndim == 1 and cu.numel() >= 2, "cu_seqlens must be [batch+1]")
    check(cu.dtype in (torch.int32, torch.int64), "cu_seqlens must be int32 or int64 before conversion")
    check(cu.device.type in ("cpu", "cuda"), "cu_seqlens must be CPU or GPU metadata")
    host = _offset_values(raw, capacity, cu.numel()) if raw is not None else None
    if _capturing(cu if reference is None else reference):
        return
    device_values = _offset_values(cu.detach().cpu().tolist(), capacity, cu.numel())
    if host is not None:
        check(host == device_values, "raw_cu_seqlens must equal device cu_seqlens")


_OPERAND_MAX = 65504.0          # largest finite fp16: the matrix products take fp16 operands


def operand_range(reference, **tensors):
    """The prefill products round their operands (v, the state, intermediate products) to fp16, so values
    beyond +-65504 or non-finite ones would turn into infinities inside the kernels.  Checks the named
    tensors (``None`` entries are skipped) outside stream capture; no-op unless the mode is on."""
    if not enabled() or _capturing(reference):
        return
    for name, t in tensors.items():
        if t is None or t.numel() == 0:
            continue
        peak = float(t.detach().abs().max().float())          # NaN propagates through max
        check(peak == peak and peak <= _OPERAND_MAX,
              f"{name} must be finite and within the fp16 operand range (|x| <= 65504), got max |x| = {peak}")
