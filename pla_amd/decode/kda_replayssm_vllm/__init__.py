"""Request-row KDA replay for a vLLM-style runner (``pla.decode.kda_replayssm_vllm``).

``kda_replay_verify`` (reference pla/decode/kda_replayssm_vllm/__init__.py:46-76, binding
src/decode/kda_replayssm_vllm/kda_replayssm_vllm.cpp:121-235): verify of up to ``Q`` draft tokens per
request against a paged FP32 checkpoint.  The conv history and the checkpoint are read-only; the
per-token records (post-conv k, v in bf16; log-decay, beta in FP32) and the conv window after every
token are written to the request's row of ``records``; only real query intervals are written.
The draft window is limited to 8 tokens here (the reference allows 32).

``KDAReplayCommitContext`` (same file :149-232): the commit plan is built on the device from the sampled
counts (and, in align mode, the block table), so nothing is read back and a commit can be captured in a
graph; per layer the committed prefix of the records is folded from the source checkpoint into the planned
final (and boundary) slot and the matching conv windows are copied into those slots' conv history.
"""

import ctypes
import os
from dataclasses import dataclass
from numbers import Integral, Real
from typing import Optional

import torch

from ... import _lib

__all__ = ["KDAReplayRecords", "KDAReplayCommitPlan", "KDAReplayCommitContext", "kda_replay_verify"]

_BYPASS = os.environ.get("PLA_BYPASS_EXEC", "0") == "1"   # read once, like src/bypass_exec.h:44-50
D = 128


@dataclass(frozen=True)
class KDAReplayRecords:
    """Per-request-row records: rawv, rawk [R,H,Q,128] bf16, g [R,H,Q,128] and beta [R,H,Q] float32,
    conv [R,Q,3*H*128,3] bf16 (the window after each token, q | k | v channels)."""
    rawv: torch.Tensor
    rawk: torch.Tensor
    g: torch.Tensor
    beta: torch.Tensor
    conv: torch.Tensor

    @classmethod
    def allocate(cls, max_num_reqs, num_heads, spec_query_len, device):
        if max_num_reqs < 0 or num_heads < 1 or not 1 <= spec_query_len <= 32:
            raise ValueError("records require R >= 0, H > 0 and Q in [1, 32]")
        shape = (max_num_reqs, num_heads, spec_query_len, D)
        return cls(torch.empty(shape, dtype=torch.bfloat16, device=device),
                   torch.empty(shape, dtype=torch.bfloat16, device=device),
                   torch.empty(shape, dtype=torch.float32, device=device),
                   torch.empty(shape[:-1], dtype=torch.float32, device=device),
                   torch.empty((max_num_reqs, spec_query_len, 3 * num_heads * D, 3),
                               dtype=torch.bfloat16, device=device))


def _need(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _index(t, ref):
    _need(t.device == ref.device and t.dim() == 1 and t.dtype in (torch.int32, torch.int64),
          "indices must be int32/int64 vectors")
    t = t.contiguous()
    return t, int(t.dtype == torch.int64)


def _paged_cache(conv, state, layout, H, slots):
    """Checks of the paged conv / checkpoint pair; returns the conv cache in [slots, channels, history] view
    (src/decode/kda_replayssm_vllm/kda_replayssm_vllm.cpp:57-82)."""
    _need(state.is_cuda and H > 0 and slots > 0, "paged state requires a GPU tensor, H > 0, slots > 0")
    _need(state.dtype == torch.float32 and tuple(state.shape) == (slots, H, D, D) and state.stride(3) == 1
          and state.stride(2) == D and state.stride(1) == D * D and state.stride(0) >= H * D * D
          and state.stride(0) % 4 == 0 and state.data_ptr() % 16 == 0,
          "state must be float4-aligned fp32 [slots,H,128,128] with contiguous pages")
    _need(layout in ("DS", "SD"), "conv_state_layout must be DS or SD")
    _need(conv.dim() == 3 and conv.size(0) == slots and conv.dtype == torch.bfloat16 and conv.device == state.device,
          "conv must be bf16 with three dimensions")
    ds = conv if layout == "DS" else conv.transpose(1, 2)
    _need(ds.size(1) == 3 * H * D and ds.size(2) >= 3,
          "conv must contain 3*H*128 channels and at least three history items")
    _need((ds.stride(2) == 1 and ds.stride(1) >= ds.size(2)) or (ds.stride(1) == 1 and ds.stride(2) >= ds.size(1)),
          "conv channel/history dimensions must not overlap")
    _need(ds.stride(0) >= (ds.size(1) - 1) * ds.stride(1) + (ds.size(2) - 1) * ds.stride(2) + 1,
          "conv pages must not overlap")
    return ds


def _check_records(records, ref, H, Q, R):
    _need(1 <= Q <= 32 and R >= 0, "records require Q in [1,32] and R >= 0")
    for t, dtype, shape in ((records.rawv, torch.bfloat16, (R, H, Q, D)), (records.rawk, torch.bfloat16, (R, H, Q, D)),
                            (records.g, torch.float32, (R, H, Q, D)), (records.beta, torch.float32, (R, H, Q)),
                            (records.conv, torch.bfloat16, (R, Q, 3 * H * D, 3))):
        _need(t.device == ref.device and t.dtype == dtype and tuple(t.shape) == shape and t.is_contiguous(),
              "invalid replay tensor shape/dtype/contiguity")
    for t in (records.rawv, records.rawk, records.g, records.beta):
        _need(t.data_ptr() % 16 == 0, "replay records must be 16-byte aligned")


def _span(t):
    if t.numel() == 0:
        return t.data_ptr(), t.data_ptr()
    extent = 1 + sum((t.size(d) - 1) * t.stride(d) for d in range(t.dim()))
    return t.data_ptr(), t.data_ptr() + extent * t.element_size()


def _disjoint(writes, reads):
    """Conservative byte-span check: written tensors alias neither each other nor anything read."""
    def overlap(a, b):
        (a0, a1), (b0, b1) = _span(a), _span(b)
        return a0 < b1 and b0 < a1
    for i, w in enumerate(writes):
        _need(not any(overlap(w, other) for other in writes[:i]), "replay writes must not alias")
        _need(not any(overlap(w, r) for r in reads), "replay writes must not alias inputs/cache")


def kda_replay_verify(*, mixed_qkv, raw_g, raw_beta, conv_weight, conv_state, checkpoint_state, A_log, dt_bias,
                      lower_bound, records, query_start_loc, state_indices, conv_state_layout,
                      out: Optional[torch.Tensor] = None, scale=None, null_block_id=0):
    """Read a paged checkpoint and write only real query intervals and records.

    mixed_qkv [T, 3*H*128], raw_g [T, H*128], raw_beta [T, H]: bf16 projection views (positive token stride,
    contiguous channels); conv_weight float32 [3*H*128, 4]; conv_state bf16 paged, ``DS`` = [slots, channels,
    history] or ``SD`` = [slots, history, channels], only its first three history items are read;
    checkpoint_state float32 [slots, H, 128, 128] with a page pitch; query_start_loc [N+1] and state_indices [N]
    int32 or int64.  A slot <= null_block_id yields zero output rows; an empty, overlong or out-of-range
    query interval is skipped.  Returns ``out`` [T, H*128] bf16 (rows outside query intervals are not written).
    """
    if not isinstance(lower_bound, Real) or (scale is not None and not isinstance(scale, Real)):
        raise TypeError("scale and lower_bound must be host numeric scalars")
    if not isinstance(null_block_id, Integral):
        raise TypeError("null_block_id must be a host integer")
    state = checkpoint_state
    _need(state.dim() == 4 and records.rawv.dim() == 4, "invalid state/records rank")
    H, slots, Q, R = state.size(1), state.size(0), records.rawv.size(2), records.rawv.size(0)
    if out is None:
        out = torch.empty(mixed_qkv.size(0), H * D, dtype=torch.bfloat16, device=mixed_qkv.device)
    if _BYPASS:
        return out
    _need(null_block_id in (-1, 0), "null_block_id must be -1 or 0")
    cs = _paged_cache(conv_state, state, conv_state_layout, H, slots)
    _check_records(records, state, H, Q, R)
    for t in (mixed_qkv, raw_g, raw_beta, conv_weight, A_log, dt_bias, out, query_start_loc, state_indices):
        _need(t.device == state.device, "replay tensors must share one device")
    x = mixed_qkv
    _need(x.dim() == 2 and x.size(1) == 3 * H * D and x.stride(1) == 1 and x.stride(0) >= 3 * H * D
          and x.dtype == torch.bfloat16, "mixed_qkv must be bf16 [T,3*H*128] with contiguous channels")
    T = x.size(0)
    for t, channels in ((raw_g, H * D), (raw_beta, H)):
        _need(tuple(t.shape) == (T, channels) and t.stride(1) == 1 and t.stride(0) >= channels
              and t.dtype == torch.bfloat16, "gate/beta must be bf16 projection views")
    _need(conv_weight.dtype == torch.float32 and tuple(conv_weight.shape) == (3 * H * D, 4) and conv_weight.is_contiguous(),
          "invalid replay tensor shape/dtype/contiguity")
    _need(A_log.numel() == H and dt_bias.numel() == H * D and A_log.is_contiguous() and dt_bias.is_contiguous()
          and A_log.dtype == torch.float32 and dt_bias.dtype == torch.float32, "gate weights must be contiguous fp32")
    _need(out.dtype == torch.bfloat16 and tuple(out.shape) == (T, H * D) and out.is_contiguous(),
          "invalid replay tensor shape/dtype/contiguity")
    scale = D ** -0.5 if scale is None else float(scale)
    _need(scale == scale and abs(scale) != float("inf") and lower_bound == lower_bound
          and abs(lower_bound) != float("inf") and lower_bound < 0, "scale/lower_bound must be finite fp32; bound < 0")
    cu, cu_wide = _index(query_start_loc, state)
    src, src_wide = _index(state_indices, state)
    N = src.numel()
    _need(cu.numel() == N + 1 and N <= R, "query index count exceeds record capacity")
    _disjoint([out, records.rawv, records.rawk, records.g, records.beta, records.conv],
              [x, raw_g, raw_beta, conv_weight, conv_state, state, A_log, dt_bias, cu, src])
    if N == 0:
        return out
    windows = records.conv
    strides = ([x.stride(0)] * 3 + [raw_g.stride(0), raw_beta.stride(0)] + list(cs.stride()) * 3
               + list(windows.stride()) * 3)
    c_strides = (ctypes.c_int64 * 26)(*strides)
    cb = H * D * 2                                           # bytes of one q / k / v channel segment
    xp, cp, wp, wtp = x.data_ptr(), conv_state.data_ptr(), windows.data_ptr(), conv_weight.data_ptr()
    with torch.cuda.device(state.device):
        _lib.call(
            "pla_kda_replay_verify_native_launch", xp, xp + cb, xp + 2 * cb, raw_g.data_ptr(), raw_beta.data_ptr(),
            wtp, wtp + H * D * 16, wtp + 2 * H * D * 16,
            cp, cp + cb * cs.stride(1), cp + 2 * cb * cs.stride(1),
            A_log.data_ptr(), dt_bias.data_ptr(), state.data_ptr(), out.data_ptr(),
            wp, wp + cb * windows.stride(2), wp + 2 * cb * windows.stride(2),
            records.rawv.data_ptr(), records.rawk.data_ptr(), records.g.data_ptr(), records.beta.data_ptr(),
            src.data_ptr(), src_wide, cu.data_ptr(), cu_wide, H, N, Q, scale, float(lower_bound),
            ctypes.cast(c_strides, ctypes.c_void_p), state.stride(0), slots, T, int(null_block_id),
            _lib.current_stream(state.device))
    return out


# ---- commit -----------------------------------------------------------------------------------------

@dataclass(frozen=True)
class KDAReplayCommitPlan:
    """Views of the device plan, ``max_num_reqs`` entries each (zeroes for inactive, invalid and
    conflicting requests)."""
    commit_lens: torch.Tensor
    final_state_indices: torch.Tensor
    boundary_state_indices: torch.Tensor
    boundary_recovery_lens: torch.Tensor


def _page_runs(conv_ds, state):
    """Writable byte runs of one layer inside a page: (page pitch in bytes, number of pages, run starts of
    page 0 as absolute addresses, run lengths).  The commit writes the whole checkpoint of a slot and the
    first three history items of every conv channel."""
    import numpy as np
    pitch_s = state.stride(0) * 4
    starts = [np.array([state.data_ptr()], dtype=np.int64)]
    lengths = [np.array([state.size(1) * D * D * 4], dtype=np.int64)]
    channels = conv_ds.size(1)
    if conv_ds.stride(2) == 1:                       # history contiguous: one 6-byte run per channel
        starts.append(conv_ds.data_ptr() + np.arange(channels, dtype=np.int64) * conv_ds.stride(1) * 2)
        lengths.append(np.full(channels, 6, dtype=np.int64))
    else:                                            # channels contiguous: three runs
        starts.append(conv_ds.data_ptr() + np.arange(3, dtype=np.int64) * conv_ds.stride(2) * 2)
        lengths.append(np.full(3, channels * 2, dtype=np.int64))
    return (pitch_s, conv_ds.stride(0) * 2), state.size(0), np.concatenate(starts), np.concatenate(lengths)


def _layers_overlap(a, b):
    """Whether the writable cache regions of two layers intersect.  Exact when both layers page with one
    common pitch (their runs are compared modulo the pitch, which may pair pages past either end of a
    pool: conservative there); otherwise the whole extents are compared."""
    import numpy as np
    (pitch_a, conv_pitch_a), pages_a, starts_a, lens_a = a
    (pitch_b, conv_pitch_b), pages_b, starts_b, lens_b = b
    if not (pitch_a == conv_pitch_a == pitch_b == conv_pitch_b):
        lo_a, hi_a = starts_a.min(), (starts_a + lens_a).max() + (pages_a - 1) * max(pitch_a, conv_pitch_a)
        lo_b, hi_b = starts_b.min(), (starts_b + lens_b).max() + (pages_b - 1) * max(pitch_b, conv_pitch_b)
        return bool(lo_a < hi_b and lo_b < hi_a)
    pitch = pitch_a
    extent_a = (starts_a + lens_a).max() + (pages_a - 1) * pitch
    extent_b = (starts_b + lens_b).max() + (pages_b - 1) * pitch
    if not (starts_a.min() < extent_b and starts_b.min() < extent_a):
        return False
    origin = min(starts_a.min(), starts_b.min())

    def circle(starts, lens):                        # intervals on [0, pitch), wrapped ones split
        s = (starts - origin) % pitch
        e = s + lens
        wrap = e > pitch
        return np.concatenate([s, np.zeros(int(wrap.sum()), dtype=np.int64)]), \
            np.concatenate([np.minimum(e, pitch), (e - pitch)[wrap]])
    sa, ea = circle(starts_a, lens_a)
    sb, eb = circle(starts_b, lens_b)
    order = np.argsort(sb)
    sb, eb = sb[order], np.maximum.accumulate(eb[order])
    # an interval of a overlaps some interval of b iff a b-interval starting before its end reaches past its start
    idx = np.searchsorted(sb, ea, side="left") - 1
    hit = (idx >= 0) & (eb[np.maximum(idx, 0)] > sa)
    return bool(hit.any())


class KDAReplayCommitContext:
    """Layer descriptors and reusable device plan buffers of the request-row commit
    (reference pla/decode/kda_replayssm_vllm/__init__.py:149-232).

    Create outside graph capture and keep the cache and record tensors in place for the lifetime of the
    context; writable cache regions of different layers must be disjoint.  Commits, reads of the returned
    plan and replays of graphs captured with this context must be ordered on one stream: the next commit
    overwrites the plan.  ``layers``: objects with ``kv_cache = (conv, state)`` and ``replay_records``.
    """

    @classmethod
    def create(cls, layers, spec_query_len, max_num_reqs, conv_state_layout="SD", null_block_id=0):
        layers = tuple(layers)
        if not layers or not 1 <= spec_query_len <= 32 or max_num_reqs < 0:
            raise ValueError("context requires layers, R >= 0 and Q in [1, 32]")
        if null_block_id not in (-1, 0):
            raise ValueError("null_block_id must be -1 or 0")
        device = layers[0].kv_cache[1].device
        if device.type != "cuda":
            raise ValueError("commit context requires GPU tensors")
        with torch.cuda.device(device):
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("create commit context before graph capture")
        slots, heads = layers[0].kv_cache[1].shape[:2]
        views, runs = [], []
        for index, layer in enumerate(layers):
            conv, state = layer.kv_cache
            records = layer.replay_records
            tensors = (conv, state, records.rawv, records.rawk, records.g, records.beta, records.conv)
            if any(t.device != device for t in tensors):
                raise ValueError("all context layers must share one device")
            ds = _paged_cache(conv, state, conv_state_layout, heads, slots)
            _check_records(records, state, heads, spec_query_len, max_num_reqs)
            _disjoint([records.rawv, records.rawk, records.g, records.beta, records.conv], [conv, state])
            layer_runs = _page_runs(ds, state)
            for previous, other in enumerate(runs):
                if _layers_overlap(layer_runs, other):
                    raise ValueError(f"context layers {previous} and {index} have overlapping writable caches")
            runs.append(layer_runs)
            views.append((ds, state, records))
        self = cls()
        self._layers, self._views = layers, tuple(views)
        # one row of base pointers and pitches per layer (include/pla_gfx950.h: PLA_LAYER_TABLE_ENTRIES), so
        # that one fold launch and one conv launch serve every layer
        table = []
        for ds, state, records in views:
            win = records.conv
            _need(state.data_ptr() % 16 == 0 and state.stride(0) % 4 == 0
                  and all(t.data_ptr() % 16 == 0 for t in (records.rawv, records.rawk, records.g, records.beta)),
                  "checkpoint pools and records require 16-byte alignment")
            table.append([state.data_ptr(), state.stride(0), records.rawv.data_ptr(), records.rawk.data_ptr(),
                          records.g.data_ptr(), records.beta.data_ptr(), ds.data_ptr(), *ds.stride(),
                          win.data_ptr(), *win.stride(), 0])
        self._table = torch.tensor(table, dtype=torch.int64).to(device)
        self._channels, self._rows = views[0][0].size(1), views[0][2].conv.size(0)
        self._candidate = torch.zeros((4, max_num_reqs), dtype=torch.int32, device=device)
        self._buffer = torch.zeros_like(self._candidate)
        self.plan = KDAReplayCommitPlan(*self._buffer.unbind(0))
        self._heads, self._slots = heads, slots
        self._q, self._capacity, self._null = spec_query_len, max_num_reqs, null_block_id
        self._device = device
        return self

    def commit(self, num_sampled, state_indices, query_start_loc, request_indices=None, block_table=None,
               num_computed_tokens=None, mamba_block_size=None, *, token_capacity):
        """Builds the plan on the device (sampled counts clamped to the query length, no bonus token
        subtracted), then, per layer, folds each request's committed prefix of records from its source
        checkpoint into the planned slots and copies the matching conv windows.  ``token_capacity`` is the
        verify projection's ``mixed_qkv.shape[0]``; query intervals beyond it are skipped.  Align mode needs
        ``block_table``, ``num_computed_tokens`` and ``mamba_block_size >= Q`` together.  Returns the plan."""
        if not isinstance(token_capacity, Integral):
            raise TypeError("token_capacity must be a host integer")
        align = (block_table is not None, num_computed_tokens is not None, mamba_block_size is not None)
        if any(align) and not all(align):
            raise ValueError("align requires block_table, computed tokens and block size")
        if all(align) and not isinstance(mamba_block_size, Integral):
            raise TypeError("mamba_block_size must be a host integer")
        if all(align) and mamba_block_size < self._q:
            raise ValueError("align block_size must be >= spec_query_len")
        if _BYPASS:
            return self.plan
        _need(0 <= token_capacity <= 2 ** 31 - 1, "token_capacity must be between 0 and INT32_MAX")
        ref = self._buffer
        sampled, sampled_wide = _index(num_sampled, ref)
        source, source_wide = _index(state_indices, ref)
        cu, cu_wide = _index(query_start_loc, ref)
        N, R = source.numel(), self._capacity
        _need(N <= R and cu.numel() == N + 1, "commit query count exceeds capacity")
        mapping = mapping_wide = None
        if request_indices is not None:
            mapping, mapping_wide = _index(request_indices, ref)
            _need(mapping.numel() == N, "mapping must have N rows")
        else:
            _need(sampled.numel() >= N, "sampler count must cover query rows")
        computed = computed_wide = None
        blocks_wide, block_rows, block_cols, row_stride, col_stride, block_size = 0, 0, 0, 0, 0, 0
        if all(align):
            computed, computed_wide = _index(num_computed_tokens, ref)
            _need(block_table.device == ref.device and block_table.dim() == 2 and block_table.size(1) > 0
                  and block_table.dtype in (torch.int32, torch.int64) and computed.numel() >= sampled.numel(),
                  "invalid align table/count/block size")
            blocks_wide = int(block_table.dtype == torch.int64)
            block_rows, block_cols = block_table.shape
            row_stride, col_stride = block_table.stride()
            block_size = int(mamba_block_size)
        if source.dtype != torch.int32:
            source32 = source.to(torch.int32)
        else:
            source32 = source
        stream = _lib.current_stream(self._device)
        with torch.cuda.device(self._device):
            _lib.call("pla_kda_commit_plan_launch", sampled.data_ptr(), sampled_wide, source.data_ptr(), source_wide,
                      cu.data_ptr(), cu_wide, _lib.ptr(mapping), int(mapping_wide or 0), _lib.ptr(computed),
                      int(computed_wide or 0), _lib.ptr(block_table) if all(align) else None, blocks_wide,
                      N, R, sampled.numel(), block_rows, block_cols, self._slots, self._q, self._null,
                      int(token_capacity), row_stride, col_stride, block_size,
                      self._candidate.data_ptr(), self._buffer.data_ptr(), stream)
            if N == 0:
                return self.plan
            lens, final, boundary, bc = (t[:N] for t in self._buffer.unbind(0))
            plan = (lens.data_ptr(), final.data_ptr(), boundary.data_ptr(), bc.data_ptr())
            nlayers = len(self._views)
            _lib.call("pla_kda_fold_native_launch", self._table.data_ptr(), nlayers, source32.data_ptr(), *plan,
                      N, self._heads, self._q, self._slots, self._null, stream)
            _lib.call("pla_kda_conv_native_launch", self._table.data_ptr(), nlayers, *plan,
                      N, self._channels, self._q, self._rows, self._slots, stream)
        return self.plan
