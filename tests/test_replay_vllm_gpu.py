"""GPU parity of the request-row (vLLM-style) KDA replay verify against the CPU oracle.

The cases follow the reference's own test of this entry (tests/test_kda_replayssm_vllm.py:45-96, 214-262):
paged conv / checkpoint caches with a poisoned page layout, projection views with a token stride and a
storage offset, sentinel-filled records, ragged query lengths including zero, null slots, DS and SD conv
layouts, int32 and int64 index vectors with a stride.  Tolerances: bf16 output atol = rtol = 2e-2, bf16
records rtol 8e-3, FP32 records rtol 1e-4; windows, untouched record rows, the persistent pages and the
input storage bit-exact.
"""
from types import SimpleNamespace

import pytest
import torch

from oracle import verify_dspark_reference
from pla_amd.decode.kda_replayssm_vllm import KDAReplayRecords, kda_replay_verify

pytestmark = pytest.mark.gpu
D = 128


def pages(slots, heads, q, layout, gen, padding=256, history=None, conv_offset=0):
    """Paged cache: every page holds a conv history (DS = [channels, history], SD = [history, channels])
    followed by the FP32 checkpoint; the rest of the page is poison."""
    c = 3 * heads * D
    history = q + 2 if history is None else history
    conv_shape = (c, history) if layout == "DS" else (history, c)
    conv_bytes = c * history * 2
    state_offset = ((conv_offset + conv_bytes + 15) // 16) * 16
    page_bytes = ((state_offset + heads * D * D * 4 + padding + 15) // 16) * 16
    raw = torch.full((slots * page_bytes,), 0x5A, dtype=torch.uint8, device="cuda")
    conv = raw.view(torch.bfloat16).as_strided((slots, *conv_shape), (page_bytes // 2, *torch.empty(conv_shape).stride()),
                                               conv_offset // 2)
    state = raw.view(torch.float32).as_strided((slots, heads, D, D), (page_bytes // 4, D * D, D, 1), state_offset // 4)
    conv.copy_((torch.randn(conv.shape, generator=gen) * 0.2).to(torch.bfloat16))
    state.copy_(torch.randn(state.shape, generator=gen) * 0.01)
    return SimpleNamespace(raw=raw, conv=conv, state=state, heads=heads, q=q, layout=layout)


def inputs(heads, capacity, gen, offset=2):
    c = heads * D
    storage = (torch.randn(offset + capacity + 2, 4 * c + heads + 3, generator=gen) * 0.4).to(torch.bfloat16).cuda()
    rows = storage[offset:offset + capacity]
    return dict(mixed_qkv=rows[:, :3 * c], raw_g=rows[:, 3 * c:4 * c], raw_beta=rows[:, 4 * c:4 * c + heads],
                storage=storage, conv_weight=(torch.randn(3 * c, 4, generator=gen) * 0.2).cuda(),
                A_log=(torch.randn(heads, generator=gen) * 0.1).cuda(),
                dt_bias=(torch.randn(c, generator=gen) * 0.2).cuda(), lower_bound=-5.0)


def records_filled(rows, heads, q):
    rec = KDAReplayRecords.allocate(rows, heads, q, "cuda")
    for name in ("rawv", "rawk", "g", "beta", "conv"):
        getattr(rec, name).fill_(-7)
    return rec


def vector(values, dtype=torch.int32, strided=False):
    t = torch.tensor(values, dtype=dtype, device="cuda")
    if strided:
        storage = torch.full((len(values) * 2 + 1,), -99, dtype=dtype, device="cuda")
        storage[1::2] = t
        t = storage[1::2]
    return t


def oracle(layer, x, offsets, slots, rec, out, null_block_id):
    """The ring-mode oracle applied per request: records and windows land in the request's row."""
    h, c = layer.heads, layer.heads * D
    conv = (layer.conv if layer.layout == "DS" else layer.conv.transpose(-1, -2)).cpu()
    state = layer.state.cpu()
    want = {k: getattr(rec, k).cpu().clone() for k in ("rawv", "rawk", "g", "beta", "conv")}
    want_out = out.cpu().clone().double()
    xc = {k: v.cpu() for k, v in x.items() if torch.is_tensor(v)}
    for row, slot in enumerate(slots):
        begin, end = offsets[row:row + 2]
        n = end - begin
        if n == 0:
            continue
        if slot <= null_block_id:
            want_out[begin:end] = 0
            continue
        qkv = xc["mixed_qkv"][begin:end].split(c, -1)
        ws = xc["conv_weight"].split(c)
        css = conv[slot].split(c)
        L = want["rawv"].shape[2]
        rings = tuple(torch.zeros(1, *want[k].shape[1:], dtype=want[k].dtype) for k in ("rawv", "rawk", "g", "beta"))
        wins = tuple(torch.zeros(1, L, c, 3, dtype=torch.bfloat16) for _ in range(3))
        ref = verify_dspark_reference(
            x_q=qkv[0].reshape(1, n, h, D), x_k=qkv[1].reshape(1, n, h, D), x_v=qkv[2].reshape(1, n, h, D),
            g=xc["raw_g"][begin:end].reshape(1, n, h, D), beta=xc["raw_beta"][begin:end][None],
            w_q=ws[0], w_k=ws[1], w_v=ws[2], cs_q=css[0][None, :, :3], cs_k=css[1][None, :, :3], cs_v=css[2][None, :, :3],
            A_log=xc["A_log"], dt_bias=xc["dt_bias"], recurrent_state=state[slot:slot + 1],
            ssm_state_indices=torch.tensor([0]), intermediate_state_indices=torch.tensor([0]),
            cu_seqlens=torch.tensor([0, n]), lower_bound=x["lower_bound"], scale=D ** -0.5, rings=rings, windows=wins)
        want_out[begin:end] = ref["out"].reshape(n, c)
        for k, name in (("rawv", "ring_rawv"), ("rawk", "ring_rawk"), ("g", "ring_g"), ("beta", "ring_beta")):
            want[k][row, :, :n] = ref[name][0, :, :n]
        want["conv"][row, :n] = torch.cat([ref["ic_" + name][0, :n] for name in ("q", "k", "v")], dim=1)
    return want_out, want


@pytest.mark.parametrize("layout", ["DS", "SD"])
@pytest.mark.parametrize("q,heads", [(1, 1), (3, 2), (5, 4), (8, 2), (11, 2), (16, 1), (21, 2), (32, 2)])
@pytest.mark.parametrize("index_dtype,null_block_id", [(torch.int32, 0), (torch.int64, -1)])
def test_replay_verify_paged(layout, q, heads, index_dtype, null_block_id):
    gen = torch.Generator().manual_seed(41 + q + heads)
    lengths = [q, max(q - 2, 0), 0, 1, 1]
    offsets = [0]
    for n in lengths:
        offsets.append(offsets[-1] + n)
    slots = [7, 2, 5, 0, -1]
    layer = pages(12, heads, q, layout, gen)
    rec = records_filled(len(slots), heads, q)
    x = inputs(heads, len(slots) * q + 3, gen)
    out = torch.full((x["mixed_qkv"].shape[0], heads * D), -11, dtype=torch.bfloat16, device="cuda")
    want_out, want = oracle(layer, x, offsets, slots, rec, out, null_block_id)
    before, storage_before = layer.raw.clone(), x["storage"].clone()
    args = {k: v for k, v in x.items() if k != "storage"}
    got = kda_replay_verify(**args, conv_state=layer.conv, checkpoint_state=layer.state, records=rec,
                            query_start_loc=vector(offsets, index_dtype, True), state_indices=vector(slots, index_dtype, True),
                            conv_state_layout=layout, out=out, null_block_id=null_block_id)
    torch.cuda.synchronize()
    assert got.data_ptr() == out.data_ptr()
    T = offsets[-1]
    torch.testing.assert_close(out[:T].cpu().double(), want_out[:T], atol=2e-2, rtol=2e-2)
    assert bool((out[T:] == -11).all())                                              # rows outside query intervals
    for name, tol in (("rawv", 8e-3), ("rawk", 8e-3), ("g", 1e-4), ("beta", 1e-4)):
        torch.testing.assert_close(getattr(rec, name).cpu().float(), want[name].float(), atol=1e-6, rtol=tol)
        untouched = want[name] == -7
        assert torch.equal(getattr(rec, name).cpu()[untouched], want[name][untouched])
    assert torch.equal(rec.conv.cpu(), want["conv"])
    assert torch.equal(layer.raw, before) and torch.equal(x["storage"], storage_before)
    for b, n in enumerate(lengths):
        if slots[b] <= null_block_id or n == 0:
            assert bool((rec.g[b] == -7).all()) and bool((rec.conv[b] == -7).all())
    default_out = kda_replay_verify(**args, conv_state=layer.conv, checkpoint_state=layer.state, records=rec,
                                    query_start_loc=vector(offsets), state_indices=vector(slots),
                                    conv_state_layout=layout, null_block_id=null_block_id)
    torch.cuda.synchronize()
    torch.testing.assert_close(default_out[:T].cpu().double(), want_out[:T], atol=2e-2, rtol=2e-2)


def test_replay_verify_skips_malformed_intervals_and_rejects_bad_arguments():
    gen = torch.Generator().manual_seed(5)
    q, heads = 3, 2
    layer = pages(6, heads, q, "DS", gen)
    rec = records_filled(4, heads, q)
    x = inputs(heads, 16, gen)
    args = {k: v for k, v in x.items() if k != "storage"}
    out = torch.full((16, heads * D), -11, dtype=torch.bfloat16, device="cuda")
    # request 1 is longer than Q, request 2 names a slot beyond the pool: both are skipped entirely
    offsets, slots = [0, 2, 7, 9, 10], [3, 1, 99, 2]
    kda_replay_verify(**args, conv_state=layer.conv, checkpoint_state=layer.state, records=rec,
                      query_start_loc=vector(offsets), state_indices=vector(slots), conv_state_layout="DS", out=out)
    torch.cuda.synchronize()
    assert bool((out[2:9] == -11).all()) and bool((rec.g[1:3] == -7).all())
    assert not bool((out[0:2] == -11).any()) and not bool((out[9:10] == -11).any())
    with pytest.raises(RuntimeError, match="null_block_id must be -1 or 0"):
        kda_replay_verify(**args, conv_state=layer.conv, checkpoint_state=layer.state, records=rec,
                          query_start_loc=vector(offsets), state_indices=vector(slots), conv_state_layout="DS",
                          null_block_id=3)
    with pytest.raises(RuntimeError, match="DS or SD"):
        kda_replay_verify(**args, conv_state=layer.conv, checkpoint_state=layer.state, records=rec,
                          query_start_loc=vector(offsets), state_indices=vector(slots), conv_state_layout="XX")
    with pytest.raises(TypeError):
        kda_replay_verify(**dict(args, lower_bound=torch.tensor(-5.0)), conv_state=layer.conv, checkpoint_state=layer.state,
                          records=rec, query_start_loc=vector(offsets), state_indices=vector(slots), conv_state_layout="DS")
    big = records_filled(8, heads, q)
    with pytest.raises(RuntimeError, match="must not alias"):
        kda_replay_verify(**args, conv_state=layer.conv, checkpoint_state=layer.state, records=big,
                          query_start_loc=vector(offsets), state_indices=vector(slots), conv_state_layout="DS",
                          out=big.rawv.view(-1)[:16 * heads * D].view(16, heads * D))


# ---- commit --------------------------------------------------------------------------------------------

from oracle import fold_reference, replay_commit_plan_reference            # noqa: E402
from pla_amd.decode.kda_replayssm_vllm import KDAReplayCommitContext        # noqa: E402
from helpers import rel_l2                                                  # noqa: E402


def _ds(layer):
    return layer.conv if layer.layout == "DS" else layer.conv.transpose(-1, -2)


def _expected_commit(layer, plan, sources):
    """Expected pools of one layer from a plan: per request, fold the committed prefix of its records from
    its source checkpoint into the final (and boundary) slot, copy the matching conv windows."""
    rec = layer.replay_records
    state0, conv0 = layer.state.cpu().clone(), _ds(layer).cpu().clone()
    state, conv = state0.clone(), conv0.clone()
    rk, rv, g, bt, win = (t.cpu() for t in (rec.rawk, rec.rawv, rec.g, rec.beta, rec.conv))
    for b, src in enumerate(sources):
        n, final, boundary, bc = (plan[c][b] for c in range(4))
        if not n:
            continue
        def folded(count):
            one = fold_reference(state0[src][None], rk[b][None], rv[b][None], g[b][None], bt[b][None], [0], [count],
                                 compute_dtype=torch.float64)
            return one[0].float()
        if bc:
            state[boundary] = folded(bc)
            conv[boundary, :, :3] = win[b, bc - 1]
        state[final] = folded(n)
        conv[final, :, :3] = win[b, n - 1]
    return state, conv


def _verify_then_commit(layers, x, offsets, slots, q, counts, *, layout, null_block_id=0, mapping=None, align=None,
                        index_dtype=torch.int32):
    rows = len(slots)
    args = {k: v for k, v in x.items() if k != "storage"}
    T = x["mixed_qkv"].shape[0]
    for layer in layers:
        layer.replay_records = records_filled(rows, layer.heads, q)
        layer.kv_cache = (layer.conv, layer.state)
        kda_replay_verify(**args, conv_state=layer.conv, checkpoint_state=layer.state, records=layer.replay_records,
                          query_start_loc=vector(offsets), state_indices=vector(slots), conv_state_layout=layout,
                          null_block_id=null_block_id)
    torch.cuda.synchronize()
    ctx = KDAReplayCommitContext.create(layers, q, rows, layout, null_block_id)
    kw = {}
    if align is not None:
        kw = dict(block_table=torch.tensor(align["table"], dtype=index_dtype, device="cuda"),
                  num_computed_tokens=vector(align["computed"], index_dtype), mamba_block_size=align["block_size"])
    want_plan = replay_commit_plan_reference(
        counts, slots, offsets, slots=layers[0].state.shape[0], Q=q, token_capacity=T, null_block_id=null_block_id,
        request_indices=mapping, block_table=None if align is None else align["table"],
        num_computed_tokens=None if align is None else align["computed"],
        block_size=None if align is None else align["block_size"], capacity=rows)
    expected = [_expected_commit(layer, want_plan, slots) for layer in layers]
    plan = ctx.commit(vector(counts, index_dtype, True), vector(slots, index_dtype, True), vector(offsets, index_dtype, True),
                      request_indices=None if mapping is None else vector(mapping, index_dtype), token_capacity=T, **kw)
    torch.cuda.synchronize()
    got_plan = [t.cpu().tolist() for t in (plan.commit_lens, plan.final_state_indices, plan.boundary_state_indices,
                                           plan.boundary_recovery_lens)]
    assert got_plan == want_plan
    for layer, (want_state, want_conv) in zip(layers, expected):
        state, conv = layer.state.cpu(), _ds(layer).cpu()
        for s in range(state.shape[0]):
            if torch.equal(want_state[s], layer._state_before[s]):
                assert torch.equal(state[s], want_state[s])                         # untouched slots stay bit-identical
            else:
                assert rel_l2(state[s], want_state[s]) <= 1e-4
        assert torch.equal(conv, want_conv)
    return ctx, want_plan


def _snapshot(layers):
    for layer in layers:
        layer._state_before = layer.state.cpu().clone()


@pytest.mark.parametrize("layout", ["DS", "SD"])
@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
def test_replay_commit_in_place(layout, index_dtype):
    gen = torch.Generator().manual_seed(11)
    q, heads = 4, 2
    lengths = [4, 2, 0, 1, 3]
    offsets = [0]
    for n in lengths:
        offsets.append(offsets[-1] + n)
    slots = [7, 2, 5, 0, 9]
    layers = [pages(12, heads, q, layout, gen)]
    x = inputs(heads, offsets[-1] + 3, gen)
    _snapshot(layers)
    _, plan = _verify_then_commit(layers, x, offsets, slots, q, [3, 9, 2, 1, -1], layout=layout, index_dtype=index_dtype)
    assert plan[0] == [3, 2, 0, 0, 0] and plan[1] == [7, 2, 0, 0, 0]                   # slot 0 is the null block


def test_replay_commit_align_boundaries_conflicts_and_mapping():
    gen = torch.Generator().manual_seed(12)
    q, heads, layout = 3, 2, "SD"
    offsets, slots = [0, 3, 5, 6, 9], [5, 9, 2, 11]
    layers = [pages(14, heads, q, layout, gen), pages(14, heads, q, layout, gen)]
    x = inputs(heads, 12, gen)
    _snapshot(layers)
    # request 0: boundary after 2 tokens (block 5 = its own source), final block 6; request 1: inside block 9;
    # request 2: exactly up to the boundary (boundary == final == 3); request 3 wants block 6 too -> cancelled with request 0
    align = dict(table=[[5, 6, 7], [8, 9, 1], [3, 3, 4], [6, 6, 6]], computed=[2, 4, 3, 1], block_size=4)
    _, plan = _verify_then_commit(layers, x, offsets, slots, q, [3, 2, 1, 2], layout=layout, align=align)
    assert plan == [[0, 2, 1, 0], [0, 9, 3, 0], [0, 0, 3, 0], [0, 0, 1, 0]]
    # the same without the conflicting request: request 0 commits with a boundary snapshot into its own source block
    layers = [pages(14, heads, q, layout, gen)]
    _snapshot(layers)
    align = dict(table=[[5, 6, 7], [8, 9, 1], [3, 3, 4], [10, 12, 13]], computed=[2, 4, 3, 1], block_size=4)
    _, plan = _verify_then_commit(layers, x, offsets, slots, q, [3, 2, 1, 2], layout=layout, align=align,
                                  index_dtype=torch.int64)
    assert plan == [[3, 2, 1, 2], [6, 9, 3, 10], [5, 0, 3, 0], [2, 0, 1, 0]]
    # request rows mapped onto sampler rows
    layers = [pages(14, heads, q, layout, gen)]
    _snapshot(layers)
    _, plan = _verify_then_commit(layers, x, offsets, slots, q, [1, 3, 0, 2], layout=layout, mapping=[3, 2, 1, 0])
    assert plan[0] == [2, 0, 1, 1]


def test_replay_commit_context_checks_and_graph_replay():
    gen = torch.Generator().manual_seed(13)
    q, heads, layout = 2, 1, "DS"
    # two layers interleaved in one set of pages: disjoint runs are accepted, overlapping ones rejected
    first = pages(6, heads, q, layout, gen, padding=3 * heads * D * 4 * 2 + heads * D * D * 4 + 512)
    span = 3 * heads * D * (q + 2) * 2
    second_offset = ((span + 15) // 16) * 16 + heads * D * D * 4 + 64
    c = 3 * heads * D
    history = q + 2
    raw = first.raw
    page_bytes = raw.numel() // 6
    conv2 = raw.view(torch.bfloat16).as_strided((6, c, history), (page_bytes // 2, history, 1), second_offset // 2)
    state_off2 = ((second_offset + c * history * 2 + 15) // 16) * 16
    state2 = raw.view(torch.float32).as_strided((6, heads, D, D), (page_bytes // 4, D * D, D, 1), state_off2 // 4)
    assert state_off2 + heads * D * D * 4 <= page_bytes
    second = SimpleNamespace(raw=raw, conv=conv2, state=state2, heads=heads, q=q, layout=layout)
    conv2.copy_((torch.randn(conv2.shape, generator=gen) * 0.2).to(torch.bfloat16))
    state2.copy_(torch.randn(state2.shape, generator=gen) * 0.01)
    layers = [first, second]
    x = inputs(heads, 8, gen)
    offsets, slots = [0, 2, 3, 5], [4, 1, 3]
    _snapshot(layers)
    ctx, _ = _verify_then_commit(layers, x, offsets, slots, q, [2, 1, 1], layout=layout)
    overlapping = SimpleNamespace(kv_cache=(first.conv, first.state), replay_records=first.replay_records)
    with pytest.raises(ValueError, match="layers 0 and 1 have overlapping writable caches"):
        KDAReplayCommitContext.create([first, overlapping], q, 3, layout, 0)
    with pytest.raises(ValueError, match="null_block_id must be -1 or 0"):
        KDAReplayCommitContext.create([first], q, 3, layout, 2)
    with pytest.raises(ValueError, match="align requires"):
        ctx.commit(vector([1, 1, 1]), vector(slots), vector(offsets), block_table=torch.zeros(3, 2, dtype=torch.int32, device="cuda"),
                   token_capacity=8)
    with pytest.raises(TypeError):
        ctx.commit(vector([1, 1, 1]), vector(slots), vector(offsets), token_capacity=torch.tensor(8))
    # graph replay: the plan is built on the device, so the captured commit follows new sampled counts
    counts = vector([2, 1, 1])
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ctx.commit(counts, vector(slots), vector(offsets), token_capacity=8)
    torch.cuda.current_stream().wait_stream(side)
    src, off = vector(slots), vector(offsets)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        plan = ctx.commit(counts, src, off, token_capacity=8)
    for new_counts, want in (([1, 0, 2], [1, 0, 2]), ([0, 5, 1], [0, 1, 1])):
        counts.copy_(torch.tensor(new_counts, dtype=torch.int32))
        before = [layer.state.clone() for layer in layers]
        graph.replay()
        torch.cuda.synchronize()
        assert plan.commit_lens.cpu().tolist() == want
        for layer, old in zip(layers, before):
            for b, s in enumerate(slots):
                changed = not torch.equal(layer.state[s], old[s])
                assert changed == (want[b] > 0)


@pytest.mark.parametrize("capacity", [384, 5000])
@pytest.mark.parametrize("align", [False, True])
def test_commit_plan_random_requests_match_the_oracle(capacity, align):
    """The plan kernel alone, through the C ABI, on 300 random requests with few slots (so that destinations
    clash), invalid sources, empty and oversized intervals and a sampler mapping; a capacity of 5000 keeps the
    requests' claims in the caller's scratch rows instead of LDS."""
    from pla_amd import _lib
    gen = torch.Generator().manual_seed(capacity + int(align))
    batch, slots, q, rows = 300, 900, 4, 320
    block_size, cols = 8, 5
    ri = lambda lo, hi, n: torch.randint(lo, hi, (n,), generator=gen)
    lengths = ri(0, q + 2, batch)
    offsets = [0] + lengths.cumsum(0).tolist()
    token_capacity = offsets[-1] - 3                       # the last intervals end beyond the capacity
    source = ri(-2, slots + 3, batch).tolist()
    sampled = ri(-1, q + 2, rows).tolist()
    mapping = ri(-1, rows + 2, batch).tolist()
    computed = ri(-1, block_size * (cols + 1), rows).tolist()
    table = ri(-1, slots + 2, rows * cols).reshape(rows, cols).tolist()
    want = replay_commit_plan_reference(
        sampled, source, offsets, slots=slots, Q=q, token_capacity=token_capacity, null_block_id=0,
        request_indices=mapping, block_table=table if align else None, num_computed_tokens=computed if align else None,
        block_size=block_size if align else None, capacity=capacity)
    dev = "cuda"
    t = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    d_sampled, d_source, d_offsets, d_mapping, d_computed, d_table = (t(x) for x in (sampled, source, offsets, mapping,
                                                                                      computed, table))
    scratch = torch.full((4, capacity), -9, dtype=torch.int32, device=dev)
    plan = torch.full((4, capacity), -9, dtype=torch.int32, device=dev)
    _lib.call("pla_kda_commit_plan_launch", d_sampled.data_ptr(), 0, d_source.data_ptr(), 0, d_offsets.data_ptr(), 0,
              d_mapping.data_ptr(), 0, d_computed.data_ptr() if align else None, 0, d_table.data_ptr() if align else None, 0,
              batch, capacity, rows, rows if align else 0, cols if align else 0, slots, q, 0, token_capacity,
              cols if align else 0, 1 if align else 0, block_size if align else 0,
              scratch.data_ptr(), plan.data_ptr(), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert plan.cpu().tolist() == want
    assert sum(1 for n in want[0] if n) >= 20 and sum(1 for n in want[0][:batch] if not n) >= 20
