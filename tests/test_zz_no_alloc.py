"""The entry point that allocates nothing (pla_gdn_prefill_launch_static: workspace = an array inside the
library) against pla_gdn_prefill_launch with a caller workspace, both through the C ABI, bit for bit on the
output, the states, the cumulative log-decay and beta: two calls in a row, the second on a smaller input (the
array still holds the first call's tiles), then the size limit."""
import pytest
import torch

pytestmark = pytest.mark.gpu

STATIC_BYTES = 64 << 20


def _launch(w, static, in_place=False, normalize=True, sync=True, outputs=None):
    from pla_amd import _lib
    m = w["_meta"]
    T, H, HV = m["T"], m["H"], m["HV"]
    packed = w["packed_qkv"]
    dev = packed.device
    stride = packed.stride(0)
    base, esz = packed.data_ptr(), packed.element_size()
    q_ptr, k_ptr, v_ptr = base, base + H * 128 * esz, base + 2 * H * 128 * esz
    pool = w["initial_state"] if in_place else w["initial_state"].clone()
    idx = w["initial_state_indices"]
    N = idx.numel()
    if outputs is None:
        o = torch.full((T, HV, 128), 7.0, dtype=packed.dtype, device=dev)
        gcum = torch.empty(T, HV, dtype=torch.float32, device=dev)
        beta = torch.empty(T, HV, dtype=torch.float32, device=dev)
    else:
        o, gcum, beta = outputs
    a, b = w["raw_gate_a"], w["raw_beta_b"]
    if normalize:
        gates = (a.data_ptr(), b.data_ptr(), a.stride(0), b.stride(0), w["A_log"].data_ptr(), w["dt_bias"].data_ptr(), None, None)
    else:
        # explicit log-decay and beta, q / k taken as they are (the workload keeps the two tensors alive)
        if "_g" not in w:
            w["_g"] = -torch.rand(T, HV, device=dev) * 0.2
            w["_beta"] = torch.rand(T, HV, device=dev)
        gates = (None, None, 0, 0, None, None, w["_g"].data_ptr(), w["_beta"].data_ptr())
    head = (q_ptr, k_ptr, v_ptr, stride, stride, stride, *gates,
            w["cu_seqlens"].data_ptr(), N, T, float(w["scale"]), 1 if normalize else 0,
            pool.data_ptr(), idx.data_ptr(), pool.stride(0), pool.data_ptr(), idx.data_ptr(), pool.stride(0), o.data_ptr())
    tail = (gcum.data_ptr(), beta.data_ptr(), H, HV, 128, 128, _lib.dtype_code(packed.dtype), _lib.current_stream(dev))
    if static:
        _lib.call("pla_gdn_prefill_launch_static", *head, *tail)
    else:
        nbytes = _lib.load().pla_gdn_prefill_workspace_bytes(T, N, H, HV)
        ws = torch.full((nbytes,), 0xFF, dtype=torch.uint8, device=dev)      # NaN as FP32 and as fp16
        _lib.call("pla_gdn_prefill_launch", *head, ws.data_ptr(), nbytes, *tail)
    if sync:
        torch.cuda.synchronize()
    tail_start = m["offsets"][-1]
    return o, pool, gcum[:tail_start], beta[:tail_start]


def test_static_scratch_prefill_equals_workspace_prefill_twice_then_rejects_oversize():
    from pla_amd import _lib
    from pla_amd.workloads import gdn_prefill_packed
    size = _lib.load().pla_gdn_prefill_workspace_bytes
    # first call: 64 chains of up to 18 chunks;
    # second call: smaller, ragged, with an empty sequence and a padded tail
    cases = [dict(lengths=[1100, 700], H=16, HV=32, tail_pad=0, seed=11),
             dict(lengths=[200, 0, 33, 450], H=2, HV=4, tail_pad=5, seed=12)]
    for case in cases:
        lengths = case["lengths"]
        w = gdn_prefill_packed(lengths, H=case["H"], HV=case["HV"], pool_slots=len(lengths) + 3, seed=case["seed"],
                               tail_pad=case["tail_pad"])
        assert size(w["_meta"]["T"], len(lengths), case["H"], case["HV"]) <= STATIC_BYTES
        want = _launch(w, static=False)
        got = _launch(w, static=True)
        for name, x, y in zip(("o", "pool", "gcum", "beta"), got, want):
            assert torch.equal(x, y), (lengths, name)
        assert torch.count_nonzero(got[0][w["_meta"]["offsets"][-1]:]) == 0
    # beyond the array: rejected before any launch, nothing written
    big = gdn_prefill_packed([9000], H=16, HV=32, pool_slots=2, seed=13)
    before = big["initial_state"].clone()
    with pytest.raises(RuntimeError, match="too large for the built-in scratch array"):
        _launch(big, static=True, in_place=True)
    assert torch.equal(big["initial_state"], before)


@pytest.mark.parametrize("lengths,H,HV,normalize", [([1100, 700], 16, 32, True), ([4096], 2, 2, True), ([900, 0, 300], 2, 4, False)])
def test_static_scratch_prefill_in_a_graph(lengths, H, HV, normalize):
    """The callers the entry point is for capture it: after one eager call on the device (which looks up the array's
    address; a first call under capture is refused) the call is captured and replayed three times, with eager work and
    a synchronisation in between, and reproduces the workspace form bit for bit.  Whole sequences, a call that is
    split into segments (few chains, one long sequence) and a call without q / k normalisation."""
    from pla_amd import _lib
    from pla_amd.workloads import gdn_prefill_packed
    w = gdn_prefill_packed(lengths, H=H, HV=HV, pool_slots=len(lengths) + 3, seed=21 + H)
    m = w["_meta"]
    assert _lib.load().pla_gdn_prefill_workspace_bytes(m["T"], len(lengths), H, HV) <= STATIC_BYTES
    if H == 2 and HV == 2:                                     # this shape carries the segment buffers
        size = _lib.load().pla_gdn_prefill_workspace_bytes
        assert size(m["T"], 1, H, HV) > 1.1 * HV * size(m["T"], 1, 65 * H, 65 * HV) / (65 * HV)
    if not normalize:
        w["packed_qkv"].mul_(0.08)                             # rows of about unit length, as a caller that normalises passes them
    pool0 = w["initial_state"].clone()
    want = _launch(w, static=False, normalize=normalize)
    assert torch.isfinite(want[0].float()).all() and torch.isfinite(want[1]).all()
    _launch(w, static=True, normalize=normalize)                # eager call: address look-up, warm-up
    dev = w["packed_qkv"].device
    outputs = (torch.empty(m["T"], HV, 128, dtype=w["packed_qkv"].dtype, device=dev),
               torch.empty(m["T"], HV, dtype=torch.float32, device=dev), torch.empty(m["T"], HV, dtype=torch.float32, device=dev))
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        _launch(w, static=True, in_place=True, normalize=normalize, sync=False, outputs=outputs)
    tail_start = m["offsets"][-1]
    for replay in range(3):
        w["initial_state"].copy_(pool0)
        for t in outputs:
            t.fill_(float("nan"))
        scratch = torch.randn(1 << 20, device=dev).sum().item()        # eager work and a sync between replays
        graph.replay()
        torch.cuda.synchronize()
        assert scratch == scratch
        got = (outputs[0], w["initial_state"], outputs[1][:tail_start], outputs[2][:tail_start])
        for name, x, y in zip(("o", "pool", "gcum", "beta"), got, want):
            assert torch.equal(x, y), (replay, name)
