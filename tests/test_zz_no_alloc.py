"""The entry point that allocates nothing (pla_gdn_prefill_launch_static: workspace = an array inside the
library) against pla_gdn_prefill_launch with a caller workspace, both through the C ABI, bit for bit on the
output, the states, the cumulative log-decay and beta: two calls in a row, the second on a smaller input (the
array still holds the first call's tiles), then the size limit."""
import pytest
import torch

pytestmark = pytest.mark.gpu

STATIC_BYTES = 64 << 20


def _launch(w, static, in_place=False):
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
    o = torch.full((T, HV, 128), 7.0, dtype=packed.dtype, device=dev)
    gcum = torch.empty(T, HV, dtype=torch.float32, device=dev)
    beta = torch.empty(T, HV, dtype=torch.float32, device=dev)
    a, b = w["raw_gate_a"], w["raw_beta_b"]
    head = (q_ptr, k_ptr, v_ptr, stride, stride, stride, a.data_ptr(), b.data_ptr(), a.stride(0), b.stride(0),
            w["A_log"].data_ptr(), w["dt_bias"].data_ptr(), None, None,
            w["cu_seqlens"].data_ptr(), N, T, float(w["scale"]), 1,
            pool.data_ptr(), idx.data_ptr(), pool.stride(0), pool.data_ptr(), idx.data_ptr(), pool.stride(0), o.data_ptr())
    tail = (gcum.data_ptr(), beta.data_ptr(), H, HV, 128, 128, _lib.dtype_code(packed.dtype), _lib.current_stream(dev))
    if static:
        _lib.call("pla_gdn_prefill_launch_static", *head, *tail)
    else:
        nbytes = _lib.load().pla_gdn_prefill_workspace_bytes(T, N, H, HV)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        _lib.call("pla_gdn_prefill_launch", *head, ws.data_ptr(), nbytes, *tail)
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
