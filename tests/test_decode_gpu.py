"""GPU parity of the k-last decode / MTP-verify kernels against the CPU oracle.

Every call goes through the C ABI of libpla_gfx950.so (via pla_amd.decode).
Tolerances: out atol 1e-3 / rtol 1e-2 and state atol 2e-3 / rtol 8e-3 on the small cases
(the reference's own bounds, tests/test_k_last_state_dtype.py:190-191), plus the
benchmark bounds (bf16 out atol 2e-2 / rtol 2e-2, FP32 state rel-L2 <= 1e-3) on the
benchmark configurations; untouched slots, guard floats and padded outputs bit-exact.
"""
import pytest
import torch

from helpers import (make_k_last_case, oracle_k_last, packed_from, oracle_packed_workload, rel_l2)

pytestmark = pytest.mark.gpu

OUT_TOL = dict(atol=1e-3, rtol=1e-2)
STATE_TOL = dict(atol=2e-3, rtol=8e-3)


def _ops():
    from pla_amd.decode import (fused_sigmoid_gating_delta_rule_forward_k_last as forward,
                                fused_sigmoid_gating_delta_rule_forward_k_last_packed as packed)
    from pla_amd.decode.private import (
        fused_sigmoid_gating_delta_rule_forward_k_last_tunable as forward_tunable,
        fused_sigmoid_gating_delta_rule_forward_k_last_packed_tunable as packed_tunable)
    return forward, packed, forward_tunable, packed_tunable


def _out_tol(dtype):
    # fp16/bf16 output rounding: one ulp of the result
    return OUT_TOL if dtype == torch.float16 else dict(atol=1e-3, rtol=1.6e-2)


def _check_case(kernel, args, backing, lengths, state_ids, cache_ids, *, tile=None, graph=False):
    forward, packed, forward_tunable, packed_tunable = _ops()
    exp_out, exp_state, exp_cache = oracle_k_last(args, lengths, state_ids, cache_ids)
    before = backing.clone()
    cache = args.get("intermediate_states_buffer")
    if kernel == "packed":
        kwargs = packed_from(args)
        call = packed if tile is None else packed_tunable
    else:
        kwargs = dict(args)
        call = forward if tile is None else forward_tunable
    if tile is not None:
        kwargs.update(tile)
    state = args["initial_state_source"]
    state_ptr = state.data_ptr()
    if graph:
        call(**kwargs)
        torch.cuda.synchronize()
        backing.copy_(before)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            out = call(**kwargs)
        for _ in range(3):
            backing.copy_(before)
            if cache is not None:
                cache.fill_(-7.0)
            g.replay()
    else:
        out = call(**kwargs)
    torch.cuda.synchronize()
    assert state.data_ptr() == state_ptr
    torch.testing.assert_close(out.reshape(exp_out.shape).cpu().float(), exp_out.float(), **_out_tol(out.dtype))
    torch.testing.assert_close(state.cpu(), exp_state, **STATE_TOL)
    assert torch.equal(backing[:, -256:], before[:, -256:])                 # guard floats
    is_sglang = True if args.get("is_sglang") is None else args["is_sglang"]
    written = {s for s, n in zip(state_ids, lengths) if n and s >= 0 and (is_sglang or s > 0)}
    if args.get("disable_state_update"):
        written = set()
    untouched = [s for s in range(backing.shape[0]) if s not in written]
    assert torch.equal(backing[untouched], before[untouched])
    if cache is not None:
        torch.testing.assert_close(cache.cpu(), exp_cache, **STATE_TOL)
        keep = exp_cache == -7.0
        assert torch.equal(cache.cpu()[keep], exp_cache[keep])
    return out


@pytest.mark.parametrize("is_kda", [False, True])
@pytest.mark.parametrize("mode", ["decode", "verify", "writeback", "tree", "ragged", "graph", "tunable"])
@pytest.mark.parametrize("H,HV", [(4, 8), (6, 6), (6, 18)])
@pytest.mark.parametrize("act_dtype", [torch.bfloat16, torch.float16])
def test_k_last_modes(is_kda, mode, H, HV, act_dtype):
    case_mode = "verify" if mode in ("graph", "tunable") else mode
    args, backing, lengths, state_ids, cache_ids = make_k_last_case(
        is_kda, case_mode, H=H, HV=HV, act_dtype=act_dtype)
    tile = dict(bv=64, wn=8, sn=4, hv_per_cta=1) if mode == "tunable" else None
    _check_case("k_last", args, backing, lengths, state_ids, cache_ids, tile=tile, graph=mode == "graph")


@pytest.mark.parametrize("is_kda", [False, True])
@pytest.mark.parametrize("mode", ["decode", "packed", "verify", "writeback", "tree", "ragged", "graph", "tunable"])
@pytest.mark.parametrize("H,HV", [(4, 8), (6, 18)])
@pytest.mark.parametrize("act_dtype", [torch.bfloat16, torch.float16])
def test_k_last_modes_bf16_state_pool(is_kda, mode, H, HV, act_dtype):
    """bf16 pools and snapshot caches: FP32 recurrence, tiles widened on load and rounded on store; a
    tree branch reloads the rounded snapshot (tests/test_k_last_state_dtype.py:108-196)."""
    case_mode = "verify" if mode in ("graph", "tunable") else ("decode" if mode == "packed" else mode)
    args, backing, lengths, state_ids, cache_ids = make_k_last_case(
        is_kda, case_mode, H=H, HV=HV, act_dtype=act_dtype, state_dtype=torch.bfloat16)
    tile = dict(bv=64, wn=8, sn=4, hv_per_cta=1) if mode == "tunable" else None
    _check_case("packed" if mode == "packed" else "k_last", args, backing, lengths, state_ids, cache_ids,
                tile=tile, graph=mode == "graph")
    assert args["initial_state_source"].dtype == torch.bfloat16


@pytest.mark.parametrize("state_dtype,cache_dtype,message", [
    (torch.float16, torch.float16, "state dtype must be"),
    (torch.float32, torch.bfloat16, "must have the same dtype"),
    (torch.bfloat16, torch.float32, "must have the same dtype")])
def test_rejects_state_dtype_combinations(state_dtype, cache_dtype, message):
    forward = _ops()[0]
    args, backing, _, _, _ = make_k_last_case(False, "verify", state_dtype=state_dtype)
    args["intermediate_states_buffer"] = args["intermediate_states_buffer"].to(cache_dtype)
    before = backing.clone()
    with pytest.raises(RuntimeError, match=message):
        forward(**args)
    torch.cuda.synchronize()
    assert torch.equal(backing.view(torch.int16 if state_dtype != torch.float32 else torch.int32),
                       before.view(torch.int16 if state_dtype != torch.float32 else torch.int32))


def test_bf16_pool_b64_kda_packed_decode_at_scale():
    """B=64 x 32 heads over a 128-slot bf16 pool with a padded pitch, 5 % padded requests."""
    from pla_amd.workloads import gdn_decode_packed
    from pla_amd.decode import fused_sigmoid_gating_delta_rule_forward_k_last_packed as packed
    w = gdn_decode_packed(64, H=32, HV=32, pool_slots=128, pad_frac=0.05, seed=77, is_kda=True, pitch_pad=64)
    pool32 = w["initial_state_source"]
    backing = torch.zeros(128, 32 * 128 * 128 + 64, dtype=torch.bfloat16, device="cuda")
    pool = backing[:, :32 * 128 * 128].view(128, 32, 128, 128)
    pool.copy_(pool32)
    w["initial_state_source"] = pool
    before = backing.clone()
    exp_out, exp_states = oracle_packed_workload(w)
    call = {k: v for k, v in w.items() if not k.startswith("_")}
    out = packed(**call)
    torch.cuda.synchronize()
    torch.testing.assert_close(out.cpu().float().reshape(exp_out.shape), exp_out.float(), atol=2e-2, rtol=2e-2)
    for slot, want in exp_states.items():
        assert want.dtype == torch.bfloat16
        torch.testing.assert_close(pool[slot].cpu(), want, **STATE_TOL)
    untouched = [s for s in range(128) if s not in exp_states]
    assert torch.equal(backing[untouched].view(torch.int16), before[untouched].view(torch.int16))
    assert torch.equal(backing[:, -64:].view(torch.int16), before[:, -64:].view(torch.int16))


@pytest.mark.parametrize("kernel", ["k_last", "packed"])
@pytest.mark.parametrize("H,HV", [(3, 3), (5, 5), (3, 6), (12, 24), (4, 12), (1, 1), (16, 32), (32, 32), (64, 64)])
@pytest.mark.parametrize("is_kda", [False, True])
def test_head_ratios(kernel, H, HV, is_kda):
    args, backing, lengths, state_ids, cache_ids = make_k_last_case(is_kda, "decode", H=H, HV=HV, B=2, padded=False)
    _check_case(kernel, args, backing, lengths, state_ids, cache_ids)


@pytest.mark.parametrize("kernel", ["k_last", "packed"])
@pytest.mark.parametrize("bv", [32, 64, 128])
@pytest.mark.parametrize("is_kda", [False, True])
@pytest.mark.parametrize("norm", [False, True])
@pytest.mark.parametrize("graph", [False, True])
def test_tile_sizes_and_norm(kernel, bv, is_kda, norm, graph):
    args, backing, lengths, state_ids, cache_ids = make_k_last_case(is_kda, "decode", H=6, HV=18)
    args["use_qk_l2norm_in_kernel"] = norm
    _check_case(kernel, args, backing, lengths, state_ids, cache_ids,
                tile=dict(bv=bv, wn=4, sn=4, hv_per_cta=1), graph=graph)


@pytest.mark.parametrize("B", [1, 2, 43])
@pytest.mark.parametrize("kernel", ["k_last", "packed", "mtp"])
def test_batch_sizes(B, kernel):
    mode = "verify" if kernel == "mtp" else "decode"
    args, backing, lengths, state_ids, cache_ids = make_k_last_case(True, mode, H=6, HV=6, B=B, padded=False)
    _check_case("k_last" if kernel == "mtp" else kernel, args, backing, lengths, state_ids, cache_ids)


@pytest.mark.parametrize("kernel", ["k_last", "packed", "mtp"])
@pytest.mark.parametrize("slot_mode", ["sglang", "vllm"])
def test_null_slots(kernel, slot_mode):
    mode = "verify" if kernel == "mtp" else "decode"
    args, backing, lengths, state_ids, cache_ids = make_k_last_case(True, mode, H=6, HV=18, B=3)
    args["is_sglang"] = slot_mode == "sglang"
    out = _check_case("k_last" if kernel == "mtp" else kernel, args, backing, lengths, state_ids, cache_ids)
    T = lengths[0]
    flat = out.reshape(-1, 18, 128)
    assert torch.count_nonzero(flat[2 * T:3 * T]) == 0            # slot -1
    if slot_mode == "vllm":
        assert torch.count_nonzero(flat[T:2 * T]) == 0            # slot 0 is vLLM's null block


@pytest.mark.parametrize("T", range(2, 9))
@pytest.mark.parametrize("mode", ["verify", "tree", "ragged", "writeback"])
@pytest.mark.parametrize("lower_bound", [None, -5.0])
def test_mtp_lengths(T, mode, lower_bound):
    args, backing, lengths, state_ids, cache_ids = make_k_last_case(True, mode, H=6, HV=6, B=3, T=T)
    if lower_bound is not None:
        args["lower_bound"] = lower_bound
    _check_case("k_last", args, backing, lengths, state_ids, cache_ids)


@pytest.mark.parametrize("is_kda,lower_bound", [(False, None), (True, None), (True, -5.0)])
@pytest.mark.parametrize("T", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("H,HV", [(4, 8), (6, 6)])
@pytest.mark.parametrize("act_dtype,state_dtype", [(torch.bfloat16, torch.float32), (torch.float16, torch.float32),
                                                   (torch.bfloat16, torch.bfloat16)])
def test_read_once_verify(is_kda, lower_bound, T, H, HV, act_dtype, state_dtype):
    """A verify that writes neither state nor snapshots (up to eight draft tokens, [B, T, ...] inputs, no
    cache) takes the read-once kernel (built for four tokens, and for eight): outputs equal the stepped
    recurrence, the pool stays bit-identical."""
    forward = _ops()[0]
    args, backing, lengths, state_ids, _ = make_k_last_case(is_kda, "verify", H=H, HV=HV, T=T, act_dtype=act_dtype,
                                                            state_dtype=state_dtype)
    B = len(lengths)
    for name in ("q", "k", "v", "a", "b"):
        args[name] = args[name].reshape(B, T, *args[name].shape[2:]).contiguous()
    args.update(cu_seqlens=None, intermediate_states_buffer=None, intermediate_state_indices=None,
                cache_steps_or_num_accept=None, disable_state_update=True)
    if lower_bound is not None:
        args["lower_bound"] = lower_bound
    flat = dict(args)
    for name in ("q", "k", "v", "a", "b"):
        flat[name] = args[name].reshape(1, B * T, *args[name].shape[2:])
    exp_out, _, _ = oracle_k_last(flat, lengths, state_ids, None)
    before = backing.clone()
    out = forward(**args)
    torch.cuda.synchronize()
    torch.testing.assert_close(out.reshape(exp_out.shape).cpu().float(), exp_out.float(), **_out_tol(out.dtype))
    assert torch.equal(backing, before)
    pad = [n for n, s in enumerate(state_ids) if s < 0]
    assert pad and all(torch.count_nonzero(out[n]) == 0 for n in pad)


@pytest.mark.parametrize("lengths,max_tokens", [([4, 2, 0, 3, 1, 4], 4), ([8, 5, 0, 3, 1, 7], 8)])
def test_read_once_verify_ragged_requests(lengths, max_tokens):
    """Requests of different numbers of draft tokens (one of them none) in one launch, a padded request among them;
    windows of up to four and of up to eight tokens."""
    from pla_amd.decode.kda_replayssm_sglang import kda_mtp_verify
    from oracle import k_last_reference
    g = torch.Generator().manual_seed(77)
    slots = [5, 0, 3, -1, 2, 6]
    nt, H, D = sum(lengths), 6, 128
    rnd = lambda *shape: torch.randn(*shape, generator=g)
    q, k, v = (rnd(1, nt, H, D).to(torch.bfloat16) for _ in range(3))
    log_decay = -torch.nn.functional.softplus(rnd(nt, H, D)) * torch.rand(nt, H, D, generator=g)
    beta = torch.sigmoid(rnd(nt, H))
    pool = rnd(8, H, D, D) * 0.1
    cu = torch.tensor([0] + torch.tensor(lengths).cumsum(0).tolist(), dtype=torch.int32)
    want, _, _ = k_last_reference(q[0], k[0], v[0], None, None, None, None, pool, slots, lengths, is_kda=True,
                                  disable_state_update=True, log_decay=log_decay, beta_activated=beta)
    pool_d = pool.cuda()
    before = pool_d.clone()
    out = kda_mtp_verify(q.cuda(), k.cuda(), v.cuda(), log_decay.cuda(), beta.cuda(), pool_d,
                         torch.tensor(slots, dtype=torch.int32, device="cuda"), cu.cuda(), max_tokens=max_tokens)
    torch.cuda.synchronize()
    torch.testing.assert_close(out[0].cpu().float(), want.float(), atol=1e-3, rtol=1.6e-2)
    assert torch.equal(pool_d, before)
    first = sum(lengths[:3])
    assert torch.count_nonzero(out[0, first:first + 3]) == 0                          # the padded request's three tokens


@pytest.mark.parametrize("layout", ["heads3", "strided_heads3", "flat2", "flat3", "batch4"])
@pytest.mark.parametrize("mode", ["decode", "tree"])
def test_kda_gate_layouts(layout, mode):
    H, HV, B = 4, 8, 3
    args, backing, lengths, state_ids, cache_ids = make_k_last_case(True, mode, H=H, HV=HV, B=B, padded=False)
    exp_out, exp_state, exp_cache = oracle_k_last(args, lengths, state_ids, cache_ids)
    nt, D = args["q"].shape[1], 128
    if layout == "heads3":
        args["a"] = args["a"].view(nt, HV, D)
    elif layout == "strided_heads3":
        storage = args["a"].new_full((nt, HV + 1, D), 17)
        storage[:, :HV].copy_(args["a"].view(nt, HV, D))
        args["a"] = storage[:, :HV]
    elif layout == "flat2":
        args["a"] = args["a"].view(nt, HV * D)
    elif layout == "flat3":
        args["a"] = args["a"].view(1, nt, HV * D)
    else:
        for key in ("q", "k", "v", "a"):
            args[key] = args[key].view(B, -1, *args[key].shape[-2:])
    forward = _ops()[0]
    out = forward(**args)
    torch.cuda.synchronize()
    torch.testing.assert_close(out.reshape(exp_out.shape).cpu().float(), exp_out.float(), atol=1e-3, rtol=1.6e-2)
    torch.testing.assert_close(args["initial_state_source"].cpu(), exp_state, **STATE_TOL)


def test_vllm_slot_table():
    forward = _ops()[0]
    args, backing, lengths, _, _ = make_k_last_case(False, "verify", H=4, HV=8)
    for key in ("a", "b", "q", "k", "v"):
        args[key] = args[key][:, :4].contiguous()
    dev = args["q"].device
    args["cu_seqlens"] = torch.tensor([0, 4], device=dev, dtype=torch.int32)
    args["initial_state_indices"] = torch.tensor([[1, 2, 3, 4]], device=dev, dtype=torch.int32)
    args["cache_steps_or_num_accept"] = torch.tensor([3], device=dev, dtype=torch.int32)
    args["intermediate_states_buffer"] = None
    args["intermediate_state_indices"] = None
    args["is_sglang"] = False
    exp_out, exp_state, _ = oracle_k_last(args, [4], [[1, 2, 3, 4]], None, num_accepted=[3])
    before = backing.clone()
    out = forward(**args)
    torch.cuda.synchronize()
    torch.testing.assert_close(out.cpu().float(), exp_out.float(), atol=1e-3, rtol=1.6e-2)
    torch.testing.assert_close(args["initial_state_source"].cpu(), exp_state, **STATE_TOL)
    assert torch.equal(backing[:, -256:], before[:, -256:])
    assert torch.equal(backing[[0, 5, 6]], before[[0, 5, 6]])
    # non-positive accepted counts start from column 0, bit-identically
    results = []
    for accepted in (1, 0, -7, -(2 ** 31)):
        backing.copy_(before)
        args["cache_steps_or_num_accept"].fill_(accepted)
        o = forward(**args).clone()
        results.append((o, args["initial_state_source"].clone()))
    for o, st in results[1:]:
        assert torch.equal(o, results[0][0]) and torch.equal(st, results[0][1])


def test_empty_and_padded_requests_consume_nothing():
    forward, packed = _ops()[:2]
    args, backing, _, _, _ = make_k_last_case(False, "decode", H=4, HV=8, B=3, padded=False)
    dev = args["q"].device
    # request 1 is empty: its slot id is garbage and must never be dereferenced
    for key in ("a", "b", "q", "k", "v"):
        args[key] = args[key][:, :2].contiguous()
    args["cu_seqlens"] = torch.tensor([0, 1, 1, 2], device=dev, dtype=torch.int32)
    args["initial_state_indices"] = torch.tensor([1, 2 ** 31 - 1, 2], device=dev, dtype=torch.int32)
    args["initial_state_source"][4:].fill_(float("nan"))
    for call, kw in ((forward, args), (packed, packed_from(args))):
        out = call(**kw)
        torch.cuda.synchronize()
        assert torch.isfinite(out).all()
        assert torch.isnan(args["initial_state_source"][4:]).all()
    # a padded slot never consumes its (NaN) token
    args, backing, _, _, _ = make_k_last_case(True, "decode", H=4, HV=8, B=2, padded=False)
    args["initial_state_indices"] = torch.tensor([0, -17], device=dev, dtype=torch.int32)
    for name in ("q", "k", "v"):
        args[name][:, 1].fill_(float("nan"))
    for call, kw in ((forward, args), (packed, packed_from(args))):
        out = call(**kw)
        torch.cuda.synchronize()
        assert torch.isfinite(out).all() and torch.count_nonzero(out.reshape(2, -1)[1]) == 0


def test_writes_caller_out_and_rejects_bad_out():
    forward = _ops()[0]
    args, _, lengths, state_ids, cache_ids = make_k_last_case(True, "verify")
    exp_out, _, _ = oracle_k_last(args, lengths, state_ids, cache_ids)
    out = torch.full_like(args["v"], 3.0)
    result = forward(**args, out=out)
    torch.cuda.synchronize()
    assert result.data_ptr() == out.data_ptr()
    torch.testing.assert_close(out.cpu().float(), exp_out.float(), atol=1e-3, rtol=1.6e-2)
    v = args["v"]
    bad = {
        "out dtype must match v": torch.empty_like(v, dtype=torch.float16),
        "out shape must match v": torch.empty_like(v[:, :-1]),
        "out must be contiguous": torch.empty(*v.shape[:-1], 2 * v.shape[-1], dtype=v.dtype, device=v.device)[..., ::2],
        "out must be on the same device as v": torch.empty_like(v, device="cpu"),
    }
    for message, o in bad.items():
        with pytest.raises(RuntimeError, match=message):
            forward(**args, out=o)


@pytest.mark.parametrize("kernel", ["k_last", "packed"])
@pytest.mark.parametrize("bad", ["zero_h", "head_ratio", "qkv_width", "a", "b", "A_log", "dt_bias", "state",
                                 "hv_cta_zero", "hv_cta_tail", "bv_zero"])
def test_rejects_bad_heads_before_touching_state(kernel, bad):
    forward, packed, forward_tunable, packed_tunable = _ops()
    tunable = bad.startswith("hv_cta") or bad == "bv_zero"
    if bad == "qkv_width" and kernel != "packed":
        pytest.skip("only the packed API accepts a QKV width")
    args, backing, _, _, _ = make_k_last_case(True, "decode", H=6, HV=18)
    kwargs = packed_from(args) if kernel == "packed" else args
    if bad in ("zero_h", "head_ratio"):
        h = 0 if bad == "zero_h" else 5
        if kernel == "packed":
            kwargs["mixed_qkv"] = kwargs["mixed_qkv"].new_zeros(3, (2 * h + 18) * 128)
        else:
            kwargs["q"] = kwargs["q"][:, :, :h].contiguous()
            kwargs["k"] = kwargs["k"][:, :, :h].contiguous()
    elif bad == "qkv_width":
        kwargs["mixed_qkv"] = kwargs["mixed_qkv"][:, :-1].contiguous()
    elif bad in ("a", "b", "A_log", "dt_bias"):
        kwargs[bad] = kwargs[bad][..., :-1].contiguous()
    elif bad == "state":
        kwargs["initial_state_source"] = kwargs["initial_state_source"][:, :-1].contiguous()
    call = packed if kernel == "packed" else forward
    if tunable:
        kwargs = dict(kwargs, bv=64, wn=8, sn=4, hv_per_cta=1)
        if bad == "hv_cta_zero":
            kwargs["hv_per_cta"] = 0
        elif bad == "hv_cta_tail":
            kwargs["hv_per_cta"] = 2
        else:
            kwargs["bv"] = 0
        call = packed_tunable if kernel == "packed" else forward_tunable
    before = backing.clone()
    with pytest.raises(RuntimeError, match="heads|head|HV|QKV|tile"):
        call(**kwargs)
    torch.cuda.synchronize()
    assert torch.equal(backing, before)


def test_lower_bound_requires_kda_and_dt_bias_dtype_rule():
    forward = _ops()[0]
    args, _, _, _, _ = make_k_last_case(False, "decode")
    with pytest.raises(RuntimeError, match="lower_bound is only supported for KDA"):
        forward(**args, lower_bound=-5.0)
    args, _, _, _, _ = make_k_last_case(True, "verify")
    args["dt_bias"] = args["dt_bias"].to(torch.bfloat16)
    with pytest.raises(RuntimeError, match="dt_bias must be"):
        forward(**args)


# ---- benchmark configurations -------------------------------------------------------------

def _check_packed_workload(w):
    packed = _ops()[1]
    exp_out, exp_states = oracle_packed_workload(w)
    call = {k: v for k, v in w.items() if not k.startswith("_")}
    pool = w["initial_state_source"]
    backing = w["_meta"]["backing"]
    before = backing.clone()
    out = packed(**call)
    torch.cuda.synchronize()
    got = out.cpu().float()
    torch.testing.assert_close(got, exp_out.float(), atol=2e-2, rtol=2e-2)
    idx = w["initial_state_indices"].cpu().tolist()
    worst = 0.0
    for slot, want in exp_states.items():
        worst = max(worst, rel_l2(pool[slot], want))
    assert worst <= 1e-3, worst
    for n, s in enumerate(idx):                       # padded entries: exact zeros
        if s < 0:
            assert torch.count_nonzero(out[n]) == 0
    untouched = torch.ones(pool.shape[0], dtype=torch.bool, device=pool.device)
    untouched[torch.tensor(sorted(exp_states), device=pool.device)] = False
    assert torch.equal(backing[untouched], before[untouched])
    return worst


def test_config0_gdn_decode_b8():
    from pla_amd.workloads import gdn_decode_packed
    _check_packed_workload(gdn_decode_packed(8, seed=100))


def test_config1_gdn_packed_decode_b256_pool4096():
    from pla_amd.workloads import gdn_decode_packed
    w = gdn_decode_packed(256, pool_slots=4096, pad_frac=0.05, seed=101)
    idx = w["initial_state_indices"].cpu()
    assert int((idx < 0).sum()) == 13 and not torch.equal(idx, torch.arange(256, dtype=torch.int32))
    _check_packed_workload(w)


def test_kda_packed_decode_b64_pool_with_padded_pitch():
    from pla_amd.workloads import gdn_decode_packed
    _check_packed_workload(gdn_decode_packed(64, H=32, HV=32, pool_slots=256, pad_frac=0.05, seed=102,
                                             is_kda=True, pitch_pad=256))


def test_sanity_mode_rejects_before_launch_and_bypass_flag(monkeypatch):
    forward, packed = _ops()[:2]
    args, backing, lengths, state_ids, cache_ids = make_k_last_case(False, "decode", H=4, HV=8, B=3, padded=False)
    monkeypatch.setenv("PLA_SANITY_CHECK", "1")
    out = forward(**args)                                   # a valid call passes the diagnostic checks
    torch.cuda.synchronize()
    before = backing.clone()
    bad = dict(args, initial_state_indices=torch.tensor([1, 1, 2], dtype=torch.int32, device="cuda"))
    with pytest.raises(RuntimeError, match=r"PLA_SANITY_CHECK \[k_last\].*alias"):
        forward(**bad)
    bad = dict(args, initial_state_indices=torch.tensor([1, 99, 2], dtype=torch.int32, device="cuda"))
    with pytest.raises(RuntimeError, match=r"PLA_SANITY_CHECK \[k_last\].*out of range"):
        forward(**bad)
    kw = packed_from(args)
    kw["cu_seqlens"] = torch.tensor([0, 2, 2, 3], dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match=r"PLA_SANITY_CHECK \[k_last_packed\]"):
        packed(**kw)
    torch.cuda.synchronize()
    assert torch.equal(backing, before)


def _reject_cases():
    """(name, kernel, edit) for calls both host layers must refuse: `edit` changes the keyword arguments of a valid
    T = 1 case (packed or not) in place."""
    def sl(key, index):
        def edit(kw):
            kw[key] = kw[key][index].contiguous()
        return edit

    def put(key, value):
        def edit(kw):
            kw[key] = value(kw) if callable(value) else value
        return edit

    cases = [
        ("no_state", "packed", put("initial_state_source", None)),
        ("state_rank", "packed", put("initial_state_source", lambda kw: kw["initial_state_source"][0])),
        ("head_dim", "packed", put("initial_state_source", lambda kw: kw["initial_state_source"][..., :64].contiguous())),
        ("qkv_rank", "packed", put("mixed_qkv", lambda kw: kw["mixed_qkv"][None])),
        ("qkv_width", "packed", sl("mixed_qkv", (slice(None), slice(0, -1)))),
        ("head_ratio", "packed", put("mixed_qkv", lambda kw: kw["mixed_qkv"].new_zeros(3, (2 * 5 + 18) * 128))),
        ("a_width", "packed", sl("a", (Ellipsis, slice(0, -1)))),
        ("b_width", "packed", sl("b", (Ellipsis, slice(0, -1)))),
        ("A_log", "packed", sl("A_log", (slice(0, -1),))),
        ("dt_bias", "packed", sl("dt_bias", (Ellipsis, slice(0, -1)))),
        ("out_shape", "packed", put("out", lambda kw: kw["out"][:, :, :-1].contiguous())),
        ("cpu_qkv", "packed", put("mixed_qkv", lambda kw: kw["mixed_qkv"].cpu())),
        ("act_dtype", "packed", put("mixed_qkv", lambda kw: kw["mixed_qkv"].float())),
        ("mixed_dtypes", "packed", put("b", lambda kw: kw["b"].half())),
        ("state_dtype", "packed", put("initial_state_source", lambda kw: kw["initial_state_source"].half())),
        ("qkv_rows", "packed", put("mixed_qkv", lambda kw: kw["mixed_qkv"].t().contiguous().t())),
        ("out_strided", "packed", put("out", lambda kw: torch.empty(*kw["out"].shape[:-1], 256, dtype=kw["out"].dtype, device="cuda")[..., ::2])),
        ("cu_dtype", "packed", put("cu_seqlens", lambda kw: kw["cu_seqlens"].long())),
        ("idx_dtype", "packed", put("initial_state_indices", lambda kw: kw["initial_state_indices"].long())),
        ("lower_bound_gdn", "k_last_gdn", put("lower_bound", -5.0)),
        ("accepted_dtype", "k_last", put("cache_steps_or_num_accept", lambda kw: torch.ones(3, dtype=torch.int64, device="cuda"))),
        ("vllm_table_sglang", "k_last", put("initial_state_indices", lambda kw: kw["initial_state_indices"][:, None].contiguous())),
        ("q_rank", "k_last", put("q", lambda kw: kw["q"][0])),
        ("zero_heads", "k_last", lambda kw: kw.update(q=kw["q"][:, :, :0].contiguous(), k=kw["k"][:, :, :0].contiguous())),
        ("head_ratio", "k_last", lambda kw: kw.update(q=kw["q"][:, :, :5].contiguous(), k=kw["k"][:, :, :5].contiguous())),
        ("qk_shapes", "k_last", put("q", lambda kw: kw["q"][:, :, :3].contiguous())),
        ("a_width", "k_last", sl("a", (Ellipsis, slice(0, -1)))),
        ("b_width", "k_last", sl("b", (Ellipsis, slice(0, -1)))),
        ("A_log", "k_last", sl("A_log", (slice(0, -1),))),
        ("state_heads", "k_last", put("initial_state_source", lambda kw: kw["initial_state_source"][:, :-1].contiguous())),
        ("state_dtype", "k_last", put("initial_state_source", lambda kw: kw["initial_state_source"].half())),
        ("cpu_q", "k_last", put("q", lambda kw: kw["q"].cpu())),
        ("act_dtype", "k_last", lambda kw: kw.update({n: kw[n].float() for n in ("q", "k", "v", "a", "b")})),
        ("mixed_dtypes", "k_last", put("k", lambda kw: kw["k"].half())),
        ("out_dtype", "k_last", put("out", lambda kw: torch.empty_like(kw["v"]).float())),
        ("out_shape", "k_last", put("out", lambda kw: torch.empty_like(kw["v"])[:, :, :-1].contiguous())),
        ("dt_bias_dtype", "k_last", put("dt_bias", lambda kw: kw["dt_bias"].float())),
        ("cu_dtype", "k_last", put("cu_seqlens", lambda kw: kw["cu_seqlens"].long())),
        ("idx_dtype", "k_last", put("initial_state_indices", lambda kw: kw["initial_state_indices"].long())),
    ]
    return cases


@pytest.mark.parametrize("name,kernel,edit", _reject_cases(), ids=lambda v: v if isinstance(v, str) else "")
def test_compiled_and_python_host_layers_reject_the_same_calls(name, kernel, edit):
    """The decode checks exist twice: compiled (pla.decode._C, the path every call takes) and in Python (the
    PLA_SANITY_CHECK diagnostics and the tunable entry points).  Every call one of them refuses the other refuses
    too, with the same exception type and the same message, and neither touches the pool."""
    import pla_amd.decode as dec
    native = dec._compiled()
    assert native, "pla_amd.decode._C is not importable"
    args, backing, _, _, _ = make_k_last_case(kernel != "k_last_gdn", "decode", H=6, HV=18)
    before = backing.clone()
    caught = []
    for layer in ("compiled", "python"):
        kw = packed_from(args) if kernel == "packed" else dict(args, lower_bound=None, is_sglang=True, out=torch.empty_like(args["v"]))
        edit(kw)
        if kernel == "packed":
            order = ["mixed_qkv", "a", "b", "A_log", "dt_bias", "softplus_beta", "softplus_threshold", "scale",
                     "initial_state_source", "initial_state_indices", "out", "use_qk_l2norm_in_kernel", "cu_seqlens",
                     "is_kda", "is_sglang"]
            call = native.fused_sigmoid_gating_delta_rule_forward_k_last_packed if layer == "compiled" else \
                (lambda *a: dec._packed_impl(*a, None))
        else:
            order = ["A_log", "a", "dt_bias", "softplus_beta", "softplus_threshold", "q", "k", "v", "b",
                     "initial_state_source", "initial_state_indices", "scale", "use_qk_l2norm_in_kernel", "cu_seqlens",
                     "is_kda", "disable_state_update", "intermediate_states_buffer", "intermediate_state_indices",
                     "cache_steps_or_num_accept", "retrieve_parent_token", "lower_bound", "is_sglang", "out"]
            call = native.fused_sigmoid_gating_delta_rule_forward_k_last if layer == "compiled" else \
                (lambda *a: dec._k_last_impl(*a, None))
        with pytest.raises(Exception) as info:
            call(*[kw[n] for n in order])
        caught.append((type(info.value), str(info.value).splitlines()[0]))
    torch.cuda.synchronize()
    assert caught[0] == caught[1], caught
    assert caught[0][0] is RuntimeError
    assert torch.equal(backing, before)
