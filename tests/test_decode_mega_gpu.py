"""GPU parity of the fused KDA decode step (conv + gate + recurrence + norm) against the CPU oracle.

Cases follow the reference's own checks for this op: the head / batch / lower-bound / norm matrix of
scripts/decode/kda_fusion/compare_kda_decode_fusion.py:102-116 and the pad-slot rules of
scripts/decode/kda_fusion/test_pad_slot.py:37-53.  Tolerances: output atol = rtol = 2e-2 (bf16) and
FP32 state rel-L2 <= 1e-3 (the measured error is far below both); the conv window is a copy of
inputs and must be bit-exact.
"""
import pytest
import torch

from helpers import rel_l2
from oracle import kda_decode_mega_reference
from pla_amd.decode.kda import fused_kda_decode_mega_forward
from pla_amd.workloads import kda_decode_mega

pytestmark = pytest.mark.gpu
D = 128


def _run(w, lower_bound, onorm, out=None):
    B, H = w["x"].shape[0], w["x"].shape[1] // (3 * D)
    out = torch.full((1, B, H, D), 7.0, dtype=w["x"].dtype, device="cuda") if out is None else out
    ret = fused_kda_decode_mega_forward(
        x=w["x"], weight=w["weight"], bias=w["bias"], conv_state=w["conv_state"], raw_g=w["raw_g"],
        raw_beta=w["raw_beta"], a_log=w["a_log"], dt_bias=w["dt_bias"], state_indices=w["state_indices"],
        state=w["state"], out=out, lower_bound=lower_bound,
        output_gate=w["output_gate"] if onorm else None, norm_weight=w["norm_weight"] if onorm else None,
        norm_eps=1e-5)
    assert ret is None
    torch.cuda.synchronize()
    return out


def _oracle(w_cpu, lower_bound, onorm):
    return kda_decode_mega_reference(
        w_cpu["x"], w_cpu["weight"], w_cpu["bias"], w_cpu["conv_state"], w_cpu["raw_g"], w_cpu["raw_beta"],
        w_cpu["a_log"], w_cpu["dt_bias"], w_cpu["state_indices"], w_cpu["state"], lower_bound=lower_bound,
        output_gate=w_cpu["output_gate"] if onorm else None, norm_weight=w_cpu["norm_weight"] if onorm else None,
        norm_eps=1e-5)


def _cpu(w):
    return {k: (v.cpu().clone() if torch.is_tensor(v) else v) for k, v in w.items() if not k.startswith("_")}


def _check(w, lower_bound, onorm, atol=2e-2):
    w_cpu = _cpu(w)
    want_o, want_s, want_c = _oracle(w_cpu, lower_bound, onorm)
    out = _run(w, lower_bound, onorm)
    torch.testing.assert_close(out.float().cpu(), want_o.float(), atol=atol, rtol=2e-2)
    assert torch.equal(w["conv_state"].cpu(), want_c)
    used = [s for s in w_cpu["state_indices"].tolist() if s >= 0]
    for s in used:
        assert rel_l2(w["state"][s], want_s[s]) <= 1e-3
    unused = [s for s in range(w_cpu["state"].shape[0]) if s not in used]
    assert torch.equal(w["state"][unused].cpu(), w_cpu["state"][unused])
    return out


@pytest.mark.parametrize("H,B,lower_bound,onorm", [
    (4, 1, -5.0, True), (6, 1, -5.0, True), (6, 4, None, False), (6, 16, -5.0, True), (8, 1, -5.0, True),
    (12, 1, -5.0, True), (12, 4, None, False), (16, 1, -5.0, True), (24, 4, None, False), (48, 1, -5.0, True),
    (64, 1, -5.0, True), (96, 1, -5.0, True), (12, 8, None, True), (4, 3, -5.0, False)])
def test_mega_matches_oracle_bf16(H, B, lower_bound, onorm):
    _check(kda_decode_mega(B, H, seed=100 + H + B), lower_bound, onorm)


@pytest.mark.parametrize("bias", [False, True])
def test_mega_matches_oracle_fp16_and_bias(bias):
    _check(kda_decode_mega(5, 12, seed=7, dtype=torch.float16, bias=bias), -5.0, True)
    _check(kda_decode_mega(5, 12, seed=8, dtype=torch.bfloat16, bias=bias), None, True)


def test_mega_four_consecutive_steps_slide_the_conv_window():
    B, H = 4, 8
    w = kda_decode_mega(B, H, seed=21)
    w_cpu = _cpu(w)
    g = torch.Generator().manual_seed(22)
    for step in range(4):
        x = torch.randn(B, 3 * H * D, generator=g).to(torch.bfloat16)
        rg = torch.randn(1, B, H, D, generator=g).to(torch.bfloat16)
        w["x"].copy_(x)
        w["raw_g"].copy_(rg)
        w_cpu["x"], w_cpu["raw_g"] = x, rg
        want_o, w_cpu["state"], w_cpu["conv_state"] = _oracle(w_cpu, -5.0, True)
        out = _run(w, -5.0, True)
        torch.testing.assert_close(out.float().cpu(), want_o.float(), atol=2e-2, rtol=2e-2)
        assert torch.equal(w["conv_state"].cpu(), w_cpu["conv_state"])
    for s in w_cpu["state_indices"].tolist():
        assert rel_l2(w["state"][s], w_cpu["state"][s]) <= 1e-3


@pytest.mark.parametrize("H,B,pad_rows", [(12, 8, (0, 3)), (12, 4, (3,)), (24, 8, (1, 7))])
def test_mega_pad_slots(H, B, pad_rows):
    """Pad rows (slot -1) emit exact zeros and touch neither pool; the other rows are bit-identical to a
    run without pad rows; slot 0 is an ordinary slot."""
    base = kda_decode_mega(B, H, seed=7)
    base["state_indices"] = torch.arange(B, dtype=torch.int32, device="cuda")
    seed_state, seed_conv = base["state"].clone(), base["conv_state"].clone()
    out_ref = _run(base, -5.0, True)
    state_ref, conv_ref = base["state"].clone(), base["conv_state"].clone()
    assert not torch.equal(state_ref[0], seed_state[0])                              # slot 0 was computed

    pad = kda_decode_mega(B, H, seed=7)
    idx = torch.arange(B, dtype=torch.int32)
    for r in pad_rows:
        idx[r] = -1
    pad["state_indices"] = idx.cuda()
    out_pad = _run(pad, -5.0, True)
    for r in range(B):
        if r in pad_rows:
            assert torch.count_nonzero(out_pad[0, r]) == 0
            assert torch.equal(pad["state"][r], seed_state[r]) and torch.equal(pad["conv_state"][r], seed_conv[r])
        else:
            assert torch.equal(out_pad[0, r], out_ref[0, r])
            assert torch.equal(pad["state"][r], state_ref[r]) and torch.equal(pad["conv_state"][r], conv_ref[r])
    # guard region of the pages (none here beyond the pools) and the extra slots stay as seeded
    assert torch.equal(pad["state"][B:], seed_state[B:]) and torch.equal(pad["conv_state"][B:], seed_conv[B:])


def test_mega_rejects_bad_arguments_before_writing():
    w = kda_decode_mega(2, 4, seed=3)
    snapshot = w["_cache"].clone()
    out = torch.full((1, 2, 4, D), 7.0, dtype=torch.bfloat16, device="cuda")
    bad = dict(w)
    bad["x"] = torch.zeros(2, 3 * 5 * D, dtype=torch.bfloat16, device="cuda")         # H = 5 is not a supported count
    with pytest.raises(RuntimeError, match="H must be"):
        _run(bad, -5.0, True, out=out)
    bad = dict(w)
    bad["state"] = w["state"].to(torch.bfloat16)
    with pytest.raises(RuntimeError, match="state must be a CUDA float32"):
        _run(bad, -5.0, True, out=out)
    bad = dict(w)
    bad["conv_state"] = w["conv_state"].contiguous()                                  # not the SD layout
    with pytest.raises(RuntimeError, match="SD cache layout"):
        _run(bad, -5.0, True, out=out)
    bad = dict(w)
    bad["norm_weight"] = None
    with pytest.raises(RuntimeError, match="provided together"):
        fused_kda_decode_mega_forward(
            x=w["x"], weight=w["weight"], bias=None, conv_state=w["conv_state"], raw_g=w["raw_g"],
            raw_beta=w["raw_beta"], a_log=w["a_log"], dt_bias=w["dt_bias"], state_indices=w["state_indices"],
            state=w["state"], out=out, lower_bound=-5.0, output_gate=w["output_gate"], norm_weight=None)
    torch.cuda.synchronize()
    assert torch.equal(w["_cache"], snapshot) and bool((out == 7.0).all())


def test_mega_in_a_graph_matches_eager():
    B, H = 8, 12
    w = kda_decode_mega(B, H, seed=31)
    seed_cache = w["_cache"].clone()
    eager = []
    for _ in range(3):
        eager.append(_run(w, -5.0, True).clone())
    eager_cache = w["_cache"].clone()
    w["_cache"].copy_(seed_cache)
    out = torch.zeros(1, B, H, D, dtype=torch.bfloat16, device="cuda")
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        _run(w, -5.0, True, out=out)                                                  # warm-up on the side stream
    torch.cuda.current_stream().wait_stream(s)
    w["_cache"].copy_(seed_cache)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fused_kda_decode_mega_forward(
            x=w["x"], weight=w["weight"], bias=None, conv_state=w["conv_state"], raw_g=w["raw_g"],
            raw_beta=w["raw_beta"], a_log=w["a_log"], dt_bias=w["dt_bias"], state_indices=w["state_indices"],
            state=w["state"], out=out, lower_bound=-5.0, output_gate=w["output_gate"],
            norm_weight=w["norm_weight"], norm_eps=1e-5)
    w["_cache"].copy_(seed_cache)
    for i in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager[i])
    assert torch.equal(w["_cache"], eager_cache)


def test_mega_sanity_mode_rejects_aliased_slots_and_bad_values(monkeypatch):
    monkeypatch.setenv("PLA_SANITY_CHECK", "1")
    w = kda_decode_mega(4, 4, seed=5)
    _run(w, -5.0, True)                                                               # a clean call passes
    snapshot = w["_cache"].clone()
    bad = dict(w)
    bad["state_indices"] = torch.tensor([2, 1, 2, -1], dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match=r"PLA_SANITY_CHECK \[fused_kda_decode\]: requests must not concurrently"):
        _run(bad, -5.0, True)
    bad["state_indices"] = torch.tensor([2, 1, 99, -1], dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="exceeds recurrent/conv pool capacity"):
        _run(bad, -5.0, True)
    with pytest.raises(RuntimeError, match="lower_bound must be a finite negative"):
        _run(w, 1.0, True)
    bad = dict(w)
    bad["x"] = w["x"].clone()
    bad["x"][1, 5] = float("nan")
    with pytest.raises(RuntimeError, match="selected x must be finite"):
        _run(bad, -5.0, True)
    bad["state_indices"] = torch.tensor([4, -1, 2, 1], dtype=torch.int32, device="cuda")   # the poisoned row is a pad
    _run(bad, -5.0, True)
    assert not torch.equal(w["_cache"], snapshot)


def test_compiled_and_python_layers_of_the_kda_entry_points_agree():
    """fused_kda_decode_mega_forward and fused_recurrent_kda exist compiled (pla.decode._C, the path a call takes) and in
    Python (the PLA_SANITY_CHECK path): the same refused calls raise the same exception type and message in both, and
    an accepted call gives the same bits."""
    import pla_amd.decode as dec
    import pla_amd.decode.kda as kda
    native = dec._compiled()
    assert native and kda._native() is native
    w = kda_decode_mega(2, 4, seed=3)
    out = torch.empty(1, 2, 4, D, dtype=torch.bfloat16, device="cuda")
    base = dict(x=w["x"], weight=w["weight"], bias=None, conv_state=w["conv_state"], raw_g=w["raw_g"], raw_beta=w["raw_beta"],
                a_log=w["a_log"], dt_bias=w["dt_bias"], state_indices=w["state_indices"], state=w["state"], out=out,
                lower_bound=-5.0, output_gate=w["output_gate"], norm_weight=w["norm_weight"], norm_eps=1e-5)
    order = list(base)
    edits = {
        "cpu_x": dict(x=w["x"].cpu()), "x_dtype": dict(x=w["x"].float()), "weight_dtype": dict(weight=w["weight"].bfloat16()),
        "heads": dict(x=torch.zeros(2, 3 * 5 * D, dtype=torch.bfloat16, device="cuda")),
        "state_dtype": dict(state=w["state"].bfloat16()), "conv_layout": dict(conv_state=w["conv_state"].contiguous()),
        "norm_pair": dict(norm_weight=None), "raw_g_shape": dict(raw_g=w["raw_g"][0]), "idx_dtype": dict(state_indices=w["state_indices"].long()),
        "out_shape": dict(out=out[0]), "eps": dict(norm_eps=-1.0), "bias": dict(bias=torch.zeros(5, device="cuda")),
        "gate_shape": dict(output_gate=w["output_gate"][..., :64]),
    }
    snapshot = w["_cache"].clone()
    for name, edit in edits.items():
        caught = []
        for call in (native.fused_kda_decode_mega_forward, kda._mega_impl):
            with pytest.raises(Exception) as info:
                call(*[dict(base, **edit)[n] for n in order])
            caught.append((type(info.value), str(info.value).splitlines()[0]))
        assert caught[0] == caught[1] and caught[0][0] is RuntimeError, (name, caught)
    torch.cuda.synchronize()
    assert torch.equal(w["_cache"], snapshot)
    # fused_recurrent_kda: refused calls
    from pla_amd.workloads import kda_mtp_verify
    H = 4
    g = torch.Generator().manual_seed(1)
    q = torch.randn(1, 3, H, 128, generator=g).bfloat16().cuda()
    args = dict(q=q, k=q.clone(), v=q.clone(), raw_g=torch.randn(1, 3, H, 128, generator=g).bfloat16().cuda(),
                raw_beta=torch.randn(1, 3, H, generator=g).bfloat16().cuda(), A_log=torch.zeros(H, device="cuda"),
                dt_bias=torch.zeros(H, 128, device="cuda"), lower_bound=-5.0, initial_state=torch.zeros(5, H, 128, 128, device="cuda"),
                cu_seqlens=torch.tensor([0, 1, 2, 3], dtype=torch.int32, device="cuda"),
                ssm_state_indices=torch.tensor([1, 2, 4], dtype=torch.int32, device="cuda"), num_accepted_tokens=None, out=None,
                fuse_gate=None, is_sglang=False)
    korder = list(args)
    kedits = {
        "fuse_gate": dict(fuse_gate=False), "no_dt_bias": dict(dt_bias=None), "q_rank": dict(q=q[0]), "batch": dict(q=q.repeat(2, 1, 1, 1)),
        "head_dim": dict(q=q[..., :64].contiguous()), "state_dtype": dict(initial_state=args["initial_state"].bfloat16()),
        "idx_rank": dict(ssm_state_indices=args["ssm_state_indices"][None, None]),
        "table_sglang": dict(ssm_state_indices=args["ssm_state_indices"][:, None].contiguous(), is_sglang=True),
        "dt_dtype": dict(dt_bias=args["dt_bias"].bfloat16()),
    }
    for name, edit in kedits.items():
        caught = []
        for call in (native.fused_recurrent_kda, kda._fused_recurrent_kda_impl):
            with pytest.raises(Exception) as info:
                call(*[dict(args, **edit)[n] for n in korder])
            caught.append((type(info.value), str(info.value).splitlines()[0]))
        assert caught[0] == caught[1] and caught[0][0] in (ValueError, NotImplementedError), (name, caught)
    # an accepted call: same output and state bits from both layers
    outs = []
    for call in (native.fused_recurrent_kda, kda._fused_recurrent_kda_impl):
        state = torch.full((5, H, 128, 128), 0.01, device="cuda")
        o, st = call(*[dict(args, initial_state=state)[n] for n in korder])
        outs.append((o.clone(), st.clone()))
    torch.cuda.synchronize()
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
