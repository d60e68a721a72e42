"""Caselist parsing (CPU) and replay of a sample of the reference's caselists with a parity check (GPU).

``tests/golden/caselist_sample.list`` holds seventeen lines of the reference's caselists (shapes only)."""
import os

import pytest
import torch

from pla_amd import caselist

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
SAMPLE = os.path.join(GOLDEN, "caselist_sample.list")
DECODE_HEAD_SHAPES = os.path.join(GOLDEN, "caselist_decode_head_shapes.list")
PREFILL_EVERY50 = os.path.join(GOLDEN, "caselist_prefill_every50.list")


def test_parse_sample_lines():
    cases = caselist.read_caselist(SAMPLE)
    assert len(cases) == 16
    first = cases[0]
    assert (first["family"], first["phase"], first["op"], first["seqlen_q"], first["batch_size"]) == ("GDN", "D", "gdn_attn", 1, 1)
    assert first["num_heads_qk"] == 16 and first["num_heads_v"] == 32 and first["dtype"] == "bf16"
    kda = [c for c in cases if c["op"] == "kda_attn" and c["phase"] == "D"]
    assert kda[0]["gate_lower_bound"] == -5.0 and "gate_lower_bound" not in kda[-1]
    prefill = [c for c in cases if c["phase"] == "P"]
    assert prefill[2]["cu_seqlens_q"] == [0, 1090, 2528, 4096, 5894, 7662, 8790] and prefill[2]["batch_size"] == 6
    assert all(c["cu_seqlens_q"][0] == 0 and len(c["cu_seqlens_q"]) == c["batch_size"] + 1 for c in prefill)
    reasons = [caselist.unsupported_reason(c) for c in cases]
    assert sum(r is not None for r in reasons) == 1 and "mamba2_ssm" in [r for r in reasons if r][0]
    assert caselist.parse_case("# comment") is None and caselist.parse_case("   ") is None
    with pytest.raises(ValueError):
        caselist.parse_case("gdn_attn:seqlen_q:1")
    assert caselist.read_caselist(SAMPLE, limit=3) == cases[:3]


def test_full_caselist_fixtures_parse_and_are_served():
    """The head shapes of every decode caselist and the sampled prefill caselists: every GDN / KDA line parses,
    and the only decode shapes without an operator here are one-token KDA head counts the fused step does not build."""
    decode = caselist.read_caselist(DECODE_HEAD_SHAPES)
    assert len(decode) == 114 and all(c["phase"] == "D" for c in decode)
    heads = {(c["family"], c["num_heads_qk"], c["num_heads_v"]) for c in decode}
    assert len([h for h in heads if h[0] == "GDN"]) == 16 and len([h for h in heads if h[0] == "KDA"]) == 11
    assert {c["seqlen_q"] for c in decode} == {1, 3, 4, 5, 8}
    unserved = {(c["num_heads_qk"], c["seqlen_q"]) for c in decode if caselist.unsupported_reason(c)}
    assert unserved == {(3, 1), (32, 1)}
    from pla_amd.autotune import shapes_from_caselists
    assert len(shapes_from_caselists([DECODE_HEAD_SHAPES])) == 27
    prefill = caselist.read_caselist(PREFILL_EVERY50)
    assert len(prefill) == 943 and all(c["phase"] == "P" for c in prefill)
    assert all(caselist.unsupported_reason(c) is None for c in prefill)
    assert all(c["cu_seqlens_q"][0] == 0 and len(c["cu_seqlens_q"]) == c["batch_size"] + 1 for c in prefill)
    assert max(c["cu_seqlens_q"][-1] for c in prefill) == 32768


@pytest.mark.gpu
def test_replay_sample_and_check_against_oracle():
    """Every supported sample shape runs; the small ones are compared with the CPU oracle."""
    from helpers import oracle_packed_workload, rel_l2
    from oracle import gdn_prefill_reference, kda_decode_mega_reference
    cases = caselist.read_caselist(SAMPLE)
    kinds = set()
    for case in cases:
        row = caselist.replay_case(case, reps=3)
        if caselist.unsupported_reason(case):
            assert row["status"] == "skipped"
            continue
        assert row["status"] == "ok" and row["us"] > 0
        kinds.add(row["kind"])
    assert kinds == {"gdn_decode", "gdn_verify", "kda_decode", "kda_verify", "gdn_prefill", "kda_prefill"}

    # parity on two small shapes through the same builders
    fns, info = caselist.build_case(cases[1], sets=1)                                  # GDN decode, batch 8
    w = info["workload"]
    exp_out, exp_states = oracle_packed_workload(w)
    fns[0]()
    torch.cuda.synchronize()
    for slot, want in exp_states.items():
        assert rel_l2(w["initial_state_source"][slot], want) <= 1e-3
    fns, info = caselist.build_case(cases[5], sets=1)                                  # KDA decode, batch 18, 12 heads
    w = {k: (v.cpu().clone() if torch.is_tensor(v) else v) for k, v in info["workload"].items()}
    want_o, want_s, _ = kda_decode_mega_reference(
        w["x"], w["weight"], None, w["conv_state"], w["raw_g"], w["raw_beta"], w["a_log"], w["dt_bias"],
        w["state_indices"], w["state"], lower_bound=-5.0, output_gate=w["output_gate"], norm_weight=w["norm_weight"])
    fns[0]()
    torch.cuda.synchronize()
    torch.testing.assert_close(info["out"].cpu().float(), want_o.float(), atol=2e-2, rtol=2e-2)
    for slot in w["state_indices"].tolist():
        assert rel_l2(info["workload"]["state"][slot], want_s[slot]) <= 1e-3
