"""Real-gate fixtures of the reference (tests/golden/): integrity, oracle pinning, GPU parity.

The reference's tests for these files (tests/test_kimi_k3_real_gate_prefill.py:58-128,
tests/test_qwen38_real_gate_prefill.py:88-140) draw q, k, v ~ 0.1 N(0,1) in bf16 and compare the
kernels with a Python reference; the same inputs are rebuilt here and compared with the oracle.
"""
import hashlib
import os

import pytest
import torch

from helpers import rel_l2
from oracle import (chunked_delta_rule_fp64, gdn_prefill_reference, kda_prefill_reference, l2norm, lower_bound_gate,
                    sigmoid_beta, softplus_gate)
from oracle.prefill import token_recurrence

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
KIMI = os.path.join(GOLDEN, "kimi_k3_layer0_tp8_rank0_gate_14x12.pt")
QWEN = os.path.join(GOLDEN, "qwen38_max_layer0_gate_2092x8.pt")
KIMI_SHA = "87dc7c462606cd1711d5c29e63b6bba11cead733a8e6c6bca56bd03db1981ab9"
QWEN_SHA = "4c7581a21824d930b49d6588c0ab45d695ae855c37067fda0d08e2dd6b05b35c"
D = 128


def _load(path, sha):
    with open(path, "rb") as f:
        assert hashlib.sha256(f.read()).hexdigest() == sha
    return torch.load(path, map_location="cpu", weights_only=True)


def _kimi_inputs():
    gate = _load(KIMI, KIMI_SHA)
    T, H = 14, 12
    gen = torch.Generator().manual_seed(20261020)
    q = (torch.randn(T, H, D, generator=gen) * 0.1).bfloat16()
    k = (torch.randn(T, H, D, generator=gen) * 0.1).bfloat16()
    v = (torch.randn(T, H, D, generator=gen) * 0.1).bfloat16()
    init = (torch.randn(1, H, D, D, generator=gen) * 0.01).bfloat16().float()
    return gate, q, k, v, init


def _qwen_inputs():
    gate = _load(QWEN, QWEN_SHA)
    total, H, HG = 2092, 8, 2
    gen = torch.Generator().manual_seed(20261013)
    q = (torch.randn(total, HG, D, generator=gen) * 0.1).bfloat16()
    k = (torch.randn(total, HG, D, generator=gen) * 0.1).bfloat16()
    v = (torch.randn(total, H, D, generator=gen) * 0.1).bfloat16()
    pool = torch.randn(6, H, D, D, generator=gen) * 0.01
    return gate, q, k, v, pool


def test_fixture_layouts():
    gate = _load(KIMI, KIMI_SHA)
    assert set(gate) == {"token_ids", "g", "beta", "A_log", "dt_bias"}
    assert gate["g"].shape == (14, 12, D) and gate["g"].dtype == torch.bfloat16
    assert gate["beta"].shape == (14, 12) and gate["beta"].dtype == torch.bfloat16
    assert gate["A_log"].shape == (12,) and gate["dt_bias"].shape == (12, D)
    gate = _load(QWEN, QWEN_SHA)
    assert set(gate) == {"raw_gate_a", "raw_beta_b", "A_log", "dt_bias"}
    assert gate["raw_gate_a"].shape == (2092, 8) and gate["raw_gate_a"].dtype == torch.bfloat16
    assert gate["raw_beta_b"].shape == (2092, 8) and gate["A_log"].shape == (8,) and gate["dt_bias"].shape == (8,)


def test_oracle_forms_agree_on_real_kda_gates():
    """Token-by-token recurrence (float64) == chunked WY form (float64) on the real KDA gates,
    whose per-channel decays span e^-5 .. ~1 inside one chunk."""
    gate, q, k, v, init = _kimi_inputs()
    g = lower_bound_gate(gate["g"], gate["dt_bias"], gate["A_log"], -5.0)
    assert g.min() >= -5.0 and g.max() <= 0.0
    beta = sigmoid_beta(gate["beta"])
    qn, kn = l2norm(q).to(q.dtype), l2norm(k).to(k.dtype)
    o_tok, s_tok = token_recurrence(qn, kn, v, g, beta, [0, 14], init, scale=D ** -0.5, compute_dtype=torch.float64)
    o_chk, s_chk = chunked_delta_rule_fp64(qn, kn, v, g, beta, init[0], scale=D ** -0.5)
    torch.testing.assert_close(o_chk, o_tok, atol=1e-9, rtol=1e-9)
    torch.testing.assert_close(s_chk, s_tok[0], atol=1e-9, rtol=1e-9)


def test_oracle_forms_agree_on_real_gdn_gates():
    gate, q, k, v, pool = _qwen_inputs()
    n = 300                                                     # a prefix keeps the token loop short
    g = softplus_gate(gate["raw_gate_a"][:n], gate["dt_bias"], gate["A_log"], 1.0, 20.0, per_channel=False)
    assert g.max() <= 0.0
    beta = sigmoid_beta(gate["raw_beta_b"][:n])
    qn, kn = l2norm(q[:n]).to(q.dtype), l2norm(k[:n]).to(k.dtype)
    o_tok, s_tok = token_recurrence(qn, kn, v[:n], g, beta, [0, n], pool[3:4], scale=D ** -0.5, compute_dtype=torch.float64)
    o_chk, s_chk = chunked_delta_rule_fp64(qn, kn, v[:n], g, beta, pool[3], scale=D ** -0.5)
    torch.testing.assert_close(o_chk, o_tok, atol=1e-9, rtol=1e-9)
    torch.testing.assert_close(s_chk, s_tok[0], atol=1e-9, rtol=1e-9)


@pytest.mark.gpu
def test_kda_prefill_on_real_kimi_gates():
    from pla_amd.prefill.flashkdapro import flashkda_fwd
    gate, q, k, v, init = _kimi_inputs()
    dev = "cuda"
    out = torch.empty(14, 12, D, dtype=torch.bfloat16, device=dev)
    final = torch.empty(1, 12, D, D, device=dev)
    flashkda_fwd(q.to(dev), k.to(dev), v.to(dev), gate["g"].to(dev), gate["beta"].to(dev), gate["A_log"].to(dev),
                 gate["dt_bias"].to(dev), out, D ** -0.5, -5.0, init.to(dev), final)
    torch.cuda.synchronize()
    exp_o, exp_final = kda_prefill_reference(q, k, v, gate["g"], gate["beta"], gate["A_log"], gate["dt_bias"], [0, 14], init)
    torch.testing.assert_close(out.cpu().float(), exp_o.float(), atol=2e-2, rtol=1e-2)     # the reference's KDA gate
    for head in range(12):
        assert rel_l2(final[0, head], exp_final[0, head]) <= 1e-3, head


@pytest.mark.gpu
@pytest.mark.parametrize("raw", [True, False])
def test_gdn_prefill_on_real_qwen_gates(raw):
    """Two sequences (654 and 1438 tokens), 2 q/k heads, 8 value heads, pool slots [3, 1] of 6."""
    from pla_amd.prefill.flashqla import chunk_gated_delta_rule_fwd
    gate, q, k, v, pool = _qwen_inputs()
    dev = "cuda"
    lengths = (654, 1438)
    offs = [0, lengths[0], sum(lengths)]
    cu = torch.tensor(offs, dtype=torch.int32, device=dev)
    idx = torch.tensor([3, 1], dtype=torch.int32, device=dev)
    dpool = pool.to(dev)
    common = dict(scale=D ** -0.5, initial_state=dpool, initial_state_indices=idx, cu_seqlens=cu,
                  output_final_state=False, normalize_qk=True, raw_cu_seqlens=tuple(offs))
    dq, dk, dv = q.to(dev)[None], k.to(dev)[None], v.to(dev)[None]
    if raw:
        res = chunk_gated_delta_rule_fwd(dq, dk, dv, None, None, raw_gate_a=gate["raw_gate_a"].to(dev),
                                         raw_beta_b=gate["raw_beta_b"].to(dev), A_log=gate["A_log"].to(dev),
                                         dt_bias=gate["dt_bias"].to(dev), **common)
    else:
        g = softplus_gate(gate["raw_gate_a"], gate["dt_bias"], gate["A_log"], 1.0, 20.0, per_channel=False)
        res = chunk_gated_delta_rule_fwd(dq, dk, dv, g.to(dev)[None], sigmoid_beta(gate["raw_beta_b"]).to(dev)[None], **common)
    torch.cuda.synchronize()
    assert res[4] is None
    exp_o, exp_final = gdn_prefill_reference(q, k, v, gate["raw_gate_a"], gate["raw_beta_b"], gate["A_log"], gate["dt_bias"],
                                             offs, pool[[3, 1]], scale=D ** -0.5, compute_dtype=torch.float64)
    o = res[2][0].cpu().float()
    assert rel_l2(o, exp_o) <= 2e-2                                              # the reference's GDN gate
    torch.testing.assert_close(o, exp_o.float(), atol=2e-2, rtol=2e-2)
    for n, slot in enumerate((3, 1)):
        for head in range(8):
            assert rel_l2(dpool[slot, head], exp_final[n, head]) <= 1e-3, (slot, head)
    assert torch.equal(dpool[[0, 2, 4, 5]].cpu(), pool[[0, 2, 4, 5]])            # unmapped slots untouched
