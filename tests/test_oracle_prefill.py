"""Pins the prefill oracle: chunked float64 evaluation == token recurrence,
chained calls == one call, closed-form scenarios, padding / empty sequences."""
import math

import pytest
import torch

from oracle import (gdn_prefill_reference, kda_prefill_reference, chunked_delta_rule_fp64,
                    k_last_reference, softplus_gate, lower_bound_gate, l2norm)
from oracle.prefill import token_recurrence


def _inputs(T, H, HV, D, per_channel, seed):
    g = torch.Generator().manual_seed(seed)
    q = l2norm(torch.randn(T, H, D, generator=g))
    k = l2norm(torch.randn(T, H, D, generator=g))
    v = torch.randn(T, HV, D, generator=g)
    if per_channel:
        gate = -torch.rand(T, HV, D, generator=g) * torch.where(torch.arange(HV) % 2 == 0, 2.0, 0.01)[None, :, None]
    else:
        gate = -torch.rand(T, HV, generator=g) * 0.5
    beta = torch.rand(T, HV, generator=g)
    S0 = torch.randn(HV, D, D, generator=g) * 0.1
    return q, k, v, gate, beta, S0


@pytest.mark.parametrize("per_channel", [False, True])
@pytest.mark.parametrize("T", [1, 63, 64, 65, 150])
def test_chunked_fp64_equals_token_recurrence(per_channel, T):
    q, k, v, gate, beta, S0 = _inputs(T, 2, 4, 16, per_channel, seed=T)
    o_tok, S_tok = token_recurrence(q, k, v, gate, beta, [0, T], S0[None], scale=0.25,
                                    compute_dtype=torch.float64)
    o_ch, S_ch = chunked_delta_rule_fp64(q, k, v, gate, beta, S0, scale=0.25, chunk=64)
    torch.testing.assert_close(o_ch, o_tok, rtol=1e-9, atol=1e-11)
    torch.testing.assert_close(S_ch, S_tok[0], rtol=1e-9, atol=1e-11)
    # the result does not depend on the chunk size
    o16, S16 = chunked_delta_rule_fp64(q, k, v, gate, beta, S0, scale=0.25, chunk=16)
    torch.testing.assert_close(o16, o_ch, rtol=1e-9, atol=1e-11)
    torch.testing.assert_close(S16, S_ch, rtol=1e-9, atol=1e-11)


def test_token_recurrence_equals_decode_oracle_step_by_step():
    T = 5
    q, k, v, gate, beta, S0 = _inputs(T, 2, 4, 8, True, seed=3)
    o, S = token_recurrence(q, k, v, gate, beta, [0, T], S0[None], scale=0.5)
    out, st, _ = k_last_reference(q, k, v, None, None, None, None, S0[None], [0], [T], scale=0.5,
                                  use_qk_l2norm=False, is_kda=True, log_decay=gate, beta_activated=beta)
    torch.testing.assert_close(o, out, rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(S[0], st[0], rtol=1e-6, atol=1e-7)


def test_two_chained_calls_equal_one_and_ragged_batch():
    lens = [0, 17, 90]
    offs = [0, 0, 17, 107]
    T = 110                                    # three padding tokens at the end
    q, k, v, gate, beta, _ = _inputs(T, 2, 4, 8, False, seed=9)
    g0 = torch.Generator().manual_seed(1)
    S0 = torch.randn(3, 4, 8, 8, generator=g0) * 0.1
    o, S = token_recurrence(q, k, v, gate, beta, offs, S0, scale=1.0)
    assert torch.equal(S[0], S0[0])                         # empty sequence keeps its state
    assert torch.count_nonzero(o[107:]) == 0                # padding rows are zero
    # split the long sequence at 48 and carry the state
    o1, S1 = token_recurrence(q[17:65], k[17:65], v[17:65], gate[17:65], beta[17:65], [0, 48], S0[2:3], scale=1.0)
    o2, S2 = token_recurrence(q[65:107], k[65:107], v[65:107], gate[65:107], beta[65:107], [0, 42], S1, scale=1.0)
    torch.testing.assert_close(torch.cat([o1, o2]), o[17:107], rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(S2[0], S[2], rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("scenario", ["initial_bits", "weak_decay", "small_update", "fresh_update"])
def test_kda_prefill_closed_forms(scenario):
    """Closed forms of tests/test_kda_prefill_flashkdapro.py:243-311 evaluated on the oracle."""
    heads, dim = 2, 128
    lengths = [0, 1, 17] if scenario == "initial_bits" else [0, 17, 200]
    offs = [0]
    for n in lengths:
        offs.append(offs[-1] + n)
    total = offs[-1]
    q = torch.zeros(total + 3, heads, dim, dtype=torch.bfloat16)
    q[..., 0] = 1
    k, v = torch.zeros_like(q), torch.zeros_like(q)
    updating = scenario in ("small_update", "fresh_update")
    if updating:
        k[..., 0] = 1
        v.fill_(1)
    raw_value = -12.0 if scenario == "weak_decay" else -100.0
    raw = torch.full_like(q, raw_value)
    beta = torch.full((total + 3, heads), -12.0, dtype=q.dtype)
    a_log = torch.zeros(heads)
    dt_bias = torch.zeros(heads, dim)
    h0 = torch.linspace(-0.25, 0.25, len(lengths) * heads * dim * dim).reshape(len(lengths), heads, dim, dim)
    if updating:
        h0.zero_()
        if scenario == "small_update":
            h0[..., 0] = 0.1253
    init = None if scenario == "fresh_update" else h0
    out, final = kda_prefill_reference(q, k, v, raw, beta, a_log, dt_bias, offs, init,
                                       compute_dtype=torch.float64)
    assert torch.count_nonzero(out[total:]) == 0
    if scenario == "initial_bits":
        assert torch.equal(final.float(), h0)               # exp(-5*sigmoid(-100)) == 1 exactly
    g = -5.0 * torch.sigmoid(torch.tensor(raw_value, dtype=torch.float64))
    b = torch.sigmoid(torch.tensor(-12.0, dtype=torch.float64))
    decay = g.exp()
    rec = decay * (1 - b) if updating else decay
    start_all = torch.zeros_like(h0) if init is None else h0
    # the oracle normalises q and k = e0 with eps inside the root and rounds to bf16 (-> exactly 1)
    for seq, length in enumerate(lengths):
        start = start_all[seq].double()
        end = start * decay.pow(length)
        steps = torch.arange(1, length + 1, dtype=torch.float64)
        values = rec.pow(steps)[:, None, None] * start[..., 0]
        if updating:
            values = values + (b * (-torch.expm1(steps * rec.log())) / (1 - rec))[:, None, None]
            end[..., 0] = rec.pow(length) * start[..., 0] + b * (-torch.expm1(length * rec.log())) / (1 - rec)
        want = (values * dim ** -0.5)
        torch.testing.assert_close(final[seq], end, rtol=1e-6, atol=1e-10)   # gates are float32
        if length:
            got = out[offs[seq]:offs[seq + 1]].double()
            torch.testing.assert_close(got, want, rtol=2 ** -7, atol=1e-12)   # out is rounded to bf16


def test_gdn_prefill_reference_preprocessing():
    T, H, HV, D = 40, 2, 4, 16
    g = torch.Generator().manual_seed(5)
    q = torch.randn(T, H, D, generator=g).bfloat16()
    k = torch.randn(T, H, D, generator=g).bfloat16()
    v = torch.randn(T, HV, D, generator=g).bfloat16()
    a = torch.randn(T, HV, generator=g).bfloat16()
    b = torch.randn(T, HV, generator=g).bfloat16()
    A = torch.rand(HV, generator=g) * math.log(16)
    dt = torch.rand(HV, generator=g) * 2 - 1
    S0 = torch.randn(1, HV, D, D, generator=g) * 0.1
    o, S = gdn_prefill_reference(q, k, v, a, b, A, dt, [0, T], S0, compute_dtype=torch.float64)
    # same thing spelled out: normalise, round to bf16, gate, chunked float64
    qn = (q.float() / torch.sqrt(q.float().square().sum(-1, keepdim=True) + 1e-6)).bfloat16()
    kn = (k.float() / torch.sqrt(k.float().square().sum(-1, keepdim=True) + 1e-6)).bfloat16()
    gate = -A.exp() * torch.nn.functional.softplus(a.float() + dt)
    o2, S2 = chunked_delta_rule_fp64(qn, kn, v, gate, torch.sigmoid(b.float()), S0[0], scale=D ** -0.5)
    torch.testing.assert_close(S[0], S2, rtol=1e-7, atol=1e-9)
    torch.testing.assert_close(o.double(), o2, rtol=2 ** -7, atol=1e-6)
    assert o.dtype == torch.bfloat16
