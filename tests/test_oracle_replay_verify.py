"""Pins the CPU oracle of the KDA verify with replay records and of the conv-window scatter.

No output vectors exist in the reference for this op; the oracle is pinned against ``F.conv1d`` /
``F.silu``, against the single-token conv oracle stepped T times, against the k-last verify oracle
(pinned in tests/test_oracle_decode.py) fed with the same post-conv activations and log-decay, against
``F.rms_norm`` and against the commit oracle replaying the records the verify wrote.
"""
import torch
import torch.nn.functional as F

from oracle import (verify_dspark_reference, causal_conv_silu_sequence, causal_conv1d_update_reference,
                    conv_window_scatter_reference, k_last_reference, fold_reference)
from pla_amd.workloads import kda_replay_verify

D = 128


def _oracle(w):
    rings = (w["replayssm_rawv"], w["replayssm_rawk"], w["replayssm_g"], w["replayssm_beta"])
    windows = (w["intermediate_conv_q"], w["intermediate_conv_k"], w["intermediate_conv_v"])
    keys = ("x_q", "x_k", "x_v", "g", "beta", "w_q", "w_k", "w_v", "cs_q", "cs_k", "cs_v", "A_log", "dt_bias",
            "recurrent_state", "ssm_state_indices", "intermediate_state_indices", "cu_seqlens", "lower_bound", "scale")
    return verify_dspark_reference(**{k: w[k] for k in keys}, rings=rings, windows=windows,
                                   onorm_gate=w.get("onorm_gate"), onorm_weight=w.get("onorm_weight"),
                                   onorm_eps=w.get("onorm_eps"))


def test_conv_sequence_is_a_depthwise_causal_convolution_and_equals_stepping():
    g = torch.Generator().manual_seed(3)
    T, C = 5, 16
    x = torch.randn(T, C, generator=g)
    window = torch.randn(C, 3, generator=g)
    w = torch.randn(C, 4, generator=g)
    y, wins = causal_conv_silu_sequence(x, window, w)
    seq = torch.cat([window, x.t()], dim=1)[None].double()                          # [1, C, 3 + T]
    want = F.silu(F.conv1d(seq, w.double()[:, None, :], groups=C))[0].t()            # [T, C]
    torch.testing.assert_close(y, want, atol=1e-12, rtol=1e-12)
    conv = window[None].clone()
    for t in range(T):
        y1, conv = causal_conv1d_update_reference(x[t][None], conv, w.t().contiguous(), None, [0])
        torch.testing.assert_close(y1[0].double(), y[t], atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(conv[0].double(), wins[t], atol=0, rtol=0)


def test_verify_is_conv_then_the_pinned_recurrence_then_rms_norm():
    w = kda_replay_verify(3, 4, 4, seed=5, device="cpu", pad_rows=(1,), onorm=True)
    N, H, T = 3, 4, 12
    res = _oracle(w)
    slots, rows = w["ssm_state_indices"].tolist(), w["intermediate_state_indices"].tolist()
    # post-conv activations from the library routines
    acts = []
    for name, cs, wt in (("x_q", "cs_q", "w_q"), ("x_k", "cs_k", "w_k"), ("x_v", "cs_v", "w_v")):
        x = w[name][0].double().reshape(N, 4, H * D)
        y = torch.zeros(N, 4, H * D, dtype=torch.float64)
        for n, slot in enumerate(slots):
            if slot < 0:
                continue
            seq = torch.cat([w[cs][slot].double(), x[n].t()], dim=1)[None]
            y[n] = F.silu(F.conv1d(seq, w[wt].double()[:, None, :], groups=H * D))[0].t()
        acts.append(y.reshape(T, H, D))
    q_c, k_c, v_c = acts
    log_decay = w["lower_bound"] * torch.sigmoid(
        w["A_log"].double().exp()[None, :, None] * (w["g"][0].double() + w["dt_bias"].double().reshape(H, D)))
    beta = torch.sigmoid(w["beta"][0].double())
    o, state_after, _ = k_last_reference(
        q_c, k_c, v_c, None, None, None, None, w["recurrent_state"].double(), slots, [4] * N,
        scale=w["scale"], use_qk_l2norm=True, is_kda=True, disable_state_update=True,
        log_decay=log_decay, beta_activated=beta, compute_dtype=torch.float64)
    want = F.rms_norm(o.double(), (D,), w["onorm_weight"].double(), w["onorm_eps"]) * torch.sigmoid(w["onorm_gate"][0].double())
    want[4:8] = 0                                                                    # the padded request
    torch.testing.assert_close(res["out"][0], want, atol=2e-6, rtol=1e-3)      # the k-last oracle normalises q, k in float32
    assert torch.equal(state_after, w["recurrent_state"].double())
    # records and windows
    for n, slot in enumerate(slots):
        if slot < 0:
            continue
        tok = slice(4 * n, 4 * n + 4)
        torch.testing.assert_close(res["ring_rawk"][slot, :, :4].double(), k_c[tok].transpose(0, 1).to(torch.bfloat16).double(), atol=0, rtol=0)
        torch.testing.assert_close(res["ring_rawv"][slot, :, :4].double(), v_c[tok].transpose(0, 1).to(torch.bfloat16).double(), atol=0, rtol=0)
        torch.testing.assert_close(res["ring_g"][slot, :, :4].double(), log_decay[tok].transpose(0, 1), atol=1e-6, rtol=1e-6)
        torch.testing.assert_close(res["ring_beta"][slot, :, :4].double(), beta[tok].t(), atol=1e-7, rtol=1e-6)
        # last window = the last three inputs; windows are exact copies of bf16 inputs
        xq = w["x_q"][0, tok].reshape(4, H * D)
        assert torch.equal(res["ic_q"][rows[n], 3].t(), xq[1:4])
        assert torch.equal(res["ic_q"][rows[n], 0, :, 2], xq[0]) and torch.equal(res["ic_q"][rows[n], 0, :, :2], w["cs_q"][slot][:, 1:])
    pad_slot_rows = [r for r in range(w["intermediate_conv_q"].shape[0]) if r not in [rows[0], rows[2]]]
    assert torch.count_nonzero(res["ic_q"][pad_slot_rows]) == 0
    untouched = [s for s in range(w["replayssm_g"].shape[0]) if s not in (slots[0], slots[2])]
    assert bool((res["ring_g"][untouched] == 3.0).all()) and bool((res["ring_g"][:, :, 4:] == 3.0).all())


def test_commit_of_the_verify_records_reproduces_the_verify_recurrence():
    """Folding the accepted prefix of the records the verify wrote gives the state of the stepped recurrence
    over that prefix (to the bf16 rounding of the recorded k and v)."""
    w = kda_replay_verify(2, 4, 4, seed=9, device="cpu", onorm=False, strided=False)
    N, H = 2, 4
    res = _oracle(w)
    slots = w["ssm_state_indices"].tolist()
    accepted = [4, 2]
    folded = fold_reference(w["recurrent_state"], res["ring_rawk"], res["ring_rawv"], res["ring_g"], res["ring_beta"],
                            slots, accepted, compute_dtype=torch.float64)
    acts = []
    for name, cs, wt in (("x_q", "cs_q", "w_q"), ("x_k", "cs_k", "w_k"), ("x_v", "cs_v", "w_v")):
        x = w[name][0].reshape(N, 4, H * D)
        acts.append(torch.stack([causal_conv_silu_sequence(x[n], w[cs][slots[n]], w[wt])[0] for n in range(N)])
                    .reshape(N * 4, H, D))
    log_decay = w["lower_bound"] * torch.sigmoid(
        w["A_log"].double().exp()[None, :, None] * (w["g"][0].double() + w["dt_bias"].double().reshape(H, D)))
    keep = torch.cat([torch.arange(4 * n, 4 * n + a) for n, a in enumerate(accepted)])
    _, stepped, _ = k_last_reference(
        acts[0][keep], acts[1][keep], acts[2][keep], None, None, None, None, w["recurrent_state"].double(), slots,
        accepted, scale=w["scale"], use_qk_l2norm=True, is_kda=True, log_decay=log_decay[keep],
        beta_activated=torch.sigmoid(w["beta"][0].double())[keep], compute_dtype=torch.float64)
    for slot in slots:
        rel = (folded[slot] - stepped[slot]).norm() / stepped[slot].norm()
        moved = (stepped[slot] - w["recurrent_state"][slot].double()).norm() / stepped[slot].norm()
        assert float(rel) < 5e-3 and float(moved) > 0.05
    other = [s for s in range(w["recurrent_state"].shape[0]) if s not in slots]
    assert torch.equal(folded[other], w["recurrent_state"][other].double())


def test_conv_window_scatter_reference_masks():
    g = torch.Generator().manual_seed(2)
    dst = torch.randn(2, 5, 8, 3, generator=g)
    src = torch.randn(2, 4, 6, 8, 3, generator=g)
    out = conv_window_scatter_reference(dst, src, torch.tensor([3, -1, 9, 0]), torch.tensor([2, 1, 0, -1]))
    assert torch.equal(out[:, 3], src[:, 0, 2])
    keep = [0, 1, 2, 4]
    assert torch.equal(out[:, keep], dst[:, keep])


def test_commit_plan_reference_known_answers():
    """Hand-derived plans (block size 4): positions count tokens already computed."""
    from oracle import replay_commit_plan_reference as plan
    # no align: counts are clamped to the query length, null / negative sources and empty queries commit nothing
    got = plan([3, 9, 2, -1, 1], [7, 2, 0, 5, 4], [0, 3, 5, 5, 6, 7], slots=12, Q=3, token_capacity=7)
    assert got == [[3, 2, 0, 0, 1], [7, 2, 0, 0, 4], [0, 0, 0, 0, 0], [0, 0, 0, 0, 0]]
    # align: request 0 at position 2 commits 3 tokens -> tokens 2, 3, 4: boundary after 2 tokens into the block of
    # position 2 (column 0), final in the block of token 4 (column 1); request 1 at position 4 commits 2 tokens inside
    # block 1 -> no boundary; request 2 at position 3 commits 1 token = exactly up to the boundary: boundary == final
    table = [[5, 6, 7], [8, 9, 1], [2, 3, 4]]
    got = plan([3, 2, 1], [5, 9, 2], [0, 3, 5, 6], slots=12, Q=3, token_capacity=6, block_table=table,
               num_computed_tokens=[2, 4, 3], block_size=4)
    assert got == [[3, 2, 1], [6, 9, 2], [5, 0, 2], [2, 0, 1]]
    # conflicts cancel both sides: request 1's final block is request 0's source
    got = plan([1, 1], [5, 9], [0, 1, 2], slots=12, Q=2, token_capacity=2, block_table=[[5], [5]],
               num_computed_tokens=[0, 0], block_size=4)
    assert got == [[0, 0], [0, 0], [0, 0], [0, 0]]
    # a live query that commits nothing still protects its source
    got = plan([0, 1], [5, 9], [0, 1, 2], slots=12, Q=2, token_capacity=2, block_table=[[5], [5]],
               num_computed_tokens=[0, 0], block_size=4)
    assert got == [[0, 0], [0, 0], [0, 0], [0, 0]]
    # mapping, capacity padding, token capacity and a boundary that differs from the final block with equal slots
    got = plan([2, 1], [3, 4], [0, 2, 3], slots=8, Q=2, token_capacity=3, request_indices=[1, 0], capacity=4)
    assert got == [[1, 1, 0, 0], [3, 4, 0, 0], [0, 0, 0, 0], [0, 0, 0, 0]]
    got = plan([2, 2], [3, 4], [0, 2, 4], slots=8, Q=2, token_capacity=3)
    assert got == [[2, 0], [3, 0], [0, 0], [0, 0]]
    got = plan([2], [3], [0, 2], slots=8, Q=2, token_capacity=2, block_table=[[6, 6]], num_computed_tokens=[3], block_size=4)
    assert got == [[0], [0], [0], [0]]                                                # boundary == final, lengths differ
