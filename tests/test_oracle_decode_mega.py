"""Pins the CPU oracle of the fused KDA decode step (conv + gate + recurrence + norm).

The reference ships no output vectors for this op, so the oracle is pinned against library
routines (``F.conv1d``, ``F.silu``, ``F.rms_norm``), against the already pinned k-last decode
oracle, against an element-wise float64 evaluation and against closed forms.
"""
import math

import torch
import torch.nn.functional as F

from oracle import kda_decode_mega_reference, causal_conv1d_update_reference, k_last_reference
from pla_amd.workloads import kda_decode_mega

D = 128


def _case(B=3, H=4, seed=5, dtype=torch.bfloat16, **kw):
    w = kda_decode_mega(B, H, seed=seed, device="cpu", dtype=dtype, **kw)
    return {k: v for k, v in w.items() if not k.startswith("_")}


def test_conv_update_is_a_depthwise_causal_convolution():
    g = torch.Generator().manual_seed(1)
    C, B = 24, 3
    x = torch.randn(B, C, generator=g)
    conv = torch.randn(5, C, 3, generator=g)
    w = torch.randn(4, C, generator=g)
    bias = torch.randn(C, generator=g)
    slots = [4, -1, 2]
    y, conv_new = causal_conv1d_update_reference(x, conv, w, bias, slots)
    for n, slot in enumerate(slots):
        if slot < 0:
            assert torch.count_nonzero(y[n]) == 0
            continue
        seq = torch.cat([conv[slot], x[n][:, None]], dim=1)[None]                   # [1, C, 4]
        want = F.silu(F.conv1d(seq, w.t()[:, None, :].contiguous(), bias, groups=C))[0, :, 0]
        torch.testing.assert_close(y[n], want, atol=1e-6, rtol=1e-6)
        assert torch.equal(conv_new[slot], seq[0, :, 1:])                           # window slides by one sample
    assert torch.equal(conv_new[[0, 1, 3]], conv[[0, 1, 3]])                         # other slots untouched


def test_conv_window_holds_the_last_three_samples():
    C = 8
    conv = torch.zeros(1, C, 3)
    w = torch.zeros(4, C)
    w[0] = 1.0                                                                       # output = silu(oldest tap)
    xs = [torch.full((1, C), float(i + 1)) for i in range(5)]
    ys = []
    for x in xs:
        y, conv = causal_conv1d_update_reference(x, conv, w, None, [0])
        ys.append(float(y[0, 0]))
    silu = lambda v: v / (1.0 + math.exp(-v))
    assert ys[:3] == [0.0, 0.0, 0.0]
    assert abs(ys[3] - silu(1.0)) < 1e-6 and abs(ys[4] - silu(2.0)) < 1e-6
    assert conv[0, 0].tolist() == [3.0, 4.0, 5.0]


def test_mega_is_conv_then_k_last_decode_then_gated_rmsnorm():
    """Composition of pinned parts: F.conv1d + F.silu, the k-last KDA decode oracle, F.rms_norm."""
    for lower_bound in (None, -5.0):
        c = _case(B=3, H=4, seed=11, bias=True)
        B, H = 3, 4
        dim = H * D
        out, state_new, conv_new = kda_decode_mega_reference(
            c["x"], c["weight"], c["bias"], c["conv_state"], c["raw_g"], c["raw_beta"], c["a_log"], c["dt_bias"],
            c["state_indices"], c["state"], lower_bound=lower_bound, output_gate=c["output_gate"],
            norm_weight=c["norm_weight"], norm_eps=1e-5, round_v=False)
        slots = c["state_indices"].tolist()
        w_dw = c["weight"].permute(0, 2, 1).reshape(3 * dim, 1, 4)                    # depthwise [C, 1, 4]
        seq = torch.cat([c["conv_state"][slots].float(), c["x"].float()[:, :, None]], dim=2)
        mixed = F.silu(F.conv1d(seq, w_dw, c["bias"], groups=3 * dim))[:, :, 0]      # [B, 3*dim]
        q, k, v = (mixed[:, i * dim:(i + 1) * dim].reshape(B, H, D) for i in range(3))
        o, st, _ = k_last_reference(
            q, k, v, c["raw_g"][0].float(), c["raw_beta"][0].float(), c["a_log"], c["dt_bias"].reshape(H, D),
            c["state"], c["state_indices"].tolist(), [1] * B, scale=D ** -0.5, use_qk_l2norm=True, is_kda=True,
            lower_bound=lower_bound)
        want = F.rms_norm(o, (D,), c["norm_weight"], 1e-5) * torch.sigmoid(c["output_gate"].float())
        torch.testing.assert_close(out[0].float(), want.to(torch.bfloat16).float(), atol=1e-2, rtol=1e-2)
        torch.testing.assert_close(state_new, st, atol=1e-6, rtol=1e-5)


def test_mega_matches_elementwise_float64_evaluation():
    c = _case(B=1, H=4, seed=3)
    H, dim = 4, 4 * D
    out, state_new, conv_new = kda_decode_mega_reference(
        c["x"], c["weight"], None, c["conv_state"], c["raw_g"], c["raw_beta"], c["a_log"], c["dt_bias"],
        c["state_indices"], c["state"], lower_bound=-5.0, round_v=False)
    slot = int(c["state_indices"][0])
    h = 2                                                                            # one head, scalar loops
    x64, cs, w = c["x"].double(), c["conv_state"].double(), c["weight"].double()
    act = []
    for seg in range(3):
        row = []
        for ch in range(h * D, (h + 1) * D):
            cc = seg * dim + ch
            acc = sum(float(cs[slot, cc, j]) * float(w[seg, j, ch]) for j in range(3)) + float(x64[0, cc]) * float(w[seg, 3, ch])
            row.append(acc / (1.0 + math.exp(-acc)))
        act.append(row)
    qn = math.sqrt(sum(t * t for t in act[0]) + 1e-6)
    kn = math.sqrt(sum(t * t for t in act[1]) + 1e-6)
    q = [t / qn * D ** -0.5 for t in act[0]]
    k = [t / kn for t in act[1]]
    eA = math.exp(float(c["a_log"][h]))
    dec = [math.exp(-5.0 / (1.0 + math.exp(-eA * (float(c["raw_g"][0, 0, h, i]) + float(c["dt_bias"][h * D + i])))))
           for i in range(D)]
    beta = 1.0 / (1.0 + math.exp(-float(c["raw_beta"][0, 0, h])))
    S = c["state"][slot, h].double()
    for vrow in (0, 17, 127):
        srow = [float(S[vrow, i]) * dec[i] for i in range(D)]
        u = (act[2][vrow] - sum(srow[i] * k[i] for i in range(D))) * beta
        srow = [srow[i] + u * k[i] for i in range(D)]
        o = sum(srow[i] * q[i] for i in range(D))
        assert abs(float(out[0, 0, h, vrow]) - o) <= 1e-2 * abs(o) + 1e-3
        torch.testing.assert_close(state_new[slot, h, vrow].double(), torch.tensor(srow, dtype=torch.float64),
                                   atol=1e-6, rtol=1e-4)


def test_mega_closed_forms():
    """beta -> 0: pure decay of the state, o = (S D) q.  Zero state and zero decay input: o = beta v (k.q)."""
    c = _case(B=2, H=4, seed=9)
    c["raw_beta"] = torch.full_like(c["raw_beta"], -60.0)                            # sigmoid -> 0
    out, state_new, _ = kda_decode_mega_reference(
        c["x"], c["weight"], None, c["conv_state"], c["raw_g"], c["raw_beta"], c["a_log"], c["dt_bias"],
        c["state_indices"], c["state"], lower_bound=None)
    H = 4
    for n, slot in enumerate(c["state_indices"].tolist()):
        x = c["raw_g"][0, n].float() + c["dt_bias"].reshape(H, D)
        decay = torch.exp(-c["a_log"].exp()[:, None] * F.softplus(x))
        torch.testing.assert_close(state_new[slot], c["state"][slot] * decay[:, None, :], atol=1e-7, rtol=1e-5)
    c = _case(B=1, H=4, seed=10)
    c["state"].zero_()
    out, state_new, _ = kda_decode_mega_reference(
        c["x"], c["weight"], None, c["conv_state"], c["raw_g"], c["raw_beta"], c["a_log"], c["dt_bias"],
        c["state_indices"], c["state"], lower_bound=-5.0, round_v=False)
    slot = int(c["state_indices"][0])
    # S = beta v k^T has rank one per head, and o = S q is parallel to v
    for h in range(H):
        S = state_new[slot, h]
        sv = torch.linalg.svdvals(S.double())
        assert float(sv[1] / sv[0]) < 1e-5                                           # rank one up to float32 rounding
        kvec = S[0] / S[0].norm()
        assert abs(float(kvec.norm()) - 1.0) < 1e-5                                  # k is L2-normalised
        ratio = out[0, 0, h].float() / S[:, 0]
        assert float(ratio.std() / ratio.abs().mean()) < 2e-2                        # bf16 output rounding


def test_mega_pad_rows_and_untouched_slots():
    c = _case(B=4, H=4, seed=2, pad_rows=(1,))
    out, state_new, conv_new = kda_decode_mega_reference(
        c["x"], c["weight"], None, c["conv_state"], c["raw_g"], c["raw_beta"], c["a_log"], c["dt_bias"],
        c["state_indices"], c["state"], lower_bound=-5.0, output_gate=c["output_gate"], norm_weight=c["norm_weight"])
    assert torch.count_nonzero(out[0, 1]) == 0
    used = [s for s in c["state_indices"].tolist() if s >= 0]
    unused = [s for s in range(c["state"].shape[0]) if s not in used]
    assert torch.equal(state_new[unused], c["state"][unused]) and torch.equal(conv_new[unused], c["conv_state"][unused])
    for s in used:
        assert not torch.equal(state_new[s], c["state"][s])
