"""GPU parity of the KDA verify with replay records, the conv-window rollback and the full commit.

Cases follow the reference's scripts for these ops (scripts/decode/kda_mtp_sglang/test_correctness.py,
test_verify_layouts.py, test_commit_layouts.py): dense and SGLang-style strided layouts, int32 / int64
indices, padded requests, the fused output norm, draft windows of 1..8 tokens.  Tolerances: bf16 output
atol = rtol = 2e-2; records: bf16 k / v within one bf16 ulp of the float64 value, FP32 log-decay and beta
rtol 1e-4; conv windows, untouched ring entries, scratch rows, states and conv pools bit-exact.
"""
import types

import pytest
import torch

from helpers import rel_l2
from oracle import verify_dspark_reference, conv_window_scatter_reference, fold_reference
from pla_amd.decode.kda_replayssm_sglang import (fused_kda_decode_mtp_dspark, commit_kda_replayssm_after_verify,
                                                 conv_window_scatter)
from pla_amd.workloads import kda_replay_verify

pytestmark = pytest.mark.gpu
D = 128
RING_KEYS = ("replayssm_rawv", "replayssm_rawk", "replayssm_g", "replayssm_beta")
WIN_KEYS = ("intermediate_conv_q", "intermediate_conv_k", "intermediate_conv_v")


def _cpu(w):
    return {k: (v.cpu().clone() if torch.is_tensor(v) else v) for k, v in w.items()}


def _oracle(c):
    keys = ("x_q", "x_k", "x_v", "g", "beta", "w_q", "w_k", "w_v", "cs_q", "cs_k", "cs_v", "A_log", "dt_bias",
            "recurrent_state", "ssm_state_indices", "intermediate_state_indices", "cu_seqlens", "lower_bound", "scale")
    return verify_dspark_reference(**{k: c[k] for k in keys}, rings=tuple(c[k] for k in RING_KEYS),
                                   windows=tuple(c[k] for k in WIN_KEYS), onorm_gate=c.get("onorm_gate"),
                                   onorm_weight=c.get("onorm_weight"), onorm_eps=c.get("onorm_eps"))


def _check(w):
    c = _cpu(w)
    want = _oracle(c)
    state_before = w["recurrent_state"].clone()
    conv_before = [w[k].clone() for k in ("cs_q", "cs_k", "cs_v")]
    out = fused_kda_decode_mtp_dspark(**w)
    torch.cuda.synchronize()
    torch.testing.assert_close(out.cpu().float(), want["out"].float(), atol=2e-2, rtol=2e-2)
    assert torch.equal(w["recurrent_state"], state_before)                           # read-only
    for k, before in zip(("cs_q", "cs_k", "cs_v"), conv_before):
        assert torch.equal(w[k], before)
    for key, name in zip(WIN_KEYS, ("ic_q", "ic_k", "ic_v")):                        # copies of bf16 inputs
        assert torch.equal(w[key].cpu(), want[name])
    torch.testing.assert_close(w["replayssm_rawk"].cpu().float(), want["ring_rawk"].float(), atol=1e-6, rtol=8e-3)
    torch.testing.assert_close(w["replayssm_rawv"].cpu().float(), want["ring_rawv"].float(), atol=1e-6, rtol=8e-3)
    torch.testing.assert_close(w["replayssm_g"].cpu(), want["ring_g"], atol=1e-6, rtol=1e-4)
    torch.testing.assert_close(w["replayssm_beta"].cpu(), want["ring_beta"], atol=1e-6, rtol=1e-4)
    for key, name in zip(RING_KEYS, ("ring_rawv", "ring_rawk", "ring_g", "ring_beta")):
        untouched = want[name] == 3.0                                                # sentinel of the workload
        assert torch.equal(w[key].cpu()[untouched], want[name][untouched])
    return out


@pytest.mark.parametrize("N,H,T", [(1, 4, 1), (3, 4, 2), (2, 6, 3), (8, 12, 4), (3, 4, 5), (2, 12, 7), (8, 12, 8), (64, 32, 4),
                                   (3, 4, 9), (2, 6, 13), (4, 4, 16), (3, 4, 17), (2, 6, 25), (4, 4, 32)])
@pytest.mark.parametrize("onorm", [False, True])
def test_verify_matches_oracle(N, H, T, onorm):
    _check(kda_replay_verify(N, H, T, seed=10 * N + T, onorm=onorm, strided=True))


@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
@pytest.mark.parametrize("strided", [False, True])
def test_verify_layouts_indices_and_padding(index_dtype, strided):
    w = kda_replay_verify(5, 6, 4, seed=33, onorm=True, strided=strided, index_dtype=index_dtype, pad_rows=(0, 3))
    out = _check(w)
    assert torch.count_nonzero(out[0, 0:4]) == 0 and torch.count_nonzero(out[0, 12:16]) == 0
    assert torch.count_nonzero(out[0, 4:8]) > 0


@pytest.mark.parametrize("T", [3, 8])
def test_verify_with_transposed_scratch_windows(T):
    """Scratch windows stored [row, step, 3, channels] (window-major) take the per-thread stores instead of
    the 16-byte vectors of the [row, step, channels, 3] layout: same results."""
    w = kda_replay_verify(3, 4, T, seed=90 + T, onorm=True)
    for key in WIN_KEYS:
        rows, steps, dim, taps = w[key].shape
        w[key] = torch.zeros(rows, steps, taps, dim, dtype=torch.bfloat16, device="cuda").transpose(2, 3)
        assert w[key].stride(3) == dim and w[key].stride(2) == 1
    _check(w)


def test_verify_rejects_bad_arguments():
    w = kda_replay_verify(2, 4, 4, seed=1)
    bad = dict(w)
    bad["replayssm_g"] = None
    with pytest.raises(ValueError, match="CACHE_RING"):
        fused_kda_decode_mtp_dspark(**bad)
    bad = dict(w)
    bad["onorm_eps"] = None
    with pytest.raises(ValueError, match="fused output norm requires"):
        fused_kda_decode_mtp_dspark(**bad)
    bad = dict(w)
    bad["recurrent_state"] = w["recurrent_state"].to(torch.bfloat16)
    with pytest.raises(RuntimeError, match="recurrent state must be fp32"):
        fused_kda_decode_mtp_dspark(**bad)
    bad = dict(w)
    bad["replayssm_rawv"] = w["replayssm_rawv"][:, :, :2]
    with pytest.raises(RuntimeError, match="ring shorter than the draft window|invalid verify ring shape"):
        fused_kda_decode_mtp_dspark(**bad)
    wide = kda_replay_verify(1, 4, 33, seed=1)
    with pytest.raises(RuntimeError, match="up to 32 draft tokens"):
        fused_kda_decode_mtp_dspark(**wide)
    torch.cuda.synchronize()
    assert bool((w["replayssm_g"] == 3.0).all())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("layout", ["dim_width", "width_dim"])
@pytest.mark.parametrize("index_dtype", [torch.int32, torch.int64])
def test_conv_window_scatter(dtype, layout, index_dtype):
    g = torch.Generator().manual_seed(4)
    layers, slots, rows, steps, dim = 3, 7, 5, 4, 300
    if layout == "dim_width":
        dst = torch.randn(layers, slots, dim, 3, generator=g).to(dtype).cuda()
        src = torch.randn(layers, rows, steps, dim, 3, generator=g).to(dtype).cuda()
    else:
        dst = torch.randn(layers, slots, 3, dim, generator=g).to(dtype).cuda().transpose(-1, -2)
        src = torch.randn(layers, rows, steps, 3, dim, generator=g).to(dtype).cuda().transpose(-1, -2)
    dst_idx = torch.tensor([4, -1, 0, 6, 99], dtype=index_dtype)
    step_idx = torch.tensor([3, 2, -1, 0, 1], dtype=index_dtype)
    want = conv_window_scatter_reference(dst.cpu(), src.cpu(), dst_idx, step_idx)
    conv_window_scatter(dst, src, dst_idx.cuda(), step_idx.cuda())
    torch.cuda.synchronize()
    assert torch.equal(dst.cpu(), want)


def test_verify_then_commit_round_trip():
    """Verify 4 draft tokens, accept 0..4 of them per request, commit: the checkpoint equals the oracle's
    fold of the recorded prefix, the conv state is the window after the last accepted token, and a second
    verify from the committed state matches the oracle run on the committed copies."""
    N, H, T, L = 6, 4, 4, 8
    w = kda_replay_verify(N, H, T, seed=71, ring_len=L, onorm=False, strided=False, pad_rows=(2,))
    w["intermediate_state_indices"] = torch.arange(N, dtype=torch.int32, device="cuda")      # row r = request r
    fused_kda_decode_mtp_dspark(**w)
    accept = torch.tensor([4, 1, 3, 0, 2, 4], dtype=torch.int32)
    last = (accept.long() - 1)
    slots = w["ssm_state_indices"].cpu()
    c = _cpu(w)
    want_state = fold_reference(c["recurrent_state"], c["replayssm_rawk"], c["replayssm_rawv"], c["replayssm_g"],
                                c["replayssm_beta"], slots.tolist(), accept.tolist())
    spec = types.SimpleNamespace(
        temporal=w["recurrent_state"][None], replayssm_rawv=w["replayssm_rawv"][None],
        replayssm_rawk=w["replayssm_rawk"][None], replayssm_g=w["replayssm_g"][None],
        replayssm_beta=w["replayssm_beta"][None],
        conv=[w["cs_q"][None], w["cs_k"][None], w["cs_v"][None]],
        intermediate_conv_window=[w["intermediate_conv_q"][None], w["intermediate_conv_k"][None],
                                  w["intermediate_conv_v"][None]])
    commit_kda_replayssm_after_verify(spec_state=spec, state_batch_indices=w["ssm_state_indices"],
                                      accept_lens=accept.cuda(), last_correct_step_indices=last.cuda())
    torch.cuda.synchronize()
    for s in range(want_state.shape[0]):
        if torch.equal(want_state[s], c["recurrent_state"][s]):
            assert torch.equal(w["recurrent_state"][s].cpu(), c["recurrent_state"][s])       # untouched slots
        else:
            assert rel_l2(w["recurrent_state"][s], want_state[s]) <= 1e-3
    for key, win in (("cs_q", "intermediate_conv_q"), ("cs_k", "intermediate_conv_k"), ("cs_v", "intermediate_conv_v")):
        want_conv = conv_window_scatter_reference(c[key][None], c[win][None], slots, last)[0]
        assert torch.equal(w[key].cpu(), want_conv)
    # the next verify starts from the committed pools
    g = torch.Generator().manual_seed(5)
    for k in ("x_q", "x_k", "x_v", "g"):
        w[k].copy_((torch.randn(w[k].shape, generator=g) * 0.5).to(torch.bfloat16))
    _check(w)


def test_verify_sanity_mode(monkeypatch):
    monkeypatch.setenv("PLA_SANITY_CHECK", "1")
    w = kda_replay_verify(4, 4, 3, seed=12, pad_rows=(1,))
    _check(w)                                                                        # a clean call passes
    rings_before = w["replayssm_g"].clone()
    bad = dict(w)
    bad["ssm_state_indices"] = torch.tensor([2, -1, 2, 0], dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match=r"PLA_SANITY_CHECK \[kda_verify_dspark\]: two requests write the rings"):
        fused_kda_decode_mtp_dspark(**bad)
    bad = dict(w)
    bad["ssm_state_indices"] = torch.tensor([2, -1, 77, 0], dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="slot is out of bounds"):
        fused_kda_decode_mtp_dspark(**bad)
    bad = dict(w)
    bad["cu_seqlens"] = torch.tensor([0, 3, 5, 9, 12], dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError, match="must own exactly 3 tokens"):
        fused_kda_decode_mtp_dspark(**bad)
    bad = dict(w)
    bad["lower_bound"] = 0.5
    with pytest.raises(RuntimeError, match="lower_bound must be a finite negative"):
        fused_kda_decode_mtp_dspark(**bad)
    bad = dict(w)
    bad["x_k"] = w["x_k"].clone()
    bad["x_k"][0, 7, 1, 3] = float("inf")
    with pytest.raises(RuntimeError, match="selected x_k must be finite"):
        fused_kda_decode_mtp_dspark(**bad)
    bad["x_k"][0, 7, 1, 3] = 0.0
    bad["x_k"][0, 4, 1, 3] = float("nan")                                              # token of the padded request
    fused_kda_decode_mtp_dspark(**bad)
    torch.cuda.synchronize()
    unused = [s for s in range(w["replayssm_g"].shape[0]) if s not in w["ssm_state_indices"].tolist()]
    assert torch.equal(w["replayssm_g"][unused], rings_before[unused])
