"""KDA MTP verify + accepted-prefix commit (benchmark configuration 2) and the KDA wrapper."""
import pytest
import torch

from helpers import rel_l2
from oracle import k_last_reference, fold_reference

pytestmark = pytest.mark.gpu


def _records_from_tokens(w, slots):
    """Lay the per-token tensors of the verify call out as per-slot records for the commit."""
    m = w["_meta"]
    B, HV, T = m["B"], m["HV"], m["T"]
    dev = w["q"].device
    idx = w["indices"].long()
    rawk = torch.zeros(slots, HV, T, 128, dtype=w["k"].dtype, device=dev)
    rawv = torch.zeros(slots, HV, T, 128, dtype=w["v"].dtype, device=dev)
    gk = torch.zeros(slots, HV, T, 128, dtype=torch.float32, device=dev)
    beta = torch.zeros(slots, HV, T, dtype=torch.float32, device=dev)
    rawk[idx] = w["k"][0].view(B, T, HV, 128).transpose(1, 2)
    rawv[idx] = w["v"][0].view(B, T, HV, 128).transpose(1, 2)
    gk[idx] = w["log_decay"].view(B, T, HV, 128).transpose(1, 2)
    beta[idx] = w["beta"].view(B, T, HV).transpose(1, 2)
    return rawk, rawv, gk, beta


@pytest.mark.parametrize("B,slots", [(6, 16), (64, 1024)])
def test_config2_kda_mtp_verify_and_commit(B, slots):
    from pla_amd.workloads import kda_mtp_verify as make
    from pla_amd.decode.kda_replayssm_sglang import kda_mtp_verify, fold_accepted_prefix
    w = make(B=B, pool_slots=slots, seed=202)
    m = w["_meta"]
    HV, T = m["HV"], m["T"]
    state = w["state"]
    before = m["backing"].clone()
    out = kda_mtp_verify(w["q"], w["k"], w["v"], w["log_decay"], w["beta"], state, w["indices"],
                         w["cu_seqlens"], scale=w["scale"])
    torch.cuda.synchronize()
    assert torch.equal(m["backing"], before)                  # verify never writes the pool

    idx = w["indices"].cpu().tolist()
    acc = w["num_accepted"].cpu().tolist()
    compact = state[w["indices"].long()].cpu()
    q, k, v = (w[n][0].cpu() for n in ("q", "k", "v"))
    exp_out, _, _ = k_last_reference(q, k, v, None, None, None, None, compact, list(range(B)), [T] * B,
                                     scale=w["scale"], use_qk_l2norm=True, is_kda=True,
                                     disable_state_update=True, log_decay=w["log_decay"].cpu(),
                                     beta_activated=w["beta"].cpu())
    torch.testing.assert_close(out[0].cpu().float(), exp_out.float(), atol=2e-2, rtol=2e-2)

    rawk, rawv, gk, beta = _records_from_tokens(w, slots)
    fold_accepted_prefix(state[None], rawv[None], rawk[None], gk[None], beta[None],
                         w["indices"], w["num_accepted"], null_block_id=-1)
    torch.cuda.synchronize()
    # expected: the state after exactly num_accepted tokens of the same recurrence
    exp_state = fold_reference(compact, rawk[w["indices"].long()].cpu(), rawv[w["indices"].long()].cpu(),
                               gk[w["indices"].long()].cpu(), beta[w["indices"].long()].cpu(),
                               list(range(B)), acc)
    for n, slot in enumerate(idx):
        if acc[n] <= 0:
            assert torch.equal(state[slot], before[slot, : HV * 16384].view(HV, 128, 128))    # untouched, bit-exact
        else:
            assert rel_l2(state[slot], exp_state[n]) <= 1e-3
            # and it is the verify recurrence truncated at num_accepted tokens
            sl = slice(n * T, n * T + acc[n])
            _, st, _ = k_last_reference(q[sl], k[sl], v[sl], None, None, None, None, compact[n:n + 1], [0],
                                        [acc[n]], scale=w["scale"], is_kda=True,
                                        log_decay=w["log_decay"].cpu()[sl], beta_activated=w["beta"].cpu()[sl])
            assert rel_l2(state[slot], st[0]) <= 1e-3
    touched = torch.zeros(slots, dtype=torch.bool, device=state.device)
    touched[torch.tensor([s for s, a in zip(idx, acc) if a > 0], device=state.device)] = True
    assert torch.equal(m["backing"][~touched], before[~touched])


@pytest.mark.parametrize("layers,padded", [(2, False), (3, True)])
def test_commit_null_slots_and_clamped_lengths(layers, padded):
    """All layers fold in one launch; with `padded` every tensor is a view with a layer pitch larger than its
    extent (two spare slots per layer), whose spare slots must stay untouched."""
    from pla_amd.decode.kda_replayssm_sglang import fold_accepted_prefix
    g = torch.Generator().manual_seed(5)
    slots, H, HV, L = 6, 2, 4, 3
    dev = "cuda"
    spare = 2 if padded else 0
    view = lambda t: t[:, :slots]
    temporal_all = (torch.randn(layers, slots + spare, HV, 128, 128, generator=g) * 0.1).to(dev)
    rawk_all = torch.randn(layers, slots + spare, H, L, 128, generator=g).bfloat16().to(dev)
    rawv_all = torch.randn(layers, slots + spare, HV, L, 128, generator=g).bfloat16().to(dev)
    gk_all = (-torch.rand(layers, slots + spare, HV, L, 128, generator=g)).to(dev)
    beta_all = torch.rand(layers, slots + spare, HV, L, generator=g).to(dev)
    temporal, rawk, rawv, gk, beta = (view(t) for t in (temporal_all, rawk_all, rawv_all, gk_all, beta_all))
    spare_before = temporal_all[:, slots:].clone()
    idx = torch.tensor([4, 0, -1, 2], dtype=torch.int32, device=dev)
    acc = torch.tensor([2, 0, 3, 99], dtype=torch.int32, device=dev)      # 99 is clamped to L
    before = temporal.clone()
    fold_accepted_prefix(temporal, rawv, rawk, gk, beta, idx, acc, null_block_id=-1)
    torch.cuda.synchronize()
    for layer in range(layers):
        exp = fold_reference(before[layer].cpu(), rawk[layer].cpu(), rawv[layer].cpu(), gk[layer].cpu(),
                             beta[layer].cpu(), idx.cpu().tolist(), [2, 0, 3, L])
        assert torch.equal(temporal[layer, [0, 1, 3, 5]], before[layer, [0, 1, 3, 5]])
        for slot in (4, 2):
            assert rel_l2(temporal[layer, slot], exp[slot]) <= 1e-4
    assert torch.equal(temporal_all[:, slots:], spare_before)
    # with null_block_id = 0 slot 0 would be a null block as well; here slot 0 had accept 0 anyway
    temporal.copy_(before)
    fold_accepted_prefix(temporal, rawv, rawk, gk, beta, idx, acc, null_block_id=4)
    torch.cuda.synchronize()
    assert torch.equal(temporal, before)                       # every slot <= null_block_id


def test_commit_track_snapshots():
    """Track snapshots: the state after step track_steps[n] also goes to slot track_indices[n]
    (src/decode/kda_replayssm/kda_mtp_fold.cu:462-478); a tracked slot <= null_block_id is skipped."""
    from pla_amd.decode.kda_replayssm_sglang import fold_accepted_prefix
    g = torch.Generator().manual_seed(8)
    slots, H, HV, L = 8, 2, 4, 4
    temporal = (torch.randn(1, slots, HV, 128, 128, generator=g) * 0.1).cuda()
    rawk = torch.randn(1, slots, H, L, 128, generator=g).bfloat16().cuda()
    rawv = torch.randn(1, slots, HV, L, 128, generator=g).bfloat16().cuda()
    gk = (-torch.rand(1, slots, HV, L, 128, generator=g)).cuda()
    beta = torch.rand(1, slots, HV, L, generator=g).cuda()
    idx = torch.tensor([4, 1, 6], dtype=torch.int32, device="cuda")
    acc = torch.tensor([4, 3, 2], dtype=torch.int32, device="cuda")
    track = torch.tensor([5, -1, 7], dtype=torch.int32, device="cuda")
    steps = torch.tensor([1, 0, 1], dtype=torch.int32, device="cuda")          # snapshot after 2, -, 2 tokens
    before = temporal.clone()
    fold_accepted_prefix(temporal, rawv, rawk, gk, beta, idx, acc, null_block_id=-1,
                         track_indices=track, track_steps=steps)
    torch.cuda.synchronize()
    c = lambda t: t[0].cpu()
    full = fold_reference(c(before), c(rawk), c(rawv), c(gk), c(beta), [4, 1, 6], [4, 3, 2])
    part = fold_reference(c(before), c(rawk), c(rawv), c(gk), c(beta), [4, 1, 6], [2, 1, 2])
    for slot in (4, 1, 6):
        assert rel_l2(temporal[0, slot], full[slot]) <= 1e-4
    assert rel_l2(temporal[0, 5], part[4]) <= 1e-4 and rel_l2(temporal[0, 7], part[6]) <= 1e-4
    assert torch.equal(temporal[0, [0, 2, 3]], before[0, [0, 2, 3]])


@pytest.mark.parametrize("spec", [False, True])
def test_fused_recurrent_kda_wrapper(spec):
    from pla_amd.decode.kda import fused_recurrent_kda
    g = torch.Generator().manual_seed(9)
    dev, H, T, N = "cuda", 4, 3, 2
    ntok = N * (T if spec else 1)
    rnd = lambda *s: torch.randn(*s, generator=g)
    q, k, v = (rnd(1, ntok, H, 128).bfloat16().to(dev) for _ in range(3))
    raw_g, raw_beta = rnd(1, ntok, H, 128).bfloat16().to(dev), rnd(1, ntok, H).bfloat16().to(dev)
    A_log, dt_bias = rnd(H).to(dev), rnd(H, 128).to(dev)
    state = (rnd(9, H, 128, 128) * 0.1).to(dev)
    before = state.clone()
    if spec:
        table = [[1, 2, 3], [4, 0, 6]]
        idx = torch.tensor(table, dtype=torch.int32, device=dev)
        acc = torch.tensor([2, 1], dtype=torch.int32, device=dev)
        cu = torch.tensor([0, T, 2 * T], dtype=torch.int32, device=dev)
        lengths, ids, accl = [T, T], table, [2, 1]
    else:
        idx = torch.tensor([5, 0], dtype=torch.int32, device=dev)     # slot 0 is vLLM's null block
        acc, cu, lengths, ids, accl = None, torch.tensor([0, 1, 2], dtype=torch.int32, device=dev), [1, 1], [5, 0], None
    out, st = fused_recurrent_kda(q, k, v, raw_g, raw_beta, A_log, dt_bias, -5.0, state, cu, idx, acc)
    torch.cuda.synchronize()
    assert st.data_ptr() == state.data_ptr()
    exp_out, exp_state, _ = k_last_reference(
        q[0].cpu(), k[0].cpu(), v[0].cpu(), raw_g[0].cpu(), raw_beta[0].cpu(), A_log.cpu(),
        dt_bias.cpu() if spec else dt_bias.cpu().bfloat16(), before.cpu(), ids, lengths,
        is_kda=True, disable_state_update=spec, num_accepted=accl, lower_bound=-5.0, is_sglang=False)
    torch.testing.assert_close(out[0].cpu().float(), exp_out.float(), atol=1e-3, rtol=1.6e-2)
    torch.testing.assert_close(state.cpu(), exp_state, atol=2e-3, rtol=8e-3)
    with pytest.raises(ValueError, match="dt_bias must be float32"):
        fused_recurrent_kda(q, k, v, raw_g, raw_beta, A_log, dt_bias.bfloat16(), -5.0, state, cu, idx, acc)
    with pytest.raises(NotImplementedError):
        fused_recurrent_kda(q, k, v, raw_g, raw_beta, A_log, dt_bias, -5.0, state, cu, idx, acc, fuse_gate=False)
