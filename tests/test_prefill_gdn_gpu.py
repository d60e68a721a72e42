"""GPU parity of the GDN chunk-64 prefill against the CPU oracle (token recurrence / float64
chunked evaluation).  Tolerances: bf16 o atol 2e-2 / rtol 2e-2, FP32 final state rel-L2 <= 1e-3;
untouched pool slots and the padded output suffix bit-exact."""
import pytest
import torch

from helpers import rel_l2
from oracle import gdn_prefill_reference, chunked_delta_rule_fp64, softplus_gate, sigmoid_beta, l2norm

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def poisoned_workspace(monkeypatch):
    """Every call of this file gets a workspace whose bytes are all 0xFF (NaN as FP32 and as fp16): a kernel that
    reads a workspace word no kernel of the same call has written turns its results into NaN.  (The workspace
    comes from torch.empty, so recycled memory may hold anything.)"""
    from pla_amd.prefill.flashqla import ops

    def workspace(T, N, Hg, H, device):
        from pla_amd import _lib
        nbytes = _lib.load().pla_gdn_prefill_workspace_bytes(T, N, Hg, H)
        return torch.full((nbytes,), 0xFF, dtype=torch.uint8, device=device), nbytes
    monkeypatch.setattr(ops, "_workspace", workspace)
    # the facade's own path allocates through _workspace; the compiled host layer (which allocates by itself) is
    # switched off here and compared with this path bit for bit in tests/test_drop_in_imports.py
    monkeypatch.setattr(ops, "_native", False)


def _run_workload(w, output_final_state=True):
    from pla_amd.prefill.flashqla import gdn_prefill_packed_qkv_fwd
    call = {k: v for k, v in w.items() if not k.startswith("_")}
    packed = call.pop("packed_qkv")
    a, b, A, dt, cu = (call.pop(n) for n in ("raw_gate_a", "raw_beta_b", "A_log", "dt_bias", "cu_seqlens"))
    return gdn_prefill_packed_qkv_fwd(packed, a, b, A, dt, cu, output_final_state=output_final_state, **call)


def _oracle_workload(w, fast=False):
    m = w["_meta"]
    T, H, HV = m["T"], m["H"], m["HV"]
    packed = w["packed_qkv"].cpu()
    q = packed[:, : H * 128].reshape(T, H, 128)
    k = packed[:, H * 128: 2 * H * 128].reshape(T, H, 128)
    v = packed[:, 2 * H * 128:].reshape(T, HV, 128)
    idx = w["initial_state_indices"].cpu().long()
    S0 = w["initial_state"][idx.to(w["initial_state"].device)].cpu()
    a, b = w["raw_gate_a"].cpu(), w["raw_beta_b"].cpu()
    A, dt = w["A_log"].cpu(), w["dt_bias"].cpu()
    if not fast:
        return gdn_prefill_reference(q, k, v, a, b, A, dt, m["offsets"], S0, scale=w["scale"])
    # float64 chunked evaluation of the same definition (validated against the token recurrence)
    qn, kn = l2norm(q).to(q.dtype), l2norm(k).to(k.dtype)
    g = softplus_gate(a, dt, A)
    beta = sigmoid_beta(b)
    o = torch.zeros(T, HV, 128, dtype=torch.float64)
    final = S0.double().clone()
    offs = m["offsets"]
    for n in range(len(offs) - 1):
        lo, hi = offs[n], offs[n + 1]
        if hi > lo:
            o[lo:hi], final[n] = chunked_delta_rule_fp64(qn[lo:hi], kn[lo:hi], v[lo:hi], g[lo:hi], beta[lo:hi],
                                                         S0[n], scale=w["scale"])
    return o, final


def _check(w, fast=False):
    m = w["_meta"]
    backing = m["backing"]
    before = backing.clone()
    exp_o, exp_final = _oracle_workload(w, fast)
    g_cum, A, o, none, final = _run_workload(w)
    torch.cuda.synchronize()
    assert none is None and o.shape == (1, m["T"], m["HV"], 128) and o.dtype == w["packed_qkv"].dtype
    torch.testing.assert_close(o[0].cpu().float(), exp_o.float(), atol=2e-2, rtol=2e-2)
    idx = w["initial_state_indices"].cpu().tolist()
    worst = max(rel_l2(final[n], exp_final[n]) for n in range(len(idx)))
    assert worst <= 1e-3, worst
    pool = w["initial_state"]
    for n, slot in enumerate(idx):
        assert torch.equal(pool[slot], final[n])               # final_state is the gathered pool rows
    untouched = torch.ones(pool.shape[0], dtype=torch.bool, device=pool.device)
    untouched[torch.tensor(idx, device=pool.device)] = False
    assert torch.equal(backing[untouched], before[untouched])
    tail = m["offsets"][-1]
    assert torch.count_nonzero(o[0, tail:]) == 0
    return worst


@pytest.mark.parametrize("lengths,tail_pad", [([64], 0), ([1], 0), ([17], 3), ([63, 65, 128], 0),
                                              ([200, 0, 33, 2049], 5), ([5555], 0)])
@pytest.mark.parametrize("H,HV", [(2, 4), (4, 4), (1, 3)])
def test_gdn_prefill_small(lengths, tail_pad, H, HV):
    from pla_amd.workloads import gdn_prefill_packed
    w = gdn_prefill_packed(lengths, H=H, HV=HV, pool_slots=len(lengths) + 3, seed=sum(lengths) + H, tail_pad=tail_pad)
    _check(w, fast=sum(lengths) > 3000)


def test_gdn_prefill_64_sequences_and_65_give_the_same_bits():
    """Calls of at most 64 whole sequences work their chunk tables out inside the kernels; with more sequences a
    table kernel runs first.  64 ragged sequences (empty ones among them, a padded tail, both staged - chains of
    unequal length - and unstaged) against the oracle, then the same tokens with one empty sequence appended (65
    sequences: the table kernel) must give the same bits in o, g_cum and the 64 states."""
    import random
    from pla_amd.workloads import gdn_prefill_packed
    rng = random.Random(5)
    for longest, H, HV in ((300, 1, 2), (2200, 2, 4)):          # 128 chains of few chunks; 256 chains, staged
        lengths = [rng.choice((0, 1, 63, 64, 65, 130, longest // 3)) for _ in range(64)]
        lengths[7] = longest
        lengths[63] = 77
        results = []
        _check(gdn_prefill_packed(lengths, H=H, HV=HV, pool_slots=70, seed=longest, tail_pad=9), fast=True)
        for extra in ([], [0]):
            w = gdn_prefill_packed(lengths + extra, H=H, HV=HV, pool_slots=70, seed=longest, tail_pad=9)
            if not extra:
                slots = w["initial_state_indices"]
            else:                                               # the same slots for the 64, a free one for the empty sequence
                free = (set(range(70)) - set(slots.cpu().tolist())).pop()
                w["initial_state_indices"] = torch.cat([slots, torch.tensor([free], dtype=slots.dtype, device=slots.device)])
            g_cum, _, o, _, final = _run_workload(w)
            torch.cuda.synchronize()
            results.append((o, g_cum.reshape(-1, HV)[:sum(lengths)], final[:64]))
        for x, y in zip(*results):
            assert torch.equal(x, y)


@pytest.mark.parametrize("lengths,tail_pad", [([17], 3), ([200, 0, 33, 2049], 5), ([5555], 0)])
def test_gdn_prefill_fp16_activations(lengths, tail_pad):
    """fp16 q / k / v / gates (the reference's FlashQLA takes both,
    src/prefill/flashqla/host/torch_extension_cute.cc:348-349): the oracle rounds the normalised q / k to fp16,
    as the kernel does; same tolerances as bf16."""
    from pla_amd.workloads import gdn_prefill_packed
    w = gdn_prefill_packed(lengths, H=2, HV=4, pool_slots=len(lengths) + 3, seed=7 + sum(lengths), tail_pad=tail_pad,
                           dtype=torch.float16)
    _check(w, fast=sum(lengths) > 3000)


def test_gdn_prefill_no_final_state_still_updates_pool_and_chained_calls():
    from pla_amd.workloads import gdn_prefill_packed
    from pla_amd.prefill.flashqla import gdn_prefill_packed_qkv_fwd
    w = gdn_prefill_packed([300], H=2, HV=4, pool_slots=4, seed=5)
    pool0 = w["initial_state"].clone()
    _, _, o_full, _, final_full = _run_workload(w)
    pool_full = w["initial_state"].clone()
    # output_final_state=False: same pool contents, no returned state
    w["initial_state"].copy_(pool0)
    _, _, o2, _, final2 = _run_workload(w, output_final_state=False)
    torch.cuda.synchronize()
    assert final2 is None and torch.equal(o2, o_full) and torch.equal(w["initial_state"], pool_full)
    # two chained calls (192 + 108 tokens, chunk aligned) == one call, bit for bit per chunk schedule
    w["initial_state"].copy_(pool0)
    parts = []
    for lo, hi in ((0, 192), (192, 300)):
        cu = torch.tensor([0, hi - lo], dtype=torch.int32, device="cuda")
        r = gdn_prefill_packed_qkv_fwd(w["packed_qkv"][lo:hi], w["raw_gate_a"][lo:hi], w["raw_beta_b"][lo:hi],
                                       w["A_log"], w["dt_bias"], cu, num_qk_heads=2, num_v_heads=4,
                                       scale=w["scale"], initial_state=w["initial_state"],
                                       initial_state_indices=w["initial_state_indices"])
        parts.append(r[2])
    torch.cuda.synchronize()
    assert torch.equal(torch.cat(parts, dim=1), o_full)
    assert torch.equal(w["initial_state"], pool_full)


def test_gdn_prefill_bf16_states():
    """A bf16 pool (or final_state_dtype=bf16) follows the reference's rule of one dtype for the incoming state,
    the pool and the returned state (pla/prefill/flashqla/ops.py:440-451): the states are widened to FP32, the
    FP32 result is rounded once, outputs equal the FP32-state call on the same (representable) values."""
    from pla_amd.workloads import gdn_prefill_packed
    w = gdn_prefill_packed([70, 0, 300], H=2, HV=4, pool_slots=6, seed=17)
    w["initial_state"].copy_(w["initial_state"].bfloat16().float())
    pool32 = w["initial_state"].clone()
    _, _, o32, _, final32 = _run_workload(w)
    after32 = w["initial_state"].clone()
    pool16 = pool32.bfloat16()
    w16 = dict(w, initial_state=pool16)
    _, _, o16, _, final16 = _run_workload(w16)
    torch.cuda.synchronize()
    assert final16.dtype == torch.bfloat16 and torch.equal(o16, o32)
    assert torch.equal(final16, final32.bfloat16()) and torch.equal(pool16, after32.bfloat16())
    # no incoming state, bf16 result requested
    call = {k: v for k, v in w.items() if not k.startswith("_") and k not in ("initial_state", "initial_state_indices")}
    from pla_amd.prefill.flashqla import gdn_prefill_packed_qkv_fwd
    packed = call.pop("packed_qkv")
    a, b, A, dt, cu = (call.pop(n) for n in ("raw_gate_a", "raw_beta_b", "A_log", "dt_bias", "cu_seqlens"))
    r32 = gdn_prefill_packed_qkv_fwd(packed, a, b, A, dt, cu, **call)
    r16 = gdn_prefill_packed_qkv_fwd(packed, a, b, A, dt, cu, final_state_dtype=torch.bfloat16, **call)
    torch.cuda.synchronize()
    assert torch.equal(r16[2], r32[2]) and torch.equal(r16[4], r32[4].bfloat16())
    with pytest.raises(ValueError, match="must match the initial_state dtype"):
        _run_workload(dict(w, final_state_dtype=torch.bfloat16))


def test_gdn_prefill_split_inputs_and_compact_state():
    """g / beta given explicitly, q/k already normalised, compact (non-indexed) state."""
    from pla_amd.prefill.flashqla import chunk_gated_delta_rule_fwd
    from oracle.prefill import token_recurrence
    g = torch.Generator().manual_seed(3)
    T, H, HV = 150, 2, 4
    q = l2norm(torch.randn(T, H, 128, generator=g)).bfloat16()
    k = l2norm(torch.randn(T, H, 128, generator=g)).bfloat16()
    v = torch.randn(T, HV, 128, generator=g).bfloat16()
    gate = -torch.rand(T, HV, generator=g) * 0.3
    beta = torch.rand(T, HV, generator=g)
    S0 = torch.randn(2, HV, 128, 128, generator=g) * 0.1
    offs = [0, 50, 150]
    exp_o, exp_final = token_recurrence(q, k, v, gate, beta, offs, S0, scale=128 ** -0.5)
    dev = "cuda"
    cu = torch.tensor(offs, dtype=torch.int32, device=dev)
    g_cum, A, o, _, final = chunk_gated_delta_rule_fwd(
        q[None].to(dev), k[None].to(dev), v[None].to(dev), gate[None].to(dev), beta[None].to(dev),
        initial_state=S0.to(dev), cu_seqlens=cu)
    torch.cuda.synchronize()
    torch.testing.assert_close(o[0].cpu().float(), exp_o, atol=2e-2, rtol=2e-2)
    assert max(rel_l2(final[n], exp_final[n]) for n in range(2)) <= 1e-3
    # chunk-local cumulative gate resets at every chunk and sequence start
    want = torch.cat([gate[0:50].cumsum(0), gate[50:114].cumsum(0), gate[114:150].cumsum(0)])
    torch.testing.assert_close(g_cum[0].cpu(), want, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("offs", [[0, 130, 130, 700], [0, 2300, 2300, 2600]])
def test_gdn_prefill_without_normalisation_on_a_poisoned_workspace_fused_sweep(offs):
    """normalize_qk=False (several chunks; whole sequences, and - the second case - a call split into segments, whose
    first sweep copies the K rows the preparation stored): the preparation then writes no 1 / |k| factors, and the
    sweeps must not read them (the workspace holds NaN)."""
    from pla_amd.prefill.flashqla import chunk_gated_delta_rule_fwd
    from oracle.prefill import token_recurrence
    g = torch.Generator().manual_seed(11)
    T, H, HV = offs[-1], 2, 4
    q = l2norm(torch.randn(T, H, 128, generator=g)).bfloat16()
    k = l2norm(torch.randn(T, H, 128, generator=g)).bfloat16()
    v = torch.randn(T, HV, 128, generator=g).bfloat16()
    gate = -torch.rand(T, HV, generator=g) * 0.3
    beta = torch.rand(T, HV, generator=g)
    S0 = torch.randn(3, HV, 128, 128, generator=g) * 0.1
    exp_o, exp_final = token_recurrence(q, k, v, gate, beta, offs, S0, scale=128 ** -0.5)
    dev = "cuda"
    cu = torch.tensor(offs, dtype=torch.int32, device=dev)
    _, _, o, _, final = chunk_gated_delta_rule_fwd(
        q[None].to(dev), k[None].to(dev), v[None].to(dev), gate[None].to(dev), beta[None].to(dev),
        initial_state=S0.to(dev), cu_seqlens=cu)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all() and torch.isfinite(final).all()
    torch.testing.assert_close(o[0].cpu().float(), exp_o, atol=2e-2, rtol=2e-2)
    assert max(rel_l2(final[n], exp_final[n]) for n in range(3)) <= 1e-3


@pytest.mark.parametrize("seed,tokens", [(348, 32810), (303, 41582)])
def test_config3_gdn_prefill_32k_varlen(seed, tokens):
    """Config 3 at full size.  Seed 348 is the workload bench.py times (32 810 tokens, its lengths sum closest to
    32K); seed 303 is a second draw of the same distribution with longer sequences."""
    from pla_amd.workloads import gdn_prefill_packed, ragged_lengths
    lengths = ragged_lengths(8, 512, 8192, seed=seed)
    assert sum(lengths) == tokens
    w = gdn_prefill_packed(lengths, H=16, HV=32, pool_slots=64, seed=seed)
    _check(w, fast=True)


@pytest.mark.parametrize("lengths,tail_pad,H,HV", [([2500, 0, 1111, 40], 5, 1, 2), ([4096], 0, 2, 2), ([1030, 2049], 0, 1, 4),
                                                    ([16384], 0, 16, 32)])
def test_gdn_prefill_split_sequences_match_oracle(lengths, tail_pad, H, HV):
    """Calls with few (sequence, head) chains and long sequences are split into 16-chunk segments that
    are swept concurrently (zero-state and identity sweeps, a combine step, a second sweep): ragged
    lengths, an empty sequence, a sequence shorter than one segment, indexed pool, against the oracle.  The last case is
    the reference report's single 16 384-token sequence of 32 value heads (8 segments of 32 chunks per head)."""
    from pla_amd import _lib
    from pla_amd.workloads import gdn_prefill_packed
    T, N = sum(lengths) + tail_pad, len(lengths)
    size = _lib.load().pla_gdn_prefill_workspace_bytes
    unsplit_per_head = size(T, N, 65 * H, 65 * HV) / (65 * HV)      # more than 64 chains are never split
    assert size(T, N, H, HV) > 1.1 * HV * unsplit_per_head           # so this call carries the segment buffers
    w = gdn_prefill_packed(lengths, H=H, HV=HV, pool_slots=N + 3, seed=99 + T, tail_pad=tail_pad)
    _check(w, fast=True)


def test_gdn_prefill_staged_pipeline_matches_oracle_and_unstaged_bits():
    """With at least 128 chains and 16 chunks per sequence on average the preparation and the sweep
    are pipelined in stages on two streams.  Ragged lengths with an empty sequence and sequences
    shorter than the number of stages (empty stages), against the oracle; and the same tokens run
    sequence by sequence (too few chains to be staged) give bit-identical o and states."""
    from pla_amd.workloads import gdn_prefill_packed
    from pla_amd.prefill.flashqla import gdn_prefill_packed_qkv_fwd
    lengths = [3000, 0, 70, 1500, 64, 2100, 1, 1500]
    H, HV = 4, 16
    w = gdn_prefill_packed(lengths, H=H, HV=HV, pool_slots=len(lengths) + 3, seed=777, tail_pad=7)
    pool0 = w["initial_state"].clone()
    _check(w, fast=True)
    # rerun staged on a fresh pool, keep o and pool
    w["initial_state"].copy_(pool0)
    _, _, o_staged, _, _ = _run_workload(w)
    pool_staged = w["initial_state"].clone()
    # one call per sequence: 16 chains each, never staged; the long ones are split into segments, so
    # only the short sequences (a single segment) are compared bit for bit
    w["initial_state"].copy_(pool0)
    offs = w["_meta"]["offsets"]
    idx = w["initial_state_indices"]
    for n, length in enumerate(lengths):
        if length == 0 or length >= 2048:
            continue
        lo, hi = offs[n], offs[n + 1]
        cu = torch.tensor([0, hi - lo], dtype=torch.int32, device="cuda")
        r = gdn_prefill_packed_qkv_fwd(w["packed_qkv"][lo:hi], w["raw_gate_a"][lo:hi], w["raw_beta_b"][lo:hi],
                                       w["A_log"], w["dt_bias"], cu, num_qk_heads=H, num_v_heads=HV, scale=w["scale"],
                                       initial_state=w["initial_state"], initial_state_indices=idx[n:n + 1])
        torch.cuda.synchronize()
        assert torch.equal(r[2][0], o_staged[0, lo:hi]), n
        slot = int(idx[n])
        assert torch.equal(w["initial_state"][slot], pool_staged[slot]), n


def test_gdn_prefill_equal_lengths_collapse_the_stages():
    """Chains of (nearly) equal length leave no idle CUs for a later preparation to hide on: the table kernel then
    puts every chunk into the first stage and the launches of the second find nothing to do.  Against the oracle,
    with initial states and final states through the pool (which the first stage now writes itself)."""
    from pla_amd.workloads import gdn_prefill_packed
    for lengths in ([1100] * 8, [1100, 1090, 1150, 1100, 1024, 1100, 1120, 1100]):
        w = gdn_prefill_packed(lengths, H=4, HV=16, pool_slots=len(lengths) + 3, seed=4242, tail_pad=3)
        _check(w, fast=True)
    # either side of the rule (one stage when the chunks fill at least 80 % of sequences x longest chain):
    # 154 of 8 x 24 chunks -> one stage, 153 -> two
    for lengths in ([1530, 1536, 1530, 1536, 955, 960, 890, 896], [1530, 1536, 1530, 1536, 955, 896, 890, 896]):
        chunks = sum((n + 63) // 64 for n in lengths)
        assert (5 * chunks < 4 * 8 * 24) == (chunks == 153)
        w = gdn_prefill_packed(lengths, H=4, HV=16, pool_slots=len(lengths) + 3, seed=chunks)
        _check(w, fast=True)


def test_gdn_prefill_with_and_without_host_offsets_gives_the_same_bits():
    """With ``raw_cu_seqlens`` the host applies the device's one-stage rule itself and enqueues nothing for a second
    stage; without it the device collapses the stages.  Both must give the same bits, on either side of the rule, for
    ragged lengths (staged either way) and through both host layers."""
    from pla_amd.prefill.flashqla import ops
    from pla_amd.workloads import gdn_prefill_packed
    for lengths in ([1100] * 8, [1530, 1536, 1530, 1536, 955, 960, 890, 896], [1530, 1536, 1530, 1536, 955, 896, 890, 896],
                    [2600, 300, 1900, 64, 0, 777, 1500, 2200]):
        results = []
        for native in (False, True):
            for with_raw in (True, False):
                ops._native = None if native else False
                w = gdn_prefill_packed(lengths, H=4, HV=16, pool_slots=len(lengths) + 3, seed=99)
                if not with_raw:
                    w["raw_cu_seqlens"] = None
                g_cum, _, o, _, final = _run_workload(w)
                torch.cuda.synchronize()
                results.append((o, g_cum.reshape(-1, 16)[:sum(lengths)], final))
        ops._native = False
        for other in results[1:]:
            for x, y in zip(results[0], other):
                assert torch.equal(x, y), lengths


@pytest.mark.parametrize("lengths,H,HV,halved,dtype", [
    ([3000, 2600, 300, 64, 0, 777, 500, 200, 900, 400], 8, 16, 1, torch.bfloat16),       # one sweep (not staged)
    ([4000, 3500, 500, 1000, 1500], 16, 32, 1, torch.bfloat16),                         # two stages: the second sweep
    ([2000, 100, 200, 300, 2000, 64, 1, 0, 500], 16, 16, 2, torch.float16),             # as many value heads as q/k heads
    ([1800, 1750, 100, 64, 0, 300, 200, 150, 400, 130, 77], 4, 12, 2, torch.bfloat16),  # three value heads per q/k head
    ([900, 100, 1500, 64, 0, 300, 2000, 150, 400, 130, 77, 700], 16, 32, 1, torch.bfloat16),     # more chains than CUs: longest first
    ([1000, 1000, 1000, 990, 1010, 1000, 1000, 1000, 1000], 16, 32, 0, torch.bfloat16),          # the same without halves
])
def test_gdn_prefill_longest_sequences_swept_as_halves(lengths, H, HV, halved, dtype):
    """Ragged whole sequences with more than 128 chains and the offsets on the host: the last sweep runs the chains
    of the longest sequences as two workgroups of 64 V columns each (the plan is host arithmetic and is asked for
    here); with more chains than CUs every sweep also starts its chains longest first.  Against the oracle, and bit for bit against the call without host offsets, which sweeps every chain
    whole."""
    import ctypes
    from pla_amd import _lib
    from pla_amd.workloads import gdn_prefill_packed
    offs = [0]
    for n in lengths:
        offs.append(offs[-1] + n)
    plan = _lib.load().pla_gdn_prefill_halved_sequences((ctypes.c_int32 * len(offs))(*offs), len(lengths), offs[-1] + 5, H, HV)
    assert plan == halved
    results = []
    for with_raw in (True, False):
        w = gdn_prefill_packed(lengths, H=H, HV=HV, pool_slots=len(lengths) + 3, seed=4711, tail_pad=5, dtype=dtype)
        assert w["raw_cu_seqlens"] == tuple(offs)
        if with_raw:
            _check(w, fast=True)
            w = gdn_prefill_packed(lengths, H=H, HV=HV, pool_slots=len(lengths) + 3, seed=4711, tail_pad=5, dtype=dtype)
        else:
            w["raw_cu_seqlens"] = None
        g_cum, _, o, _, final = _run_workload(w)
        torch.cuda.synchronize()
        results.append((o, g_cum.reshape(-1, HV)[:offs[-1]], final, w["initial_state"]))
    for x, y in zip(*results):
        assert torch.equal(x, y)


@pytest.mark.parametrize("lengths,H,HV", [([1500, 2100, 900, 1500, 1300, 1100, 700, 1200], 4, 16), ([2600, 70], 2, 4),
                                          ([4000, 3500, 500, 1000, 1500], 8, 32)])
def test_gdn_prefill_staged_pipeline_in_a_graph(lengths, H, HV):
    """The staged call forks to a side stream and joins again, so it can be captured: three replays with
    eager work and synchronisation in between reproduce the eager result bit for bit.  The second case is a call
    split into segments (two sweeps and the combine step, tables written by the preparation's appended workgroup),
    the third a staged call whose last sweep runs the chains of its longest sequence as two workgroups each."""
    from pla_amd.workloads import gdn_prefill_packed
    w = gdn_prefill_packed(lengths, H=H, HV=HV, pool_slots=len(lengths) + 2, seed=31)
    pool0 = w["initial_state"].clone()
    _, _, o_eager, _, _ = _run_workload(w, output_final_state=False)
    torch.cuda.synchronize()
    pool_eager = w["initial_state"].clone()
    w["initial_state"].copy_(pool0)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        _run_workload(w, output_final_state=False)            # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    w["initial_state"].copy_(pool0)
    with torch.cuda.graph(graph, stream=stream):
        _, _, o_graph, _, _ = _run_workload(w, output_final_state=False)
    for replay in range(3):
        w["initial_state"].copy_(pool0)
        o_graph.zero_()
        scratch = torch.randn(1 << 20, device="cuda").sum().item()     # eager work and a sync between replays
        graph.replay()
        torch.cuda.synchronize()
        assert scratch == scratch
        assert torch.equal(o_graph, o_eager), replay
        assert torch.equal(w["initial_state"], pool_eager), replay


def test_gdn_prefill_twenty_staged_calls_in_one_graph():
    """One capture holding more staged calls than the library keeps side streams (a model with twenty GDN layers):
    a side stream that has joined a capture is taken again by the later calls of that capture.  The calls chain on
    one pool, so every call's result depends on all calls before it; three replays reproduce the eager chain bit
    for bit."""
    from pla_amd.workloads import gdn_prefill_packed
    lengths = [1500, 2100, 900, 1500, 1300, 1100, 700, 1200]
    layers = 20
    w = gdn_prefill_packed(lengths, H=4, HV=16, pool_slots=len(lengths) + 2, seed=77)
    pool0 = w["initial_state"].clone()
    o_eager = [_run_workload(w, output_final_state=False)[2] for _ in range(layers)]
    torch.cuda.synchronize()
    pool_eager = w["initial_state"].clone()
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    w["initial_state"].copy_(pool0)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=stream):
        o_graph = [_run_workload(w, output_final_state=False)[2] for _ in range(layers)]
    for replay in range(3):
        w["initial_state"].copy_(pool0)
        for o in o_graph:
            o.zero_()
        scratch = torch.randn(1 << 20, device="cuda").sum().item()     # eager work and a sync between replays
        graph.replay()
        torch.cuda.synchronize()
        assert scratch == scratch
        for layer in range(layers):
            assert torch.equal(o_graph[layer], o_eager[layer]), (replay, layer)
        assert torch.equal(w["initial_state"], pool_eager), replay
    # an eager call afterwards finds a side stream again (the capture has ended)
    w["initial_state"].copy_(pool0)
    o_after = _run_workload(w, output_final_state=False)[2]
    torch.cuda.synchronize()
    assert torch.equal(o_after, o_eager[0])


@pytest.mark.parametrize("lengths", [[130, 0, 77], [2100, 40]])
def test_gdn_prefill_rows_aligned_to_4_bytes_only(lengths):
    """A packed Q|K|V view whose rows start 4 bytes into a 16-byte piece: the library copies such q and k rows into
    dense buffers of its workspace before its kernels read them, v (copied to LDS in 16-byte pieces) is materialised
    by the facade; the results equal those of the aligned buffer (bit for bit: the same kernels run on the same
    values) and the oracle's.  Whole sequences and (the second case) a call split into segments."""
    from pla_amd.prefill.flashqla import gdn_prefill_packed_qkv_fwd
    from pla_amd.workloads import gdn_prefill_packed
    outs = []
    for shifted in (False, True):
        w = gdn_prefill_packed(lengths, H=2, HV=4, pool_slots=6, seed=23)
        call = {k: v for k, v in w.items() if not k.startswith("_")}
        packed = call.pop("packed_qkv")
        if shifted:
            T, width = packed.shape
            wide = torch.zeros(T, width + 6, dtype=packed.dtype, device=packed.device)
            wide[:, 2:2 + width] = packed
            packed = wide[:, 2:2 + width]
            assert packed.data_ptr() % 8 == 4 and packed.stride(0) % 4 == 2
        a, b, A, dt, cu = (call.pop(n) for n in ("raw_gate_a", "raw_beta_b", "A_log", "dt_bias", "cu_seqlens"))
        g_cum, _, o, _, final = gdn_prefill_packed_qkv_fwd(packed, a, b, A, dt, cu, **call)
        torch.cuda.synchronize()
        outs.append((o.float().cpu(), final.cpu()))
    assert torch.equal(outs[1][0], outs[0][0]) and torch.equal(outs[1][1], outs[0][1])
    w = gdn_prefill_packed(lengths, H=2, HV=4, pool_slots=6, seed=23)
    exp_o, exp_final = _oracle_workload(w, fast=sum(lengths) > 1000)
    torch.testing.assert_close(outs[1][0][0], exp_o.float(), atol=2e-2, rtol=2e-2)


def _correlated_keys(w, noise, seed=5):
    """Keys = one direction per head plus `noise` x N(0, 1), beta = 0.982, log-decay of a few 1e-3 per token."""
    m = w["_meta"]
    T, H = m["T"], m["H"]
    g = torch.Generator().manual_seed(seed)
    base = torch.randn(1, H, 128, generator=g)
    k = base + noise * torch.randn(T, H, 128, generator=g)
    packed = w["packed_qkv"].cpu().clone()
    packed[:, H * 128: 2 * H * 128] = k.reshape(T, -1).to(packed.dtype)
    w["packed_qkv"] = packed.to(w["packed_qkv"].device)
    w["raw_beta_b"] = torch.full_like(w["raw_beta_b"], 4.0)
    w["raw_gate_a"] = torch.full_like(w["raw_gate_a"], -6.0)
    return w


@pytest.mark.parametrize("lengths,noise", [([200, 131], 0.1), ([1000, 700], 0.1), ([640], 0.03)])
def test_gdn_prefill_correlated_keys_dense_triangular_system(lengths, noise):
    """Keys that nearly repeat, beta near 1 and a slow decay: every entry of the chunk's triangular system I + L is
    of order one, so the off-diagonal blocks of its inverse (formed on MFMA from hi/lo operand pairs) carry the
    result, U = W X cancels heavily, and each token overwrites what the state holds along the shared direction: the
    final state is the work of the last few tokens and operand roundings show unaveraged.  W and the U of the state
    update therefore travel as fp16 hi + lo pairs (single fp16 operands measure 1.0e-3 .. 3.5e-3 on these cases,
    the pairs 2.5e-4 .. 2.7e-4 in a float64 simulation of the rounding points); the bounds are the usual ones."""
    from pla_amd.workloads import gdn_prefill_packed
    w = _correlated_keys(gdn_prefill_packed(lengths, H=2, HV=4, pool_slots=5, seed=41 + len(lengths)), noise)
    exp_o, exp_final = _oracle_workload(w, fast=sum(lengths) > 600)
    g_cum, A, o, _, final = _run_workload(w)
    torch.cuda.synchronize()
    torch.testing.assert_close(o[0].cpu().float(), exp_o.float(), atol=2e-2, rtol=2e-2)
    worst = max(rel_l2(final[n], exp_final[n]) for n in range(len(lengths)))
    print("correlated keys", lengths, noise, "state rel-L2 %.3e" % worst)
    assert worst <= 1e-3, worst


def test_gdn_prefill_operands_beyond_the_fp16_range_stay_finite():
    """|v| around 1e5 and an incoming state of the same size are beyond what the fp16 MFMA operands hold (65504; a
    bf16 pipeline would carry them).  The operand roundings saturate instead of producing infinities: the output and
    the state stay finite and of the inputs' order of magnitude (|o| and |S| below 64 x the largest input), and a
    sequence of ordinary magnitude in the same call is unaffected (usual bounds)."""
    from pla_amd.workloads import gdn_prefill_packed
    lengths = [150, 90]
    w = gdn_prefill_packed(lengths, H=2, HV=4, pool_slots=4, seed=77)
    offs = w["_meta"]["offsets"]
    exp_o, exp_final = _oracle_workload(w)
    packed = w["packed_qkv"].clone()
    H = 2
    packed[offs[0]:offs[1], 2 * H * 128:] = (packed[offs[0]:offs[1], 2 * H * 128:].float() * 1e5).to(packed.dtype)
    w["packed_qkv"] = packed
    slot0 = int(w["initial_state_indices"][0])
    w["initial_state"][slot0] *= 1e6                      # N(0, 0.1) -> magnitudes around 1e5
    big = float(max(packed[offs[0]:offs[1], 2 * H * 128:].float().abs().max(), w["initial_state"][slot0].abs().max()))
    g_cum, A, o, _, final = _run_workload(w)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all() and torch.isfinite(final).all()
    assert float(o[0, offs[0]:offs[1]].float().abs().max()) <= 64 * big and float(final[0].abs().max()) <= 64 * big
    torch.testing.assert_close(o[0, offs[1]:offs[2]].cpu().float(), exp_o[offs[1]:offs[2]].float(), atol=2e-2, rtol=2e-2)
    assert rel_l2(final[1], exp_final[1]) <= 1e-3


def test_gdn_prefill_staged_calls_from_two_threads_on_two_streams():
    """Two host threads, each on a stream of its own, enqueue staged calls (fork to a side stream, join again) at
    the same time: every call takes a side stream and events of its own for the time it enqueues, so neither waits
    on the other's events nor reads workspace tiles that are not prepared yet.  Each thread's results equal, bit
    for bit, what the same call gives when it runs alone."""
    import threading
    from pla_amd.workloads import gdn_prefill_packed
    works = [gdn_prefill_packed([1500, 2100, 900, 1500, 1300, 1100, 700, 1200], H=4, HV=16, pool_slots=10, seed=31),
             gdn_prefill_packed([2300, 1700, 1100, 1900, 1600, 1250, 1800, 1400], H=4, HV=16, pool_slots=10, seed=32)]
    pools = [w["initial_state"].clone() for w in works]
    alone = []
    for w in works:
        _, _, o, _, _ = _run_workload(w, output_final_state=False)
        torch.cuda.synchronize()
        alone.append((o.clone(), w["initial_state"].clone()))
    rounds = 6
    errors = []
    start = threading.Barrier(2)

    def worker(i):
        try:
            stream = torch.cuda.Stream()
            w, pool0 = works[i], pools[i]
            with torch.cuda.stream(stream):
                start.wait()
                for _ in range(rounds):
                    w["initial_state"].copy_(pool0)
                    _, _, o, _, _ = _run_workload(w, output_final_state=False)
                    stream.synchronize()
                    if not (torch.equal(o, alone[i][0]) and torch.equal(w["initial_state"], alone[i][1])):
                        errors.append(i)
        except Exception as exc:          # surfaced in the main thread
            errors.append(repr(exc))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
