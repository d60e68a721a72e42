"""GPU parity of the KDA chunk-64 prefill against the CPU oracle, plus the reference's closed-form
scenarios (tests/test_kda_prefill_flashkdapro.py:243-357) evaluated on the GPU path."""
import pytest
import torch

from helpers import rel_l2
from oracle import kda_prefill_reference, chunked_delta_rule_fp64, lower_bound_gate, sigmoid_beta, l2norm

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def poisoned_workspace(monkeypatch):
    """Every call of this file gets a workspace of 0xFF bytes (NaN as FP32 and as fp16), so a kernel that reads a
    workspace word no kernel of the same call has written turns its results into NaN."""
    from pla_amd.prefill.flashkdapro import ops

    def workspace(T, N, H, device):
        from pla_amd import _lib
        nbytes = _lib.load().pla_kda_prefill_workspace_bytes(T, N, H)
        return torch.full((nbytes,), 0xFF, dtype=torch.uint8, device=device), nbytes
    monkeypatch.setattr(ops, "_workspace", workspace)
    # the facade's own path allocates through _workspace; the compiled host layer (which allocates by itself) is
    # switched off here and compared with this path bit for bit in tests/test_drop_in_imports.py
    monkeypatch.setattr(ops, "_native", False)


def _inputs(lengths, H, seed, pad=0, gate_scale=1.0):
    g = torch.Generator().manual_seed(seed)
    T = sum(lengths) + pad
    q = torch.randn(T, H, 128, generator=g).bfloat16()
    k = torch.randn(T, H, 128, generator=g).bfloat16()
    v = torch.randn(T, H, 128, generator=g).bfloat16()
    raw = (torch.randn(T, H, 128, generator=g) * gate_scale).bfloat16()
    beta = torch.randn(T, H, generator=g).bfloat16()
    A_log = torch.randn(H, generator=g) * 0.5
    dt_bias = torch.randn(H, 128, generator=g) * 0.5
    offs = [0]
    for n in lengths:
        offs.append(offs[-1] + n)
    S0 = torch.randn(len(lengths), H, 128, 128, generator=g) * 0.1
    return q, k, v, raw, beta, A_log, dt_bias, offs, S0


def _oracle(q, k, v, raw, beta, A_log, dt_bias, offs, S0, fast):
    if not fast:
        return kda_prefill_reference(q, k, v, raw, beta, A_log, dt_bias, offs, S0)
    qn, kn = l2norm(q).to(q.dtype), l2norm(k).to(k.dtype)
    gate = lower_bound_gate(raw, dt_bias, A_log, -5.0)
    b = sigmoid_beta(beta)
    T, H = q.shape[0], q.shape[1]
    o = torch.zeros(T, H, 128, dtype=torch.float64)
    final = S0.double().clone()
    for n in range(len(offs) - 1):
        lo, hi = offs[n], offs[n + 1]
        if hi > lo:
            o[lo:hi], final[n] = chunked_delta_rule_fp64(qn[lo:hi], kn[lo:hi], v[lo:hi], gate[lo:hi], b[lo:hi],
                                                         S0[n], scale=128 ** -0.5)
    return o, final


@pytest.mark.parametrize("lengths,pad", [([64], 0), ([1], 0), ([17], 3), ([63, 65, 128], 0), ([0, 17, 300], 2),
                                         ([2049], 0)])
@pytest.mark.parametrize("H", [2, 4])
def test_kda_prefill_small(lengths, pad, H):
    from pla_amd.prefill.flashkdapro import flashkda_fwd
    q, k, v, raw, beta, A_log, dt_bias, offs, S0 = _inputs(lengths, H, seed=sum(lengths) + H, pad=pad)
    exp_o, exp_final = _oracle(q, k, v, raw, beta, A_log, dt_bias, offs, S0, fast=sum(lengths) > 1000)
    dev = "cuda"
    cu = torch.tensor(offs, dtype=torch.int32, device=dev)
    out = torch.full((q.shape[0], H, 128), 7.0, dtype=torch.bfloat16, device=dev)
    init = S0.to(dev)
    init_before = init.clone()
    final = torch.empty_like(init)
    args = [t.to(dev) for t in (q, k, v, raw, beta, A_log, dt_bias)]
    assert flashkda_fwd(*args, out, initial_state=init, final_state=final, cu_seqlens=cu) is None
    torch.cuda.synchronize()
    torch.testing.assert_close(out.cpu().float(), exp_o.float(), atol=2e-2, rtol=2e-2)
    worst = max(rel_l2(final[n], exp_final[n]) for n in range(len(lengths)))
    assert worst <= 1e-3, worst
    assert torch.equal(init, init_before)                        # read-only initial state
    assert torch.count_nonzero(out[offs[-1]:]) == 0              # padded suffix zeroed
    # final_state=None must not change out
    out2 = torch.full_like(out, 9.0)
    flashkda_fwd(*args, out2, initial_state=init, final_state=None, cu_seqlens=cu)
    # indexed pool == compact states, unmapped slots untouched
    slots = len(lengths) + 4
    idx = torch.tensor(list(range(len(lengths) + 1, 1, -1))[:len(lengths)], dtype=torch.int32, device=dev)
    pool = torch.full((slots, H, 128, 128), 11.0, device=dev)
    pool[idx.long()] = init
    before = pool.clone()
    out3 = torch.full_like(out, 13.0)
    flashkda_fwd(*args, out3, state_pool=pool, state_indices=idx, cu_seqlens=cu)
    torch.cuda.synchronize()
    assert torch.equal(out2, out) and torch.equal(out3, out)
    assert torch.equal(pool[idx.long()], final)
    untouched = [i for i in range(slots) if i not in idx.cpu().tolist()]
    assert torch.equal(pool[untouched], before[untouched])


def test_kda_prefill_bf16_and_strided_states():
    """States may be bf16 or arbitrarily strided (pla/prefill/flashkdapro/ops.py:104-118 of the reference): they
    are staged through dense FP32 copies, so the outputs equal the FP32-state call bit for bit when the bf16
    initial state holds the same values, and the final state is the FP32 result rounded once."""
    from pla_amd.prefill.flashkdapro import flashkda_fwd
    lengths, H, dev = [0, 17, 300], 2, "cuda"
    q, k, v, raw, beta, A_log, dt_bias, offs, S0 = _inputs(lengths, H, seed=91, pad=2)
    S0 = S0.bfloat16().float()                                   # representable in both dtypes
    cu = torch.tensor(offs, dtype=torch.int32, device=dev)
    args = [t.to(dev) for t in (q, k, v, raw, beta, A_log, dt_bias)]
    out32 = torch.empty(q.shape[0], H, 128, dtype=torch.bfloat16, device=dev)
    fin32 = torch.empty(len(lengths), H, 128, 128, device=dev)
    flashkda_fwd(*args, out32, initial_state=S0.to(dev), final_state=fin32, cu_seqlens=cu)
    # bf16 states
    out16 = torch.empty_like(out32)
    init16 = S0.to(dev).bfloat16()
    fin16 = torch.full((len(lengths), H, 128, 128), 5.0, dtype=torch.bfloat16, device=dev)
    flashkda_fwd(*args, out16, initial_state=init16, final_state=fin16, cu_seqlens=cu)
    torch.cuda.synchronize()
    assert torch.equal(out16, out32) and torch.equal(fin16, fin32.bfloat16())
    # a bf16 pool with a padded slot pitch, updated in place at the indexed slots only
    backing = torch.full((6, H * 128 * 128 + 24), 3.0, dtype=torch.bfloat16, device=dev)
    pool = backing[:, 8:8 + H * 128 * 128].view(6, H, 128, 128)
    idx = torch.tensor([4, 1, 3], dtype=torch.int32, device=dev)
    pool[idx.long()] = init16
    before = backing.clone()
    outp = torch.empty_like(out32)
    flashkda_fwd(*args, outp, state_pool=pool, state_indices=idx, cu_seqlens=cu)
    torch.cuda.synchronize()
    assert torch.equal(outp, out32) and torch.equal(pool[idx.long()], fin32.bfloat16())
    untouched = torch.ones_like(backing, dtype=torch.bool)
    untouched[idx.long(), 8:8 + H * 128 * 128] = False
    assert torch.equal(backing[untouched], before[untouched])
    # transposed FP32 states (strided V / K axes)
    init_t = S0.to(dev).transpose(2, 3).contiguous().transpose(2, 3)
    fin_t = torch.empty(len(lengths), H, 128, 128, device=dev).transpose(2, 3)
    outt = torch.empty_like(out32)
    flashkda_fwd(*args, outt, initial_state=init_t, final_state=fin_t, cu_seqlens=cu)
    torch.cuda.synchronize()
    assert torch.equal(outt, out32) and torch.equal(fin_t, fin32)
    with pytest.raises(ValueError, match="same dtype"):
        flashkda_fwd(*args, outt, initial_state=init16, final_state=fin32, cu_seqlens=cu)


@pytest.mark.parametrize("scenario", ["initial_bits", "weak_decay", "small_update", "fresh_update"])
def test_kda_prefill_closed_forms(scenario):
    from pla_amd.prefill.flashkdapro import flashkda_fwd
    heads, dim, dev = 4, 128, "cuda"
    lengths = [0, 1, 17] if scenario == "initial_bits" else [0, 17, 4099]
    offs = [0]
    for n in lengths:
        offs.append(offs[-1] + n)
    total = offs[-1]
    q = torch.zeros(total + 3, heads, dim, dtype=torch.bfloat16, device=dev)
    q[..., 0] = 1
    k, v = torch.zeros_like(q), torch.zeros_like(q)
    updating = scenario in ("small_update", "fresh_update")
    if updating:
        k[..., 0] = 1
        v.fill_(1)
    raw_value = -12.0 if scenario == "weak_decay" else -100.0
    raw = torch.full_like(q, raw_value)
    beta = torch.full((total + 3, heads), -12.0, dtype=q.dtype, device=dev)
    a_log = torch.zeros(heads, device=dev)
    dt_bias = torch.zeros(heads, dim, device=dev)
    h0 = torch.linspace(-0.25, 0.25, len(lengths) * heads * dim * dim).reshape(len(lengths), heads, dim, dim)
    if updating:
        h0.zero_()
        if scenario == "small_update":
            h0[..., 0] = 0.1253
    h0_before = h0.clone()
    h0 = h0.to(dev)
    initial = None if scenario == "fresh_update" else h0
    cu = torch.tensor(offs, dtype=torch.int32, device=dev)
    out = torch.full_like(q, 7)
    final = torch.empty_like(h0)
    flashkda_fwd(q, k, v, raw, beta, a_log, dt_bias, out, initial_state=initial, final_state=final,
                 cu_seqlens=cu, raw_cu_seqlens=tuple(offs))
    torch.cuda.synchronize()
    assert torch.count_nonzero(out[total:]) == 0
    if scenario == "initial_bits":
        assert torch.equal(final.cpu(), h0_before)              # identity recurrence keeps every bit
    gg = -5.0 * torch.sigmoid(torch.tensor(raw_value, dtype=torch.float64))
    b = torch.sigmoid(torch.tensor(-12.0, dtype=torch.float64))
    decay = gg.exp()
    rec = decay * (1 - b) if updating else decay
    for seq, length in enumerate(lengths):
        start = h0_before[seq].double() if scenario != "fresh_update" else torch.zeros(heads, dim, dim, dtype=torch.float64)
        end = start * decay.pow(length)
        steps = torch.arange(1, length + 1, dtype=torch.float64)
        values = rec.pow(steps)[:, None, None] * start[..., 0]
        if updating:
            values = values + (b * (-torch.expm1(steps * rec.log())) / (1 - rec))[:, None, None]
            end[..., 0] = rec.pow(length) * start[..., 0] + b * (-torch.expm1(length * rec.log())) / (1 - rec)
        want = values * dim ** -0.5
        for head in range(heads):
            d = final[seq, head].cpu().double() - end[head]
            rms = float(d.square().mean().sqrt()); ref = float(end[head].square().mean().sqrt())
            assert (rms / ref if ref > 0 else rms) <= 1e-3 or float(d.abs().max()) <= 1e-6, (seq, head, rms, ref)
            if length:
                got = out[offs[seq]:offs[seq + 1], head].cpu().double()
                d = got - want[:, head]
                rms = float(d.square().mean().sqrt()); ref = float(want[:, head].square().mean().sqrt())
                assert (rms / ref if ref > 0 else rms) <= 0.01 or float(d.abs().max()) <= 1e-6, (seq, head, rms, ref)


def test_kda_prefill_two_chained_calls_equal_one():
    from pla_amd.prefill.flashkdapro import flashkda_fwd
    q, k, v, raw, beta, A_log, dt_bias, offs, S0 = _inputs([320], 2, seed=77)
    dev = "cuda"
    args = [t.to(dev) for t in (q, k, v, raw, beta)]
    A_log, dt_bias = A_log.to(dev), dt_bias.to(dev)
    out = torch.empty(320, 2, 128, dtype=torch.bfloat16, device=dev)
    final = torch.empty(1, 2, 128, 128, device=dev)
    flashkda_fwd(*args, A_log, dt_bias, out, initial_state=S0.to(dev), final_state=final)
    carry = S0.to(dev)
    parts = []
    for lo, hi in ((0, 128), (128, 320)):
        part = torch.empty(hi - lo, 2, 128, dtype=torch.bfloat16, device=dev)
        nxt = torch.empty_like(carry)
        flashkda_fwd(*(t[lo:hi] for t in args), A_log, dt_bias, part, initial_state=carry, final_state=nxt)
        parts.append(part)
        carry = nxt
    torch.cuda.synchronize()
    assert torch.equal(torch.cat(parts), out) and torch.equal(carry, final)


def test_config4_kda_prefill_strong_and_weak_decay_prefix():
    """Config 4 distributions (strong-decay and weak-decay heads) on a 8192-token prefix, checked
    against the float64 chunked oracle; the full 65536-token run is checked through the
    chained-calls invariant in bench / DESIGN."""
    from pla_amd.workloads import kda_prefill
    from pla_amd.prefill.flashkdapro import flashkda_fwd
    w = kda_prefill(T=8192, H=8, seed=404)
    call = {k: v for k, v in w.items() if not k.startswith("_")}
    flashkda_fwd(call["q"], call["k"], call["v"], call["g"], call["beta"], call["A_log"], call["dt_bias"], call["out"],
                 scale=call["scale"], lower_bound=call["lower_bound"], initial_state=call["initial_state"],
                 final_state=call["final_state"], cu_seqlens=call["cu_seqlens"])
    torch.cuda.synchronize()
    cpu = {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in call.items()}
    exp_o, exp_final = _oracle(cpu["q"], cpu["k"], cpu["v"], cpu["g"], cpu["beta"], cpu["A_log"], cpu["dt_bias"],
                               [0, 8192], cpu["initial_state"], fast=True)
    torch.testing.assert_close(call["out"].cpu().float(), exp_o.float(), atol=2e-2, rtol=2e-2)
    for head in range(8):
        assert rel_l2(call["final_state"][0, head], exp_final[0, head]) <= 1e-3, head


def test_config4_kda_prefill_full_size():
    """Config 4 at its full size (one sequence of 65536 tokens, 32 heads).  Eight heads (four that decay
    strongly, four that decay weakly) are checked against the float64 chunked oracle over
    the whole sequence; every head is checked through the chained-calls invariant: two calls
    that split the sequence at a chunk boundary and pass the state on give the same o and final
    state."""
    from pla_amd.workloads import kda_prefill
    from pla_amd.prefill.flashkdapro import flashkda_fwd
    T, H = 65536, 32
    w = kda_prefill(T=T, H=H, seed=4)
    call = {k: v for k, v in w.items() if not k.startswith("_")}

    def run(lo, hi, init, out, final):
        cu = torch.tensor([0, hi - lo], dtype=torch.int32, device="cuda")
        flashkda_fwd(call["q"][lo:hi], call["k"][lo:hi], call["v"][lo:hi], call["g"][lo:hi], call["beta"][lo:hi],
                     call["A_log"], call["dt_bias"], out, scale=call["scale"], lower_bound=call["lower_bound"],
                     initial_state=init, final_state=final, cu_seqlens=cu)

    run(0, T, call["initial_state"], call["out"], call["final_state"])
    torch.cuda.synchronize()
    assert torch.isfinite(call["out"].float()).all() and torch.isfinite(call["final_state"]).all()

    split = 40 * 64 * 16                                    # chunk-aligned, not the middle
    o2 = torch.empty_like(call["out"])
    mid = torch.empty_like(call["final_state"])
    fin = torch.empty_like(call["final_state"])
    run(0, split, call["initial_state"], o2[:split], mid)
    run(split, T, mid, o2[split:], fin)
    torch.cuda.synchronize()
    # A call with this few chains splits the sequence into concurrently swept segments, and the two
    # shorter calls split differently, so the results agree to the rounding of the fp16 operands (2^-12
    # relative per operand) rather than bit for bit: a few percent of the bf16 outputs move by one ulp.
    torch.testing.assert_close(o2.float(), call["out"].float(), atol=2e-2, rtol=2e-2)
    assert (o2 != call["out"]).float().mean().item() < 0.10
    for head in range(H):
        assert rel_l2(fin[0, head], call["final_state"][0, head]) <= 5e-4, head

    heads = [0, 5, 10, 15, 16, 21, 26, 31]                  # four strongly and four weakly decaying heads
    cpu = {k: (v.cpu() if torch.is_tensor(v) else v) for k, v in call.items()}
    sel = lambda t: t[:, heads].contiguous()
    exp_o, exp_final = _oracle(sel(cpu["q"]), sel(cpu["k"]), sel(cpu["v"]), sel(cpu["g"]), sel(cpu["beta"]),
                               cpu["A_log"][heads], cpu["dt_bias"][heads], [0, T], cpu["initial_state"][:, heads], fast=True)
    torch.testing.assert_close(call["out"][:, heads].cpu().float(), exp_o.float(), atol=2e-2, rtol=2e-2)
    for i, head in enumerate(heads):
        assert rel_l2(call["final_state"][0, head], exp_final[0, i]) <= 1e-3, head


@pytest.mark.parametrize("lengths,H", [([700, 0, 130, 64, 1], 24), ([4096, 40], 2), ([1500, 200, 300, 400, 700], 32)])
def test_kda_prefill_in_a_graph(lengths, H):
    """flashkda_fwd allocates (workspace) and launches only, so it can be captured: a call of whole sequences (more
    than 64 chains) and a call that is split into segments (zero-state / identity sweeps, combine, second sweep),
    each replayed three times with eager work and a synchronisation in between, reproduce the eager result bit for
    bit (outputs and written-back states)."""
    from pla_amd.prefill.flashkdapro import flashkda_fwd
    q, k, v, raw, beta, A_log, dt_bias, offs, S0 = _inputs(lengths, H, seed=77 + H, pad=3)
    dev = "cuda"
    T, N = q.shape[0], len(lengths)
    dq, dk, dv, dg, db = (t.to(dev) for t in (q, k, v, raw, beta))
    dA, dD, dS = A_log.to(dev), dt_bias.to(dev), S0.to(dev)
    cu = torch.tensor(offs, dtype=torch.int32, device=dev)

    def run(out, final):
        # (with the host offsets: the third case then runs the chains of its longest sequence as two workgroups each)
        flashkda_fwd(dq, dk, dv, dg, db, dA, dD, out, initial_state=dS, final_state=final, cu_seqlens=cu,
                     raw_cu_seqlens=tuple(offs))

    o_eager = torch.empty(T, H, 128, dtype=torch.bfloat16, device=dev)
    f_eager = torch.empty(N, H, 128, 128, device=dev)
    run(o_eager, f_eager)
    torch.cuda.synchronize()
    o_graph, f_graph = torch.empty_like(o_eager), torch.empty_like(f_eager)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        run(o_graph, f_graph)                                  # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(stream)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        run(o_graph, f_graph)
    for replay in range(3):
        o_graph.fill_(float("nan"))
        f_graph.fill_(float("nan"))
        scratch = torch.randn(1 << 20, device=dev).sum().item()        # eager work and a sync between replays
        graph.replay()
        torch.cuda.synchronize()
        assert scratch == scratch
        assert torch.equal(o_graph.view(torch.int16), o_eager.view(torch.int16)), replay
        assert torch.equal(f_graph.view(torch.int32), f_eager.view(torch.int32)), replay


@pytest.mark.parametrize("lengths,pad,H", [([2500, 0, 1111, 40], 5, 2), ([4096], 0, 1), ([1030, 2049], 0, 3)])
def test_kda_prefill_split_sequences_match_oracle(lengths, pad, H):
    """Few, long sequences are split into 16-chunk segments that are swept concurrently (zero-state
    and identity sweeps, a combine step, a second sweep).  Ragged lengths, an empty sequence, a
    sequence shorter than one segment, initial and final states, against the float64 oracle."""
    from pla_amd.prefill.flashkdapro import flashkda_fwd
    from pla_amd import _lib
    q, k, v, raw, beta, A_log, dt_bias, offs, S0 = _inputs(lengths, H, seed=515, pad=pad)
    T, N = q.shape[0], len(lengths)
    size = _lib.load().pla_kda_prefill_workspace_bytes
    unsplit_per_head = size(T, N, 65 * H) / (65 * H)          # more than 64 chains are never split
    assert size(T, N, H) > 1.1 * H * unsplit_per_head           # so this call carries the segment buffers
    dev = "cuda"
    out = torch.full((T, H, 128), float("nan"), dtype=torch.bfloat16, device=dev)
    final = torch.full((N, H, 128, 128), float("nan"), device=dev)
    cu = torch.tensor(offs, dtype=torch.int32, device=dev)
    flashkda_fwd(q.to(dev), k.to(dev), v.to(dev), raw.to(dev), beta.to(dev), A_log.to(dev), dt_bias.to(dev), out,
                 initial_state=S0.to(dev), final_state=final, cu_seqlens=cu)
    torch.cuda.synchronize()
    exp_o, exp_final = _oracle(q, k, v, raw, beta, A_log, dt_bias, offs, S0, fast=True)
    real = offs[-1]
    torch.testing.assert_close(out[:real].cpu().float(), exp_o[:real].float(), atol=2e-2, rtol=2e-2)
    assert (out[real:] == 0).all()
    for n, length in enumerate(lengths):
        for head in range(H):
            if length == 0:
                assert torch.equal(final[n, head].cpu(), S0[n, head])   # an empty sequence publishes its incoming state
            else:
                assert rel_l2(final[n, head], exp_final[n, head]) <= 1e-3, (n, head)


@pytest.mark.parametrize("lengths,H,halved", [([1500, 1300, 300, 64, 0, 777, 500, 200, 900], 16, 2),
                                              ([900, 800, 100, 64, 0, 300, 200, 150, 400, 130, 77, 60], 12, 2),
                                              ([1500, 200, 300, 400, 700], 32, 1),
                                              ([900, 100, 1500, 64, 0, 300, 2000, 150, 400, 130, 77, 700], 32, 1),
                                              ([500, 500, 500, 490, 510, 500, 500, 500, 500], 32, 0)])
def test_kda_prefill_longest_sequences_swept_as_halves(lengths, H, halved):
    """Ragged whole sequences with more than 128 chains and the offsets on the host: the chains of the longest
    sequences run as two workgroups of 64 V columns each (the plan is host arithmetic and is asked for here); with
    more chains than CUs the chains also start longest first.  Against the oracle, and bit for bit against the call without host offsets, which sweeps every chain whole, through
    both host layers."""
    import ctypes
    from pla_amd import _lib
    from pla_amd.prefill.flashkdapro import flashkda_fwd, ops
    q, k, v, raw, beta, A_log, dt_bias, offs, S0 = _inputs(lengths, H, seed=4711, pad=5)
    plan = _lib.load().pla_kda_prefill_halved_sequences((ctypes.c_int32 * len(offs))(*offs), len(lengths), q.shape[0], H)
    assert plan == halved
    exp_o, exp_final = _oracle(q, k, v, raw, beta, A_log, dt_bias, offs, S0, fast=True)
    dev = "cuda"
    args = [t.to(dev) for t in (q, k, v, raw, beta, A_log, dt_bias)]
    cu = torch.tensor(offs, dtype=torch.int32, device=dev)
    results = []
    for native in (False, True):
        for host_offsets in (tuple(offs), None):
            ops._native = None if native else False
            out = torch.full((q.shape[0], H, 128), 7.0, dtype=torch.bfloat16, device=dev)
            final = torch.empty_like(S0, device=dev)
            flashkda_fwd(*args, out, initial_state=S0.to(dev), final_state=final, cu_seqlens=cu, raw_cu_seqlens=host_offsets)
            torch.cuda.synchronize()
            results.append((out, final))
    ops._native = False
    out, final = results[0]
    torch.testing.assert_close(out[:offs[-1]].float().cpu(), exp_o[:offs[-1]].float(), atol=2e-2, rtol=2e-2)
    assert torch.count_nonzero(out[offs[-1]:]) == 0
    worst = max(rel_l2(final[n].cpu(), exp_final[n]) for n in range(len(lengths)))
    assert worst <= 1e-3, worst
    for other in results[1:]:
        assert torch.equal(other[0], out) and torch.equal(other[1], final)


def test_kda_prefill_many_chains_match_oracle_and_single_sequence_bits():
    """128 chains of ragged lengths (an empty sequence, sequences of one token and of one chunk) in one call, against
    the oracle; the short sequences run alone give the same bits.  (The shape is the one a pipelined call of
    preparation and sweep would take: that variant passes this test too and is switched off for its speed.)"""
    from pla_amd.prefill.flashkdapro import flashkda_fwd
    lengths = [3000, 0, 70, 1500, 64, 2100, 1, 1500]
    H = 16
    q, k, v, raw, beta, A_log, dt_bias, offs, S0 = _inputs(lengths, H, seed=91, pad=5)
    exp_o, exp_final = _oracle(q, k, v, raw, beta, A_log, dt_bias, offs, S0, fast=True)
    dev = "cuda"
    args = [t.to(dev) for t in (q, k, v, raw, beta, A_log, dt_bias)]
    cu = torch.tensor(offs, dtype=torch.int32, device=dev)
    out = torch.full((q.shape[0], H, 128), 7.0, dtype=torch.bfloat16, device=dev)
    final = torch.empty_like(S0, device=dev)
    flashkda_fwd(*args, out, initial_state=S0.to(dev), final_state=final, cu_seqlens=cu)
    torch.cuda.synchronize()
    torch.testing.assert_close(out[:offs[-1]].float().cpu(), exp_o[:offs[-1]].float(), atol=2e-2, rtol=2e-2)
    assert torch.count_nonzero(out[offs[-1]:]) == 0
    worst = max(rel_l2(final[n].cpu(), exp_final[n]) for n in range(len(lengths)))
    assert worst <= 1e-3, worst
    for n, length in enumerate(lengths):
        if length == 0 or length >= 2048:
            continue
        lo, hi = offs[n], offs[n + 1]
        one = torch.empty(hi - lo, H, 128, dtype=torch.bfloat16, device=dev)
        fin1 = torch.empty(1, H, 128, 128, device=dev)
        flashkda_fwd(*[t[lo:hi] for t in args[:5]], args[5], args[6], one, initial_state=S0[n:n + 1].to(dev),
                     final_state=fin1, cu_seqlens=torch.tensor([0, hi - lo], dtype=torch.int32, device=dev))
        torch.cuda.synchronize()
        assert torch.equal(one, out[lo:hi]), n
        assert torch.equal(fin1[0], final[n]), n


@pytest.mark.parametrize("lengths,noise", [([200, 131], 0.1), ([1000, 700], 0.1), ([640], 0.03)])
def test_kda_prefill_correlated_keys_dense_triangular_system(lengths, noise):
    """The correlated-key stress of the GDN prefill on the KDA path: keys = one direction per head plus `noise` x
    N(0, 1), beta = 0.982, a per-channel log-decay of -1.7e-3 per token.  Every entry of the chunk's triangular
    system is of order one, U = W X cancels heavily and the final state is the work of the last few tokens, so
    operand roundings show unaveraged; the bounds are the usual ones."""
    from pla_amd.prefill.flashkdapro import flashkda_fwd
    H = 2
    q, k, v, raw, beta, A_log, dt_bias, offs, S0 = _inputs(lengths, H, seed=41 + len(lengths))
    g = torch.Generator().manual_seed(5)
    k = (torch.randn(1, H, 128, generator=g) + noise * torch.randn(q.shape[0], H, 128, generator=g)).bfloat16()
    beta = torch.full_like(beta, 4.0)
    raw = torch.full_like(raw, -8.0)
    A_log = torch.zeros_like(A_log)
    dt_bias = torch.zeros_like(dt_bias)
    exp_o, exp_final = _oracle(q, k, v, raw, beta, A_log, dt_bias, offs, S0, fast=sum(lengths) > 600)
    dev = "cuda"
    cu = torch.tensor(offs, dtype=torch.int32, device=dev)
    out = torch.empty(q.shape[0], H, 128, dtype=torch.bfloat16, device=dev)
    final = torch.empty(len(lengths), H, 128, 128, device=dev)
    flashkda_fwd(*[t.to(dev) for t in (q, k, v, raw, beta, A_log, dt_bias)], out, initial_state=S0.to(dev),
                 final_state=final, cu_seqlens=cu)
    torch.cuda.synchronize()
    torch.testing.assert_close(out.cpu().float(), exp_o.float(), atol=2e-2, rtol=2e-2)
    worst = max(rel_l2(final[n], exp_final[n]) for n in range(len(lengths)))
    print("KDA correlated keys", lengths, noise, "state rel-L2 %.3e" % worst)
    assert worst <= 1e-3, worst
