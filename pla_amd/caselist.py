"""Replay of OperatorsForge caselists on the gfx950 kernels.

A caselist line names one operator shape, e.g.::

    [GDN]:[D][8]gdn_attn:seqlen_q:1,head_dim_qk:128,...,num_heads_qk:16,num_heads_v:32,...,batch_size:8,dtype:bf16.
    [KDA]:[P][6,1798]kda_attn:head_dim_qk:128,...,gate_lower_bound:-5.0,batch_size:6,dtype:bf16,cu_seqlens_q:[0,1090,...].

(the format of the reference's ``caselist/decode/*.list`` and ``caselist/prefill/*.list``, which its
``tests/test_op_forge.py`` replays).  ``parse_case`` turns a line into a dict, ``replay_case`` runs the
shape on synthetic inputs through the operator that serves it here and times it:

==========================  =====================================================================
GDN decode, 1 token         ``fused_sigmoid_gating_delta_rule_forward_k_last_packed``
GDN decode, T tokens        ``fused_sigmoid_gating_delta_rule_forward_k_last`` (verify, state read-only)
KDA decode, 1 token         ``fused_kda_decode_mega_forward`` (conv + gate + recurrence + norm)
KDA decode, T tokens        ``fused_kda_decode_mtp_dspark`` (verify with replay records, T <= 32)
GDN / KDA prefill           ``gdn_prefill_packed_qkv_fwd`` / ``flashkda_fwd``
==========================  =====================================================================

Shapes outside head_dim 128 and other operator families (``mamba2_ssm``) are reported as skipped.
Decode shapes are timed as graph replays over rotating slot sets (the host-side argument checks cost
more than the small kernels, and a fixed slot set would be served from the last-level cache).

Command line: ``python -m pla_amd.caselist FILE [--limit N] [--csv OUT]`` times every case;
``python -m pla_amd.caselist FILE --check N`` checks N seeded small prefill shapes of the list instead (each against
itself fed in two chained calls per sequence; ``check_case`` also takes a reference, which the tests use).
"""

import argparse
import ast
import csv
import gzip
import re
import sys

import torch

_LINE = re.compile(r"^\[(?P<family>\w+)\]:\[(?P<phase>[DP])\]\[(?P<tag>[^\]]*)\](?P<op>\w+):(?P<body>.*?)\.?$")
_MEGA_HEADS = (4, 6, 8, 12, 16, 24, 48, 64, 96)
ROUNDING_TIE_BOUND = 4e-3          # relative L2 deviation of a final state that one rounding tie of a key may cause


def parse_case(line):
    """One caselist line -> dict (``family``, ``phase``, ``op`` and the line's own keys with integers,
    floats and the ``cu_seqlens_q`` list converted); ``None`` for blank and comment lines."""
    line = line.strip()
    if not line or line.startswith("#"):
        return None
    m = _LINE.match(line)
    if m is None:
        raise ValueError(f"not a caselist line: {line[:80]!r}")
    case = dict(family=m["family"], phase=m["phase"], op=m["op"], tag=m["tag"])
    body = m["body"]
    lists = {}
    for key, value in re.findall(r"(\w+):(\[[^\]]*\])", body):
        lists[key] = list(ast.literal_eval(value))
    body = re.sub(r"\w+:\[[^\]]*\],?", "", body)
    for item in filter(None, body.split(",")):
        key, _, value = item.partition(":")
        try:
            case[key] = int(value)
        except ValueError:
            try:
                case[key] = float(value)
            except ValueError:
                case[key] = value
    case.update(lists)
    return case


def read_caselist(path, limit=None):
    """The cases of a list file (plain text, or gzip when the name ends in .gz), in file order."""
    cases = []
    opener = gzip.open if str(path).endswith(".gz") else open
    with opener(path, "rt") as fh:
        for line in fh:
            case = parse_case(line)
            if case is not None:
                cases.append(case)
                if limit is not None and len(cases) >= limit:
                    break
    return cases


def unsupported_reason(case):
    """Why a case cannot be replayed here, or ``None``."""
    if case["op"] not in ("gdn_attn", "kda_attn"):
        return f"operator family {case['op']} is not part of this library"
    if case.get("head_dim_qk") != 128 or case.get("head_dim_v") != 128:
        return "head_dim must be 128"
    if case.get("dtype") not in ("bf16", "fp16"):
        return f"dtype {case.get('dtype')}"
    H, HV = case["num_heads_qk"], case["num_heads_v"]
    if HV % H:
        return "num_heads_v must be a multiple of num_heads_qk"
    if case["phase"] == "D" and case["op"] == "kda_attn":
        if case.get("seqlen_q", 1) == 1 and H not in _MEGA_HEADS:
            return f"the fused KDA decode step supports H in {_MEGA_HEADS}"
        if case.get("seqlen_q", 1) > 32:
            return "the KDA verify handles up to 32 draft tokens"
    if case["phase"] == "P" and case["op"] == "kda_attn" and case.get("dtype") != "bf16":
        return "KDA prefill takes bf16 activations"
    return None


def _graph_time_us(fns, reps):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for fn in fns:
            fn()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for fn in fns:
            fn()
    for _ in range(2):
        graph.replay()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        graph.replay()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / reps / len(fns) * 1e3


def _eager_time_us(fn, reps):
    for _ in range(2):
        fn()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / reps * 1e3


def _prefill_case_on_device(case, device, seed):
    """A prefill case whose inputs are drawn on the GPU (same distributions as the CPU-seeded inputs of the checks,
    other values): for replays of long lists, where drawing up to 32 768 tokens x 128 heads on the host would take
    most of the time.  Returns ``(fn, kind)``."""
    import math
    from .prefill.flashqla import gdn_prefill_packed_qkv_fwd
    from .prefill.flashkdapro import flashkda_fwd
    dtype = torch.bfloat16 if case["dtype"] == "bf16" else torch.float16
    H, HV = case["num_heads_qk"], case["num_heads_v"]
    offs = list(case["cu_seqlens_q"])
    N, T = len(offs) - 1, offs[-1]
    lb = case.get("gate_lower_bound")
    g = torch.Generator(device=device).manual_seed(seed)
    rnd = lambda *s: torch.randn(*s, generator=g, device=device)
    cu = torch.tensor(offs, dtype=torch.int32, device=device)
    if case["op"] == "gdn_attn":
        slots = max(8, N + 3)
        packed = rnd(T, (2 * H + HV) * 128).to(dtype)
        a, b = rnd(T, HV).to(dtype), rnd(T, HV).to(dtype)
        A_log = torch.rand(HV, generator=g, device=device) * math.log(16.0)
        dt_bias = torch.rand(HV, generator=g, device=device) * 2 - 1
        pool = rnd(slots, HV, 128, 128) * 0.1
        idx = torch.randperm(slots, generator=g, device=device)[:N].to(torch.int32)
        fn = lambda: gdn_prefill_packed_qkv_fwd(packed, a, b, A_log, dt_bias, cu, num_qk_heads=H, num_v_heads=HV,
                                                scale=128 ** -0.5, initial_state=pool, initial_state_indices=idx,
                                                raw_cu_seqlens=tuple(offs), output_final_state=False)
        return fn, "gdn_prefill"
    q, k, v, gate = (rnd(T, H, 128).to(dtype) for _ in range(4))
    beta = rnd(T, H).to(dtype)
    A_log, dt_bias = rnd(H) * 0.5, rnd(H, 128) * 0.1
    out = torch.empty(T, H, 128, dtype=dtype, device=device)
    state = rnd(N, H, 128, 128) * 0.1
    final = torch.empty(N, H, 128, 128, dtype=torch.float32, device=device)
    fn = lambda: flashkda_fwd(q, k, v, gate, beta, A_log, dt_bias, out, scale=128 ** -0.5,
                              lower_bound=-5.0 if lb is None else lb, initial_state=state, final_state=final,
                              cu_seqlens=cu)
    return fn, "kda_prefill"


def build_case(case, device="cuda", seed=0, sets=None):
    """Synthetic inputs for a case: returns ``(fns, info)`` where every ``fn()`` runs the operator once
    (several closures = rotating slot sets) and ``info`` holds the algorithmic bytes / tokens of one run
    plus the tensors a checker needs (``info["workload"]``)."""
    from . import workloads
    from .decode import (fused_sigmoid_gating_delta_rule_forward_k_last as k_last,
                         fused_sigmoid_gating_delta_rule_forward_k_last_packed as packed)
    from .decode.kda import fused_kda_decode_mega_forward as mega
    from .decode.kda_replayssm_sglang import fused_kda_decode_mtp_dspark as verify_dspark
    from .prefill.flashqla import gdn_prefill_packed_qkv_fwd
    from .prefill.flashkdapro import flashkda_fwd
    dtype = torch.bfloat16 if case["dtype"] == "bf16" else torch.float16
    H, HV = case["num_heads_qk"], case["num_heads_v"]
    B = case["batch_size"]
    kda = case["op"] == "kda_attn"
    lb = case.get("gate_lower_bound")
    if case["phase"] == "D":
        T = case.get("seqlen_q", 1)
        if sets is None:
            sets = max(1, min(8, (1 << 31) // max(1, B * HV * 65536 * 2)))     # at most 4 GiB of state per case
        if not kda and T == 1:
            w = workloads.gdn_decode_packed(B, H=H, HV=HV, pool_slots=B * sets, seed=seed, device=device, dtype=dtype)
            call = {k: v for k, v in w.items() if not k.startswith("_")}
            g = torch.Generator().manual_seed(seed + 1)
            idx = [torch.randperm(B * sets, generator=g)[:B].to(torch.int32).to(device) for _ in range(sets)]
            idx[0] = call["initial_state_indices"]
            fns = [lambda i=i: packed(**dict(call, initial_state_indices=i)) for i in idx]
            return fns, dict(kind="gdn_decode", state_bytes=B * HV * 131072, workload=w)
        if not kda:
            g = torch.Generator().manual_seed(seed)
            rnd = lambda *s: torch.randn(*s, generator=g)
            pool = (rnd(B + 1, HV, 128, 128) * 0.1).to(device)
            args = dict(
                A_log=rnd(HV).to(device), a=rnd(B, T, HV).to(dtype).to(device), dt_bias=rnd(HV).to(dtype).to(device),
                softplus_beta=1.0, softplus_threshold=20.0,
                q=rnd(B, T, H, 128).to(dtype).to(device), k=rnd(B, T, H, 128).to(dtype).to(device),
                v=rnd(B, T, HV, 128).to(dtype).to(device), b=rnd(B, T, HV).to(dtype).to(device),
                initial_state_source=pool,
                initial_state_indices=torch.randperm(B + 1, generator=g)[:B].to(torch.int32).to(device),
                scale=128 ** -0.5, use_qk_l2norm_in_kernel=True, cu_seqlens=None, is_kda=False,
                disable_state_update=True, intermediate_states_buffer=None, intermediate_state_indices=None,
                cache_steps_or_num_accept=None, retrieve_parent_token=None)
            out = torch.empty(B, T, HV, 128, dtype=dtype, device=device)
            return [lambda: k_last(**args, out=out)], dict(kind="gdn_verify", state_bytes=B * HV * 65536,
                                                           workload=args, out=out)
        if T == 1:
            w = workloads.kda_decode_mega(B, H, seed=seed, device=device, dtype=dtype, slots=B * sets + 2)
            out = torch.empty(1, B, H, 128, dtype=dtype, device=device)
            base = w["state_indices"]
            call = dict(x=w["x"], weight=w["weight"], bias=None, conv_state=w["conv_state"], raw_g=w["raw_g"],
                        raw_beta=w["raw_beta"], a_log=w["a_log"], dt_bias=w["dt_bias"], state=w["state"], out=out,
                        lower_bound=lb, output_gate=w["output_gate"], norm_weight=w["norm_weight"], norm_eps=1e-5)
            idx = [(base + i * B).contiguous() for i in range(sets)]
            fns = [lambda i=i: mega(**call, state_indices=i) for i in idx]
            return fns, dict(kind="kda_decode", state_bytes=B * H * 131072, workload=w, out=out)
        if dtype != torch.bfloat16:
            raise ValueError("the KDA verify takes bf16 activations")
        w = workloads.kda_replay_verify(B, H, T, seed=seed, device=device, ring_len=max(8, T), slots=B + 2,
                                        lower_bound=-5.0 if lb is None else lb, onorm=True, strided=True)
        out = torch.empty(1, B * T, H, 128, dtype=dtype, device=device)
        return [lambda: verify_dspark(out=out, **w)], dict(kind="kda_verify", state_bytes=B * H * 65536,
                                                           workload=w, out=out)
    lengths = [b - a for a, b in zip(case["cu_seqlens_q"], case["cu_seqlens_q"][1:])]
    tokens = sum(lengths)
    if not kda:
        w = workloads.gdn_prefill_packed(lengths, H=H, HV=HV, pool_slots=max(8, len(lengths) + 3), seed=seed,
                                         device=device, dtype=dtype)
        call = {k: v for k, v in w.items() if not k.startswith("_")}
        packed_qkv = call.pop("packed_qkv")
        a, b, A, dt, cu = (call.pop(n) for n in ("raw_gate_a", "raw_beta_b", "A_log", "dt_bias", "cu_seqlens"))
        fn = lambda: gdn_prefill_packed_qkv_fwd(packed_qkv, a, b, A, dt, cu, output_final_state=False, **call)
        return [fn], dict(kind="gdn_prefill", tokens=tokens, workload=w)
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *s: torch.randn(*s, generator=g)
    N = len(lengths)
    w = dict(q=rnd(tokens, H, 128).to(dtype).to(device), k=rnd(tokens, H, 128).to(dtype).to(device),
             v=rnd(tokens, H, 128).to(dtype).to(device), g=rnd(tokens, H, 128).to(dtype).to(device),
             beta=rnd(tokens, H).to(dtype).to(device), A_log=(rnd(H) * 0.5).to(device),
             dt_bias=(rnd(H, 128) * 0.1).to(device),
             out=torch.empty(tokens, H, 128, dtype=dtype, device=device), scale=128 ** -0.5,
             lower_bound=-5.0 if lb is None else lb, initial_state=(rnd(N, H, 128, 128) * 0.1).to(device),
             final_state=torch.empty(N, H, 128, 128, dtype=torch.float32, device=device),
             cu_seqlens=torch.tensor(case["cu_seqlens_q"], dtype=torch.int32, device=device))
    fn = lambda: flashkda_fwd(w["q"], w["k"], w["v"], w["g"], w["beta"], w["A_log"], w["dt_bias"], w["out"],
                              scale=w["scale"], lower_bound=w["lower_bound"], initial_state=w["initial_state"],
                              final_state=w["final_state"], cu_seqlens=w["cu_seqlens"])
    return [fn], dict(kind="kda_prefill", tokens=tokens, workload=w)


def select_check_cases(cases, n, seed=0, max_tokens=2048):
    """``n`` prefill cases of a list for a correctness check: drawn with a seeded generator from the served prefill
    cases of at most ``max_tokens`` tokens (small enough for a CPU reference), in the order of the list."""
    import random
    small = [c for c in cases if c["phase"] == "P" and unsupported_reason(c) is None and c["cu_seqlens_q"][-1] <= max_tokens]
    if len(small) <= n:
        return small
    keep = set(random.Random(seed).sample(range(len(small)), n))
    return [c for i, c in enumerate(small) if i in keep]


def run_prefill_case(case, device="cuda", seed=0, split=False):
    """One prefill case on seeded synthetic inputs: returns ``(o, final_states, inputs)`` with ``o`` [T, HV, 128],
    the final states [N, HV, 128, 128] and the input tensors (what a CPU reference needs).  With ``split`` every
    sequence is fed in two calls - its first ``len // 2`` tokens, then the rest from the state the first call left -
    and the outputs are put back into the order of the single call: both ways must agree to rounding."""
    from . import workloads
    from .prefill.flashqla import gdn_prefill_packed_qkv_fwd
    from .prefill.flashkdapro import flashkda_fwd
    dtype = torch.bfloat16 if case["dtype"] == "bf16" else torch.float16
    H, HV = case["num_heads_qk"], case["num_heads_v"]
    offs = list(case["cu_seqlens_q"])
    N, T = len(offs) - 1, offs[-1]
    lb = case.get("gate_lower_bound")
    mids = [lo + (hi - lo) // 2 for lo, hi in zip(offs, offs[1:])]
    # token rows of the two calls of a split run, and the offsets of each call
    parts = [[(lo, mid) for lo, mid in zip(offs, mids)], [(mid, hi) for mid, hi in zip(mids, offs[1:])]] if split else \
            [[(lo, hi) for lo, hi in zip(offs, offs[1:])]]

    def rows_and_offsets(part):
        rows = torch.cat([torch.arange(lo, hi) for lo, hi in part] + [torch.arange(0)]).to(device)
        cu = [0]
        for lo, hi in part:
            cu.append(cu[-1] + hi - lo)
        return rows, cu

    if case["op"] == "gdn_attn":
        w = workloads.gdn_prefill_packed([hi - lo for lo, hi in zip(offs, offs[1:])], H=H, HV=HV,
                                         pool_slots=max(8, N + 3), seed=seed, device=device, dtype=dtype)
        pool = w["initial_state"].clone()
        idx = w["initial_state_indices"]
        o = torch.zeros(T, HV, 128, dtype=dtype, device=device)
        for part in parts:
            rows, cu = rows_and_offsets(part)
            if rows.numel() == 0:
                continue
            out = gdn_prefill_packed_qkv_fwd(
                w["packed_qkv"][rows].contiguous(), w["raw_gate_a"][rows].contiguous(), w["raw_beta_b"][rows].contiguous(),
                w["A_log"], w["dt_bias"], torch.tensor(cu, dtype=torch.int32, device=device), num_qk_heads=H,
                num_v_heads=HV, scale=w["scale"], initial_state=pool, initial_state_indices=idx,
                raw_cu_seqlens=tuple(cu), output_final_state=False)
            o[rows] = out[2][0]
        torch.cuda.synchronize()
        return o, pool[idx.long()], w
    g = torch.Generator().manual_seed(seed)
    rnd = lambda *s: torch.randn(*s, generator=g)
    w = dict(q=rnd(T, H, 128).to(dtype).to(device), k=rnd(T, H, 128).to(dtype).to(device),
             v=rnd(T, H, 128).to(dtype).to(device), g=rnd(T, H, 128).to(dtype).to(device),
             beta=rnd(T, H).to(dtype).to(device), A_log=(rnd(H) * 0.5).to(device), dt_bias=(rnd(H, 128) * 0.1).to(device),
             scale=128 ** -0.5, lower_bound=-5.0 if lb is None else lb, initial_state=(rnd(N, H, 128, 128) * 0.1).to(device),
             offsets=offs)
    o = torch.zeros(T, H, 128, dtype=dtype, device=device)
    state = w["initial_state"]
    for part in parts:
        rows, cu = rows_and_offsets(part)
        final = torch.empty(N, H, 128, 128, dtype=torch.float32, device=device)
        if rows.numel() == 0:
            continue
        out = torch.empty(rows.numel(), H, 128, dtype=dtype, device=device)
        flashkda_fwd(w["q"][rows].contiguous(), w["k"][rows].contiguous(), w["v"][rows].contiguous(),
                     w["g"][rows].contiguous(), w["beta"][rows].contiguous(), w["A_log"], w["dt_bias"], out,
                     scale=w["scale"], lower_bound=w["lower_bound"], initial_state=state, final_state=final,
                     cu_seqlens=torch.tensor(cu, dtype=torch.int32, device=device))
        o[rows] = out
        state = final
    torch.cuda.synchronize()
    return o, state, w


def check_case(case, reference=None, device="cuda", seed=0):
    """Correctness of one prefill case.  ``reference(case, inputs) -> (o, final_states)`` supplies the expected
    result (the tests pass the CPU oracle); without one the case is compared with itself fed in two chained calls
    per sequence.  Returns a row with the largest output error in units of the tolerance ``2e-2 + 2e-2 |o|``
    (``o_err`` <= 1 passes), the worst relative L2 error of a final state (bound 1e-3 against a reference, 2e-3
    between the two ways of calling, which round differently) and ``ok``.

    A normalised q / k element that lies within an FP32 rounding error of the midpoint between two values of the
    activation dtype rounds one way here and the other way in a reference that sums the row's squares in another
    order; both are correct roundings of the same number.  Where the gate decays strongly the final state is the
    outer product of the last token, and one such element shows as a rank-one deviation of up to one unit of the
    activation dtype (2^-8) in one channel.  So a state may exceed the bound in at most one of sixteen (sequence,
    head) pairs, and then by no more than ``ROUNDING_TIE_BOUND``; ``states_over_bound`` counts them."""
    o, final, w = run_prefill_case(case, device=device, seed=seed)
    if reference is not None:
        want_o, want_final = reference(case, w)
        bound = 1e-3
    else:
        want_o, want_final, _ = run_prefill_case(case, device=device, seed=seed, split=True)
        bound = 2e-3
    want_o = want_o.to(o.device).float()
    want_final = want_final.to(final.device).float()
    o_err = float(((o.float() - want_o).abs() / (2e-2 + 2e-2 * want_o.abs())).max()) if o.numel() else 0.0
    errors = []
    for n in range(final.shape[0]):
        for h in range(final.shape[1]):
            den = float(want_final[n, h].norm())
            num = float((final[n, h] - want_final[n, h]).norm())
            errors.append(num / den if den > 0 else num)
    worst = max(errors, default=0.0)
    over = sum(e > bound for e in errors)
    finite = bool(torch.isfinite(o.float()).all() and torch.isfinite(final).all())
    states_ok = over == 0 or (16 * over <= len(errors) and worst <= ROUNDING_TIE_BOUND)
    return dict(family=case["family"], heads=f"{case['num_heads_qk']}/{case['num_heads_v']}", batch=case["batch_size"],
                tokens=case["cu_seqlens_q"][-1], against="reference" if reference is not None else "split calls",
                o_err=round(o_err, 4), state_rel_l2=float("%.3e" % worst), states_over_bound=over,
                ok=finite and o_err <= 1.0 and states_ok)


def replay_case(case, device="cuda", reps=20, seed=0, device_inputs=False):
    """Runs and times one case.  Returns a result row (dict).  device_inputs: prefill inputs are drawn on the GPU."""
    row = dict(family=case["family"], phase=case["phase"], batch=case.get("batch_size"),
               heads=f"{case.get('num_heads_qk')}/{case.get('num_heads_v')}", seqlen_q=case.get("seqlen_q"))
    reason = unsupported_reason(case)
    if reason is not None:
        row.update(status="skipped", reason=reason)
        return row
    if device_inputs and case["phase"] == "P":
        fn, kind = _prefill_case_on_device(case, device, seed)
        us = _eager_time_us(fn, max(3, reps // 4))
        tokens = case["cu_seqlens_q"][-1]
        row.update(status="ok", kind=kind, us=round(us, 1), tokens=tokens, tokens_per_s=round(tokens / us * 1e6))
        return row
    fns, info = build_case(case, device=device, seed=seed)
    if case["phase"] == "D":
        us = _graph_time_us(fns, reps)
        row.update(status="ok", kind=info["kind"], us=round(us, 2),
                   state_GBps=round(info["state_bytes"] / us / 1e3, 1))
    else:
        us = _eager_time_us(fns[0], max(3, reps // 4))
        row.update(status="ok", kind=info["kind"], us=round(us, 1), tokens=info["tokens"],
                   tokens_per_s=round(info["tokens"] / us * 1e6))
    return row


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("caselist")
    ap.add_argument("--limit", type=int, default=None)
    ap.add_argument("--start", type=int, default=0, help="skip this many cases of the list (a long list replayed in parts)")
    ap.add_argument("--csv", default=None)
    ap.add_argument("--min-seqlen-q", type=int, default=0, metavar="N",
                    help="decode lists: only the cases with at least N tokens per request (2: the verify shapes)")
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--check", type=int, default=0, metavar="N",
                    help="instead of timing, check N seeded small prefill shapes of the list: each case against itself "
                         "fed in two chained calls per sequence; exit status 1 if a case fails")
    ap.add_argument("--check-max-tokens", type=int, default=2048)
    ap.add_argument("--device-inputs", action="store_true",
                    help="draw prefill inputs on the GPU instead of the host (long lists; same distributions)")
    ap.add_argument("--quiet", action="store_true", help="print every 500th row only (the CSV holds them all)")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("a GPU is required to replay a caselist", file=sys.stderr)
        return 2
    if args.check > 0:
        chosen = select_check_cases(read_caselist(args.caselist, args.limit), args.check, max_tokens=args.check_max_tokens)
        failed = 0
        for case in chosen:
            row = check_case(case)
            failed += not row["ok"]
            print(row, flush=True)
        print(f"checked {len(chosen)} cases, {failed} failed", flush=True)
        return 1 if failed else 0
    # rows are written as they are measured, so that an interrupted replay keeps what it has
    keys = ["family", "phase", "kind", "batch", "heads", "seqlen_q", "tokens", "us", "tokens_per_s", "state_GBps",
            "status", "reason"]
    fh = open(args.csv, "w", newline="") if args.csv else None
    writer = csv.DictWriter(fh, fieldnames=keys) if fh else None
    if writer:
        writer.writeheader()
    try:
        for i, case in enumerate(read_caselist(args.caselist, args.limit)[args.start:]):
            if args.min_seqlen_q and int(case.get("seqlen_q") or 1) < args.min_seqlen_q:
                continue
            row = replay_case(case, reps=args.reps, device_inputs=args.device_inputs)
            if not args.quiet or i % 500 == 0:
                print(args.start + i, row, flush=True)
            if writer:
                writer.writerow(row)
                fh.flush()
            if not args.device_inputs or i % 100 == 99:      # (the caching allocator reuses the blocks in between)
                torch.cuda.empty_cache()
    finally:
        if fh:
            fh.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
