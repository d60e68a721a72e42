#!/usr/bin/env python3
"""Headline benchmark: packed GDN decode at batch 256 over an indexed FP32 k-last pool.

One step = one call of ``fused_sigmoid_gating_delta_rule_forward_k_last_packed`` on the
benchmark configuration (B=256, H=16, HV=32, K=V=128, pool of 4096 slots, 5 % of the
entries padded with -1).  Inputs are resident in HBM before the timed region.  To keep the
256 MB last-level cache from serving the state, consecutive steps use disjoint slot sets
drawn from one seeded permutation of the pool (16 sets of 256 slots = 8.6 GB between two
uses of a slot), which is what a model with many layers does to the cache.

Prints ONE JSON line (see README / DESIGN for the fields).  ``value`` is the state
traffic rate: n_active * HV * 131072 bytes per step / step time.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch of the headline decode kernel, from two rocprofv3 --pmc runs (FETCH_SIZE, then
# WRITE_SIZE, KiB per dispatch) scaled by the same counters of a 1 GiB device copy (x2.00 and x1.00);
# the runs and figures are in profiles/k_last_decode_kernel_gdn_b256.txt.
DECODE_TRAFFIC_BYTES_PER_LAUNCH = 1027728285
BF16_PEAK_TFLOPS = 2500.0


def build_decode_sets(w, n_sets, pool_slots, B, pad_frac, seed, device):
    """Disjoint slot sets for consecutive steps, each with the same number of padded entries."""
    import torch
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(pool_slots, generator=g).to(torch.int32)
    n_pad = int(round(B * pad_frac))
    pad_pos = torch.randperm(B, generator=g)[:n_pad]
    sets = []
    for i in range(n_sets):
        idx = perm[i * B:(i + 1) * B].clone()
        idx[pad_pos] = -1
        sets.append(idx.to(device))
    return sets, B - n_pad


def prepare_decode(device):
    """The headline workload (inputs resident in HBM) and the closure that runs one step on slot set i."""
    from pla_amd.decode import fused_sigmoid_gating_delta_rule_forward_k_last_packed as packed
    from pla_amd.workloads import gdn_decode_packed

    B, H, HV, slots, pad = 256, 16, 32, 4096, 0.05
    w = gdn_decode_packed(B, H=H, HV=HV, pool_slots=slots, pad_frac=pad, seed=101, device=device)
    call = {k: v for k, v in w.items() if not k.startswith("_")}
    sets, n_active = build_decode_sets(w, slots // B, slots, B, pad, 11, device)

    def step(i):
        call["initial_state_indices"] = sets[i % len(sets)]
        packed(**call)

    return dict(workload=w, step=step, n_active=n_active, bytes_state=n_active * HV * 131072)


def time_decode(prep, steps, warmup):
    """W untimed warm-up steps, then exactly K timed steps bracketed by synchronisations."""
    import torch
    step, bytes_state = prep["step"], prep["bytes_state"]
    filler = torch.empty(16 << 20, dtype=torch.float32, device=prep["workload"]["mixed_qkv"].device)
    filler.zero_()                      # the fill kernel is loaded before anything is timed
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    # The op launches on torch's current stream, so torch events bracket exactly these launches.
    # One event pair around the K back-to-back launches: their mean is the kernel's average
    # launch duration (rocprofv3 --kernel-trace reports the same average within 2 %).  A 64 MB fill (about 13 us) runs
    # in front of the start event: while it runs the host enqueues the event and the first steps, so the event's
    # time stamp is followed at once by the first kernel and the K steps are back to back from the first one on
    # (with an idle stream the 10-20 us between enqueueing the event and the first launch would be counted, which
    # is 0.5 % of a 20-step run).  The wall clock below includes the fill.
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    filler.zero_()
    start.record()
    for i in range(steps):
        step(warmup + i)
    end.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    avg_kernel_s = start.elapsed_time(end) * 1e-3 / steps
    return dict(
        wall_s=wall, ms_per_step=wall / steps * 1e3, bytes_state=bytes_state, n_active=prep["n_active"],
        kernel_us_avg=avg_kernel_s * 1e6,
        achieved_gbps=bytes_state / avg_kernel_s / 1e9,
        value_gbps=bytes_state * steps / wall / 1e9, workload=prep["workload"])


def bench_decode_bf16_pool(w, steps, device):
    """The headline workload with the pool stored in bf16 (FP32 recurrence, tiles widened on load and
    rounded on store): half the state bytes per step."""
    import torch
    from pla_amd.decode import fused_sigmoid_gating_delta_rule_forward_k_last_packed as packed
    B, HV, slots, pad = 256, 32, 4096, 0.05
    call = {k: v for k, v in w.items() if not k.startswith("_")}
    sets, n_active = build_decode_sets(w, slots // B, slots, B, pad, 11, device)
    pool32 = call["initial_state_source"]
    pool16 = torch.empty(pool32.shape, dtype=torch.bfloat16, device=device)
    for s0 in range(0, slots, 256):
        pool16[s0:s0 + 256].copy_(pool32[s0:s0 + 256])
    call["initial_state_source"] = pool16

    def step(i):
        call["initial_state_indices"] = sets[i % len(sets)]
        packed(**call)

    for i in range(16):
        step(i)
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(steps):
        step(i)
    end.record()
    torch.cuda.synchronize()
    us = start.elapsed_time(end) / steps * 1e3
    nbytes = n_active * HV * 65536
    return {"config1_bf16_pool_us": round(us, 2), "config1_bf16_pool_state_GBps": round(nbytes / us / 1e3, 1)}


PREFILL_SEED = 348      # ragged_lengths(8, 512, 8192, 348) sums to 32 810 tokens
GDN_FLOP_PER_TOKEN = 4718592      # 2 * [HV (3 K V + 2 C V) + H (2 C K)], C = 64, K = V = 128, HV = 32, H = 16
KDA_FLOP_PER_TOKEN = 5242880      # same with HV = H = 32 (one gram per head)
# HBM bytes per call from rocprofv3 --pmc FETCH_SIZE (x2.00) and WRITE_SIZE (x1.00), summed over the kernels of
# one call (profiles/gdn_prefill_kernels_32k.txt, profiles/kda_prefill_kernels_64k.txt)
GDN_PREFILL_TRAFFIC_BYTES_PER_CALL = 1532000000
KDA_PREFILL_TRAFFIC_BYTES_PER_CALL = 11129000000


def cpu_baseline_prefill(w):
    """The CPU oracle's token recurrence (FP32, vectorised over heads) over ALL tokens of config 3, one pass, all
    host cores: tokens/s beside the GPU figure."""
    import torch
    from oracle import gdn_prefill_reference
    m = w["_meta"]
    T, H, HV = m["T"], m["H"], m["HV"]
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    packed = w["packed_qkv"].cpu()
    q = packed[:, : H * 128].reshape(T, H, 128)
    k = packed[:, H * 128: 2 * H * 128].reshape(T, H, 128)
    v = packed[:, 2 * H * 128:].reshape(T, HV, 128)
    S0 = w["initial_state"][w["initial_state_indices"].long()].cpu()
    args = (q, k, v, w["raw_gate_a"].cpu(), w["raw_beta_b"].cpu(), w["A_log"].cpu(), w["dt_bias"].cpu(), m["offsets"], S0)
    t0 = time.perf_counter()
    gdn_prefill_reference(*args, scale=w["scale"])
    t = time.perf_counter() - t0
    tokens = m["offsets"][-1]
    return dict(value=round(tokens / t, 1), unit="tokens/s", cores=threads, kind="port",
                sample="all %d tokens of the 8 sequences, one pass of the token recurrence (%.1f s)" % (tokens, t),
                threads_torch=torch.get_num_threads())


def time_calls(run, steps, warmup, device):
    """Mean milliseconds of `steps` back-to-back calls of `run` after `warmup` untimed ones.

    A prefill call is a Python wrapper around several kernel launches: on an idle stream the time between
    enqueueing the start event and the first kernel of the first call (allocations, argument checks, the first
    launches: a few hundred microseconds) would be counted, which is a tenth of a five-call run.  A 2 GiB fill runs in
    front of the start event instead: while it runs the host enqueues the event and the first calls, so the event's
    time stamp is followed at once by the first kernel and the calls are back to back from the first one on."""
    import torch
    filler = torch.empty(512 << 20, dtype=torch.float32, device=device)
    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    filler.zero_()
    start.record()
    for _ in range(steps):
        run()
    end.record()
    torch.cuda.synchronize()
    del filler
    return start.elapsed_time(end) / steps


def bench_prefill(steps, warmup, device, cpu_leg=False):
    """Config 3: GDN chunk-64 prefill, 8 ragged sequences (about 32K tokens), indexed FP32 pool."""
    import torch
    from pla_amd.prefill.flashqla import gdn_prefill_packed_qkv_fwd
    from pla_amd.workloads import gdn_prefill_packed, ragged_lengths
    lengths = ragged_lengths(8, 512, 8192, PREFILL_SEED)
    w = gdn_prefill_packed(lengths, H=16, HV=32, pool_slots=64, seed=PREFILL_SEED, device=device)
    call = {k: v for k, v in w.items() if not k.startswith("_")}
    packed = call.pop("packed_qkv")
    a, b, A, dt, cu = (call.pop(n) for n in ("raw_gate_a", "raw_beta_b", "A_log", "dt_bias", "cu_seqlens"))

    def run():
        return gdn_prefill_packed_qkv_fwd(packed, a, b, A, dt, cu, output_final_state=False, **call)

    ms = time_calls(run, steps, warmup, device)
    T = sum(lengths)
    tflops = GDN_FLOP_PER_TOKEN * T / (ms * 1e-3) / 1e12
    extra = dict(cpu_baseline=cpu_baseline_prefill(w)) if cpu_leg else {}
    return dict(tokens=T, lengths=lengths, steps=steps, warmup=warmup, ms_per_call=round(ms, 4),
                tokens_per_s=round(T / ms * 1e3, 1), **extra,
                roofline=dict(bound="mfma", achieved=round(tflops, 2), peak=BF16_PEAK_TFLOPS, unit="TFLOP/s",
                              frac=round(tflops / BF16_PEAK_TFLOPS, 4), traffic=GDN_PREFILL_TRAFFIC_BYTES_PER_CALL,
                              hbm_GBps=round(GDN_PREFILL_TRAFFIC_BYTES_PER_CALL / ms / 1e6, 1),
                              flop_per_token=GDN_FLOP_PER_TOKEN,
                              note="algorithmic flops (dense) over the whole call; fp16 operands, FP32 accumulation "
                                   "(v_mfma_f32_16x16x32_f16, the rate of the bf16 instruction): "
                                   "key-side preparation + fused sweeps (chunk tables worked out inside them), two pipelined stages, steady state after "
                                   "%d warm-up calls; " % warmup +
                                   "traffic is a constant from rocprofv3 --pmc runs (profiles/gdn_prefill_kernels_32k.txt)"))


# GDN prefill shapes the reference publishes timings for (reports/prefill_bench_20260911.json, family gdn,
# num_v_heads 32 / 16 q/k heads, bf16, measured by its authors on a ZW-M890P PPU): lengths -> published ms
REFERENCE_GDN_PREFILL_MS = (([2048] * 8, 1.4865), ([4096] * 4, 1.5035), ([16384], 2.241))


def bench_prefill_reference_shapes(steps, device, only=None, host_offsets=True):
    """The batch x length shapes of the reference's own prefill report, next to its published times (other
    hardware: a ratio of two machines, not a like-for-like comparison).  only: a "BxL" string, that shape alone
    (any batch and length, for profiling; without a published time unless it is one of the report's), or ragged
    lengths joined by "+" ("8000+7000+1000").  host_offsets False: the call goes without ``raw_cu_seqlens``."""
    import torch
    from pla_amd.prefill.flashqla import gdn_prefill_packed_qkv_fwd
    from pla_amd.workloads import gdn_prefill_packed
    rows = []
    shapes = REFERENCE_GDN_PREFILL_MS
    if only is not None:
        if "+" in only:
            shapes = (([int(x) for x in only.split("+")], None),)
        else:
            batch, length = (int(x) for x in only.lower().split("x"))
            published = dict(((len(l), l[0]), ms) for l, ms in REFERENCE_GDN_PREFILL_MS)
            shapes = (([length] * batch, published.get((batch, length))),)
    for lengths, published_ms in shapes:
        w = gdn_prefill_packed(lengths, H=16, HV=32, pool_slots=len(lengths) + 2, seed=1, device=device)
        call = {k: v for k, v in w.items() if not k.startswith("_")}
        packed = call.pop("packed_qkv")
        a, b, A, dt, cu = (call.pop(n) for n in ("raw_gate_a", "raw_beta_b", "A_log", "dt_bias", "cu_seqlens"))
        if not host_offsets:
            call["raw_cu_seqlens"] = None
        run = lambda: gdn_prefill_packed_qkv_fwd(packed, a, b, A, dt, cu, **call)
        ms = time_calls(run, steps, 20, device)
        ragged = len(set(lengths)) > 1
        rows.append({"shape": "+".join(str(n) for n in lengths) + " tokens" if ragged else "%d x %d tokens" % (len(lengths), lengths[0]),
                     "host_offsets": bool(host_offsets), "ms_per_call": round(ms, 4),
                     "tokens_per_s": round(sum(lengths) / ms * 1e3, 1), "reference_ppu_ms": published_ms,
                     "reference_ms_over_ours": round(published_ms / ms, 2) if published_ms else None})
        del w, call, packed
        torch.cuda.empty_cache()
    return rows


def bench_prefill_kda(steps, device, cpu_leg=False):
    """Config 4: KDA chunk-64 prefill of one 65 536-token sequence, 32 heads (32 independent chains)."""
    import torch
    from pla_amd.prefill.flashkdapro import flashkda_fwd
    from pla_amd.workloads import kda_prefill
    T = 65536
    c = {k: v for k, v in kda_prefill(T=T, H=32, seed=4, device=device).items() if not k.startswith("_")}

    def run():
        flashkda_fwd(c["q"], c["k"], c["v"], c["g"], c["beta"], c["A_log"], c["dt_bias"], c["out"], scale=c["scale"],
                     lower_bound=c["lower_bound"], initial_state=c["initial_state"], final_state=c["final_state"],
                     cu_seqlens=c["cu_seqlens"])

    extra = {}
    if cpu_leg:                                   # ahead of the GPU leg: what follows this function finds a busy GPU
        # the CPU oracle's token recurrence over a prefix of the same sequence (the whole of it would take minutes)
        import time as _time
        from oracle import kda_prefill_reference
        prefix = 8192
        threads = os.cpu_count() or 1
        torch.set_num_threads(threads)
        cpu = {k: (v[:prefix].cpu() if k in ("q", "k", "v", "g", "beta") else v.cpu() if torch.is_tensor(v) else v)
               for k, v in c.items()}
        t0 = _time.perf_counter()
        kda_prefill_reference(cpu["q"], cpu["k"], cpu["v"], cpu["g"], cpu["beta"], cpu["A_log"], cpu["dt_bias"],
                              [0, prefix], cpu["initial_state"], scale=c["scale"], lower_bound=c["lower_bound"])
        t = _time.perf_counter() - t0
        extra["cpu_baseline"] = dict(value=round(prefix / t, 1), unit="tokens/s", cores=threads, kind="port",
                                     sample="the first %d tokens of the 65 536-token sequence, all 32 heads, one pass of "
                                            "the token recurrence (%.1f s)" % (prefix, t),
                                     threads_torch=torch.get_num_threads())
    ms = time_calls(run, steps, 3, device)
    tflops = KDA_FLOP_PER_TOKEN * T / (ms * 1e-3) / 1e12
    return dict(tokens=T, steps=steps, warmup=3, ms_per_call=round(ms, 4), tokens_per_s=round(T / ms * 1e3, 1), **extra,
                roofline=dict(bound="mfma", achieved=round(tflops, 2), peak=BF16_PEAK_TFLOPS, unit="TFLOP/s",
                              frac=round(tflops / BF16_PEAK_TFLOPS, 4), traffic=KDA_PREFILL_TRAFFIC_BYTES_PER_CALL,
                              hbm_GBps=round(KDA_PREFILL_TRAFFIC_BYTES_PER_CALL / ms / 1e6, 1),
                              flop_per_token=KDA_FLOP_PER_TOKEN))


def bench_prefill_host_time(device, calls=200):
    """Host time of one prefill call (argument checks, workspace from torch's allocator, launches; the stream is not
    waited for): 8 x 2048-token GDN prefill and 1 x 2048-token KDA prefill, eager, best of three batches.  The GPU
    needs longer than the host for these shapes, so the launch queue is drained between batches and the batch is
    short enough not to fill it."""
    import torch
    from pla_amd.prefill.flashqla import gdn_prefill_packed_qkv_fwd
    from pla_amd.prefill.flashkdapro import flashkda_fwd
    from pla_amd.workloads import gdn_prefill_packed, kda_prefill
    out = {}
    w = gdn_prefill_packed([2048] * 8, H=16, HV=32, pool_slots=10, seed=1, device=device)
    call = {k: v for k, v in w.items() if not k.startswith("_")}
    packed = call.pop("packed_qkv")
    a, b, A, dt, cu = (call.pop(n) for n in ("raw_gate_a", "raw_beta_b", "A_log", "dt_bias", "cu_seqlens"))
    c = {k: v for k, v in kda_prefill(T=2048, H=32, seed=4, device=device).items() if not k.startswith("_")}
    runs = {
        "gdn_8x2048": lambda: gdn_prefill_packed_qkv_fwd(packed, a, b, A, dt, cu, output_final_state=False, **call),
        "kda_1x2048": lambda: flashkda_fwd(c["q"], c["k"], c["v"], c["g"], c["beta"], c["A_log"], c["dt_bias"], c["out"],
                                           scale=c["scale"], lower_bound=c["lower_bound"], initial_state=c["initial_state"],
                                           final_state=c["final_state"], cu_seqlens=c["cu_seqlens"]),
    }
    for name, run in runs.items():
        for _ in range(20):
            run()
        best = 1e9
        for _ in range(3):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(calls // 10):
                run()
            best = min(best, (time.perf_counter() - t0) / (calls // 10) * 1e6)
        torch.cuda.synchronize()
        out[name] = round(best, 1)
    return out


def copy_calibration(device, reps=5):
    """A plain device-to-device copy of known size (1 GiB read + 1 GiB written per launch): the
    reference point that scales the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run."""
    import torch
    src = torch.empty(1 << 28, dtype=torch.float32, device=device).normal_()
    dst = torch.empty_like(src)
    for _ in range(reps):
        dst.copy_(src)
    torch.cuda.synchronize()
    return dict(bytes_read=src.numel() * 4, bytes_written=src.numel() * 4, launches=reps)


def bench_small_decode(device, steps=200):
    """Config 0 (B=8 packed GDN decode) and config 2 (KDA MTP verify T=4, B=64 + commit): kernel times."""
    import torch
    from pla_amd.decode import fused_sigmoid_gating_delta_rule_forward_k_last_packed as packed
    from pla_amd.decode.kda_replayssm_sglang import kda_mtp_verify
    from pla_amd.workloads import gdn_decode_packed, kda_mtp_verify as make_verify
    out = {}
    w = gdn_decode_packed(8, seed=100, device=device)
    call = {k: v for k, v in w.items() if not k.startswith("_")}

    def timed(fn):
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(steps):
            fn()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / steps * 1e3

    us = timed(lambda: packed(**call))
    out["config0_gdn_decode_b8_us"] = round(us, 2)
    out["config0_state_GBps"] = round(8 * 32 * 131072 / us / 1e3, 1)
    v = make_verify(B=64, pool_slots=1024, seed=202, device=device)
    # Consecutive steps take disjoint sets of 64 slots (16 sets cover the pool of 1024: 2.1 GB of state), so that no
    # step finds its tiles in the 256 MB last-level cache, as the headline does.
    B, slots = 64, 1024
    perm = torch.randperm(slots, generator=torch.Generator().manual_seed(7)).to(device=device, dtype=torch.int32)
    slot_sets = [perm[i * B:(i + 1) * B].contiguous() for i in range(slots // B)]
    turn = [0]

    def next_set():
        turn[0] = (turn[0] + 1) % len(slot_sets)
        return slot_sets[turn[0]]

    us = timed(lambda: kda_mtp_verify(v["q"], v["k"], v["v"], v["log_decay"], v["beta"], v["state"], next_set(),
                                      v["cu_seqlens"], scale=v["scale"]))
    out["config2_kda_verify_t4_b64_us"] = round(us, 2)
    out["config2_verify_state_read_GBps"] = round(64 * 32 * 65536 / us / 1e3, 1)
    out["config2_slot_sets"] = len(slot_sets)
    # accepted-prefix commit of the same window: per-slot records, num_accepted ~ U{0..4}
    from pla_amd.decode.kda_replayssm_sglang import fold_accepted_prefix
    T, HV = 4, 32
    rawk = torch.zeros(slots, HV, T, 128, dtype=torch.bfloat16, device=device)
    rawv = torch.zeros_like(rawk)
    gk = torch.zeros(slots, HV, T, 128, dtype=torch.float32, device=device)
    beta = torch.zeros(slots, HV, T, dtype=torch.float32, device=device)
    for ids in slot_sets:                             # every set of slots holds the records of the same draft window
        idx = ids.long()
        rawk[idx] = v["k"][0].view(B, T, HV, 128).transpose(1, 2)
        rawv[idx] = v["v"][0].view(B, T, HV, 128).transpose(1, 2)
        gk[idx] = v["log_decay"].view(B, T, HV, 128).transpose(1, 2)
        beta[idx] = v["beta"].view(B, T, HV).transpose(1, 2)
    us = timed(lambda: fold_accepted_prefix(v["state"][None], rawv[None], rawk[None], gk[None], beta[None],
                                            next_set(), v["num_accepted"], null_block_id=-1))
    touched = int((v["num_accepted"] > 0).sum().item())
    out["config2_kda_commit_b64_us"] = round(us, 2)
    out["config2_commit_state_GBps"] = round(touched * 32 * 2 * 65536 / us / 1e3, 1)     # tiles read and written
    return out


def bench_decode_mega(device, steps=100, B=256, H=12, sets=16):
    """Fused KDA decode step (conv + gate + recurrence + gated RMSNorm), B=256 requests x 12 heads
    (the per-rank head count of the reference's Kimi K3 TP8 fixture).  Consecutive steps use
    disjoint slot sets so that no state tile is served from a cache."""
    import torch
    from pla_amd.decode.kda import fused_kda_decode_mega_forward as mega
    from pla_amd.workloads import kda_decode_mega
    w = kda_decode_mega(B, H, seed=404, device=device, slots=sets * B + 2)
    base = w["state_indices"].clone()
    idx = [(base + i * B).contiguous() for i in range(sets)]
    out = torch.empty(1, B, H, 128, dtype=torch.bfloat16, device=device)

    def step(i):
        mega(x=w["x"], weight=w["weight"], bias=None, conv_state=w["conv_state"], raw_g=w["raw_g"],
             raw_beta=w["raw_beta"], a_log=w["a_log"], dt_bias=w["dt_bias"], state_indices=idx[i % sets],
             state=w["state"], out=out, lower_bound=-5.0, output_gate=w["output_gate"],
             norm_weight=w["norm_weight"], norm_eps=1e-5)

    for i in range(sets):
        step(i)
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for i in range(steps):
        step(i)
    e.record()
    torch.cuda.synchronize()
    us = s.elapsed_time(e) / steps * 1e3
    state_bytes = B * H * 131072
    return {"workload": "fused KDA decode step, B=%d, H=%d, bf16 activations, lower-bound gate, gated RMSNorm" % (B, H),
            "us_per_step": round(us, 2), "state_GBps": round(state_bytes / us / 1e3, 1),
            "frac_of_hbm_peak": round(state_bytes / us / 1e3 / HBM_PEAK_GBPS, 4)}


def bench_replay_verify(device, steps=100, N=64, H=32, T=4):
    """Config 2 through the production contract: conv front end + gate + verify of 4 draft tokens with replay
    records and scratch windows in one launch, then the commit (fold of the accepted prefix + conv rollback)."""
    import types
    import torch
    from pla_amd.decode.kda_replayssm_sglang import fused_kda_decode_mtp_dspark, commit_kda_replayssm_after_verify
    from pla_amd.workloads import kda_replay_verify
    w = kda_replay_verify(N, H, T, seed=505, device=device, slots=1024, ring_len=max(8, T), onorm=True, strided=False)
    w["intermediate_state_indices"] = torch.arange(N, dtype=torch.int32, device=device)
    out = torch.empty(1, N * T, H, 128, dtype=torch.bfloat16, device=device)

    def timed(fn):
        # replayed from a graph: the Python facade (argument checks) costs more than these kernels
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            fn()
        for _ in range(10):
            graph.replay()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(steps):
            graph.replay()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / steps * 1e3

    us_verify = timed(lambda: fused_kda_decode_mtp_dspark(out=out, **w))
    g = torch.Generator().manual_seed(6)
    accept = torch.randint(0, T + 1, (N,), generator=g).to(torch.int32).to(device)
    spec = types.SimpleNamespace(
        temporal=w["recurrent_state"][None], replayssm_rawv=w["replayssm_rawv"][None],
        replayssm_rawk=w["replayssm_rawk"][None], replayssm_g=w["replayssm_g"][None],
        replayssm_beta=w["replayssm_beta"][None],
        conv=[w["cs_q"][None], w["cs_k"][None], w["cs_v"][None]],
        intermediate_conv_window=[w["intermediate_conv_q"][None], w["intermediate_conv_k"][None],
                                  w["intermediate_conv_v"][None]])
    last = accept.long() - 1
    us_commit = timed(lambda: commit_kda_replayssm_after_verify(
        spec_state=spec, state_batch_indices=w["ssm_state_indices"], accept_lens=accept,
        last_correct_step_indices=last))
    return {"workload": "KDA verify with replay records + commit, B=%d, H=%d, %d draft tokens, gated RMSNorm" % (N, H, T),
            "verify_us": round(us_verify, 2), "verify_state_read_GBps": round(N * H * 65536 / us_verify / 1e3, 1),
            "commit_us": round(us_commit, 2)}


def bench_replay_paged(device, steps=100, N=64, H=32, Q=4, layout="SD"):
    """The same verify + commit through the request-row (vLLM) contract: paged conv history + FP32 checkpoints,
    records per request row, device-side commit plan, fold into the final slot, conv windows into the paged history."""
    import torch
    from pla_amd.decode.kda_replayssm_vllm import KDAReplayCommitContext, kda_replay_verify
    from pla_amd.workloads import kda_replay_paged
    w = kda_replay_paged(N, H, Q, slots=1024, layout=layout, seed=606, device=device)
    out = torch.empty(w.tokens, H * 128, dtype=torch.bfloat16, device=device)

    def timed(fn):
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            fn()
        for _ in range(10):
            graph.replay()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(steps):
            graph.replay()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / steps * 1e3

    us_verify = timed(lambda: kda_replay_verify(out=out, **w.verify))
    ctx = KDAReplayCommitContext.create([w.layer], Q, N, layout, 0)
    g = torch.Generator().manual_seed(7)
    sampled = torch.randint(0, Q + 1, (N,), generator=g).to(torch.int32).to(device)
    us_commit = timed(lambda: ctx.commit(sampled, w.source, w.offsets, token_capacity=w.tokens))
    touched = int((sampled > 0).sum())
    return {"workload": "request-row KDA replay verify + commit over paged checkpoints (%s pages), B=%d, H=%d, %d draft tokens"
                        % (layout, N, H, Q),
            "verify_us": round(us_verify, 2), "verify_state_read_GBps": round(N * H * 65536 / us_verify / 1e3, 1),
            "commit_us": round(us_commit, 2), "commit_state_GBps": round(touched * H * 131072 / us_commit / 1e3, 1)}


def cpu_baseline_decode(w, reps=20):
    """The CPU oracle (a PyTorch restatement of the reference recurrence) timed on the whole workload: all 256
    requests (the padded ones are skipped, as on the GPU), one step, median of `reps` steps, all host cores."""
    import torch
    from oracle import k_last_reference
    meta = w["_meta"]
    B, H, HV = meta["B"], meta["H"], meta["HV"]
    threads = os.cpu_count() or 1
    torch.set_num_threads(threads)
    idx = w["initial_state_indices"].cpu().tolist()
    active = [s for s in idx if s >= 0]
    remap = {s: i for i, s in enumerate(active)}
    state = w["initial_state_source"][torch.tensor(active, device=w["initial_state_source"].device)].cpu()
    mixed = w["mixed_qkv"].cpu()
    q = mixed[:, : H * 128].reshape(B, H, 128)
    k = mixed[:, H * 128: 2 * H * 128].reshape(B, H, 128)
    v = mixed[:, 2 * H * 128:].reshape(B, HV, 128)
    a, b = w["a"].cpu(), w["b"].cpu()
    slots = [remap.get(s, -1) for s in idx]
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        k_last_reference(q, k, v, a, b, w["A_log"].cpu(), w["dt_bias"].cpu(), state, slots, [1] * B,
                         scale=w["scale"], use_qk_l2norm=True, is_kda=False)
        times.append(time.perf_counter() - t0)
    t = statistics.median(times)
    n = len(active)
    # the same oracle on one thread, on the first 32 requests (a bounded sample: the whole batch takes seconds per step)
    sub = 32
    sub_slots = slots[:sub]
    n_sub = sum(1 for x in sub_slots if x >= 0)
    torch.set_num_threads(1)
    t0 = time.perf_counter()
    k_last_reference(q[:sub], k[:sub], v[:sub], a[:sub], b[:sub], w["A_log"].cpu(), w["dt_bias"].cpu(), state, sub_slots,
                     [1] * sub, scale=w["scale"], use_qk_l2norm=True, is_kda=False)
    t1 = time.perf_counter() - t0
    torch.set_num_threads(threads)
    single = dict(value=round(n_sub * HV * 131072 / t1 / 1e9, 2), unit="GB/s", cores=1,
                  sample="the first %d requests (%d active), one step (%.1f ms)" % (sub, n_sub, t1 * 1e3))
    return dict(value=n * HV * 131072 / t / 1e9, unit="GB/s", cores=threads, kind="port", single_thread=single,
                sample="all 256 requests (%d active), one step, median of %d steps (%.1f ms/step; %.0f us per "
                       "active request)" % (n, reps, t * 1e3, t / n * 1e6),
                threads_torch=torch.get_num_threads())


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--decode-only", action="store_true", help="skip the secondary decode / prefill measurements")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the two prefill workloads (for rocprofv3 --pmc byte counters) and print their objects")
    ap.add_argument("--prefill-shape", metavar="BxL", default=None,
                    help="run only the GDN prefill of B sequences of L tokens (H=16, HV=32), e.g. 1x16384, or of ragged "
                         "lengths joined by +, e.g. 8000+7000+1000+2000+3000, and print its row")
    ap.add_argument("--no-host-offsets", action="store_true",
                    help="with --prefill-shape: call without raw_cu_seqlens (the host then plans nothing from the lengths)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch a 1 GiB device copy (reference for scaling rocprofv3 --pmc byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the decode and prefill "
              "kernels shard by request / head without communication); run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (MI355X)", file=sys.stderr)
        sys.exit(2)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.prefill_shape:
        print(json.dumps({"prefill_reference_shapes": bench_prefill_reference_shapes(max(args.steps // 2, 10), device,
                                                                                     only=args.prefill_shape,
                                                                                     host_offsets=not args.no_host_offsets)}))
        return
    if args.prefill_only:
        result = {"prefill": bench_prefill(max(args.steps, 50), 50, device)}
        torch.cuda.empty_cache()
        result["prefill_kda"] = bench_prefill_kda(max(args.steps // 4, 5), device)
        if args.copy_calibration:
            result["copy_calibration"] = copy_calibration(device)
        print(json.dumps(result))
        return
    # Order of the run: the CPU legs and the secondary workloads first, the headline decode last.  The driver's
    # short runs (5 warm-up steps are under a millisecond of GPU work) then measure the headline on a GPU that has
    # been busy for a while, as it is in serving, instead of one that has just left idle clocks.
    prep = prepare_decode(device)
    cpu_leg = None if args.no_cpu_baseline else cpu_baseline_decode(prep["workload"])
    extra = {}
    if not args.decode_only:
        extra["other_decode"] = bench_small_decode(device)
        extra["other_decode"].update(bench_decode_bf16_pool(prep["workload"], args.steps, device))
        extra["decode_mega"] = bench_decode_mega(device)
        extra["replay_verify"] = bench_replay_verify(device)
        extra["replay_paged"] = bench_replay_paged(device)
        torch.cuda.empty_cache()
        # (the host-time leg keeps the GPU nearly idle, so it does not run last: what precedes the headline is GPU work)
        extra["prefill_host_us"] = bench_prefill_host_time(device)
        torch.cuda.empty_cache()
        extra["prefill"] = bench_prefill(max(args.steps, 50), 50, device, cpu_leg=not args.no_cpu_baseline)
        torch.cuda.empty_cache()
        # (at least 50 timed calls per shape: the first calls of a process run 10-20 % slower, and ten calls of 0.2 ms
        # after twenty warm-up calls still show it)
        extra["prefill_reference_shapes"] = bench_prefill_reference_shapes(max(args.steps // 2, 50), device)
        extra["prefill_kda"] = bench_prefill_kda(max(args.steps // 4, 5), device, cpu_leg=not args.no_cpu_baseline)
        torch.cuda.empty_cache()
    d = time_decode(prep, args.steps, args.warmup)
    result = {
        "metric": "gdn_packed_decode_state_hbm_GBps@B=256",
        "value": round(d["value_gbps"], 1),
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(d["ms_per_step"], 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: GDN packed-QKV decode, 1 step, B=256 (243 active, 13 padded), "
                               "H=16, HV=32, K=V=128, FP32 k-last pool of 4096 slots, bf16 activations",
                   "batch": 256, "n_active": d["n_active"], "pool_slots": 4096,
                   "slot_rotation": "16 disjoint slot sets, one per consecutive step"},
        "decode_us_per_step": round(d["kernel_us_avg"], 2),
        "roofline": {"bound": "hbm", "achieved": round(d["achieved_gbps"], 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(d["achieved_gbps"] / HBM_PEAK_GBPS, 4),
                     "traffic": DECODE_TRAFFIC_BYTES_PER_LAUNCH,
                     "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per launch, scaled by a 1 GiB device copy "
                                       "(profiles/k_last_decode_kernel_gdn_b256.txt); a constant here, not measured in this run",
                     "kernel": "k_last_decode_kernel<bf16,GDN,rows_per_wave=32>",
                     "bytes_per_launch": d["bytes_state"], "launch_us_avg": round(d["kernel_us_avg"], 2)},
        "run_order": "CPU baselines and the secondary workloads first, the headline steps last",
    }
    if cpu_leg is not None:
        result["cpu_baseline"] = cpu_leg
    result.update(extra)
    if args.copy_calibration:
        result["copy_calibration"] = copy_calibration(device)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
