"""Auto-tuner of the k-last decode kernels and the tuned table they are built with.

The reference sweeps its tile tuple (BV, WARP_NUM, STAGE_NUM, HV_PER_CTA) over every decode shape of its
caselists, keeps the fastest combination per (kernel, B, H, HV, dtype, state dtype, mode) in
``lut/tuned_result_<device>.csv`` and generates its dispatch from that file at build time
(scripts/decode/auto_tune.py:57-375, scripts/decode/generate_kernel_instantiations.py).  The gfx950 kernels
have one tile parameter, the rows of the 128-row state tile a wavefront owns (8, 16 or 32), which the
tunable entry points take as BV = 4 x rows (WARP_NUM 4, nothing staged, one value head per workgroup).
This module

* times the three candidates through ``pla_amd.decode.private``'s tunable entry points (graph replays
  over rotating slot sets, so neither the Python facade nor the last-level cache is in the number),
* upserts the winners into ``pla_amd/lut/tuned_result_gfx950.csv`` (same columns as the reference's
  tables; rows of other kernels, modes and state dtypes are preserved),
* renders the tables under ``pla_amd/lut/`` into ``pla_amd/csrc/generated/tuned_table.inc``, which the
  library's row-count choice consults before its size thresholds (``pla_amd.build`` re-renders it on
  every build, so a stale header cannot be compiled in).

Usage:
    python -m pla_amd.autotune --caselist tests/golden/caselist_sample.list
    python -m pla_amd.autotune --case 16,32[,256] [--kernel k_last_packed] [--state-dtype bf16]
    python -m pla_amd.autotune --render-only
"""
import argparse
import csv
import glob
import os
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LUT_DIR = os.path.join(PKG_DIR, "lut")
DEFAULT_TABLE = os.path.join(LUT_DIR, "tuned_result_gfx950.csv")
GENERATED_HEADER = os.path.join(PKG_DIR, "csrc", "generated", "tuned_table.inc")
DEVICE_NAME = "gfx950"

FIELDNAMES = ["device_name", "kernel", "B", "H", "HV", "K", "V", "dtype", "state_dtype",
              "BV", "WARP_NUM", "STAGE_NUM", "HV_PER_CTA", "latency", "unit", "mode"]
KEY_FIELDS = ("device_name", "kernel", "B", "H", "HV", "K", "V", "dtype", "state_dtype", "mode")
KERNELS = ("k_last", "k_last_packed", "k_last_mtp")
# (BV, WARP_NUM, STAGE_NUM, HV_PER_CTA): 8, 16 and 32 rows per wavefront
CANDIDATES = ((32, 4, 1, 1), (64, 4, 1, 1), (128, 4, 1, 1))
ROWS_OF_BV = {32: 8, 64: 16, 128: 32}
KERNEL_CODE = {"k_last": 0, "k_last_packed": 1, "k_last_mtp": 2}
DTYPE_CODE = {"fp32": 0, "bf16": 1, "fp16": 2}          # include/pla_gfx950.h: PLA_F32, PLA_BF16, PLA_F16


# ---- table files --------------------------------------------------------------------------------------

def _normalised(row):
    out = {name: str(row.get(name, "") or "") for name in FIELDNAMES}
    out["device_name"] = out["device_name"] or DEVICE_NAME
    out["state_dtype"] = out["state_dtype"] or "fp32"
    return out


def read_table(path):
    if not os.path.exists(path):
        return []
    with open(path, newline="") as fh:
        return [_normalised(r) for r in csv.DictReader(fh)]


def merge_tuned_rows(path, new_rows):
    """Upsert ``new_rows`` into the table at ``path``: a row replaces the row with the same key (device,
    kernel, shape, dtypes, mode), every other row stays (scripts/decode/auto_tune.py:117-170).
    Returns (rows before, rows after)."""
    existing = read_table(path)
    merged = {tuple(r[k] for k in KEY_FIELDS): r for r in existing}
    for r in new_rows:
        r = _normalised(r)
        merged[tuple(r[k] for k in KEY_FIELDS)] = r

    def order(r):
        return (r["device_name"], KERNELS.index(r["kernel"]) if r["kernel"] in KERNELS else 99, r["mode"],
                r["dtype"], r["state_dtype"], int(r["H"]), int(r["HV"]), int(r["B"]))

    rows = sorted(merged.values(), key=order)
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    with open(path, "w", newline="") as fh:
        writer = csv.DictWriter(fh, fieldnames=FIELDNAMES, lineterminator="\n")
        writer.writeheader()
        writer.writerows(rows)
    return len(existing), len(rows)


def sample_batch_sizes(all_batches, interval=16, max_batch=None):
    """1, interval, 2 x interval, ... and the largest batch of the shape
    (scripts/decode/auto_tune.py:173-184)."""
    top = max(all_batches)
    if max_batch is not None:
        top = min(top, max_batch)
    sampled = [1]
    b = interval
    while b <= top:
        sampled.append(b)
        b += interval
    if top not in sampled:
        sampled.append(top)
    return sampled


def shapes_from_caselists(paths):
    """{(H, HV, dtype): set of batch sizes} over the decode lines of the given caselist files."""
    from .caselist import read_caselist
    shapes = {}
    for path in paths:
        for case in read_caselist(path):
            if case.get("phase") != "D" or case.get("dtype") not in ("bf16", "fp16"):
                continue
            H = case.get("num_heads_qk")
            HV = case.get("num_heads_v", H)
            if not isinstance(H, int) or not isinstance(HV, int) or H <= 0 or HV % H:
                continue
            if case.get("head_dim_qk", 128) != 128 or case.get("head_dim_v", 128) != 128:
                continue
            shapes.setdefault((H, HV, case["dtype"]), set()).add(case.get("batch_size", 1))
    return shapes


# ---- generated header ---------------------------------------------------------------------------------

def render_header(table_paths):
    """Text of the generated table: one row per tuned (kernel, mode, dtypes, H, HV, B), sorted the way
    the library's lookup expects (rows of one shape are consecutive, ascending in B)."""
    rows = []
    for path in sorted(table_paths):
        for r in read_table(path):
            if r["device_name"] != DEVICE_NAME or r["kernel"] not in KERNEL_CODE:
                continue
            if r["K"] != "128" or r["V"] != "128" or int(r["BV"]) not in ROWS_OF_BV:
                continue
            if r["dtype"] not in ("bf16", "fp16") or r["state_dtype"] not in ("fp32", "bf16"):
                continue
            tree = 1 if r["mode"] == "tree" else 0
            rows.append((KERNEL_CODE[r["kernel"]], tree, DTYPE_CODE[r["dtype"]], DTYPE_CODE[r["state_dtype"]],
                         int(r["H"]), int(r["HV"]), int(r["B"]), ROWS_OF_BV[int(r["BV"])]))
    rows = sorted(set(rows))
    lines = ["// Generated by `python -m pla_amd.autotune --render-only` from pla_amd/lut/*.csv.  Do not edit.",
             "// {kernel, tree, act dtype, state dtype, H, HV, B, rows per wavefront}",
             "static const TunedRow kTunedRows[] = {"]
    lines += ["  {%d, %d, %d, %d, %d, %d, %d, %d}," % r for r in rows]
    if not rows:
        lines.append("  {-1, 0, 0, 0, 0, 0, 0, 0},")
    lines += ["};", "static const int kTunedRowCount = %d;" % len(rows), ""]
    return "\n".join(lines)


def table_paths():
    return sorted(glob.glob(os.path.join(LUT_DIR, "*.csv")))


def write_header(path=GENERATED_HEADER):
    text = render_header(table_paths())
    os.makedirs(os.path.dirname(path), exist_ok=True)
    if not os.path.exists(path) or open(path).read() != text:
        with open(path, "w") as fh:
            fh.write(text)
    return path


def header_is_current(path=GENERATED_HEADER):
    return os.path.exists(path) and open(path).read() == render_header(table_paths())


# ---- measurement --------------------------------------------------------------------------------------

def _decode_calls(kernel, B, H, HV, dtype, state_dtype, mtp_t, mode, device, seed=0):
    """Closures ``fn(tile)`` over rotating slot sets for one shape: each runs the tunable entry once."""
    import torch
    from . import workloads
    from .decode.private import (fused_sigmoid_gating_delta_rule_forward_k_last_packed_tunable as packed_tunable,
                                 fused_sigmoid_gating_delta_rule_forward_k_last_tunable as k_last_tunable)
    act = torch.bfloat16 if dtype == "bf16" else torch.float16
    st = torch.float32 if state_dtype == "fp32" else torch.bfloat16
    tile_bytes = 16384 * (4 if state_dtype == "fp32" else 2)
    sets = max(1, min(8, (1 << 31) // max(1, B * HV * tile_bytes)))          # at most 2 GiB of state
    slots = B * sets
    g = torch.Generator().manual_seed(seed)
    idx = [torch.randperm(slots, generator=g)[:B].to(torch.int32).to(device) for _ in range(sets)]
    if kernel == "k_last_packed":
        w = workloads.gdn_decode_packed(B, H=H, HV=HV, pool_slots=slots, seed=seed, device=device, dtype=act)
        call = {k: v for k, v in w.items() if not k.startswith("_")}
        if st != torch.float32:
            call["initial_state_source"] = call["initial_state_source"].to(st)
        return [lambda tile, i=i: packed_tunable(**dict(call, initial_state_indices=i), bv=tile[0], wn=tile[1],
                                                 sn=tile[2], hv_per_cta=tile[3]) for i in idx]
    T = 1 if kernel == "k_last" else mtp_t
    rnd = lambda *s: torch.randn(*s, generator=g)
    pool = (rnd(slots, HV, 128, 128) * 0.1).to(st).to(device)
    parents = None
    if kernel == "k_last_mtp" and mode == "tree":
        parents = torch.tensor([[max(0, t - 2) for t in range(T)]] * B, dtype=torch.int32, device=device)
    mtp = kernel == "k_last_mtp"
    args = dict(
        A_log=rnd(HV).to(device), a=rnd(1, B * T, HV).to(act).to(device), dt_bias=rnd(HV).to(act).to(device),
        softplus_beta=1.0, softplus_threshold=20.0,
        q=rnd(1, B * T, H, 128).to(act).to(device), k=rnd(1, B * T, H, 128).to(act).to(device),
        v=rnd(1, B * T, HV, 128).to(act).to(device), b=rnd(1, B * T, HV).to(act).to(device),
        initial_state_source=pool, scale=128 ** -0.5, use_qk_l2norm_in_kernel=True,
        cu_seqlens=torch.arange(0, B * T + 1, T, dtype=torch.int32, device=device), is_kda=False,
        disable_state_update=mtp,
        intermediate_states_buffer=torch.empty(B, T, HV, 128, 128, dtype=st, device=device) if mtp else None,
        intermediate_state_indices=torch.arange(B, dtype=torch.int32, device=device) if mtp else None,
        cache_steps_or_num_accept=T if mtp else None, retrieve_parent_token=parents)
    out = torch.empty(1, B * T, HV, 128, dtype=act, device=device)
    return [lambda tile, i=i: k_last_tunable(**dict(args, initial_state_indices=i), bv=tile[0], wn=tile[1], sn=tile[2],
                                             hv_per_cta=tile[3], out=out) for i in idx]


def threshold_candidate(tiles):
    """The library's choice for a shape the table does not hold (pick_rows_per_wave, decode_k_last.hip)."""
    return CANDIDATES[2] if tiles >= 512 else CANDIDATES[1] if tiles >= 192 else CANDIDATES[0]


def pick_candidate(timings, tiles, margin=0.015):
    """Fastest candidate, except that the threshold choice stays when it is within ``margin`` of the
    fastest: run-to-run noise must not flip table rows."""
    best = min(CANDIDATES, key=lambda t: timings[t[0]])
    default = threshold_candidate(tiles)
    return default if timings[default[0]] <= timings[best[0]] * (1.0 + margin) else best


def tune_shape(kernel, B, H, HV, dtype="bf16", state_dtype="fp32", mtp_t=4, mode="", device="cuda", reps=20):
    """Times every candidate on one shape.  Returns (best table row, {BV: microseconds})."""
    import torch
    from .caselist import _graph_time_us
    if kernel == "k_last_mtp" and not mode:
        mode = "chain"
    calls = _decode_calls(kernel, B, H, HV, dtype, state_dtype, mtp_t, mode, device)
    timings = {}
    for _ in range(2):                                     # two rounds, the faster counts (clock ramp, first touch)
        for tile in CANDIDATES:
            us = _graph_time_us([lambda fn=fn: fn(tile) for fn in calls], reps)
            timings[tile[0]] = min(us, timings.get(tile[0], us))
    best = pick_candidate(timings, B * HV)
    del calls
    torch.cuda.empty_cache()
    row = dict(device_name=DEVICE_NAME, kernel=kernel, B=B, H=H, HV=HV, K=128, V=128, dtype=dtype,
               state_dtype=state_dtype, BV=best[0], WARP_NUM=best[1], STAGE_NUM=best[2], HV_PER_CTA=best[3],
               latency=f"{timings[best[0]]:.2f}", unit="us", mode=mode)
    return row, timings


def main(argv=None):
    ap = argparse.ArgumentParser(description="Auto-tune the rows-per-wavefront choice of the k-last decode kernels")
    ap.add_argument("--caselist", nargs="*", default=[], help="caselist files or directories of *.list files")
    ap.add_argument("--case", default=None, help="one shape: H,HV[,B]")
    ap.add_argument("--kernel", choices=KERNELS, default=None, help="tune one kernel only (default: all three)")
    ap.add_argument("--dtype", choices=("bf16", "fp16"), default=None, help="activation dtype with --case (default bf16)")
    ap.add_argument("--state-dtype", choices=("fp32", "bf16"), default="fp32")
    ap.add_argument("--mtp-t", type=int, default=4, help="draft tokens of the k_last_mtp shapes")
    ap.add_argument("--mtp-mode", choices=("chain", "tree"), default="chain")
    ap.add_argument("--batch-interval", type=int, default=16)
    ap.add_argument("--max-batch", type=int, default=512)
    ap.add_argument("--batches", default=None, help="explicit batch sizes (comma separated) instead of the sampled ones")
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--output", default=DEFAULT_TABLE)
    ap.add_argument("--render-only", action="store_true", help="only re-render the generated header from the tables")
    args = ap.parse_args(argv)

    if args.render_only:
        print(write_header())
        return 0
    import torch
    if not torch.cuda.is_available():
        print("a GPU is required to tune; --render-only needs none", file=sys.stderr)
        return 2

    if args.case:
        parts = [int(x) for x in args.case.split(",")]
        if len(parts) not in (2, 3):
            ap.error("--case expects H,HV[,B]")
        H, HV = parts[:2]
        batches = [parts[2]] if len(parts) == 3 else sample_batch_sizes([args.max_batch], args.batch_interval)
        shapes = {(H, HV, args.dtype or "bf16"): batches}
    else:
        files = []
        for path in args.caselist:
            files += sorted(glob.glob(os.path.join(path, "*.list"))) if os.path.isdir(path) else [path]
        if not files:
            ap.error("give --caselist or --case")
        shapes = {key: sample_batch_sizes(bs, args.batch_interval, args.max_batch)
                  for key, bs in shapes_from_caselists(files).items()}

    if args.batches:
        explicit = sorted({int(x) for x in args.batches.split(",")})
        shapes = {key: explicit for key in shapes}
    kernels = [args.kernel] if args.kernel else list(KERNELS)
    rows = []
    for (H, HV, dtype), batches in sorted(shapes.items()):
        for kernel in kernels:
            for B in batches:
                mode = args.mtp_mode if kernel == "k_last_mtp" else ""
                row, timings = tune_shape(kernel, B, H, HV, dtype, args.state_dtype, args.mtp_t, mode, reps=args.reps)
                rows.append(row)
                shown = " ".join(f"BV={bv}:{us:.1f}" for bv, us in timings.items())
                print(f"{kernel:>14} H={H} HV={HV} {dtype} state={args.state_dtype} B={B:>4} {mode:>5}  {shown}  -> BV={row['BV']}",
                      flush=True)
    before, after = merge_tuned_rows(args.output, rows)
    print(f"upserted {len(rows)} rows into {args.output} ({before} before, {after} after)")
    if os.path.abspath(args.output).startswith(LUT_DIR):
        print(f"rendered {write_header()}; rebuild the library (python -m pla_amd.build) to compile it in")
    return 0


if __name__ == "__main__":
    sys.exit(main())
