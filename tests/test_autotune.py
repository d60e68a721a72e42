"""Auto-tuner: table upserts, batch sampling, the generated header and the compiled-in lookup.

Modelled on the reference's tests of its tuned tables (tests/test_generated_k_last.py:114-203, 247-276:
upserts preserve other kernels / modes / state dtypes, the built header follows the table files)."""
import os

import pytest
import torch

from pla_amd import _lib, autotune


def _row(kernel, B, bv, mode="", state_dtype="fp32", H=16, HV=32, dtype="bf16"):
    return dict(device_name="gfx950", kernel=kernel, B=B, H=H, HV=HV, K=128, V=128, dtype=dtype,
                state_dtype=state_dtype, BV=bv, WARP_NUM=4, STAGE_NUM=1, HV_PER_CTA=1, latency="1.00", unit="us", mode=mode)


def test_upsert_replaces_same_key_and_preserves_the_rest(tmp_path):
    path = str(tmp_path / "tuned_result_gfx950.csv")
    first = [_row("k_last_packed", 8, 32), _row("k_last_packed", 8, 64, state_dtype="bf16"),
             _row("k_last_mtp", 8, 32, mode="chain"), _row("k_last_mtp", 8, 64, mode="tree"), _row("k_last", 8, 32)]
    assert autotune.merge_tuned_rows(path, first) == (0, 5)
    assert autotune.merge_tuned_rows(path, [_row("k_last_packed", 8, 128), _row("k_last_mtp", 8, 128, mode="chain"),
                                            _row("k_last_packed", 16, 64)]) == (5, 6)
    rows = {(r["kernel"], r["B"], r["state_dtype"], r["mode"]): r["BV"] for r in autotune.read_table(path)}
    assert rows == {("k_last_packed", "8", "fp32", ""): "128", ("k_last_packed", "8", "bf16", ""): "64",
                    ("k_last_packed", "16", "fp32", ""): "64", ("k_last_mtp", "8", "fp32", "chain"): "128",
                    ("k_last_mtp", "8", "fp32", "tree"): "64", ("k_last", "8", "fp32", ""): "32"}
    header = open(path).readline().strip().split(",")
    assert header == autotune.FIELDNAMES            # the reference's columns, mode last


def test_table_without_state_dtype_and_mode_columns_is_migrated(tmp_path):
    path = str(tmp_path / "legacy.csv")
    with open(path, "w") as fh:
        fh.write("device_name,kernel,B,H,HV,K,V,dtype,BV,WARP_NUM,STAGE_NUM,HV_PER_CTA,latency,unit\n"
                 "gfx950,k_last,4,16,32,128,128,bf16,32,4,1,1,5.0,us\n")
    autotune.merge_tuned_rows(path, [_row("k_last", 64, 128)])
    rows = autotune.read_table(path)
    assert [(r["B"], r["state_dtype"], r["mode"]) for r in rows] == [("4", "fp32", ""), ("64", "fp32", "")]


def test_sample_batch_sizes():
    assert autotune.sample_batch_sizes({1, 70}, 16) == [1, 16, 32, 48, 64, 70]
    assert autotune.sample_batch_sizes({3, 2000}, 16, max_batch=40) == [1, 16, 32, 40]
    assert autotune.sample_batch_sizes({1}, 16) == [1]


def test_pick_candidate_keeps_the_threshold_choice_within_the_margin():
    assert autotune.pick_candidate({32: 10.0, 64: 10.05, 128: 11.0}, 256)[0] == 64      # threshold choice, 0.5 % off
    assert autotune.pick_candidate({32: 10.0, 64: 10.5, 128: 11.0}, 256)[0] == 32       # 5 % off: the fastest wins
    assert [autotune.threshold_candidate(t)[0] for t in (32, 191, 192, 511, 512)] == [32, 32, 64, 64, 128]


def test_shapes_from_the_sample_caselist():
    here = os.path.dirname(os.path.abspath(__file__))
    shapes = autotune.shapes_from_caselists([os.path.join(here, "golden", "caselist_sample.list")])
    assert shapes[(16, 32, "bf16")] >= {1, 8, 1823}
    assert all(HV % H == 0 for H, HV, _ in shapes)


def test_render_skips_foreign_rows(tmp_path):
    path = str(tmp_path / "t.csv")
    rows = [_row("k_last_packed", 8, 64), dict(_row("k_last_packed", 8, 32), device_name="ZW-M890P"),
            dict(_row("k_last_packed", 9, 16)), dict(_row("k_last_packed", 10, 64), K=64),
            _row("k_last_mtp", 4, 128, mode="tree", dtype="fp16", state_dtype="bf16")]
    autotune.merge_tuned_rows(path, rows)
    text = autotune.render_header([path])
    assert "{1, 0, 1, 0, 16, 32, 8, 16}," in text and "{2, 1, 2, 1, 16, 32, 4, 32}," in text
    assert "kTunedRowCount = 2;" in text
    assert "kTunedRowCount = 0;" in autotune.render_header([])


def test_generated_header_follows_the_tables():
    assert autotune.table_paths(), "pla_amd/lut holds no table"
    assert autotune.header_is_current(), "pla_amd/csrc/generated/tuned_table.inc is stale: python -m pla_amd.autotune --render-only"


def _nearest(rows, B):
    return min(rows, key=lambda r: max(r[0] / B, B / r[0]))[1]


def test_library_lookup_matches_the_table():
    """The compiled-in table answers like the table file: nearest tuned batch size in ratio for a shape it
    holds, size thresholds for any other (host function, no GPU)."""
    lib = _lib.load()
    by_shape = {}
    for r in autotune.read_table(autotune.DEFAULT_TABLE):
        key = (autotune.KERNEL_CODE[r["kernel"]], 1 if r["mode"] == "tree" else 0, autotune.DTYPE_CODE[r["dtype"]],
               autotune.DTYPE_CODE[r["state_dtype"]], int(r["H"]), int(r["HV"]))
        by_shape.setdefault(key, []).append((int(r["B"]), autotune.ROWS_OF_BV[int(r["BV"])]))
    assert by_shape
    for key, rows in by_shape.items():
        for B, rpw in rows:
            assert lib.pla_tuned_rows_per_wave(*key, B) == rpw
        for B in (3, 5, 40, 100, 300, 4000):
            ratios = sorted(max(b / B, B / b) for b, _ in rows)
            if len(ratios) > 1 and ratios[0] == ratios[1]:
                continue                                   # equidistant neighbours: either answer is valid
            assert lib.pla_tuned_rows_per_wave(*key, B) == _nearest(rows, B)
    # a shape the table does not hold: thresholds on B * HV
    for B, want in ((1, 8), (2, 8), (3, 16), (7, 16), (8, 32), (100, 32)):
        assert lib.pla_tuned_rows_per_wave(1, 0, 1, 0, 32, 64, B) == want
    assert lib.pla_tuned_rows_per_wave(7, 0, 1, 0, 16, 32, 8) == 0
    assert lib.pla_tuned_rows_per_wave(1, 0, 1, 0, 16, 32, 0) == 0


@pytest.mark.gpu
def test_tune_one_shape_on_the_gpu(tmp_path):
    for kernel, mode in (("k_last_packed", ""), ("k_last", ""), ("k_last_mtp", "chain"), ("k_last_mtp", "tree")):
        row, timings = autotune.tune_shape(kernel, 4, 4, 8, mode=mode, reps=3)
        assert set(timings) == {32, 64, 128} and all(t > 0 for t in timings.values())
        assert row["kernel"] == kernel and row["BV"] in (32, 64, 128) and row["mode"] == mode
    row, _ = autotune.tune_shape("k_last_packed", 4, 4, 8, state_dtype="bf16", reps=3)
    path = str(tmp_path / "t.csv")
    assert autotune.merge_tuned_rows(path, [row]) == (0, 1)
    assert autotune.read_table(path)[0]["state_dtype"] == "bf16"


@pytest.mark.gpu
def test_untuned_and_tuned_row_counts_give_identical_results():
    """The row count only changes how a tile is spread over wavefronts: outputs and states are bit-identical."""
    from pla_amd.decode import fused_sigmoid_gating_delta_rule_forward_k_last_packed as packed
    from pla_amd.decode.private import fused_sigmoid_gating_delta_rule_forward_k_last_packed_tunable as tunable
    from pla_amd.workloads import gdn_decode_packed
    results = []
    for bv in (None, 32, 64, 128):
        w = gdn_decode_packed(8, H=16, HV=32, pool_slots=16, pad_frac=0.1, seed=5)
        call = {k: v for k, v in w.items() if not k.startswith("_")}
        out = packed(**call) if bv is None else tunable(**call, bv=bv, wn=4, sn=1, hv_per_cta=1)
        torch.cuda.synchronize()
        results.append((out.clone(), w["_meta"]["backing"].clone()))
    for out, backing in results[1:]:
        assert torch.equal(out, results[0][0]) and torch.equal(backing, results[0][1])
