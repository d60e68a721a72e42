"""CPU-only checks: the C-ABI library loads and exports every symbol the header declares, the
ctypes signatures have the header's arity, and host-side argument validation rejects bad calls
before anything native runs (no compute call is made here)."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "pla_gfx950.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for m in re.finditer(r"\b(pla_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if args in ("", "void") else len(args.split(","))
    return out


def test_library_exports_every_declared_symbol():
    from pla_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build the library first: python -m pla_amd.build"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    declared = _declared()
    assert {"pla_version", "pla_last_error", "pla_k_last_packed_launch", "pla_k_last_launch",
            "pla_kda_fold_launch", "pla_kda_fold_native_launch", "pla_kda_conv_native_launch", "pla_kda_commit_plan_launch", "pla_kda_decode_mega_launch", "pla_kda_verify_dspark_launch", "pla_kda_replay_verify_native_launch", "pla_conv_window_scatter_launch",
            "pla_gdn_prefill_launch", "pla_gdn_prefill_launch_raw", "pla_gdn_prefill_workspace_bytes", "pla_gdn_prefill_halved_sequences",
            "pla_kda_prefill_launch", "pla_kda_prefill_launch_raw", "pla_kda_prefill_halved_sequences", "pla_kda_prefill_workspace_bytes"} <= set(declared)
    for name in declared:
        assert hasattr(lib, name), name
    lib.pla_version.restype = ctypes.c_char_p
    assert b"gfx950" in lib.pla_version()


def test_ctypes_signatures_match_header_arity():
    from pla_amd import _lib
    declared = _declared()
    for name, argtypes in _lib.SIGNATURES.items():
        assert declared[name] == len(argtypes), name


def test_workspace_sizes_are_monotone_and_aligned():
    from pla_amd import _lib
    lib = _lib.load()
    a = lib.pla_gdn_prefill_workspace_bytes(4096, 2, 16, 32)
    b = lib.pla_gdn_prefill_workspace_bytes(8192, 2, 16, 32)
    assert 0 < a < b and a % 256 == 0 and b % 256 == 0
    assert lib.pla_gdn_prefill_workspace_bytes(0, 1, 1, 1) == 0
    c = lib.pla_kda_prefill_workspace_bytes(4096, 1, 32)
    assert c > 0 and c % 256 == 0


def test_plan_of_the_halved_sequences_is_host_arithmetic():
    """Which sequences the last sweep of a ragged GDN prefill call runs as two workgroups per chain is decided from
    the host offsets alone: more than 128 chains of whole sequences, a price that falls by 5 % or more."""
    from pla_amd import _lib
    lib = _lib.load()

    def plan(lengths, H, HV):
        offs = [0]
        for n in lengths:
            offs.append(offs[-1] + n)
        return lib.pla_gdn_prefill_halved_sequences((ctypes.c_int32 * len(offs))(*offs), len(lengths), offs[-1], H, HV)
    assert plan([8000, 7000, 1000, 2000, 3000], 16, 32) == 1           # 0.9 x 79 chunks is still above the runner-up's 69
    assert plan([5000, 4800, 300, 2000, 1000, 100, 64], 16, 32) == 2   # two long sequences of nearly equal length
    assert plan([4000] * 4 + [1000], 16, 32) == 0                      # four long ones as halves would fill every CU
    assert plan([2646, 6988, 1342, 6924, 3410, 2250, 1978, 7272], 16, 32) == 0      # 256 chains: no idle CU to gain from
    assert plan([4000, 3900, 3800, 3700, 500, 600, 700, 800, 900], 16, 32) == 0
    assert plan([1500, 200, 300, 400, 700], 16, 32) == 1               # a single sweep (too short for stages)
    assert plan([16384], 16, 32) == 0                                  # split into segments instead
    assert plan([3000, 100], 16, 32) == 0                              # at most 128 chains: every chain runs as halves anyway
    assert plan([100] * 65, 16, 32) == 0                               # more than 64 sequences: table kernel path
    assert lib.pla_gdn_prefill_halved_sequences(None, 5, 1000, 16, 32) == 0

    def kda_plan(lengths, H):
        offs = [0]
        for n in lengths:
            offs.append(offs[-1] + n)
        return lib.pla_kda_prefill_halved_sequences((ctypes.c_int32 * len(offs))(*offs), len(lengths), offs[-1], H)
    # a KDA half costs less of a whole chain's time and a full chip slows its chunks less: the plan splits more
    assert kda_plan([8000, 7000, 1000, 2000, 3000], 32) == 2
    assert kda_plan([2646, 6988, 1342, 6924, 3410, 2250, 1978, 7272], 32) == 3
    assert kda_plan([4000] * 4 + [1000], 32) == 0                      # halves of all four would leave the fifth no CU
    assert kda_plan([65536], 32) == 0 and kda_plan([3000, 100], 32) == 0 and kda_plan([100] * 65, 32) == 0
    assert lib.pla_kda_prefill_halved_sequences(None, 5, 1000, 32) == 0


def test_native_entry_points_reject_bad_arguments_without_a_gpu():
    """Argument checks run before any launch, so they are testable on a CPU-only host."""
    from pla_amd import _lib
    lib = _lib.load()
    rc = lib.pla_k_last_packed_launch(None, 0, None, None, 1.0, 20.0, None, None, None, None, _lib.F32, None, None,
                                      0.1, 1, 0, 0, 0, 0, 4, 2, 4, 64, 64, 1, 1, 0, _lib.BF16, 0, None)
    assert rc != 0 and b"K == V == 128" in lib.pla_last_error()
    rc = lib.pla_k_last_packed_launch(None, 0, None, None, 1.0, 20.0, None, None, None, None, _lib.F32, None, None,
                                      0.1, 1, 0, 0, 0, 0, 4, 3, 4, 128, 128, 1, 1, 0, _lib.BF16, 0, None)
    assert rc != 0 and b"multiple of H" in lib.pla_last_error()
    rc = lib.pla_kda_prefill_launch(None, None, None, None, None, 0, 0, 0, 0, 0, None, None, -7.0, 1.0,
                                    None, 1, 64, None, None, 0, None, None, 0, None, None, 0, 4, 128, 128,
                                    _lib.BF16, None)
    assert rc != 0


def test_facade_validation_raises_before_native_code():
    from pla_amd.decode import fused_sigmoid_gating_delta_rule_forward_k_last_packed as packed
    from pla_amd.prefill.flashqla import gdn_prefill_packed_qkv_fwd
    from pla_amd.prefill.flashkdapro import flashkda_fwd
    HV, H = 4, 2
    state = torch.zeros(3, HV, 128, 128)
    mixed = torch.zeros(2, (2 * H + HV) * 128 - 1, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="packed QKV width"):
        packed(mixed, torch.zeros(2, HV, dtype=torch.bfloat16), torch.zeros(2, HV, dtype=torch.bfloat16),
               torch.zeros(HV), torch.zeros(HV, dtype=torch.bfloat16), 1.0, 20.0, None, state,
               torch.zeros(2, dtype=torch.int32), torch.zeros(2, 1, HV, 128, dtype=torch.bfloat16), True, None, False)
    with pytest.raises(RuntimeError, match="initial_state_source is required"):
        packed(mixed, torch.zeros(2, HV, dtype=torch.bfloat16), torch.zeros(2, HV, dtype=torch.bfloat16),
               torch.zeros(HV), torch.zeros(HV, dtype=torch.bfloat16), 1.0, 20.0, None, None, None,
               torch.zeros(2, 1, HV, 128, dtype=torch.bfloat16), True, None, False)
    with pytest.raises(ValueError, match="CUDA tensor"):
        gdn_prefill_packed_qkv_fwd(torch.zeros(4, 1024, dtype=torch.bfloat16), None, None, None, None, None,
                                   num_qk_heads=2, num_v_heads=4)
    with pytest.raises(ValueError, match="CUDA tensor"):
        flashkda_fwd(*([torch.zeros(4, 2, 128, dtype=torch.bfloat16)] * 4), torch.zeros(4, 2), torch.zeros(2),
                     torch.zeros(2, 128), torch.zeros(4, 2, 128, dtype=torch.bfloat16))


def test_missing_library_fails_loudly(monkeypatch):
    from pla_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libpla_gfx950.so")
    with pytest.raises(RuntimeError, match="there is no fallback path"):
        _lib.load()


def test_prefill_sanity_mode_checks_offsets(monkeypatch):
    """PLA_SANITY_CHECK=1: offsets are validated before they are narrowed to int32 (reference helper
    pla/prefill/_sanity.py:46-110); violations raise AssertionError with the reference's prefix."""
    import torch
    from pla_amd.prefill import _sanity
    cu = torch.tensor([0, 5, 5, 9], dtype=torch.int64)
    monkeypatch.delenv("PLA_SANITY_CHECK", raising=False)
    _sanity.offsets(torch.tensor([3, 1]), 2)                                         # off: nothing is checked
    monkeypatch.setenv("PLA_SANITY_CHECK", "1")
    _sanity.offsets(cu, 9, (0, 5, 5, 9))
    _sanity.offsets(None, 7, (0, 7))
    for bad_cu, cap, raw, msg in (
            (torch.tensor([1, 5]), 9, None, "start at zero"),
            (torch.tensor([0, 5, 4]), 9, None, "monotonic"),
            (torch.tensor([0, 5, 10]), 9, None, "within token capacity"),
            (torch.tensor([0, 2 ** 31], dtype=torch.int64), 2 ** 31 + 5, None, "token capacity must fit int32"),
            (cu, 9, (0, 5, 6, 9), "raw_cu_seqlens must equal device cu_seqlens"),
            (cu, 9, (0, 5, 9), "batch\\+1 entries"),
            (cu.float(), 9, None, "int32 or int64"),
            (cu.reshape(2, 2), 9, None, r"\[batch\+1\]"),
            (None, 7, (0, 6), r"must be \[0,T\]")):
        with pytest.raises(AssertionError, match=r"PLA_SANITY_CHECK \[prefill\]: .*" + msg):
            _sanity.offsets(bad_cu, cap, raw)
    # operands of the fp16 matrix products: finite and within +-65504
    ref = torch.zeros(1)
    _sanity.operand_range(ref, v=torch.tensor([1.0, -65504.0]), initial_state=None)
    for bad in (torch.tensor([7e4]), torch.tensor([float("nan")]), torch.tensor([float("-inf")])):
        with pytest.raises(AssertionError, match=r"PLA_SANITY_CHECK \[prefill\]: v must be finite and within the fp16"):
            _sanity.operand_range(ref, v=bad)
    monkeypatch.delenv("PLA_SANITY_CHECK")
    _sanity.operand_range(ref, v=torch.tensor([7e4]))                                 # off: nothing is checked


def test_namespace_mirrors_the_reference_packages():
    """`import pla_amd as pla` gives the reference's sub-packages and public names for the path
    (pla/decode/__init__.py:63-66, pla/decode/kda/__init__.py:51-52, pla/decode/private/__init__.py:46-47,
    pla/decode/kda_mtp_sglang/__init__.py:35-41, pla/decode/kda_replayssm_vllm/__init__.py,
    pla/prefill/flashqla/__init__.py:48, pla/prefill/flashkdapro/__init__.py:39)."""
    import importlib
    expected = {
        "decode": ["fused_sigmoid_gating_delta_rule_forward_k_last", "fused_sigmoid_gating_delta_rule_forward_k_last_packed"],
        "decode.private": ["fused_sigmoid_gating_delta_rule_forward_k_last_tunable",
                           "fused_sigmoid_gating_delta_rule_forward_k_last_packed_tunable"],
        "decode.kda": ["fused_recurrent_kda", "fused_kda_decode_mega_forward"],
        "decode.kda_replayssm_sglang": ["fused_kda_decode_mtp_dspark", "commit_kda_replayssm_after_verify"],
        "decode.kda_mtp_sglang": ["fused_kda_decode_mtp_dspark", "commit_kda_replayssm_after_verify"],
        "decode.kda_replayssm_vllm": ["KDAReplayRecords", "KDAReplayCommitPlan", "KDAReplayCommitContext", "kda_replay_verify"],
        "prefill.flashqla": ["chunk_gated_delta_rule_fwd", "gdn_prefill_packed_qkv_fwd"],
        "prefill.flashkdapro": ["flashkda_fwd"],
    }
    for sub, names in expected.items():
        mod = importlib.import_module("pla_amd." + sub)
        for name in names:
            assert callable(getattr(mod, name)), (sub, name)
    a = importlib.import_module("pla_amd.decode.kda_mtp_sglang")
    b = importlib.import_module("pla_amd.decode.kda_replayssm_sglang")
    assert a.fused_kda_decode_mtp_dspark is b.fused_kda_decode_mtp_dspark
