"""The reference's import paths resolve to this implementation: ``pla.*`` modules are the ``pla_amd.*`` module
objects, and ``pla.decode._C`` is a compiled pybind11 module with the reference's function names and argument
names (src/decode/k-last/fused_sigmoid_gating.cpp:167-235).  CPU only: nothing is launched."""
import inspect
import re

import pytest


def test_reference_import_paths_resolve_to_the_same_modules():
    import pla
    import pla_amd
    from pla.decode import (fused_sigmoid_gating_delta_rule_forward_k_last,
                            fused_sigmoid_gating_delta_rule_forward_k_last_packed)
    from pla.decode.private import (fused_sigmoid_gating_delta_rule_forward_k_last_tunable,
                                    fused_sigmoid_gating_delta_rule_forward_k_last_packed_tunable)
    from pla.decode.kda import fused_recurrent_kda, fused_kda_decode_mega_forward
    from pla.prefill.flashqla import chunk_gated_delta_rule_fwd, gdn_prefill_packed_qkv_fwd
    from pla.prefill.flashkdapro import flashkda_fwd
    import pla.decode.kda_replayssm_sglang
    import pla.decode.kda_mtp_sglang
    import pla.decode.kda_replayssm_vllm
    import pla.prefill.flashqla.ops
    import pla_amd.decode
    import pla_amd.prefill.flashqla.ops
    assert pla.decode is pla_amd.decode and pla.prefill.flashqla.ops is pla_amd.prefill.flashqla.ops
    # the alias import leaves the module's own spec in place (relative imports, reload and pkgutil keep working)
    assert pla_amd.decode.__spec__.name == "pla_amd.decode" and pla_amd.decode.__package__ == "pla_amd.decode"
    assert pla_amd.prefill.flashqla.ops.__spec__.name == "pla_amd.prefill.flashqla.ops"
    assert fused_sigmoid_gating_delta_rule_forward_k_last_packed is pla_amd.decode.fused_sigmoid_gating_delta_rule_forward_k_last_packed
    assert pla.__all__ == []
    params = list(inspect.signature(fused_sigmoid_gating_delta_rule_forward_k_last).parameters)
    assert params[:5] == ["A_log", "a", "dt_bias", "softplus_beta", "softplus_threshold"] and params[-3:] == ["lower_bound", "is_sglang", "out"]
    assert len(params) == 23
    assert len(inspect.signature(fused_sigmoid_gating_delta_rule_forward_k_last_packed).parameters) == 15
    assert list(inspect.signature(gdn_prefill_packed_qkv_fwd).parameters)[:6] == [
        "packed_qkv", "raw_gate_a", "raw_beta_b", "A_log", "dt_bias", "cu_seqlens"]
    assert list(inspect.signature(flashkda_fwd).parameters)[:8] == ["q", "k", "v", "g", "beta", "A_log", "dt_bias", "out"]
    with pytest.raises(ModuleNotFoundError):
        import pla.no_such_namespace  # noqa: F401


def test_compiled_decode_module_has_the_reference_functions_and_argument_names():
    import torch  # noqa: F401  (the extension links torch's libraries; importing torch loads them)
    import pla.decode
    import pla_amd.decode._C as direct
    C = pla.decode._C
    assert C is direct
    names = {
        "fused_sigmoid_gating_delta_rule_forward_k_last": 23,
        "fused_sigmoid_gating_delta_rule_forward_k_last_packed": 15,
        "fused_sigmoid_gating_delta_rule_forward_k_last_tunable": 27,
        "fused_sigmoid_gating_delta_rule_forward_k_last_packed_tunable": 19,
    }
    for name, count in names.items():
        doc = getattr(C, name).__doc__
        args = re.findall(r"(\w+): ", doc.split("->")[0])
        assert len(args) == count, (name, args)
    doc = C.fused_sigmoid_gating_delta_rule_forward_k_last.__doc__
    args = re.findall(r"(\w+): ", doc.split("->")[0])
    assert args[9:11] == ["initial_state_source", "initial_state_indices"] and args[18] == "cache_steps_or_num_accept"
    assert re.search(r"lower_bound: [^,]* = None, is_sglang: [^,]* = None, out: [^,)]* = None\)", doc)
    # a rejected call raises RuntimeError from the compiled checks, before anything touches a GPU
    x = torch.zeros(2, 4)
    with pytest.raises(RuntimeError, match="initial_state_source is required"):
        C.fused_sigmoid_gating_delta_rule_forward_k_last_packed(x, x, x, x, x, 1.0, 20.0, None, None, None, x, True, None, False)


@pytest.mark.gpu
def test_decode_calls_go_through_the_compiled_module_on_the_gpu():
    """On a GPU box the public decode entry points run the compiled host layer (not the ctypes path).  The host
    time of one packed config-0 call (B=8; launch included, kernel excluded: the stream is not waited for) is
    printed, not asserted: a loaded host must not turn a correctness run red (bench.py reports the figure)."""
    import time
    import torch
    import pla_amd.decode as dec
    from pla_amd.workloads import gdn_decode_packed
    assert dec._compiled(), "pla_amd.decode._C is not importable"
    w = gdn_decode_packed(8, pool_slots=32, pad_frac=0.0, seed=1)
    call = {k: v for k, v in w.items() if not k.startswith("_")}
    packed = dec.fused_sigmoid_gating_delta_rule_forward_k_last_packed
    for _ in range(200):
        packed(**call)
    torch.cuda.synchronize()
    best = 1e9
    for _ in range(5):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(500):
            packed(**call)
        best = min(best, (time.perf_counter() - t0) / 500 * 1e6)
        torch.cuda.synchronize()
    print("host time per packed call: %.2f us" % best)
