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


def test_compiled_prefill_modules_exist_and_decline_calls_they_do_not_take():
    """pla.prefill.flashqla._C and pla.prefill.flashkdapro._C are compiled modules (as the reference ships one per
    namespace); _C.flashkda_fwd has the 15 positional arguments of the reference's call
    (pla/prefill/flashkdapro/ops.py:215-219).  Calls outside the plain GPU form are declined without a launch: the
    try_* functions return None / False and the facade's own checks speak."""
    import torch
    import pla.prefill.flashqla._C as QC
    import pla.prefill.flashkdapro._C as KC
    import pla_amd.prefill.flashqla.ops as qops
    assert QC.__file__.endswith(".so") and KC.__file__.endswith(".so") and qops._compiled() is QC
    doc = KC.flashkda_fwd.__doc__.split("->")[0]
    assert re.findall(r"(\w+): ", doc) == ["q", "k", "v", "g", "beta", "A_log", "dt_bias", "out", "scale", "lower_bound",
                                            "initial_state", "final_state", "cu_seqlens", "state_indices", "raw_cu_seqlens"]
    x = torch.zeros(4, 2, 128, dtype=torch.bfloat16)
    assert KC.try_flashkda_fwd(x, x, x, x, torch.zeros(4, 2, dtype=torch.bfloat16), torch.zeros(2), torch.zeros(2, 128), x,
                               0.1, -5.0, None, None, None, None, None) is False
    with pytest.raises(ValueError, match="compiled entry point takes"):
        KC.flashkda_fwd(x, x, x, x, torch.zeros(4, 2, dtype=torch.bfloat16), torch.zeros(2), torch.zeros(2, 128), x,
                        0.1, -5.0, None, None, None, None, None)
    assert QC.try_gdn_prefill_packed_qkv_fwd(torch.zeros(4, 1024, dtype=torch.bfloat16), None, None, None, None, None, 2, 4,
                                             None, None, None, True, None, None, None) is None
    # the facade then refuses the call with its own message
    from pla.prefill.flashqla import gdn_prefill_packed_qkv_fwd
    with pytest.raises(ValueError, match="must be a CUDA tensor"):
        gdn_prefill_packed_qkv_fwd(torch.zeros(4, 1024, dtype=torch.bfloat16), None, None, None, None, None,
                                   num_qk_heads=2, num_v_heads=4)


@pytest.mark.gpu
def test_compiled_prefill_layer_equals_the_facade_path_bit_for_bit(monkeypatch):
    """The compiled host layer and the facade's own path launch the same C ABI call: same bits for GDN (packed rows
    with an indexed pool; separate q / k / v with explicit gates and compact states, with and without a returned
    state) and KDA (compact states, indexed pool), and forms the compiled layer does not take (bf16 states) still
    work through the facade.  Host time per call is printed."""
    import time
    import torch
    import pla_amd.prefill.flashqla.ops as qops
    import pla_amd.prefill.flashkdapro.ops as kops
    from pla_amd.workloads import gdn_prefill_packed
    assert qops._compiled() and kops._compiled()
    taken = {"q": 0, "k": 0}
    real_q, real_k = qops._compiled(), kops._compiled()

    class Counting:
        def __init__(self, real, key):
            self._real, self._key = real, key

        def __getattr__(self, name):
            fn = getattr(self._real, name)

            def call(*args):
                r = fn(*args)
                if r is not None and r is not False:
                    taken[self._key] += 1
                return r
            return call

    def both(run):
        monkeypatch.setattr(qops, "_native", Counting(real_q, "q"))
        monkeypatch.setattr(kops, "_native", Counting(real_k, "k"))
        fast = run()
        monkeypatch.setattr(qops, "_native", False)
        monkeypatch.setattr(kops, "_native", False)
        slow = run()
        torch.cuda.synchronize()
        return fast, slow

    # GDN, packed rows, indexed pool
    w = gdn_prefill_packed([300, 0, 70, 1100], H=2, HV=4, pool_slots=7, seed=3, tail_pad=2)
    call = {k: v for k, v in w.items() if not k.startswith("_")}
    packed = call.pop("packed_qkv")
    a, b, A, dt, cu = (call.pop(n) for n in ("raw_gate_a", "raw_beta_b", "A_log", "dt_bias", "cu_seqlens"))
    pool0 = call["initial_state"].clone()

    def run_packed():
        call["initial_state"].copy_(pool0)
        r = qops.gdn_prefill_packed_qkv_fwd(packed, a, b, A, dt, cu, **call)
        return r[0][:, :w["_meta"]["offsets"][-1]], r[2], r[4], call["initial_state"].clone()      # g_cum is defined for real tokens
    fast, slow = both(run_packed)
    assert taken["q"] == 1
    for x, y in zip(fast, slow):
        assert torch.equal(x, y)
    # GDN, separate tensors, explicit gates, compact states
    T, H, HV = 700, 2, 4
    g = torch.Generator().manual_seed(5)
    q = torch.nn.functional.normalize(torch.randn(1, T, H, 128, generator=g), dim=-1).bfloat16().cuda()
    k = torch.nn.functional.normalize(torch.randn(1, T, H, 128, generator=g), dim=-1).bfloat16().cuda()
    v = torch.randn(1, T, HV, 128, generator=g).bfloat16().cuda()
    gate = (-torch.rand(1, T, HV, generator=g) * 0.3).cuda()
    beta = torch.rand(1, T, HV, generator=g).cuda()
    S0 = (torch.randn(3, HV, 128, 128, generator=g) * 0.1).cuda()
    cu2 = torch.tensor([0, 130, 130, 700], dtype=torch.int32, device="cuda")
    for final in (True, False):
        fast, slow = both(lambda: qops.chunk_gated_delta_rule_fwd(q, k, v, gate, beta, initial_state=S0, cu_seqlens=cu2,
                                                                  output_final_state=final, raw_cu_seqlens=(0, 130, 130, 700)))
        assert torch.equal(fast[0], slow[0]) and torch.equal(fast[2], slow[2]) and fast[3] is None
        assert (fast[4] is None and slow[4] is None) if not final else torch.equal(fast[4], slow[4])
    assert taken["q"] == 3
    # a bf16 pool is not the compiled layer's form: declined, the facade widens the states and calls again in FP32
    # (that inner call is taken), then rounds the result
    fast, slow = both(lambda: qops.chunk_gated_delta_rule_fwd(q, k, v, gate, beta, initial_state=S0.bfloat16(), cu_seqlens=cu2))
    assert taken["q"] == 4 and torch.equal(fast[2], slow[2]) and fast[4].dtype == torch.bfloat16 and torch.equal(fast[4], slow[4])
    # KDA: compact states, then an indexed pool
    qk = torch.randn(T, H, 128, generator=g).bfloat16().cuda()
    kk = torch.randn(T, H, 128, generator=g).bfloat16().cuda()
    vk = torch.randn(T, H, 128, generator=g).bfloat16().cuda()
    gk = torch.randn(T, H, 128, generator=g).bfloat16().cuda()
    bk = torch.randn(T, H, generator=g).bfloat16().cuda()
    Ak, dk = (torch.randn(H, generator=g) * 0.5).cuda(), (torch.randn(H, 128, generator=g) * 0.5).cuda()
    S0k = (torch.randn(5, H, 128, 128, generator=g) * 0.1).cuda()
    idx = torch.tensor([4, 0, 2], dtype=torch.int32, device="cuda")

    def run_kda(indexed):
        out = torch.empty(T, H, 128, dtype=torch.bfloat16, device="cuda")
        if indexed:
            pool = S0k.clone()
            kops.flashkda_fwd(qk, kk, vk, gk, bk, Ak, dk, out, cu_seqlens=cu2, state_pool=pool, state_indices=idx)
            return out, pool
        fin = torch.full((3, H, 128, 128), float("nan"), device="cuda")
        kops.flashkda_fwd(qk, kk, vk, gk, bk, Ak, dk, out, initial_state=S0k, final_state=fin, cu_seqlens=cu2)
        return out, fin
    for indexed in (False, True):
        fast, slow = both(lambda: run_kda(indexed))
        assert torch.equal(fast[0], slow[0]) and torch.equal(fast[1], slow[1])
    assert taken["k"] == 2
    # host time per call through the compiled layer (printed, not asserted)
    monkeypatch.setattr(qops, "_native", real_q)
    for _ in range(20):
        run_packed()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(20):
        qops.gdn_prefill_packed_qkv_fwd(packed, a, b, A, dt, cu, **call)
    print("host time per compiled GDN prefill call: %.1f us" % ((time.perf_counter() - t0) / 20 * 1e6))
    torch.cuda.synchronize()
