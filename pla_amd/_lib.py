"""ctypes binding of libpla_gfx950.so (the C ABI declared in include/pla_gfx950.h).

The library is the only compute path of this package: if it is missing or does
not load, importing an operator raises; there is no CPU or PyTorch fallback.
"""

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libpla_gfx950.so")

F32, BF16, F16 = 0, 1, 2
GATE_SOFTPLUS, GATE_LOWER_BOUND, GATE_LOG_DECAY = 0, 1, 2

_c_int, _c_i64, _c_f, _c_p = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p

# name -> argtypes, in the order of include/pla_gfx950.h
SIGNATURES = {
    "pla_k_last_packed_launch": [
        _c_p, _c_int, _c_p, _c_p, _c_f, _c_f, _c_p, _c_p, _c_p, _c_p, _c_int, _c_p, _c_p,
        _c_f, _c_int, _c_i64, _c_i64, _c_i64, _c_i64,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_p],
    "pla_k_last_launch": [
        _c_p, _c_int, _c_p, _c_p, _c_int, _c_f, _c_f, _c_int,
        _c_p, _c_p, _c_p, _c_p, _c_int,
        _c_p, _c_p, _c_int, _c_p, _c_p, _c_p, _c_p, _c_int,
        _c_p, _c_i64, _c_i64, _c_f, _c_int,
        _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
        _c_p, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_p],
    "pla_kda_fold_launch": [
        _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p,
        _c_i64, _c_i64, _c_i64, _c_i64, _c_i64,
        _c_int, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_p],
    "pla_kda_fold_native_launch": [
        _c_p, _c_int, _c_p, _c_p, _c_p, _c_p, _c_p,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_p],
    "pla_kda_conv_native_launch": [
        _c_p, _c_int, _c_p, _c_p, _c_p, _c_p,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_p],
    "pla_kda_decode_mega_launch": [
        _c_int, _c_int, _c_int, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p,
        _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p,
        _c_p, _c_p, _c_f, _c_p, _c_p, _c_p,
        _c_f, _c_f, _c_int, _c_int, _c_int,
        _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_p],
    "pla_kda_verify_dspark_launch": [
        _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p,
        _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p,
        _c_p, _c_int, _c_p, _c_int, _c_p, _c_int,
        _c_int, _c_int, _c_int, _c_int, _c_f, _c_f, _c_p,
        _c_p, _c_p, _c_i64, _c_f, _c_p],
    "pla_kda_replay_verify_native_launch": [
        _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p,
        _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p, _c_p,
        _c_p, _c_int, _c_p, _c_int,
        _c_int, _c_int, _c_int, _c_f, _c_f, _c_p,
        _c_i64, _c_int, _c_int, _c_int, _c_p],
    "pla_kda_commit_plan_launch": [
        _c_p, _c_int, _c_p, _c_int, _c_p, _c_int, _c_p, _c_int, _c_p, _c_int, _c_p, _c_int,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
        _c_i64, _c_i64, _c_i64, _c_p, _c_p, _c_p],
    "pla_conv_window_scatter_launch": [
        _c_int, _c_int, _c_p, _c_p, _c_p, _c_int, _c_p, _c_int, _c_int, _c_int, _c_int,
        _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64,
        _c_int, _c_int, _c_int, _c_p],
    "pla_gdn_prefill_launch": [
        _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64,
        _c_p, _c_p, _c_i64, _c_i64,
        _c_p, _c_p, _c_p, _c_p,
        _c_p, _c_int, _c_int, _c_f, _c_int,
        _c_p, _c_p, _c_i64, _c_p, _c_p, _c_i64,
        _c_p, _c_p, _c_i64, _c_p, _c_p,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_p],
    "pla_gdn_prefill_launch_raw": [
        _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64,
        _c_p, _c_p, _c_i64, _c_i64,
        _c_p, _c_p, _c_p, _c_p,
        _c_p, _c_int, _c_int, _c_f, _c_int,
        _c_p, _c_p, _c_i64, _c_p, _c_p, _c_i64,
        _c_p, _c_p, _c_i64, _c_p, _c_p,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_p, _c_p],
    "pla_gdn_prefill_launch_static": [
        _c_p, _c_p, _c_p, _c_i64, _c_i64, _c_i64,
        _c_p, _c_p, _c_i64, _c_i64,
        _c_p, _c_p, _c_p, _c_p,
        _c_p, _c_int, _c_int, _c_f, _c_int,
        _c_p, _c_p, _c_i64, _c_p, _c_p, _c_i64,
        _c_p, _c_p, _c_p,
        _c_int, _c_int, _c_int, _c_int, _c_int, _c_p],
    "pla_kda_prefill_launch": [
        _c_p, _c_p, _c_p, _c_p, _c_p,
        _c_i64, _c_i64, _c_i64, _c_i64, _c_i64,
        _c_p, _c_p, _c_f, _c_f,
        _c_p, _c_int, _c_int,
        _c_p, _c_p, _c_i64, _c_p, _c_p, _c_i64,
        _c_p, _c_p, _c_i64,
        _c_int, _c_int, _c_int, _c_int, _c_p],
    "pla_kda_prefill_launch_raw": [
        _c_p, _c_p, _c_p, _c_p, _c_p,
        _c_i64, _c_i64, _c_i64, _c_i64, _c_i64,
        _c_p, _c_p, _c_f, _c_f,
        _c_p, _c_int, _c_int,
        _c_p, _c_p, _c_i64, _c_p, _c_p, _c_i64,
        _c_p, _c_p, _c_i64,
        _c_int, _c_int, _c_int, _c_int, _c_p, _c_p],
}

_lib = None


def load():
    """Return the loaded library; raises RuntimeError when it is absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "pla_amd: %s is missing. Build it with `python -m pla_amd.build` "
            "(hipcc, --offload-arch=gfx950); there is no fallback path." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    lib.pla_version.restype = ctypes.c_char_p
    lib.pla_version.argtypes = []
    lib.pla_last_error.restype = ctypes.c_char_p
    lib.pla_last_error.argtypes = []
    lib.pla_gdn_prefill_workspace_bytes.restype = _c_i64
    lib.pla_gdn_prefill_workspace_bytes.argtypes = [_c_int, _c_int, _c_int, _c_int]
    lib.pla_gdn_prefill_halved_sequences.restype = _c_int
    lib.pla_gdn_prefill_halved_sequences.argtypes = [_c_p, _c_int, _c_int, _c_int, _c_int]
    lib.pla_kda_prefill_halved_sequences.restype = _c_int
    lib.pla_kda_prefill_halved_sequences.argtypes = [_c_p, _c_int, _c_int, _c_int]
    lib.pla_kda_prefill_workspace_bytes.restype = _c_i64
    lib.pla_kda_prefill_workspace_bytes.argtypes = [_c_int, _c_int, _c_int]
    lib.pla_tuned_rows_per_wave.restype = _c_int
    lib.pla_tuned_rows_per_wave.argtypes = [_c_int] * 7
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = _c_int
        fn.argtypes = argtypes
    _lib = lib
    return lib


def call(name, *args):
    """Invoke an entry point; a non-zero return becomes RuntimeError(pla_last_error())."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise RuntimeError(lib.pla_last_error().decode())


def ptr(t):
    return None if t is None else t.data_ptr()


def dtype_code(dtype):
    import torch
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    if dtype == torch.float16:
        return F16
    raise RuntimeError("unsupported dtype %s" % dtype)


def current_stream(device):
    import torch
    return torch.cuda.current_stream(device).cuda_stream
