"""Test-side glue: runs the CPU oracle on the arguments of a GPU call."""
import torch

from oracle import k_last_reference, fold_reference


def rel_l2(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    den = want.norm().clamp_min(1e-30)
    return float((got - want).norm() / den)


def make_k_last_case(is_kda, mode, *, H=4, HV=8, B=3, T=None, seed=2026, padded=True,
                     act_dtype=torch.bfloat16, device="cuda", state_dtype=torch.float32):
    """Small decode / MTP case in the style of the reference's k-last tests
    (tests/test_k_last_state_dtype.py:55-105): slot pool with a padded pitch and guard
    floats, non-trivial slot ids including an SGLang pad, a sentinel-filled cache."""
    g = torch.Generator().manual_seed(seed)
    D = 128
    T = 1 if mode == "decode" else (4 if T is None else T)
    lengths = [T] * B
    if mode == "ragged":
        assert B == 3
        lengths = [T, T // 2, 0]
    nt = sum(lengths)

    def rand(*shape, dtype=act_dtype):
        return torch.randn(*shape, generator=g).to(dtype).to(device)

    slots = max(7, B + 2)
    backing = (torch.randn(slots, HV * D * D + 256, generator=g) * 0.1).to(state_dtype).to(device)
    state = backing[:, : HV * D * D].view(slots, HV, D, D)
    state_ids = [3, 0, -1] if padded and B == 3 else list(range(B))
    cache_ids = [2, 0, 1] if padded and B == 3 else list(reversed(range(B)))
    cache = None if mode == "decode" else torch.full(
        (max(4, B + 1), T + 3, HV, D, D), -7.0, dtype=state_dtype, device=device)
    parents = None
    if mode == "tree":
        parents = torch.tensor([[max(0, t - 2) for t in range(T)]] * B, dtype=torch.int32, device=device)
    cu = torch.tensor([0] + torch.tensor(lengths).cumsum(0).tolist(), dtype=torch.int32, device=device)
    args = dict(
        A_log=rand(HV, dtype=torch.float32),
        a=rand(1, nt, HV, D) if is_kda else rand(1, nt, HV),
        dt_bias=rand(HV, D, dtype=torch.float32 if mode != "decode" else act_dtype) if is_kda else rand(HV),
        softplus_beta=1.0, softplus_threshold=20.0,
        q=rand(1, nt, H, D), k=rand(1, nt, H, D), v=rand(1, nt, HV, D), b=rand(1, nt, HV),
        initial_state_source=state,
        initial_state_indices=torch.tensor(state_ids, dtype=torch.int32, device=device),
        scale=D ** -0.5, use_qk_l2norm_in_kernel=True, cu_seqlens=cu, is_kda=is_kda,
        disable_state_update=mode not in ("decode", "writeback"),
        intermediate_states_buffer=cache,
        intermediate_state_indices=None if mode == "decode" else torch.tensor(cache_ids, dtype=torch.int32, device=device),
        cache_steps_or_num_accept=None if mode == "decode" else T,
        retrieve_parent_token=parents,
    )
    return args, backing, lengths, state_ids, cache_ids


def oracle_k_last(args, lengths, state_ids, cache_ids=None, num_accepted=None, compute_dtype=torch.float32):
    """Oracle result for a (non-packed) k-last call; returns CPU tensors."""
    cpu = lambda t: None if t is None else t.detach().cpu()
    q, k, v = (cpu(args[n]).reshape(-1, *args[n].shape[-2:]) for n in ("q", "k", "v"))
    HV, D = v.shape[1], v.shape[2]
    a = cpu(args["a"])
    a = a.reshape(-1, HV, D) if args["is_kda"] else a.reshape(-1, HV)
    dt = cpu(args["dt_bias"])
    dt = dt.reshape(HV, D) if args["is_kda"] else dt.reshape(HV)
    parents = args.get("retrieve_parent_token")
    out, state, cache = k_last_reference(
        q, k, v, a, cpu(args["b"]).reshape(-1, HV), cpu(args["A_log"]), dt,
        cpu(args["initial_state_source"]), state_ids, lengths,
        scale=args["scale"], use_qk_l2norm=args["use_qk_l2norm_in_kernel"], is_kda=args["is_kda"],
        disable_state_update=args.get("disable_state_update", False),
        cache=cpu(args.get("intermediate_states_buffer")), cache_indices=cache_ids,
        num_accepted=num_accepted, parents=None if parents is None else parents.cpu().tolist(),
        lower_bound=args.get("lower_bound"),
        is_sglang=True if args.get("is_sglang") is None else args["is_sglang"],
        softplus_beta=args["softplus_beta"], softplus_threshold=args["softplus_threshold"],
        compute_dtype=compute_dtype)
    return out.reshape(args["v"].shape), state, cache


def packed_from(args):
    """Packed-call arguments equivalent to a T=1 non-packed case."""
    nt = args["q"].shape[1]
    return dict(
        mixed_qkv=torch.cat([args[k].reshape(nt, -1) for k in ("q", "k", "v")], -1),
        a=args["a"].reshape(nt, -1), b=args["b"].reshape(nt, -1),
        A_log=args["A_log"], dt_bias=args["dt_bias"],
        softplus_beta=args["softplus_beta"], softplus_threshold=args["softplus_threshold"],
        scale=args["scale"], initial_state_source=args["initial_state_source"],
        initial_state_indices=args["initial_state_indices"], out=torch.empty_like(args["v"]),
        use_qk_l2norm_in_kernel=args["use_qk_l2norm_in_kernel"], cu_seqlens=args["cu_seqlens"],
        is_kda=args["is_kda"], is_sglang=args.get("is_sglang", True),
    )


def oracle_packed_workload(w):
    """Oracle for a ``pla_amd.workloads.gdn_decode_packed`` dict; only the selected slots are
    copied to the host.  Returns (out [B,1,HV,128] cpu, {slot: state_after [HV,128,128]})."""
    meta = w["_meta"]
    B, H, HV = meta["B"], meta["H"], meta["HV"]
    idx = w["initial_state_indices"].cpu().tolist()
    active = [s for s in idx if s >= 0]
    remap = {s: i for i, s in enumerate(active)}
    compact = w["initial_state_source"][torch.tensor(active, device=w["initial_state_source"].device)].cpu()
    mixed = w["mixed_qkv"].cpu()
    q = mixed[:, : H * 128].reshape(B, H, 128)
    k = mixed[:, H * 128: 2 * H * 128].reshape(B, H, 128)
    v = mixed[:, 2 * H * 128:].reshape(B, HV, 128)
    is_kda = w["is_kda"]
    a = w["a"].cpu().reshape(B, HV, 128) if is_kda else w["a"].cpu()
    dt = w["dt_bias"].cpu().reshape(HV, 128) if is_kda else w["dt_bias"].cpu()
    out, st, _ = k_last_reference(
        q, k, v, a, w["b"].cpu(), w["A_log"].cpu(), dt, compact,
        [remap.get(s, -1) for s in idx], [1] * B, scale=w["scale"],
        use_qk_l2norm=w["use_qk_l2norm_in_kernel"], is_kda=is_kda)
    return out.reshape(B, 1, HV, 128), {s: st[i] for s, i in remap.items()}
