"""Seeded synthetic workloads of the five benchmark configurations.

Used by ``bench.py``, the smoke run and the parity tests so that all of them see
identical inputs.  Small tensors are drawn on the CPU with a seeded
``torch.Generator`` and copied to the device; state pools (up to 8.6 GB) are
drawn on the device with a seeded device generator.

Distributions: q, k ~ N(0,1) rounded to bf16, L2-normalised per head in float32
and stored as bf16; v ~ N(0,1); b ~ N(0,1) (beta = sigmoid(b)); A_log ~
U(0, ln 16); a ~ N(0,1); dt_bias ~ U(-1,1); state ~ N(0, 0.1); scale = 128^-0.5.
"""

import math

import torch

D = 128


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _normalised(shape, g, dtype):
    x = torch.randn(*shape, generator=g).to(dtype).float()
    x = x * torch.rsqrt(x.square().sum(-1, keepdim=True) + 1e-6)
    return x.to(dtype)


def _pool(slots, HV, device, seed, pitch_pad=0):
    """FP32 k-last pool [slots, HV, 128, 128] ~ N(0, 0.1); optional padded slot pitch."""
    width = HV * D * D
    if device.type == "cuda":
        g = torch.Generator(device=device).manual_seed(seed)
        backing = torch.empty(slots, width + pitch_pad, dtype=torch.float32, device=device)
        backing.normal_(0.0, 0.1, generator=g)
    else:
        backing = torch.randn(slots, width + pitch_pad, generator=_gen(seed)) * 0.1
    return backing, backing[:, :width].view(slots, HV, D, D)


def slot_subset(slots, B, pad_frac, g, pad_value=-1):
    """First B entries of a seeded permutation (never arange), pad_frac of them set to pad_value."""
    perm = torch.randperm(slots, generator=g)[:B].to(torch.int32)
    n_pad = int(round(B * pad_frac))
    if n_pad:
        pos = torch.randperm(B, generator=g)[:n_pad]
        perm[pos] = pad_value
    return perm


def gdn_decode_packed(B, H=16, HV=32, pool_slots=None, pad_frac=0.0, seed=0, device="cuda",
                      dtype=torch.bfloat16, is_kda=False, pitch_pad=0):
    """Configs 0/1: packed one-token decode. Returns a dict of call arguments + metadata."""
    device = torch.device(device)
    g = _gen(seed)
    pool_slots = pool_slots or B
    q = _normalised((B, H, D), g, dtype)
    k = _normalised((B, H, D), g, dtype)
    v = torch.randn(B, HV, D, generator=g).to(dtype)
    mixed = torch.cat([q.reshape(B, -1), k.reshape(B, -1), v.reshape(B, -1)], dim=1)
    a = torch.randn(B, HV * D if is_kda else HV, generator=g).to(dtype)
    b = torch.randn(B, HV, generator=g).to(dtype)
    A_log = torch.rand(HV, generator=g) * math.log(16.0)
    dt_bias = (torch.rand(HV * D if is_kda else HV, generator=g) * 2 - 1).to(dtype)
    if pool_slots == B and pad_frac == 0.0:
        indices = torch.arange(B, dtype=torch.int32)
    else:
        indices = slot_subset(pool_slots, B, pad_frac, g)
    backing, state = _pool(pool_slots, HV, device, seed + 1, pitch_pad)
    to = lambda t: t.to(device)
    return dict(
        mixed_qkv=to(mixed), a=to(a), b=to(b), A_log=to(A_log), dt_bias=to(dt_bias),
        softplus_beta=1.0, softplus_threshold=20.0, scale=D ** -0.5,
        initial_state_source=state, initial_state_indices=to(indices),
        out=torch.empty(B, 1, HV, D, dtype=dtype, device=device),
        use_qk_l2norm_in_kernel=True,
        cu_seqlens=to(torch.arange(B + 1, dtype=torch.int32)),
        is_kda=is_kda, is_sglang=True,
        _meta=dict(B=B, H=H, HV=HV, backing=backing, n_active=int((indices >= 0).sum()),
                   state_bytes=int((indices >= 0).sum()) * HV * D * D * 4 * 2),
    )


def kda_mtp_verify(B=64, HV=32, T=4, pool_slots=1024, seed=0, device="cuda", dtype=torch.bfloat16):
    """Config 2: KDA MTP verify with a supplied per-channel log-decay and accepted-prefix commit.

    g = -softplus(N(0,1)) * U(0.01, 1) float32 [B*T, HV, 128]; num_accepted ~ U{0..T}.
    Records for the commit are laid out per slot: rawk/rawv [slots, HV, T, 128] bf16,
    gk [slots, HV, T, 128] float32, beta [slots, HV, T] float32.
    """
    device = torch.device(device)
    g = _gen(seed)
    H = HV
    nt = B * T
    q = _normalised((nt, H, D), g, dtype)
    k = _normalised((nt, H, D), g, dtype)
    v = torch.randn(nt, HV, D, generator=g).to(dtype)
    log_decay = -torch.nn.functional.softplus(torch.randn(nt, HV, D, generator=g)) * \
        (torch.rand(nt, HV, D, generator=g) * 0.99 + 0.01)
    beta = torch.sigmoid(torch.randn(nt, HV, generator=g))
    indices = slot_subset(pool_slots, B, 0.0, g)
    num_accepted = torch.randint(0, T + 1, (B,), generator=g).to(torch.int32)
    backing, state = _pool(pool_slots, HV, device, seed + 1)
    to = lambda t: t.to(device)
    return dict(
        q=to(q.view(1, nt, H, D)), k=to(k.view(1, nt, H, D)), v=to(v.view(1, nt, HV, D)),
        log_decay=to(log_decay), beta=to(beta), state=state, indices=to(indices),
        num_accepted=to(num_accepted), cu_seqlens=to(torch.arange(0, nt + 1, T, dtype=torch.int32)),
        scale=D ** -0.5, _meta=dict(B=B, H=H, HV=HV, T=T, backing=backing),
    )


def ragged_lengths(n_seq, lo, hi, seed):
    g = _gen(seed)
    return torch.randint(lo, hi + 1, (n_seq,), generator=g).tolist()


def gdn_prefill_packed(lengths, H=16, HV=32, pool_slots=64, seed=0, device="cuda", dtype=torch.bfloat16,
                       tail_pad=0):
    """Config 3: packed varlen GDN prefill with raw gating and an indexed FP32 pool."""
    device = torch.device(device)
    g = _gen(seed)
    T = sum(lengths) + tail_pad
    N = len(lengths)
    q = torch.randn(T, H, D, generator=g).to(dtype)
    k = torch.randn(T, H, D, generator=g).to(dtype)
    v = torch.randn(T, HV, D, generator=g).to(dtype)
    packed = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], dim=1)
    a = torch.randn(T, HV, generator=g).to(dtype)
    b = torch.randn(T, HV, generator=g).to(dtype)
    A_log = torch.rand(HV, generator=g) * math.log(16.0)
    dt_bias = torch.rand(HV, generator=g) * 2 - 1
    offs = [0]
    for n in lengths:
        offs.append(offs[-1] + n)
    indices = slot_subset(pool_slots, N, 0.0, g)
    backing, state = _pool(pool_slots, HV, device, seed + 1)
    to = lambda t: t.to(device)
    return dict(
        packed_qkv=to(packed), raw_gate_a=to(a), raw_beta_b=to(b), A_log=to(A_log), dt_bias=to(dt_bias),
        cu_seqlens=to(torch.tensor(offs, dtype=torch.int32)), num_qk_heads=H, num_v_heads=HV,
        scale=D ** -0.5, initial_state=state, initial_state_indices=to(indices),
        raw_cu_seqlens=tuple(offs),
        _meta=dict(T=T, N=N, H=H, HV=HV, offsets=offs, backing=backing),
    )


def kda_prefill(T=65536, H=32, seed=0, device="cuda", dtype=torch.bfloat16, lower_bound=-5.0):
    """Config 4: one long KDA sequence; heads [0, H/2) decay strongly (g ~ -U(0.5, 2) per token
    and channel), heads [H/2, H) weakly (g ~ -U(1e-4, 1e-2)).

    The operator takes the RAW gate: with A_log = 0 and dt_bias = 0 the lower-bound gate is
    g = lower_bound * sigmoid(raw), so raw = logit(g / lower_bound), stored in bf16.
    """
    device = torch.device(device)
    g = _gen(seed)
    q = torch.randn(T, H, D, generator=g).to(dtype)
    k = torch.randn(T, H, D, generator=g).to(dtype)
    v = torch.randn(T, H, D, generator=g).to(dtype)
    u = torch.rand(T, H, D, generator=g)
    strong = -(0.5 + 1.5 * u)
    weak = -(1e-4 + (1e-2 - 1e-4) * u)
    target = torch.where((torch.arange(H) < H // 2)[None, :, None], strong, weak)
    frac = (target / lower_bound).clamp(1e-7, 1 - 1e-7)
    raw = torch.log(frac) - torch.log1p(-frac)
    beta_raw = torch.randn(T, H, generator=g).to(dtype)
    g2 = torch.Generator().manual_seed(seed + 1)
    state = torch.randn(1, H, D, D, generator=g2) * 0.1
    to = lambda t: t.to(device)
    return dict(
        q=to(q), k=to(k), v=to(v), g=to(raw.to(dtype)), beta=to(beta_raw),
        A_log=to(torch.zeros(H)), dt_bias=to(torch.zeros(H, D)),
        out=torch.empty(T, H, D, dtype=dtype, device=device),
        scale=D ** -0.5, lower_bound=lower_bound, initial_state=to(state),
        final_state=torch.empty(1, H, D, D, dtype=torch.float32, device=device),
        cu_seqlens=to(torch.tensor([0, T], dtype=torch.int32)), raw_cu_seqlens=(0, T),
        _meta=dict(T=T, H=H),
    )


def kda_decode_mega(B, H, seed=0, device="cuda", dtype=torch.bfloat16, pad_rows=(), bias=False, slots=None):
    """Fused KDA decode step (conv + gate + recurrence + norm), one token per request.

    Layouts follow the reference's own input builder for this op
    (scripts/decode/kda_fusion/compare_kda_decode_fusion.py:124-186, :288-312): rows of ``x``,
    ``raw_beta`` and ``output_gate`` are views into wider storage, the conv window and the FP32
    state of a slot share one page of a paged cache (conv in the SD layout: channel stride 1, tap
    stride 3*H*128), slot ids count down from ``B`` so that none equals its row.  ``pad_rows``
    get slot -1.  Returns call arguments (device tensors) under their argument names plus
    ``_cache`` (the page storage, uint8).
    """
    device = torch.device(device)
    g = _gen(seed)
    dim = H * D
    slots = slots or B + 2
    W = 4
    eb = torch.empty((), dtype=dtype).element_size()

    def rand(*shape, scale=1.0):
        return torch.randn(*shape, generator=g) * scale

    x_store = rand(B, 3 * dim + 24).to(dtype).to(device)
    beta_store = rand(1, B, H + 1).to(dtype).to(device)
    gate_store = rand(B, dim + 8).to(dtype).to(device)
    conv_elems = 3 * dim * (W - 1)
    page_bytes = conv_elems * eb + H * D * D * 4
    cache = torch.zeros(slots * page_bytes, dtype=torch.uint8, device=device)
    conv = torch.as_strided(cache.view(dtype), (slots, 3 * dim, W - 1), (page_bytes // eb, 1, 3 * dim))
    state = torch.as_strided(cache.view(torch.float32), (slots, H, D, D), (page_bytes // 4, D * D, D, 1),
                             storage_offset=conv_elems * eb // 4)
    if device.type == "cuda":                      # the pools can be several GB: draw them on the device
        dg = torch.Generator(device=device).manual_seed(seed + 1)
        conv.copy_((torch.randn(slots, W - 1, 3 * dim, generator=dg, device=device) * 0.1).to(dtype).transpose(1, 2))
        for s0 in range(0, slots, 256):
            n = min(256, slots - s0)
            state[s0:s0 + n].copy_(torch.randn(n, H, D, D, generator=dg, device=device) * 0.01)
    else:
        conv.copy_(rand(slots, W - 1, 3 * dim, scale=0.1).to(dtype).transpose(1, 2))
        state.copy_(rand(slots, H, D, D, scale=0.01))
    idx = torch.arange(B, 0, -1, dtype=torch.int32)
    for r in pad_rows:
        idx[r] = -1
    return {
        "x": x_store[:, :3 * dim],
        "weight": rand(3, W, dim, scale=0.1).to(device),
        "bias": rand(3 * dim, scale=0.1).to(device) if bias else None,
        "conv_state": conv,
        "raw_g": rand(1, B, H, D).to(dtype).to(device),
        "raw_beta": beta_store[:, :, :H],
        "a_log": rand(H, scale=0.5).to(device),
        "dt_bias": rand(dim, scale=0.1).to(device),
        "state_indices": idx.to(device),
        "state": state,
        "output_gate": gate_store[:, :dim].view(B, H, D),
        "norm_weight": rand(D).to(device),
        "_cache": cache,
    }


def kda_replay_verify(N, H, num_draft, seed=0, device="cuda", ring_len=None, slots=None, lower_bound=-8.0,
                      onorm=True, pad_rows=(), strided=True, index_dtype=torch.int32):
    """KDA speculative verify with replay records (ring mode): ``N`` requests of ``num_draft`` tokens.

    Shapes and distributions follow the reference's input builder
    (scripts/decode/kda_mtp_sglang/private/_common.py:84-166).  With ``strided`` the q/k/v inputs are the
    three segments of one mixed row, the conv states the transposed segments of a [slots, 3, 3*H*128]
    pool and the scratch windows segments of one [rows, steps, 3*H*128, 3] buffer, as SGLang passes them.
    Slot ids are a seeded permutation, scratch rows a different one; ``pad_rows`` get slot -1.
    Returns the keyword arguments of ``fused_kda_decode_mtp_dspark``.
    """
    device = torch.device(device)
    g = _gen(seed)
    dim, T, W = H * D, N * num_draft, 4
    ring_len = ring_len or max(16, num_draft)
    slots = slots or N + 2

    def bf16(*shape, scale=1.0):
        return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)

    if strided:
        mixed = bf16(1, T, 3 * dim + 64, scale=0.5).to(device)
        x_q, x_k, x_v = (mixed[:, :, i * dim:(i + 1) * dim].view(1, T, H, D) for i in range(3))
        pool = bf16(slots, W - 1, 3 * dim, scale=0.3).to(device)
        cs_q, cs_k, cs_v = (pool[:, :, i * dim:(i + 1) * dim].transpose(-1, -2) for i in range(3))
        ic = torch.zeros(N + 1, num_draft + 1, 3 * dim, W - 1, dtype=torch.bfloat16, device=device)
        ic_q, ic_k, ic_v = (ic[:, :, i * dim:(i + 1) * dim] for i in range(3))
        gate_store = bf16(1, T, dim + 32, scale=0.5).to(device)
        onorm_gate = gate_store[:, :, :dim].view(1, T, H, D)
    else:
        x_q, x_k, x_v = (bf16(1, T, H, D, scale=0.5).to(device) for _ in range(3))
        cs_q, cs_k, cs_v = (bf16(slots, dim, W - 1, scale=0.3).to(device) for _ in range(3))
        ic_q, ic_k, ic_v = (torch.zeros(N + 1, num_draft, dim, W - 1, dtype=torch.bfloat16, device=device)
                            for _ in range(3))
        onorm_gate = bf16(1, T, H, D, scale=0.5).to(device)
    conv_w = (torch.randn(3 * dim, W, generator=g) * 0.3).to(device)
    idx = torch.randperm(slots, generator=g)[:N].to(index_dtype)
    for r in pad_rows:
        idx[r] = -1
    out = dict(
        x_q=x_q, x_k=x_k, x_v=x_v, w_q=conv_w[:dim], w_k=conv_w[dim:2 * dim], w_v=conv_w[2 * dim:],
        cs_q=cs_q, cs_k=cs_k, cs_v=cs_v,
        g=bf16(1, T, H, D, scale=0.5).to(device), beta=bf16(1, T, H).to(device),
        A_log=(torch.rand(H, generator=g) * 0.5 + 0.5).to(device),
        dt_bias=(torch.randn(dim, generator=g) * 0.1).to(device),
        recurrent_state=(torch.randn(slots, H, D, D, generator=g) * 0.1).to(device),
        intermediate_ssm=None,
        intermediate_state_indices=torch.randperm(N + 1, generator=g)[:N].to(index_dtype).to(device),
        intermediate_conv_q=ic_q, intermediate_conv_k=ic_k, intermediate_conv_v=ic_v,
        ssm_state_indices=idx.to(device),
        cu_seqlens=torch.arange(0, T + 1, num_draft, dtype=index_dtype).to(device),
        lower_bound=lower_bound, scale=D ** -0.5,
        replayssm_rawv=torch.full((slots, H, ring_len, D), 3.0, dtype=torch.bfloat16, device=device),
        replayssm_rawk=torch.full((slots, H, ring_len, D), 3.0, dtype=torch.bfloat16, device=device),
        replayssm_g=torch.full((slots, H, ring_len, D), 3.0, dtype=torch.float32, device=device),
        replayssm_beta=torch.full((slots, H, ring_len), 3.0, dtype=torch.float32, device=device),
    )
    if onorm:
        out.update(onorm_gate=onorm_gate, onorm_weight=(torch.rand(D, generator=g) * 0.5 + 0.75).to(device),
                   onorm_eps=1e-6)
    return out


def kda_replay_paged(N, H, Q, slots=None, layout="DS", seed=0, device="cuda", lower_bound=-5.0, history=None):
    """Request-row (vLLM-style) KDA replay workload: ``N`` requests of ``Q`` draft tokens over paged caches.

    Every page holds the conv history of the 3*H*128 channels (``DS`` = [channels, history], ``SD`` =
    [history, channels]) followed by the FP32 checkpoint [H, 128, 128], as the reference's test lays its
    pages out (tests/test_kda_replayssm_vllm.py:45-96).  Returns a namespace with the keyword arguments of
    ``kda_replay_verify`` (``verify``), the layer object a ``KDAReplayCommitContext`` takes (``layer``) and
    the index vectors."""
    from types import SimpleNamespace
    from .decode.kda_replayssm_vllm import KDAReplayRecords
    device = torch.device(device)
    g = _gen(seed)
    slots = slots or 2 * N + 1
    c = 3 * H * D
    history = history or Q + 2
    conv_shape = (c, history) if layout == "DS" else (history, c)
    state_offset = ((c * history * 2 + 15) // 16) * 16
    page_bytes = ((state_offset + H * D * D * 4 + 255) // 256) * 256
    raw = torch.zeros(slots * page_bytes, dtype=torch.uint8, device=device)
    conv = raw.view(torch.bfloat16).as_strided((slots, *conv_shape), (page_bytes // 2, *torch.empty(conv_shape).stride()))
    state = raw.view(torch.float32).as_strided((slots, H, D, D), (page_bytes // 4, D * D, D, 1), state_offset // 4)
    for s0 in range(0, slots, 64):                      # bounded host staging
        n = min(64, slots - s0)
        conv[s0:s0 + n].copy_((torch.randn(n, *conv_shape, generator=g) * 0.2).to(torch.bfloat16))
        state[s0:s0 + n].copy_(torch.randn(n, H, D, D, generator=g) * 0.1)
    T = N * Q
    rows = (torch.randn(T, 4 * H * D + H, generator=g) * 0.4).to(torch.bfloat16).to(device)
    hd = H * D
    records = KDAReplayRecords.allocate(N, H, Q, device)
    source = (1 + torch.randperm(slots - 1, generator=g)[:N]).to(torch.int32).to(device)      # slot 0 is the null block
    offsets = torch.arange(0, T + 1, Q, dtype=torch.int32, device=device)
    verify = dict(mixed_qkv=rows[:, :3 * hd], raw_g=rows[:, 3 * hd:4 * hd], raw_beta=rows[:, 4 * hd:],
                  conv_weight=(torch.randn(3 * hd, 4, generator=g) * 0.2).to(device),
                  A_log=(torch.randn(H, generator=g) * 0.1).to(device), dt_bias=(torch.randn(hd, generator=g) * 0.2).to(device),
                  lower_bound=lower_bound, conv_state=conv, checkpoint_state=state, records=records,
                  query_start_loc=offsets, state_indices=source, conv_state_layout=layout, null_block_id=0)
    layer = SimpleNamespace(kv_cache=(conv, state), replay_records=records)
    return SimpleNamespace(verify=verify, layer=layer, source=source, offsets=offsets, raw=raw, tokens=T)
