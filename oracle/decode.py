"""Token-recurrence oracle for k-last decode, MTP verify and accepted-prefix commit.

Test infrastructure only; see ``oracle/__init__.py``.

State layout is k-last: ``S[hv, v, k]``.  One step, per value head
(scripts/decode/kda_mtp_sglang/private/_reference.py:44-50)::

    S[v,k] *= exp(g[k]);  d[v] = sum_k S[v,k] k[k];  u[v] = (v[v] - d[v]) * beta
    S[v,k] += u[v] k[k];  o[v] = sum_k S[v,k] q[k]        (q carries ``scale``)
"""

import torch

from .gates import softplus_gate, lower_bound_gate, sigmoid_beta, l2norm


def recurrent_step(S, q, k, v, log_decay, beta):
    """One gated delta-rule step on ``S [HV,V,K]`` (updated copy returned).

    ``q,k [HV,K]`` (already normalised / scaled / head-expanded), ``v [HV,V]``,
    ``log_decay [HV,K]`` or ``[HV,1]``, ``beta [HV]``.  Returns ``(S_new, o [HV,V])``.
    Follows tests/test_k_last_state_dtype.py:146-149.
    """
    S = S * log_decay.exp()[:, None, :]
    d = torch.einsum("hvk,hk->hv", S, k)
    u = (v - d) * beta[:, None]
    S = S + u[:, :, None] * k[:, None, :]
    o = torch.einsum("hvk,hk->hv", S, q)
    return S, o


def _invalid_slot(slot, is_sglang):
    # sglang: pad id is negative, slot 0 is real; vLLM: block 0 is the null block
    # (src/decode/k-last/fused_sigmoid_gating_k_last_kernel.cuh:232-248).
    return slot < 0 if is_sglang else slot <= 0


def k_last_reference(q, k, v, a, b, A_log, dt_bias, state, state_indices, lengths, *,
                     scale=None, use_qk_l2norm=True, is_kda=False,
                     disable_state_update=False,
                     cache=None, cache_indices=None, num_accepted=None, parents=None,
                     lower_bound=None, is_sglang=True,
                     softplus_beta=1.0, softplus_threshold=20.0,
                     log_decay=None, beta_activated=None, compute_dtype=torch.float32):
    """Reference for ``fused_sigmoid_gating_delta_rule_forward_k_last{,_packed}``.

    Restates tests/test_k_last_state_dtype.py:108-156 (``reference``) and adds
    the vLLM 2-D slot-table mode of
    src/decode/k-last/fused_sigmoid_gating_k_last_kernel.cuh:215-229, 847-863.

    Token tensors are flat over requests: ``q,k [ntok,H,K]``, ``v [ntok,HV,V]``,
    ``a [ntok,HV]`` (GDN) or ``[ntok,HV,K]`` (KDA), ``b [ntok,HV]``;
    ``lengths[n]`` tokens belong to request ``n``.  ``state [slots,HV,V,K]``.
    ``state_indices``: list ``[B]`` or nested list ``[B][S]`` (vLLM, requires
    ``is_sglang=False``).  ``log_decay`` (same shape as ``a``, float) replaces
    the gate computed from ``a/A_log/dt_bias``; ``beta_activated`` replaces
    ``sigmoid(b)``.

    Returns ``(out [ntok,HV,V] in v.dtype, state_after, cache_after)``; inputs
    are not modified.
    """
    cd = compute_dtype
    K = q.shape[-1]
    HV = v.shape[1]
    if scale is None:
        scale = K ** -0.5
    qf, kf = q.float(), k.float()
    if use_qk_l2norm:
        qf, kf = l2norm(qf), l2norm(kf)
    qf = qf * scale
    rep = HV // q.shape[1]
    qf = qf.repeat_interleave(rep, dim=1).to(cd)
    kf = kf.repeat_interleave(rep, dim=1).to(cd)
    vf = v.to(cd)
    if log_decay is None:
        if lower_bound is not None:
            g = lower_bound_gate(a, dt_bias, A_log, lower_bound, per_channel=is_kda)
        else:
            g = softplus_gate(a, dt_bias, A_log, softplus_beta, softplus_threshold,
                              per_channel=is_kda)
    else:
        g = log_decay.float()
    g = g.to(cd)
    if not is_kda:
        g = g[..., None]
    beta = (sigmoid_beta(b) if beta_activated is None else beta_activated.float()).to(cd)

    state = state.clone()
    cache = None if cache is None else cache.clone()
    out = torch.zeros_like(vf)
    two_d = len(state_indices) > 0 and isinstance(state_indices[0], (list, tuple))
    bos = 0
    for n, length in enumerate(lengths):
        if length == 0:                      # empty request: nothing is read or written
            continue
        if two_d:
            acc = 1 if num_accepted is None else int(num_accepted[n])
            col = acc - 1 if acc > 0 else 0
            slot = int(state_indices[n][col])
        else:
            slot = int(state_indices[n])
        if _invalid_slot(slot, is_sglang):   # zeros in o, no state / cache access
            bos += length
            continue
        cidx = -1
        if cache is not None and cache_indices is not None:
            cidx = int(cache_indices[n])
        h = state[slot].to(cd)
        for t in range(length):
            if parents is not None and t > 0 and cidx >= 0:
                parent = int(parents[n][t])
                if parent >= 0 and parent != t - 1:
                    h = cache[cidx, parent].to(cd)
            i = bos + t
            h, o = recurrent_step(h, qf[i], kf[i], vf[i], g[i], beta[i])
            out[i] = o
            if is_sglang:
                if cache is not None and cidx >= 0:
                    cache[cidx, t] = h.to(cache.dtype)
            elif two_d:
                step_slot = int(state_indices[n][t])
                if step_slot > 0:
                    state[step_slot] = h.to(state.dtype)
        if not disable_state_update:
            state[slot] = h.to(state.dtype)
        bos += length
    return out.to(v.dtype), state, cache


def fold_reference(state, rawk, rawv, g, beta, slot_indices, accept_lens, *,
                   null_block_id=-1, compute_dtype=torch.float32):
    """Accepted-prefix commit: replay ``accept_lens[n]`` recorded tokens into the state.

    Restates scripts/decode/kda_mtp_sglang/private/_reference.py:183-216
    (``fold_reference``; one layer): raw k is L2-normalised in division form
    with eps inside the square root, then decay -> delta -> rank-1.  A request
    whose slot is ``<= null_block_id`` or whose accepted length is ``<= 0``
    leaves its slot untouched (src/decode/kda_replayssm/kda_mtp_fold.cu:306).

    ``state [slots,HV,V,K]``; records are indexed by slot: ``rawk [slots,H,L,K]``,
    ``rawv [slots,HV,L,V]``, ``g [slots,HV,L,K]`` (log-decay), ``beta [slots,HV,L]``.
    Returns the folded copy of ``state``.
    """
    cd = compute_dtype
    state = state.clone()
    HV = state.shape[1]
    H = rawk.shape[1]
    rep = HV // H
    for n, slot in enumerate(slot_indices):
        slot = int(slot)
        n_acc = int(accept_lens[n])
        if slot <= null_block_id or n_acc <= 0:
            continue
        h = state[slot].to(cd)
        for t in range(n_acc):
            kk = rawk[slot, :, t].to(cd)
            kk = kk / torch.sqrt((kk * kk).sum(-1, keepdim=True) + 1e-6)
            kk = kk.repeat_interleave(rep, dim=0)
            h = h * g[slot, :, t].to(cd).exp()[:, None, :]
            d = torch.einsum("hvk,hk->hv", h, kk)
            u = (rawv[slot, :, t].to(cd) - d) * beta[slot, :, t].to(cd)[:, None]
            h = h + u[:, :, None] * kk[:, None, :]
        state[slot] = h.to(state.dtype)
    return state


def causal_conv1d_update_reference(x, conv_state, weight, bias, slots):
    """Width-4 causal conv1d update + SiLU for one new sample per request.

    ``x [B, C]``, ``conv_state [slots, C, 3]`` (oldest tap first; updated copy returned),
    ``weight [4, C]`` width-major float32, ``bias [C]`` or None, ``slots`` a list of ints
    (negative: the request is skipped).  Returns ``(y [B, C] float32, conv_state_new)``.
    Follows scripts/decode/kda_fusion/compare_kda_decode_fusion.py:243-255: the window is the
    three stored taps followed by the new sample; the stored taps shift by one and the new sample
    (unrounded copy of ``x``) becomes the newest tap.
    """
    conv = conv_state.clone()
    y = torch.zeros(x.shape, dtype=torch.float32)
    w = weight.float()
    for n, slot in enumerate(slots):
        if slot < 0:
            continue
        window = torch.cat([conv[slot].float(), x[n].float()[:, None]], dim=1)      # [C, 4]
        acc = (window * w.t()).sum(-1)
        if bias is not None:
            acc = acc + bias.float()
        y[n] = acc * torch.sigmoid(acc)
        conv[slot, :, 0] = conv_state[slot, :, 1]
        conv[slot, :, 1] = conv_state[slot, :, 2]
        conv[slot, :, 2] = x[n]
    return y, conv


def kda_decode_mega_reference(x, weight, bias, conv_state, raw_g, raw_beta, a_log, dt_bias, state_indices,
                              state, *, lower_bound=None, output_gate=None, norm_weight=None, norm_eps=1e-5,
                              round_v=True):
    """Reference for ``fused_kda_decode_mega_forward`` (one decode token per request).

    Follows the reference's own step-by-step float32 golden
    scripts/decode/kda_fusion/compare_kda_decode_fusion.py:209-282 (conv + SiLU, q/k L2 norm with
    eps 1e-6 inside the root, q scaled by 128^-0.5, softplus or lower-bound per-channel decay,
    sigmoid beta, k-last recurrence, RMSNorm * weight * sigmoid(gate)), and the pad rule of
    scripts/decode/kda_fusion/test_pad_slot.py:37-53 (slot < 0: zero output, no pool write).
    ``round_v``: the activated v is rounded to the activation dtype before the recurrence, as the
    reference kernel does (src/decode/k-last/fused_kda_decode_mega_kernel.cuh:384, :463); the
    float32 golden of the script does not round.

    ``x [B,3*H*128]``, ``weight [3,4,H*128]``, ``bias [3*H*128]`` or None,
    ``conv_state [slots,3*H*128,3]``, ``raw_g [1,B,H,128]``, ``raw_beta [1,B,H]``, ``a_log [H]``,
    ``dt_bias [H*128]``, ``state [slots,H,128,128]`` float32, ``output_gate [B,H,128]``.
    Returns ``(out [1,B,H,128] in x.dtype, state_new, conv_state_new)``.
    """
    B = x.shape[0]
    D = 128
    H = x.shape[1] // (3 * D)
    dim = H * D
    slots = [int(s) for s in state_indices.tolist()]
    w_flat = weight.float().permute(1, 0, 2).reshape(4, 3 * dim)                   # [4, 3*dim] width-major
    mixed, conv_new = causal_conv1d_update_reference(x, conv_state, w_flat, bias, slots)
    state_new = state.clone()
    out = torch.zeros(1, B, H, D, dtype=x.dtype)
    dt = dt_bias.float().reshape(H, D)
    for n, slot in enumerate(slots):
        if slot < 0:
            continue
        q = l2norm(mixed[n, :dim].reshape(H, D)) * (float(D) ** -0.5)
        k = l2norm(mixed[n, dim:2 * dim].reshape(H, D))
        v = mixed[n, 2 * dim:].reshape(H, D)
        if round_v:
            v = v.to(x.dtype).float()
        g = raw_g[0, n].float()
        if lower_bound is not None:
            log_decay = lower_bound_gate(g, dt, a_log, lower_bound, per_channel=True)
        else:
            log_decay = softplus_gate(g, dt, a_log, per_channel=True)
        beta = sigmoid_beta(raw_beta[0, n])
        S, o = recurrent_step(state_new[slot].float(), q, k, v, log_decay, beta)
        state_new[slot] = S
        if output_gate is not None:
            gate = torch.sigmoid(output_gate.reshape(B, H, D)[n].float())
            o = o * torch.rsqrt(o.square().mean(-1, keepdim=True) + norm_eps) * norm_weight.float()[None, :] * gate
        out[0, n] = o.to(x.dtype)
    return out, state_new, conv_new


def causal_conv_silu_sequence(x_seq, window, weight):
    """Width-4 causal conv + SiLU of ``x_seq [T, C]`` seeded by ``window [C, 3]`` (oldest tap first),
    ``weight [C, 4]`` (taps oldest first).  Returns ``(y [T, C] float64, windows [T, C, 3])`` where
    ``windows[t]`` is the window after token ``t`` was consumed
    (scripts/decode/kda_mtp_sglang/private/_reference.py:66-85)."""
    T, C = x_seq.shape
    full = torch.cat([window.double().t(), x_seq.double()], dim=0)                  # [3 + T, C]
    w = weight.double()
    y = torch.empty(T, C, dtype=torch.float64)
    wins = torch.empty(T, C, 3, dtype=torch.float64)
    for t in range(T):
        acc = (full[t:t + 4] * w.t()).sum(0)
        y[t] = acc * torch.sigmoid(acc)
        wins[t] = full[t + 1:t + 4].t()
    return y, wins


def verify_dspark_reference(*, x_q, x_k, x_v, g, beta, w_q, w_k, w_v, cs_q, cs_k, cs_v, A_log, dt_bias,
                            recurrent_state, ssm_state_indices, intermediate_state_indices, cu_seqlens,
                            lower_bound, scale, rings, windows, onorm_gate=None, onorm_weight=None, onorm_eps=None):
    """Reference for ``fused_kda_decode_mtp_dspark`` (ring mode), float64 throughout.

    Restates scripts/decode/kda_mtp_sglang/private/_reference.py:88-177: per request and head, conv +
    SiLU of the draft tokens from the (read-only) conv state, records of the post-conv k (before its
    L2 norm) and v, of the log-decay ``lower_bound * sigmoid(exp(A_log) (g + dt_bias))`` and of
    ``sigmoid(beta)`` at ring position t, the window after every token in the request's scratch row,
    and the delta-rule recurrence from the (read-only) state with ``q`` scaled after its L2 norm;
    optional ``o * rsqrt(mean(o^2) + eps) * weight * sigmoid(gate)``.  ``rings`` = (rawv, rawk, g, beta)
    and ``windows`` = (ic_q, ic_k, ic_v) are copied and returned updated in their own dtypes; slots < 0
    are skipped (their output rows stay zero).

    Returns ``dict(out [1,T,H,128] float64, ring_rawv, ring_rawk, ring_g, ring_beta, ic_q, ic_k, ic_v)``.
    """
    D = 128
    T, H = x_q.shape[1], x_q.shape[2]
    out = torch.zeros(1, T, H, D, dtype=torch.float64)
    rawv, rawk, ring_g, ring_beta = (r.clone() for r in rings)
    ic = [w.clone() for w in windows]
    cu = [int(v) for v in cu_seqlens.tolist()]
    slots = [int(v) for v in ssm_state_indices.tolist()]
    rows = [int(v) for v in intermediate_state_indices.tolist()]
    xs = [x_q[0].double(), x_k[0].double(), x_v[0].double()]
    ws = [w_q, w_k, w_v]
    css = [cs_q, cs_k, cs_v]
    graw, braw = g[0].double(), beta[0].double()
    dt = dt_bias.double().reshape(H, D)
    for n, slot in enumerate(slots):
        if slot < 0:
            continue
        bos, eos = cu[n], cu[n + 1]
        nt = eos - bos
        for h in range(H):
            sl = slice(h * D, (h + 1) * D)
            conv = []
            for i in range(3):
                y, wins = causal_conv_silu_sequence(xs[i][bos:eos, h], css[i][slot, sl], ws[i][sl])
                conv.append(y)
                ic[i][rows[n], :nt, sl] = wins.to(ic[i].dtype)
            q_c, k_c, v_c = conv
            rawk[slot, h, :nt] = k_c.to(rawk.dtype)
            rawv[slot, h, :nt] = v_c.to(rawv.dtype)
            q_n = q_c / torch.sqrt((q_c * q_c).sum(-1, keepdim=True) + 1e-6) * scale
            k_n = k_c / torch.sqrt((k_c * k_c).sum(-1, keepdim=True) + 1e-6)
            b = torch.sigmoid(braw[bos:eos, h])
            ring_beta[slot, h, :nt] = b.to(ring_beta.dtype)
            gk = lower_bound * torch.sigmoid(A_log[h].double().exp() * (graw[bos:eos, h] + dt[h]))
            ring_g[slot, h, :nt] = gk.to(ring_g.dtype)
            S = recurrent_state[slot, h].double()[None]
            for t in range(nt):
                S, o = recurrent_step(S, q_n[t][None], k_n[t][None], v_c[t][None], gk[t][None], b[t][None])
                out[0, bos + t, h] = o[0]
    if onorm_gate is not None:
        gate = torch.sigmoid(onorm_gate[0].double())
        rms = torch.rsqrt((out[0] * out[0]).mean(-1, keepdim=True) + onorm_eps)
        out = (out[0] * rms * onorm_weight.double()[None, None, :] * gate)[None]
    return dict(out=out, ring_rawv=rawv, ring_rawk=rawk, ring_g=ring_g, ring_beta=ring_beta,
                ic_q=ic[0], ic_k=ic[1], ic_v=ic[2])


def conv_window_scatter_reference(dst, src, dst_idx, step_idx):
    """``dst[layer, dst_idx[r]] = src[layer, r, step_idx[r]]`` for requests with a non-negative step and an
    in-range destination (src/decode/kda_replayssm/kda_mtp_fold.cu:602-634).  Returns the updated copy."""
    out = dst.clone()
    for r, (d, s) in enumerate(zip(dst_idx.tolist(), step_idx.tolist())):
        if s < 0 or d < 0 or d >= dst.shape[1] or r >= src.shape[1] or s >= src.shape[2]:
            continue
        out[:, d] = src[:, r, s]
    return out


def replay_commit_plan_reference(num_sampled, state_indices, query_start_loc, *, slots, Q, token_capacity,
                                 null_block_id=0, request_indices=None, block_table=None, num_computed_tokens=None,
                                 block_size=None, capacity=None):
    """Commit plan of the request-row replay as four lists of ``capacity`` integers (commit length, final
    slot, boundary slot, boundary length).

    Restates src/decode/kda_replayssm_vllm/commit_plan.cu:19-117 (``build_plan`` + ``protect_plan``) and the
    expected plan of the reference's test oracle tests/test_kda_replayssm_vllm.py:148-178: a request commits
    ``min(max(sampled, 0), query length)`` tokens if its source slot and query interval are valid; in align
    mode the final state belongs to the block of token ``p + n - 1`` and, when the window reaches the next
    block boundary, the state after ``block_size - p % block_size`` tokens to the block of position ``p``;
    requests whose destinations collide with another live source or another committing request's
    destinations (or whose source is another's destination) are cancelled on both sides.
    """
    N = len(state_indices)
    capacity = N if capacity is None else capacity
    valid_slot = lambda s: s > null_block_id and 0 <= s < slots
    valid_iv = lambda a, b: a >= 0 and b > a and b <= token_capacity and b - a <= Q
    cand = [[0, 0, 0, 0] for _ in range(capacity)]
    for b in range(N):
        row = b if request_indices is None else request_indices[b]
        src = state_indices[b]
        begin, end = query_start_loc[b], query_start_loc[b + 1]
        if not (query_start_loc[0] == 0 and 0 <= row < len(num_sampled) and valid_slot(src) and valid_iv(begin, end)):
            continue
        n = min(max(num_sampled[row], 0), end - begin)
        final, boundary, bc = src, 0, 0
        if n and block_table is not None:
            if row >= len(block_table) or num_computed_tokens[row] < 0:
                n = 0
            else:
                p = num_computed_tokens[row]
                cols = len(block_table[row])
                f = block_table[row][min((p + n - 1) // block_size, cols - 1)]
                if not valid_slot(f):
                    n = 0
                else:
                    final = f
                distance = block_size - p % block_size
                if n and n >= distance:
                    col = p // block_size
                    if col >= cols:
                        n = 0
                    else:
                        dest = block_table[row][col]
                        if not valid_slot(dest) or (dest == final and distance != n):
                            n = 0
                        else:
                            boundary, bc = dest, distance
        if n:
            cand[b] = [n, final, boundary, bc]
    plan = [list(c) for c in cand]
    for b in range(N):
        if not cand[b][0]:
            continue
        _, f, d, bc = cand[b]
        src = state_indices[b]
        conflict = False
        for o in range(N):
            if o == b:
                continue
            os_ = state_indices[o]
            if valid_slot(os_) and valid_iv(query_start_loc[o], query_start_loc[o + 1]):
                conflict |= f == os_ or (bc > 0 and d == os_)
            if not cand[o][0]:
                continue
            _, of, od, obc = cand[o]
            conflict |= (f == os_ or f == of or (obc > 0 and f == od)
                         or (bc > 0 and (d == os_ or d == of or (obc > 0 and d == od)))
                         or src == of or (obc > 0 and src == od))
        if conflict:
            plan[b] = [0, 0, 0, 0]
    return [[plan[b][c] for b in range(capacity)] for c in range(4)]
