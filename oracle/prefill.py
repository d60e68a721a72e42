"""Prefill oracles: token recurrence (the definition) and a float64 chunked form.

Test infrastructure only; see ``oracle/__init__.py``.
"""

import torch

from .gates import softplus_gate, lower_bound_gate, sigmoid_beta, l2norm


def token_recurrence(q, k, v, g, beta, offsets, state0, *, scale, compute_dtype=torch.float32):
    """Gated delta rule, one token at a time, vectorised over value heads.

    ``q,k [T,H,K]`` (already normalised, NOT scaled), ``v [T,HV,V]``,
    ``g [T,HV]`` (scalar gate) or ``[T,HV,K]`` (per channel), log-decay per token,
    ``beta [T,HV]`` activated; ``offsets`` python list of N+1 packed sequence
    boundaries (tokens past ``offsets[-1]`` are padding: output zero, no state
    effect); ``state0 [N,HV,V,K]`` or ``None``.

    Follows tests/test_kda_prefill_flashkdapro.py:547-556 (float64 natural-log
    recurrence, k-last state) and scripts/decode/_kda_reference.py:83-92.
    Returns ``(o [T,HV,V] compute_dtype, final_state [N,HV,V,K] compute_dtype)``.
    """
    cd = compute_dtype
    T, HV, V = v.shape
    K = q.shape[-1]
    rep = HV // q.shape[1]
    qf = (q.to(cd) * scale).repeat_interleave(rep, dim=1)
    kf = k.to(cd).repeat_interleave(rep, dim=1)
    vf = v.to(cd)
    gf = g.to(cd)
    if gf.dim() == 2:
        gf = gf[..., None]
    decay = gf.exp()
    bf = beta.to(cd)
    N = len(offsets) - 1
    out = torch.zeros(T, HV, V, dtype=cd)
    final = torch.zeros(N, HV, V, K, dtype=cd) if state0 is None else state0.to(cd).clone()
    for n in range(N):
        S = final[n]
        for t in range(offsets[n], offsets[n + 1]):
            S = S * decay[t][:, None, :]
            d = torch.einsum("hvk,hk->hv", S, kf[t])
            u = (vf[t] - d) * bf[t][:, None]
            S = S + u[:, :, None] * kf[t][:, None, :]
            out[t] = torch.einsum("hvk,hk->hv", S, qf[t])
        final[n] = S
    return out, final


def chunked_delta_rule_fp64(q, k, v, g, beta, S0, *, scale, chunk=64):
    """Float64 chunked (WY / UT) evaluation of one sequence; an independent
    second evaluation order used to cross-check ``token_recurrence`` and to
    provide an accurate target at sizes where the token loop is too slow.

    Same algebra as scripts/prefill/flashqla/private/ref_gdr.py:78-298
    (``torch_kkt_fwd`` / ``torch_solve`` / ``torch_w_u_fwd`` /
    ``torch_chunk_gdr_fwd`` / ``torch_chunk_o_fwd``), written for a k-last state
    and a per-channel gate with all decays in difference form
    ``exp(G_i - G_j)``, ``i >= j`` (never larger than one).

    ``q,k [T,H,K]`` normalised, ``v [T,HV,V]``, ``g [T,HV]`` or ``[T,HV,K]``,
    ``beta [T,HV]``, ``S0 [HV,V,K]`` or None.  Returns ``(o [T,HV,V], S [HV,V,K])`` float64.
    """
    f64 = torch.float64
    T, HV, V = v.shape
    K = q.shape[-1]
    rep = HV // q.shape[1]
    qd = (q.to(f64) * scale).repeat_interleave(rep, dim=1).transpose(0, 1)   # [HV,T,K]
    kd = k.to(f64).repeat_interleave(rep, dim=1).transpose(0, 1)
    vd = v.to(f64).transpose(0, 1)                                           # [HV,T,V]
    gd = g.to(f64)
    if gd.dim() == 2:
        gd = gd[..., None].expand(T, HV, K)
    gd = gd.transpose(0, 1)                                                  # [HV,T,K]
    bd = beta.to(f64).transpose(0, 1)                                        # [HV,T]
    S = torch.zeros(HV, V, K, dtype=f64) if S0 is None else S0.to(f64).clone()
    o = torch.zeros(HV, T, V, dtype=f64)
    for c0 in range(0, T, chunk):
        c1 = min(c0 + chunk, T)
        C = c1 - c0
        kc, qc, vc, bc = kd[:, c0:c1], qd[:, c0:c1], vd[:, c0:c1], bd[:, c0:c1]
        G = gd[:, c0:c1].cumsum(1)                                           # [HV,C,K]
        diff = G[:, :, None, :] - G[:, None, :, :]                           # [HV,i,j,K]
        low = torch.tril(torch.ones(C, C, dtype=torch.bool))
        E = torch.where(low[None, :, :, None], diff, torch.full_like(diff, -float("inf"))).exp()
        M = torch.einsum("hik,hjk,hijk->hij", kc, kc, E)
        P = torch.einsum("hik,hjk,hijk->hij", qc, kc, E)                     # j <= i kept
        strict = torch.tril(torch.ones(C, C, dtype=f64), -1)
        L = torch.eye(C, dtype=f64) + bc[:, :, None] * M * strict
        rhs = bc[:, :, None] * (vc - torch.einsum("hik,hvk->hiv", kc * G.exp(), S))
        U = torch.linalg.solve_triangular(L, rhs, upper=False)               # [HV,C,V]
        o[:, c0:c1] = torch.einsum("hik,hvk->hiv", qc * G.exp(), S) + torch.einsum("hij,hjv->hiv", P, U)
        Gl = G[:, -1:, :]
        S = S * Gl.exp() + torch.einsum("hjv,hjk->hvk", U, kc * (Gl - G).exp())
    return o.transpose(0, 1).contiguous(), S


def gdn_prefill_reference(q, k, v, a, b, A_log, dt_bias, offsets, state0, *,
                          scale=None, normalize_qk=True, compute_dtype=torch.float32):
    """Reference for ``gdn_prefill_packed_qkv_fwd`` / ``chunk_gated_delta_rule_fwd``
    with raw gating.

    Pre-processing follows
    src/prefill/flashqla/kernels/chunk_cumsum_cute.cu:260-318: q and k are
    L2-normalised in float32 (eps 1e-6 inside the root) and ROUNDED to the
    activation dtype; ``g = -exp(A_log) * softplus(a + dt_bias)`` with the
    linear branch above 20; ``beta = sigmoid(b)``; all gate math in float32.
    The recurrence then follows ``token_recurrence``.

    ``q,k [T,H,K]``, ``v [T,HV,V]``, ``a,b [T,HV]`` activation dtype,
    ``A_log, dt_bias [HV]`` float32.  Returns ``(o [T,HV,V] v.dtype, final [N,HV,V,K])``.
    """
    if scale is None:
        scale = q.shape[-1] ** -0.5
    if normalize_qk:
        q = l2norm(q).to(q.dtype)
        k = l2norm(k).to(k.dtype)
    g = softplus_gate(a, dt_bias, A_log, 1.0, 20.0, per_channel=False)
    beta = sigmoid_beta(b)
    o, final = token_recurrence(q, k, v, g, beta, offsets, state0, scale=scale,
                                compute_dtype=compute_dtype)
    return o.to(v.dtype), final


def kda_prefill_reference(q, k, v, g_raw, beta_raw, A_log, dt_bias, offsets, state0, *,
                          scale=None, lower_bound=-5.0, compute_dtype=torch.float32):
    """Reference for ``flashkda_fwd``.

    Follows tests/test_kda_prefill_flashkdapro.py:538-556: q and k L2-normalised
    then rounded to bf16 (the public normalisation boundary), per-channel
    lower-bound gate ``exp(lb * sigmoid(exp(A_log) * (g_raw + dt_bias)))``,
    ``beta = sigmoid(beta_raw)``, k-last state.

    ``q,k,v,g_raw [T,H,128]``, ``beta_raw [T,H]``, ``A_log [H]``, ``dt_bias [H,K]``.
    """
    if scale is None:
        scale = q.shape[-1] ** -0.5
    q = l2norm(q).to(q.dtype)
    k = l2norm(k).to(k.dtype)
    g = lower_bound_gate(g_raw, dt_bias, A_log, lower_bound, per_channel=True)
    beta = sigmoid_beta(beta_raw)
    o, final = token_recurrence(q, k, v, g, beta, offsets, state0, scale=scale,
                                compute_dtype=compute_dtype)
    return o.to(v.dtype), final
