"""Pins the decode oracle without importing anything from the reference:
textbook library routines, element-wise float64 loops on tiny shapes, closed
forms and prefix/commit invariants."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import (softplus_gate, lower_bound_gate, l2norm, k_last_reference,
                    fold_reference, recurrent_step)


def test_softplus_gate_matches_library_and_threshold_branch():
    torch.manual_seed(0)
    a = torch.randn(7, 5) * 12
    dt = torch.randn(5)
    A = torch.rand(5) * math.log(16)
    g = softplus_gate(a, dt, A)
    want = -A.exp() * F.softplus(a + dt, beta=1.0, threshold=20.0)
    torch.testing.assert_close(g, want, rtol=1e-6, atol=1e-7)
    # above the threshold the gate is exactly linear
    x = torch.tensor([[25.0, 40.0]])
    g2 = softplus_gate(x, torch.zeros(2), torch.zeros(2))
    assert torch.equal(g2, -x)
    # softplus_beta scales the argument and divides the result
    g3 = softplus_gate(a, dt, A, softplus_beta=2.0, softplus_threshold=20.0)
    want3 = -A.exp() * F.softplus(a + dt, beta=2.0, threshold=20.0)
    torch.testing.assert_close(g3, want3, rtol=1e-6, atol=1e-7)


def test_per_channel_gates():
    torch.manual_seed(1)
    a = torch.randn(3, 4, 8)
    dt = torch.randn(4, 8)
    A = torch.randn(4)
    g = softplus_gate(a, dt, A, per_channel=True)
    for h in range(4):
        torch.testing.assert_close(g[:, h], -math.exp(A[h]) * F.softplus(a[:, h] + dt[h]))
    lb = lower_bound_gate(a, dt, A, -5.0)
    for h in range(4):
        torch.testing.assert_close(lb[:, h], -5.0 * torch.sigmoid(math.exp(A[h]) * (a[:, h] + dt[h])))
    assert (lb <= 0).all() and (lb >= -5).all()


def test_l2norm_eps_inside_root():
    x = torch.tensor([[3.0, 4.0], [0.0, 0.0]])
    y = l2norm(x)
    torch.testing.assert_close(y[0], x[0] / math.sqrt(25 + 1e-6))
    assert torch.equal(y[1], torch.zeros(2))           # finite at zero thanks to eps


def _brute_force(q, k, v, g, beta, S0, scale):
    """Scalar float64 loops; S[v][k] k-last."""
    T, K, V = len(q), len(q[0]), len(v[0])
    S = [[float(S0[i][j]) for j in range(K)] for i in range(V)]
    outs = []
    for t in range(T):
        for i in range(V):
            for j in range(K):
                S[i][j] *= math.exp(g[t][j])
        u = []
        for i in range(V):
            d = sum(S[i][j] * k[t][j] for j in range(K))
            u.append((v[t][i] - d) * beta[t])
        for i in range(V):
            for j in range(K):
                S[i][j] += u[i] * k[t][j]
        outs.append([sum(S[i][j] * q[t][j] * scale for j in range(K)) for i in range(V)])
    return outs, S


@pytest.mark.parametrize("is_kda", [False, True])
def test_k_last_reference_vs_scalar_loops(is_kda):
    torch.manual_seed(3)
    T, H, HV, K, V = 3, 1, 2, 4, 3
    q = torch.randn(T, H, K, dtype=torch.float64)
    k = torch.randn(T, H, K, dtype=torch.float64)
    v = torch.randn(T, HV, V, dtype=torch.float64)
    a = torch.randn(T, HV, K) if is_kda else torch.randn(T, HV)
    dt = torch.randn(HV, K) if is_kda else torch.randn(HV)
    A = torch.randn(HV)
    b = torch.randn(T, HV)
    state = torch.randn(5, HV, V, K, dtype=torch.float64)
    out, st, _ = k_last_reference(q, k, v, a, b, A, dt, state, [3], [T], scale=0.7,
                                  use_qk_l2norm=True, is_kda=is_kda,
                                  compute_dtype=torch.float64)
    g = softplus_gate(a, dt, A, per_channel=is_kda).double()
    beta = torch.sigmoid(b.float()).double()
    for hv in range(HV):
        qn = q[:, 0] / torch.sqrt((q[:, 0] ** 2).sum(-1, keepdim=True) + 1e-6)
        kn = k[:, 0] / torch.sqrt((k[:, 0] ** 2).sum(-1, keepdim=True) + 1e-6)
        gl = [[float(g[t, hv, j]) if is_kda else float(g[t, hv]) for j in range(K)] for t in range(T)]
        outs, S = _brute_force(qn.tolist(), kn.tolist(), v[:, hv].tolist(), gl,
                               beta[:, hv].tolist(), state[3, hv].tolist(), 0.7)
        torch.testing.assert_close(out[:, hv], torch.tensor(outs, dtype=torch.float64), rtol=1e-6, atol=1e-7)
        torch.testing.assert_close(st[3, hv], torch.tensor(S, dtype=torch.float64), rtol=1e-6, atol=1e-7)
    untouched = [0, 1, 2, 4]
    assert torch.equal(st[untouched], state[untouched])


def test_step_pure_decay_when_beta_zero():
    torch.manual_seed(4)
    S = torch.randn(2, 3, 4, dtype=torch.float64)
    g = -torch.rand(2, 4, dtype=torch.float64)
    S2, o = recurrent_step(S, torch.randn(2, 4, dtype=torch.float64), torch.randn(2, 4, dtype=torch.float64),
                           torch.randn(2, 3, dtype=torch.float64), g, torch.zeros(2, dtype=torch.float64))
    torch.testing.assert_close(S2, S * g.exp()[:, None, :])


def test_step_projection_when_no_decay_and_beta_one():
    torch.manual_seed(5)
    S = torch.randn(1, 3, 4, dtype=torch.float64)
    k = torch.randn(1, 4, dtype=torch.float64)
    k = k / k.norm()
    v = torch.randn(1, 3, dtype=torch.float64)
    q = torch.randn(1, 4, dtype=torch.float64)
    S2, o = recurrent_step(S, q, k, v, torch.zeros(1, 4, dtype=torch.float64), torch.ones(1, dtype=torch.float64))
    want = S[0] @ (torch.eye(4, dtype=torch.float64) - torch.outer(k[0], k[0])) + torch.outer(v[0], k[0])
    torch.testing.assert_close(S2[0], want)
    # after the update the state maps k exactly onto v
    torch.testing.assert_close(S2[0] @ k[0], v[0])
    # and from a zero state o = v * (k . q)
    S3, o3 = recurrent_step(torch.zeros_like(S), q, k, v, torch.zeros(1, 4, dtype=torch.float64),
                            torch.ones(1, dtype=torch.float64))
    torch.testing.assert_close(o3[0], v[0] * (k[0] @ q[0]))


def test_geometric_series_closed_form():
    """k = e0, v = 1, constant gate and beta: S[:,0] follows a geometric series
    (the scenario of tests/test_kda_prefill_flashkdapro.py:293-311)."""
    T, K, V = 9, 4, 3
    g0, beta0 = -0.3, 0.25
    e0 = torch.zeros(T, 1, K, dtype=torch.float64)
    e0[..., 0] = 1
    v = torch.ones(T, 1, V, dtype=torch.float64)
    state = torch.zeros(1, 1, V, K, dtype=torch.float64)
    state[..., 0] = 0.125
    log_decay = torch.full((T, 1), g0)
    out, st, _ = k_last_reference(e0, e0, v, None, None, None, None, state, [0], [T], scale=1.0,
                                  use_qk_l2norm=False, log_decay=log_decay,
                                  beta_activated=torch.full((T, 1), beta0), compute_dtype=torch.float64)
    r = math.exp(g0) * (1 - beta0)
    for t in range(1, T + 1):
        want = r ** t * 0.125 + beta0 * (1 - r ** t) / (1 - r)
        torch.testing.assert_close(out[t - 1, 0], torch.full((V,), want, dtype=torch.float64))
    torch.testing.assert_close(st[0, 0, :, 0], torch.full((V,), r ** T * 0.125 + beta0 * (1 - r ** T) / (1 - r), dtype=torch.float64))
    assert torch.count_nonzero(st[0, 0, :, 1:]) == 0


def _mtp_case(seed=7, B=3, T=4, H=2, HV=4, D=8, is_kda=True):
    torch.manual_seed(seed)
    nt = B * T
    c = dict(
        q=torch.randn(nt, H, D), k=torch.randn(nt, H, D), v=torch.randn(nt, HV, D),
        a=torch.randn(nt, HV, D) if is_kda else torch.randn(nt, HV), b=torch.randn(nt, HV),
        A_log=torch.randn(HV), dt_bias=torch.randn(HV, D) if is_kda else torch.randn(HV),
        state=torch.randn(9, HV, D, D) * 0.1)
    return c


@pytest.mark.parametrize("is_kda", [False, True])
def test_sglang_cache_holds_prefix_states_and_pool_untouched(is_kda):
    B, T = 3, 4
    c = _mtp_case(is_kda=is_kda)
    cache = torch.full((4, T + 1, 4, 8, 8), -7.0)
    out, st, ca = k_last_reference(c["q"], c["k"], c["v"], c["a"], c["b"], c["A_log"], c["dt_bias"],
                                   c["state"], [5, 0, -1], [T] * B, is_kda=is_kda,
                                   disable_state_update=True, cache=cache, cache_indices=[2, 0, 1])
    assert torch.equal(st, c["state"])                       # verify never writes the pool
    assert torch.equal(ca[1], cache[1]) and torch.equal(ca[3], cache[3])   # padded / unused rows
    assert torch.equal(ca[:, T], cache[:, T])                # step beyond T untouched
    assert torch.count_nonzero(out[2 * T:]) == 0             # padded request -> zeros
    for n, (slot, cidx) in enumerate([(5, 2), (0, 0)]):
        for t in range(T):
            sl = slice(n * T, n * T + t + 1)
            _, st_t, _ = k_last_reference(c["q"][sl], c["k"][sl], c["v"][sl], c["a"][sl], c["b"][sl],
                                          c["A_log"], c["dt_bias"], c["state"], [slot], [t + 1], is_kda=is_kda)
            torch.testing.assert_close(ca[cidx, t], st_t[slot], rtol=1e-5, atol=1e-6)


def test_eagle_tree_parent_reload():
    B, T = 1, 4
    c = _mtp_case(B=B)
    cache = torch.zeros(2, T, 4, 8, 8)
    parents = [[0, 0, 0, 1]]     # step 2 branches from step 0, step 3 from step 1
    out, _, ca = k_last_reference(c["q"], c["k"], c["v"], c["a"], c["b"], c["A_log"], c["dt_bias"],
                                  c["state"], [4], [T], is_kda=True, disable_state_update=True,
                                  cache=cache, cache_indices=[1], parents=parents)
    # step 2 computed from the state after step 0 only
    idx = torch.tensor([0, 2])
    o02, st02, _ = k_last_reference(c["q"][idx], c["k"][idx], c["v"][idx], c["a"][idx], c["b"][idx],
                                    c["A_log"], c["dt_bias"], c["state"], [4], [2], is_kda=True)
    torch.testing.assert_close(out[2], o02[1], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(ca[1, 2], st02[4], rtol=1e-5, atol=1e-6)
    idx = torch.tensor([0, 1, 3])
    o013, st013, _ = k_last_reference(c["q"][idx], c["k"][idx], c["v"][idx], c["a"][idx], c["b"][idx],
                                      c["A_log"], c["dt_bias"], c["state"], [4], [3], is_kda=True)
    torch.testing.assert_close(out[3], o013[2], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(ca[1, 3], st013[4], rtol=1e-5, atol=1e-6)


def test_vllm_slot_table_and_num_accepted():
    B, T = 2, 4
    c = _mtp_case(B=B)
    table = [[1, 2, 3, 4], [5, 0, 7, 8]]
    acc = [3, 0]
    out, st, _ = k_last_reference(c["q"], c["k"], c["v"], c["a"], c["b"], c["A_log"], c["dt_bias"],
                                  c["state"], table, [T] * B, is_kda=True, disable_state_update=True,
                                  num_accepted=acc, is_sglang=False)
    # request 0 starts from slot table[0][2] = 3; request 1 (accepted <= 0) from column 0 = slot 5
    for n, start in enumerate([3, 5]):
        for t in range(T):
            sl = slice(n * T, n * T + t + 1)
            o_t, st_t, _ = k_last_reference(c["q"][sl], c["k"][sl], c["v"][sl], c["a"][sl], c["b"][sl],
                                            c["A_log"], c["dt_bias"], c["state"], [start], [t + 1],
                                            is_kda=True, is_sglang=False)
            torch.testing.assert_close(out[n * T + t], o_t[t], rtol=1e-5, atol=1e-6)
            slot = table[n][t]
            if slot > 0:
                torch.testing.assert_close(st[slot], st_t[start], rtol=1e-5, atol=1e-6)
    assert torch.equal(st[0], c["state"][0]) and torch.equal(st[6], c["state"][6])   # null / unmapped
    # negative accepted counts behave like zero
    out2, st2, _ = k_last_reference(c["q"], c["k"], c["v"], c["a"], c["b"], c["A_log"], c["dt_bias"],
                                    c["state"], table, [T] * B, is_kda=True, disable_state_update=True,
                                    num_accepted=[3, -(2 ** 31)], is_sglang=False)
    assert torch.equal(out, out2) and torch.equal(st, st2)


def test_pad_rules_and_empty_requests():
    c = _mtp_case(B=3, T=1)
    common = (c["q"], c["k"], c["v"], c["a"], c["b"], c["A_log"], c["dt_bias"], c["state"])
    out, st, _ = k_last_reference(*common, [0, -1, 2], [1, 1, 1], is_kda=True, is_sglang=True)
    assert torch.count_nonzero(out[1]) == 0 and torch.count_nonzero(out[0]) > 0
    out, st, _ = k_last_reference(*common, [0, -1, 2], [1, 1, 1], is_kda=True, is_sglang=False)
    assert torch.count_nonzero(out[0]) == 0 and torch.equal(st[0], c["state"][0])   # slot 0 is vLLM's null block
    # empty request consumes no token and no slot (its index may be garbage)
    out, st, _ = k_last_reference(c["q"][:2], c["k"][:2], c["v"][:2], c["a"][:2], c["b"][:2], c["A_log"],
                                  c["dt_bias"], c["state"], [1, 2 ** 31 - 1, 2], [1, 0, 1], is_kda=True)
    assert torch.count_nonzero(out[1]) > 0 and not torch.equal(st[2], c["state"][2])


def test_fold_equals_recurrence_over_accepted_prefix():
    torch.manual_seed(11)
    slots, H, HV, L, D = 6, 2, 4, 4, 8
    state = torch.randn(slots, HV, D, D) * 0.1
    rawk = torch.randn(slots, H, L, D).bfloat16()
    rawv = torch.randn(slots, HV, L, D).bfloat16()
    g = -torch.rand(slots, HV, L, D)
    beta = torch.rand(slots, HV, L)
    idx, acc = [4, 1, -1, 2], [3, 0, 2, 4]
    folded = fold_reference(state, rawk, rawv, g, beta, idx, acc)
    assert torch.equal(folded[1], state[1]) and torch.equal(folded[[0, 3, 5]], state[[0, 3, 5]])
    for slot, n_acc in [(4, 3), (2, 4)]:
        _, st, _ = k_last_reference(rawk[slot].transpose(0, 1)[:n_acc], rawk[slot].transpose(0, 1)[:n_acc],
                                    rawv[slot].transpose(0, 1)[:n_acc], None, None, None, None,
                                    state, [slot], [n_acc], is_kda=True, use_qk_l2norm=True,
                                    log_decay=g[slot].transpose(0, 1)[:n_acc],
                                    beta_activated=beta[slot].transpose(0, 1)[:n_acc])
        torch.testing.assert_close(folded[slot], st[slot], rtol=1e-5, atol=1e-6)
