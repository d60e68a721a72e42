"""Gate, beta and q/k normalisation of the gated delta rule (oracle, CPU).

Test infrastructure only; see ``oracle/__init__.py``.
"""

import torch


def _head_scale(A_log, per_channel):
    eA = A_log.float().exp()
    return eA[:, None] if per_channel else eA


def softplus_gate(a, dt_bias, A_log, softplus_beta=1.0, softplus_threshold=20.0,
                  per_channel=False):
    """Log-decay ``g = -exp(A_log) * softplus(a + dt_bias)``.

    Follows src/pla_device_helpers.cuh:215-225 (``compute_bg``: the linear
    branch is taken when ``softplus_beta * x > threshold``) and
    scripts/decode/_kda_reference.py:27-39 (``naive_kda_gate``).

    ``a``: [..., HV] (GDN, ``per_channel=False``) or [..., HV, K] (KDA,
    ``per_channel=True``); ``dt_bias`` broadcastable to ``a``'s trailing dims;
    ``A_log``: [HV].  Returns float32 log-decay of a's shape.
    """
    x = a.float() + dt_bias.float()
    bx = x * softplus_beta
    # log1p(exp(.)) evaluated without overflow; beyond the threshold the
    # reference returns x itself.
    soft = torch.where(bx <= softplus_threshold,
                       torch.log1p(torch.exp(torch.clamp(bx, max=softplus_threshold))) / softplus_beta,
                       x)
    return -_head_scale(A_log, per_channel) * soft


def lower_bound_gate(a, dt_bias, A_log, lower_bound, per_channel=True):
    """Log-decay ``g = lower_bound * sigmoid(exp(A_log) * (a + dt_bias))``.

    Follows src/pla_device_helpers.cuh:227-246 (``USE_LOWER_BOUND``) and
    scripts/decode/_kda_reference.py:42-54 (``naive_kda_lowerbound_gate``).
    """
    x = a.float() + dt_bias.float()
    return float(lower_bound) * torch.sigmoid(_head_scale(A_log, per_channel) * x)


def sigmoid_beta(b):
    """``beta = sigmoid(b)`` in float32
    (src/decode/k-last/fused_sigmoid_gating_k_last_packed_kernel.cuh:211-217)."""
    return torch.sigmoid(b.float())


def l2norm(x, eps=1e-6):
    """``x * rsqrt(sum(x^2) + eps)`` over the last dim, float32, eps inside the
    square root (tests/test_k_last_state_dtype.py:111-113;
    src/prefill/flashqla/kernels/chunk_cumsum_cute.cu:279-286)."""
    x = x.float()
    return x * torch.rsqrt(x.square().sum(-1, keepdim=True) + eps)
