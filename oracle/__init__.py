"""CPU oracle for the gated delta-rule path.  TEST INFRASTRUCTURE ONLY.

Nothing under this package is part of the product: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it, and only as the checker.  The product path (``pla_amd``) never
imports it and raises when its HIP library is missing.

The oracle is a plain PyTorch (CPU) restatement of the reference repository's
own PyTorch reference recurrences; each function cites the reference file and
lines it follows.  The reference ships no golden output vectors, so every
function is pinned by closed forms, invariants and brute force in
``tests/test_oracle_*.py`` (geometric-series decay, pure-decay, projection,
element-wise float64 loops on tiny shapes, chunked == token recurrence,
prefix/commit consistency).  No function here is "parity unpinned".
"""

from .gates import softplus_gate, lower_bound_gate, l2norm, sigmoid_beta  # noqa: F401
from .decode import (  # noqa: F401
    k_last_reference, fold_reference, recurrent_step,
    causal_conv1d_update_reference, kda_decode_mega_reference,
    causal_conv_silu_sequence, verify_dspark_reference, conv_window_scatter_reference,
    replay_commit_plan_reference,
)
from .prefill import (  # noqa: F401
    gdn_prefill_reference,
    kda_prefill_reference,
    chunked_delta_rule_fp64,
)
