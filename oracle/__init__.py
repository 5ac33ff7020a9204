"""CPU oracle for the dropless-MoE hot path.

TEST INFRASTRUCTURE ONLY.  This package is a CPU restatement (torch-CPU / numpy)
of the semantics of databricks/megablocks' single-GPU dMoE path.  It exists so
that the HIP kernels can be checked against it; nothing in ``megablocks_amd``
imports it, and only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may call it.

Every function cites the reference file:line whose behaviour it restates.  The integer routing ops exist
twice: as torch code (``oracle/routing.py``) and as plain C (``oracle/routing_c.c``, bound by
``oracle/routing_c.py``, compiled with gcc by ``__graft_entry__.build()``); the tests hold the two
against each other.
The reference itself (Python + CUDA/CUB + Triton + two un-vendored packages,
``grouped_gemm==0.3.0`` and ``stanford-stk==0.7.1``) can neither be imported nor
compiled in this environment, so there is no ``oracle/_ref`` build.

Pinning status (see ``tests/test_oracle_pins.py``): every function below is
pinned by an independent brute-force loop on small inputs modelled on the
in-test oracles of the reference's own ``tests/ops/*_test.py`` and by
closed-form invariants.  No function is "parity unpinned".
"""
from oracle.routing import (  # noqa: F401
    histogram, sort, inclusive_cumsum, exclusive_cumsum, round_up, replicate,
    replicate_backward, topology, indices_and_bins, indices_and_padded_bins,
    sparse_transpose, row_indices,
)
from oracle.permute import (  # noqa: F401
    gather, scatter, padded_gather, padded_scatter, scatter_wgrad,
    padded_scatter_wgrad, binned_gather, binned_scatter, binned_scatter_wgrad,
)
from oracle.gmm import gmm  # noqa: F401
from oracle.layers import (  # noqa: F401
    gelu_tanh_backward, router_forward, dmoe_forward,
)
from oracle.losses import (  # noqa: F401
    load_balancing_loss, layer_load_balancing_loss, router_zloss, uniform_expert_assignment,
)
