"""MI355X-native dropless-MoE hot path behind the megablocks operator and layer interface
(megablocks/__init__.py:4-20)."""
from megablocks_amd import ops  # noqa: F401  (loads libmbx.so; raises if it was not built)
from megablocks_amd.layers.arguments import Arguments
from megablocks_amd.layers.dmoe import ParallelDroplessMLP, dMoE
from megablocks_amd.layers.glu import SparseGLU
from megablocks_amd.layers.mlp import MLP, SparseMLP
from megablocks_amd.layers.moe import MoE, ParallelMLP, get_load_balancing_loss

__all__ = ['MoE', 'dMoE', 'get_load_balancing_loss', 'ParallelMLP', 'ParallelDroplessMLP', 'SparseMLP', 'MLP',
           'SparseGLU', 'Arguments', 'ops']
