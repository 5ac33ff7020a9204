"""megablocks/layers/dmlp_registry.py:11-42: expert MLP by (mlp_type, mlp_impl)."""
from megablocks_amd.layers import glu, mlp
from megablocks_amd.layers.arguments import Arguments

_REGISTRY = {
    'mlp': {'grouped': mlp.GroupedMLP, 'sparse': mlp.SparseMLP},
    'glu': {'grouped': glu.GroupedGLU, 'sparse': glu.SparseGLU},
}


def get(args: Arguments):
    if args.mlp_type not in _REGISTRY:
        raise ValueError(f'Unsupported mlp type: {args.mlp_type}')
    if args.mlp_impl not in _REGISTRY[args.mlp_type]:
        raise ValueError(f'{args.mlp_type} does not support {args.mlp_impl} backend.',)
    return _REGISTRY[args.mlp_type][args.mlp_impl](args)
