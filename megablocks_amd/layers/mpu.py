"""Sharding-degree helpers of megablocks/layers/mpu.py:24-93 for one GPU holding all experts:
every degree is 1."""
import torch

from megablocks_amd.layers.arguments import Arguments


def get_expert_parallel_world_size(args: Arguments) -> int:
    return 1


def get_expert_parallel_rank(args: Arguments) -> int:
    return 0


def set_expert_model_parallel_attributes(tensor: torch.Tensor, is_parallel: bool):
    assert not hasattr(tensor, 'expert_model_parallel')
    setattr(tensor, 'expert_model_parallel', is_parallel)


def param_is_expert_model_parallel(param) -> bool:
    return hasattr(param, 'expert_model_parallel') and param.expert_model_parallel


def expert_sharding_degree(args: Arguments) -> int:
    return 1


def hidden_sharding_degree(args: Arguments) -> int:
    return 1


def experts_per_rank(args: Arguments) -> int:
    return args.moe_num_experts


def features_per_rank(args: Arguments) -> int:
    return args.ffn_hidden_size
