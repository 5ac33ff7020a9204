"""megablocks/layers/common.py:9-26."""
import torch

from megablocks_amd import _lib
from megablocks_amd.layers.arguments import Arguments


def dtype(args: Arguments):
    if args.fp16:
        return torch.float16
    elif args.bf16:
        return torch.bfloat16
    return None


def cast_if_autocast_enabled(tensor):
    if torch.is_autocast_enabled():
        if tensor.device.type == 'cuda':
            target = _lib.autocast_gpu_dtype()
        elif tensor.device.type == 'cpu':
            target = torch.get_autocast_cpu_dtype()
        else:
            raise NotImplementedError()
        return tensor.to(dtype=target)
    return tensor
