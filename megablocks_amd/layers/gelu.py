"""megablocks/layers/gelu.py:9-29: closed-form tanh-GELU backward, in place on the gradient."""
import torch

from megablocks_amd import _lib
from megablocks_amd._lib import lib


def gelu_backward_(grad: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """grad *= d/dx gelu_tanh(x); returns grad."""
    _lib.require_cuda(grad, x)
    if grad.shape != x.shape or grad.dtype != x.dtype:
        raise ValueError('gelu_backward_: grad and x must match in shape and dtype')
    if not grad.is_contiguous() or not x.is_contiguous():
        raise ValueError('gelu_backward_: expected contiguous tensors')
    with _lib.device_of(grad):
        _lib.check(lib.mbx_gelu_backward_inplace(_lib.ptr(grad), _lib.ptr(x), _lib.dtype_of(grad), grad.numel(),
                                                 _lib.stream()), 'gelu_backward_')
    return grad
