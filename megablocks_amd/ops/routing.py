"""Routing / bookkeeping operators: same names, arguments and results as
megablocks/ops/{histogram,sort,cumsum,topology,replicate,round_up,repeat,sum}.py, running the
HIP kernels of libmbx.so on the current stream.  None of them is differentiable except
`replicate`.
"""
from typing import Any, Optional

import torch

from megablocks_amd import _lib
from megablocks_amd._lib import lib

_BITS_FOR_DTYPE = {torch.int16: 16, torch.int32: 32, torch.int64: 64}


def _histogram(x: torch.Tensor, num_bins: int) -> torch.Tensor:
    # argument checks of csrc/histogram.h:62-67
    _lib.require_cuda(x)
    if x.ndim not in (1, 2):
        raise RuntimeError('histogram expects a 1-D or 2-D tensor')
    it = _lib.itype_of(x)
    num_bins = int(num_bins)
    x = x.contiguous()
    rows, n = (1, x.numel()) if x.ndim == 1 else x.shape
    out = torch.empty((rows, num_bins), dtype=torch.int32, device=x.device)
    with _lib.device_of(x):
        _lib.check(lib.mbx_histogram(_lib.ptr(x), it, rows, n, num_bins, _lib.ptr(out), _lib.stream()), 'histogram')
    return out.flatten() if x.ndim == 1 else out


class HistogramOp(torch.autograd.Function):
    """megablocks/ops/histogram.py:20-27."""

    @staticmethod
    def forward(ctx: Any, x: torch.Tensor, max_val: float):
        return _histogram(x, max_val)


histogram = HistogramOp.apply


def _sort(x, end_bit, x_out, iota_out):
    # argument checks of csrc/sort.h:63-74
    _lib.require_cuda(x, x_out, iota_out)
    if x.ndim != 1 or x_out.ndim != 1 or iota_out.ndim != 1:
        raise RuntimeError('sort expects 1-D tensors')
    it = _lib.itype_of(x)
    if x_out.dtype != x.dtype or iota_out.dtype != x.dtype:
        raise RuntimeError('sort outputs must have the dtype of the input')
    if x_out.numel() == 0:
        return
    x = x.contiguous()
    n = x.numel()
    nbytes = lib.mbx_sort_scratch_bytes(n, it, end_bit)
    scratch = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=x.device)
    with _lib.device_of(x):
        _lib.check(lib.mbx_sort(_lib.ptr(x), it, n, end_bit, _lib.ptr(x_out), _lib.ptr(iota_out), _lib.ptr(scratch),
                                nbytes, _lib.stream()), 'sort')


class SortOp(torch.autograd.Function):
    """megablocks/ops/sort.py:26-35: returns (sorted keys, permutation), both in x's dtype."""

    @staticmethod
    def forward(ctx: Any, x: torch.Tensor, end_bit: Optional[int] = None):
        if end_bit is None:
            end_bit = _BITS_FOR_DTYPE[x.dtype]
        x_out = torch.empty_like(x, memory_format=torch.contiguous_format)
        iota_out = torch.empty_like(x, memory_format=torch.contiguous_format)
        _sort(x, int(end_bit), x_out, iota_out)
        ctx.mark_non_differentiable(x_out, iota_out)
        return (x_out, iota_out)


sort = SortOp.apply


def route_supported(expert_ids: torch.Tensor, num_experts: int, end_bit: int) -> bool:
    """Whether `route` takes these ids: int32 on the GPU, one 8-bit sort pass whose digits are the expert ids."""
    return (expert_ids.is_cuda and expert_ids.dtype == torch.int32 and expert_ids.ndim == 1 and
            0 < end_bit <= 8 and 0 < num_experts <= (1 << end_bit))


def route(expert_ids: torch.Tensor, num_experts: int, end_bit: int, blocking: int = 0):
    """The routing bookkeeping of a layer step (moe.py:152-183, dmoe.py:131-154) in three launches:
    (indices, bin_ids, tokens_per_expert, bins, padded_bins) with the values `sort`, `histogram`, `inclusive_cumsum`
    and `round_up` give for ids inside [0, num_experts); padded_bins is None without `blocking`.  The slot -> row map
    of the permutation kernels comes out of the same launches and is left where they look for it."""
    from megablocks_amd.backend import kernels
    n = expert_ids.shape[0]
    expert_ids = expert_ids.contiguous()
    dev = expert_ids.device
    indices = torch.empty(n, dtype=torch.int32, device=dev)
    bin_ids = torch.empty(n, dtype=torch.int32, device=dev)
    tokens_per_expert = torch.empty(num_experts, dtype=torch.int32, device=dev)
    bins = torch.empty(num_experts, dtype=torch.int32, device=dev)
    padded_bins = torch.empty(num_experts, dtype=torch.int32, device=dev) if blocking else None
    slot_rows = torch.empty(max(n, 1), dtype=torch.int32, device=dev)
    with _lib.device_of(expert_ids):
        nbytes = max(lib.mbx_sort_scratch_bytes(max(n, 1), _lib.I32, end_bit), 1)
        scratch = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        _lib.check(lib.mbx_route(_lib.ptr(expert_ids), n, num_experts, end_bit, int(blocking), _lib.ptr(indices),
                                 _lib.ptr(bin_ids), _lib.ptr(tokens_per_expert), _lib.ptr(bins), _lib.ptr(padded_bins),
                                 _lib.ptr(slot_rows), _lib.ptr(scratch), nbytes, _lib.stream()), 'route')
    kernels.remember_slot_rows(indices, bins, padded_bins, slot_rows)
    return indices, bin_ids, tokens_per_expert, bins, padded_bins


def _cumsum(x, dim, exclusive):
    _lib.require_cuda(x)
    it = _lib.itype_of(x)
    squeeze = x.ndim == 1
    if squeeze:
        x = x.view([1, -1])           # megablocks/ops/cumsum.py:24-25
    elif x.ndim != 2 or dim != 1:
        raise RuntimeError('cumsum expects a 2-D tensor scanned along dim 1')  # csrc/cumsum.h:115-117
    x = x.contiguous()
    out = torch.empty_like(x)
    with _lib.device_of(x):
        _lib.check(lib.mbx_cumsum(_lib.ptr(x), it, x.shape[0], x.shape[1], int(exclusive), _lib.ptr(out),
                                  _lib.stream()), 'cumsum')
    return out.squeeze() if squeeze else out  # a one-element 1-D input comes back 0-dim, as in the reference


class ExclusiveCumsumOp(torch.autograd.Function):
    """megablocks/ops/cumsum.py:20-31."""

    @staticmethod
    def forward(ctx: Any, x: torch.Tensor, dim: int):
        return _cumsum(x, dim, True)


class InclusiveCumsumOp(torch.autograd.Function):
    """megablocks/ops/cumsum.py:37-48."""

    @staticmethod
    def forward(ctx: Any, x: torch.Tensor, dim: int):
        return _cumsum(x, dim, False)


exclusive_cumsum = ExclusiveCumsumOp.apply
inclusive_cumsum = InclusiveCumsumOp.apply


class TopologyOp(torch.autograd.Function):
    """megablocks/ops/topology.py:20-42 (argument checks of csrc/indices.h:74-83)."""

    @staticmethod
    def forward(ctx: Any, padded_bins: torch.Tensor, block_size: int, output_block_rows: int,
                output_block_columns: int):
        _lib.require_cuda(padded_bins)
        if padded_bins.ndim != 1 or padded_bins.dtype != torch.int32:
            raise RuntimeError('topology expects a 1-D int32 padded_bins')
        padded_bins = padded_bins.contiguous()
        out = torch.empty(output_block_rows * output_block_columns, dtype=torch.int16, device=padded_bins.device)
        with _lib.device_of(padded_bins):
            _lib.check(lib.mbx_topology(_lib.ptr(padded_bins), padded_bins.numel(), int(block_size),
                                        int(output_block_rows), int(output_block_columns), _lib.ptr(out),
                                        _lib.stream()), 'topology')
        return out


topology = TopologyOp.apply

_REPLICATE_FWD = (torch.float16, torch.bfloat16, torch.int16, torch.int32, torch.float32)


def replicate_forward(x, bins, out):
    """csrc/replicate.h:130-183."""
    _lib.require_cuda(x, bins, out)
    if x.ndim != 2 or bins.ndim != 1 or out.ndim != 2:
        raise RuntimeError('replicate expects x [batch, bins], bins [bins], out [batch, columns]')
    if bins.dtype != torch.int32 or x.dtype not in _REPLICATE_FWD or out.dtype != x.dtype:
        raise RuntimeError('replicate: unsupported dtype')
    if x.shape[1] != bins.shape[0] or out.shape[0] != x.shape[0]:
        raise RuntimeError('replicate: shape mismatch')
    if out.numel() == 0:
        return
    x, bins = x.contiguous(), bins.contiguous()
    assert out.is_contiguous()
    with _lib.device_of(x):
        _lib.check(lib.mbx_replicate_forward(_lib.ptr(x), x.element_size(), x.shape[0], bins.shape[0], _lib.ptr(bins),
                                             _lib.ptr(out), out.shape[1], _lib.stream()), 'replicate_forward')


def replicate_backward(grad, bins, out):
    """csrc/replicate.h:185-206."""
    _lib.require_cuda(grad, bins, out)
    if grad.ndim != 2 or bins.ndim != 1 or out.ndim != 2:
        raise RuntimeError('replicate_backward expects grad [batch, columns], bins [bins], out [batch, bins]')
    if bins.dtype != torch.int32 or out.dtype != grad.dtype:
        raise RuntimeError('replicate_backward: unsupported dtype')
    dt = _lib.dtype_of(grad)
    if out.shape[0] != grad.shape[0] or out.shape[1] != bins.shape[0]:
        raise RuntimeError('replicate_backward: shape mismatch')
    if out.numel() == 0:
        return
    grad, bins = grad.contiguous(), bins.contiguous()
    assert out.is_contiguous()
    with _lib.device_of(grad):
        _lib.check(lib.mbx_replicate_backward(_lib.ptr(grad), dt, grad.shape[0], grad.shape[1], _lib.ptr(bins),
                                              bins.shape[0], _lib.ptr(out), _lib.stream()), 'replicate_backward')


class ReplicateOp(torch.autograd.Function):
    """megablocks/ops/replicate.py:19-33."""

    @staticmethod
    def forward(ctx: Any, x: torch.Tensor, bins: torch.Tensor, num_outputs: int):
        ctx.save_for_backward(bins)
        out = torch.empty((x.shape[0], num_outputs), dtype=x.dtype, device=x.device)
        replicate_forward(x, bins, out)
        return out

    @staticmethod
    def backward(ctx: Any, grad: torch.Tensor):
        bins, = ctx.saved_tensors
        out = torch.empty((grad.shape[0], bins.shape[0]), dtype=grad.dtype, device=grad.device)
        replicate_backward(grad.contiguous(), bins, out)
        return out, None, None


replicate = ReplicateOp.apply


def round_up(x: torch.Tensor, value: int):
    """megablocks/ops/round_up.py:7-14."""
    assert isinstance(value, int)
    assert x.dtype == torch.int32
    return torch.div(x + (value - 1), value, rounding_mode='trunc') * value


def repeat(x: torch.Tensor, tiling):
    """megablocks/ops/repeat.py:7-10."""
    if all((t == 1 for t in tiling)):
        return x
    return x.repeat(*tiling)


def sum(x: torch.Tensor, dim: int = 0):
    """megablocks/ops/sum.py:6-9."""
    if x.shape[dim] == 1:
        return x.squeeze(dim=dim)
    return x.sum(dim=dim)
