"""Differentiable token permutation operators with the signatures and gradient pairing of
megablocks/ops/{gather,scatter,padded_gather,padded_scatter,binned_gather,binned_scatter}.py:

    gather.backward          = unweighted scatter
    scatter.backward         = weighted gather (+ scatter_wgrad when the weights need a gradient;
                               x is saved only in that case)
and likewise for the padded and binned forms.
"""
from typing import Any

import torch
from torch.amp import custom_bwd, custom_fwd

from megablocks_amd.backend import kernels

_fwd = custom_fwd(device_type='cuda')
_bwd = custom_bwd(device_type='cuda')


class GatherOp(torch.autograd.Function):
    """megablocks/ops/gather.py:12-35."""

    @staticmethod
    @_fwd
    def forward(ctx: Any, x, indices, bin_ids, bins, top_k: int):
        ctx.save_for_backward(indices, bin_ids, bins)
        ctx.top_k = top_k
        return kernels.gather(x, indices, bin_ids, None, bins, top_k)

    @staticmethod
    @_bwd
    def backward(ctx: Any, grad):
        indices, bin_ids, bins = ctx.saved_tensors
        out = kernels.scatter(grad.contiguous(), indices, bin_ids, None, bins, ctx.top_k)
        return out, None, None, None, None, None


gather = GatherOp.apply


class ScatterOp(torch.autograd.Function):
    """megablocks/ops/scatter.py:13-61."""

    @staticmethod
    @_fwd
    def forward(ctx: Any, x, indices, bin_ids, weights, bins, top_k: int):
        keep_x = [x] if ctx.needs_input_grad[3] else []
        ctx.save_for_backward(indices, bin_ids, weights, bins, *keep_x)
        ctx.top_k = top_k
        ctx.x_shape = x.shape
        return kernels.scatter(x, indices, bin_ids, weights, bins, top_k)

    @staticmethod
    @_bwd
    def backward(ctx: Any, grad):
        grad = grad.contiguous()
        saved = ctx.saved_tensors
        indices, bin_ids, weights, bins = saved[:4]
        if ctx.needs_input_grad[0] and ctx.needs_input_grad[3] and weights is not None:   # both read grad's rows: one pass
            dgrad, wgrad = kernels.scatter_backward(saved[-1], grad, indices, bin_ids, weights, bins, None, ctx.top_k)
            return dgrad, None, None, wgrad, None, None, None
        dgrad = None
        if ctx.needs_input_grad[0]:
            dgrad = kernels.gather(grad, indices, bin_ids, weights, bins, ctx.top_k)
        wgrad = None
        if ctx.needs_input_grad[3]:
            wgrad = kernels.scatter_wgrad(saved[-1], grad, indices, bin_ids, bins, ctx.top_k)
        return dgrad, None, None, wgrad, None, None, None


def scatter(x, indices, bin_ids, weights, bins, top_k: int):
    return ScatterOp.apply(x, indices, bin_ids, weights, bins, top_k)


class PaddedGatherOp(torch.autograd.Function):
    """megablocks/ops/padded_gather.py:12-52."""

    @staticmethod
    @_fwd
    def forward(ctx: Any, x, indices, bin_ids, bins, padded_bins, top_k: int):
        ctx.save_for_backward(indices, bin_ids, bins, padded_bins)
        ctx.top_k = top_k
        return kernels.padded_gather(x, indices, bin_ids, None, bins, padded_bins, top_k)

    @staticmethod
    @_bwd
    def backward(ctx: Any, grad):
        indices, bin_ids, bins, padded_bins = ctx.saved_tensors
        out = kernels.padded_scatter(grad.contiguous(), indices, bin_ids, None, bins, padded_bins, ctx.top_k)
        return out, None, None, None, None, None


padded_gather = PaddedGatherOp.apply


class PaddedScatterOp(torch.autograd.Function):
    """megablocks/ops/padded_scatter.py:12-77."""

    @staticmethod
    @_fwd
    def forward(ctx: Any, x, indices, bin_ids, weights, bins, padded_bins, top_k: int):
        keep_x = [x] if ctx.needs_input_grad[3] else []
        ctx.save_for_backward(indices, bin_ids, weights, bins, padded_bins, *keep_x)
        ctx.top_k = top_k
        ctx.x_shape = x.shape
        return kernels.padded_scatter(x, indices, bin_ids, weights, bins, padded_bins, top_k)

    @staticmethod
    @_bwd
    def backward(ctx: Any, grad):
        grad = grad.contiguous()
        saved = ctx.saved_tensors
        indices, bin_ids, weights, bins, padded_bins = saved[:5]
        if ctx.needs_input_grad[0] and ctx.needs_input_grad[3] and weights is not None:   # both read grad's rows: one pass
            dgrad, wgrad = kernels.scatter_backward(saved[-1], grad, indices, bin_ids, weights, bins, padded_bins,
                                                    ctx.top_k)
            return dgrad, None, None, wgrad, None, None, None, None
        dgrad = None
        if ctx.needs_input_grad[0]:
            dgrad = kernels.padded_gather(grad, indices, bin_ids, weights, bins, padded_bins, ctx.top_k)
        wgrad = None
        if ctx.needs_input_grad[3]:
            wgrad = kernels.padded_scatter_wgrad(saved[-1], grad, indices, bin_ids, bins, padded_bins, ctx.top_k)
        return dgrad, None, None, wgrad, None, None, None, None


def padded_scatter(x, indices, bin_ids, weights, bins, padded_bins, top_k: int):
    return PaddedScatterOp.apply(x, indices, bin_ids, weights, bins, padded_bins, top_k)


class BinnedGatherOp(torch.autograd.Function):
    """megablocks/ops/binned_gather.py:12-34."""

    @staticmethod
    @_fwd
    def forward(ctx: Any, x, indices, bins, bin_size: int, top_k: int):
        ctx.save_for_backward(indices, bins)
        ctx.top_k = top_k
        return kernels.binned_gather(x, indices, None, bins, bin_size, top_k)

    @staticmethod
    @_bwd
    def backward(ctx: Any, grad):
        indices, bins = ctx.saved_tensors
        out = kernels.binned_scatter(grad.contiguous(), indices, None, bins, ctx.top_k)
        return out, None, None, None, None


binned_gather = BinnedGatherOp.apply


class BinnedScatterOp(torch.autograd.Function):
    """megablocks/ops/binned_scatter.py:12-56."""

    @staticmethod
    @_fwd
    def forward(ctx: Any, x, indices, weights, bins, top_k: int):
        assert len(x.size()) == 3
        ctx.bin_size = x.size(1)
        ctx.top_k = top_k
        ctx.save_for_backward(x, indices, weights, bins)
        return kernels.binned_scatter(x, indices, weights, bins, top_k)

    @staticmethod
    @_bwd
    def backward(ctx: Any, grad):
        grad = grad.contiguous()
        x, indices, weights, bins = ctx.saved_tensors
        out = kernels.binned_gather(grad, indices, weights, bins, ctx.bin_size, ctx.top_k)
        wgrad = None
        if ctx.needs_input_grad[2]:
            wgrad = kernels.binned_scatter_wgrad(x, grad, indices, bins, ctx.top_k)
        return out, None, wgrad, None, None


binned_scatter = BinnedScatterOp.apply
