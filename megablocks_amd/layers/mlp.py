"""Expert MLPs of the dropless MoE: megablocks/layers/mlp.py.

Weights keep the reference layout `[num_experts * ffn_hidden_size, hidden_size]` for both
w1 and w2 (mlp.py:315-330), so the first product is `x @ w1[e].T` (NT) and the second
`h @ w2[e]` (NN).  The block-sparse formulation of the reference (`mlp_impl='sparse'`, stk
sdd/dsd on a block-diagonal topology) is the same pair of grouped products taken over
128-padded row groups, and is computed that way here.
"""
from typing import Any, Optional

import torch

from megablocks_amd import grouped_gemm_util as gg
from megablocks_amd.layers import common, gelu, mpu
from megablocks_amd.layers.arguments import DEFAULT_ACTIVATION_FN, Arguments, InitFn


class ScaleGradient(torch.autograd.Function):
    """mlp.py:18-31."""

    @staticmethod
    @torch.amp.custom_fwd(device_type='cuda')
    def forward(ctx: Any, x: torch.Tensor, scale: float):
        ctx.scale = scale
        return x

    @staticmethod
    @torch.amp.custom_bwd(device_type='cuda')
    def backward(ctx: Any, grad: torch.Tensor):
        return grad * ctx.scale, None


scale_gradient = ScaleGradient.apply


def resolve_dtensor(weight: torch.Tensor):
    """mlp.py:35-40."""
    try:
        from torch.distributed._tensor import DTensor
    except Exception:  # torch built without distributed
        return weight
    if isinstance(weight, DTensor):
        return weight.to_local()
    return weight


def create_moe_expert_weights(args: Arguments, num_experts: int, ffn_hidden_size: int, hidden_size: int,
                              init_method: InitFn):
    """mlp.py:43-88 without the expert-parallel slicing: [E, ffn, hidden], initialised in one call
    so that the values do not depend on how experts are later divided."""
    master_weights = torch.empty(num_experts, ffn_hidden_size, hidden_size, device=args.device,
                                 dtype=common.dtype(args))
    init_method(master_weights)
    return master_weights


def create_dmoe_expert_weights(args: Arguments, num_experts: int, rows: int, columns: int, init_method: InitFn):
    """mlp.py:170-184."""
    return create_moe_expert_weights(args, num_experts, rows, columns, init_method).view([-1, columns])


class MLP(torch.nn.Module):
    """Batched expert MLP of the capacity-factor MoE (mlp.py:91-167): w1 [E, hidden, ffn],
    w2 [E, ffn, hidden], x [E, capacity, hidden]."""

    def __init__(self, args: Arguments):
        super().__init__()
        self.args = args
        experts = mpu.experts_per_rank(args)
        self.w1 = torch.nn.Parameter(torch.empty(experts, args.hidden_size, mpu.features_per_rank(args),
                                                 device=args.device, dtype=common.dtype(args)))
        self.w2 = torch.nn.Parameter(torch.empty(experts, mpu.features_per_rank(args), args.hidden_size,
                                                 device=args.device, dtype=common.dtype(args)))
        mpu.set_expert_model_parallel_attributes(self.w1, args.moe_expert_model_parallelism)
        mpu.set_expert_model_parallel_attributes(self.w2, args.moe_expert_model_parallelism)
        with torch.no_grad():
            w1 = create_moe_expert_weights(args, args.moe_num_experts, args.ffn_hidden_size, args.hidden_size,
                                           args.init_method)
            self.w1.copy_(w1.transpose(1, 2).contiguous())
            self.w2.copy_(create_moe_expert_weights(args, args.moe_num_experts, args.ffn_hidden_size,
                                                    args.hidden_size, args.output_layer_init_method))
        self.gradient_scale = None

    def scale_grad(self, w):
        if self.gradient_scale is None:
            return w
        return scale_gradient(w, self.gradient_scale)

    def equal_groups(self, experts: int, capacity: int, device):
        """Row counts of a batched product seen as a grouped one: `capacity` rows for every expert (kept on
        the device, with their cached bins, as long as the shape stays the same)."""
        key = (experts, capacity, device)
        if getattr(self, '_groups_key', None) != key:
            self._groups = torch.full((experts,), capacity, dtype=torch.int32, device=device)
            self._groups_key = key
        return self._groups

    def forward(self, x):
        # mlp.py:162-167 computes the two batched products with torch.bmm; the same products as grouped ones
        # with equal groups run on this library's kernel (forward and both gradients)
        w1, w2 = resolve_dtensor(self.scale_grad(self.w1)), resolve_dtensor(self.scale_grad(self.w2))
        experts, capacity, hidden = x.shape
        sizes = self.equal_groups(experts, capacity, x.device)
        x = gg.ops.gmm(x.reshape(experts * capacity, hidden), w1, sizes, False)
        x = self.args.activation_fn(x)
        return gg.ops.gmm(x, w2, sizes, False).view(experts, capacity, -1)


class Topology:
    """Metadata of the block-diagonal sparse matrix the reference hands to stk (what
    `stk.Matrix(shape, data, row_indices, column_indices, offsets, column_indices_t, offsets_t,
    block_offsets_t)` carries at dmoe.py:120-129), plus the padded row groups it was built from.

    The products here are grouped GEMMs over `padded_tokens_per_expert` and read none of the index arrays, so
    those are built (by `build`, a callable returning them by name) the first time one of them is asked for:
    a layer step that never looks at them spares the dozen small launches of dmoe.py:35-129."""
    _INDEX_ARRAYS = ('row_indices', 'column_indices', 'offsets', 'column_indices_t', 'offsets_t', 'block_offsets_t')

    def __init__(self, shape, blocking: int, padded_tokens_per_expert: torch.Tensor, build):
        self.shape = shape
        self.blocking = blocking
        self.padded_tokens_per_expert = padded_tokens_per_expert   # int32 [E], multiples of `blocking`
        self._build = build

    def __getattr__(self, name):
        # reached only for attributes that are not set yet
        if name in Topology._INDEX_ARRAYS and self.__dict__.get('_build') is not None:
            build, self._build = self._build, None
            for key, value in build().items():
                setattr(self, key, value)
            return self.__dict__[name]
        raise AttributeError(name)

    def size(self):
        return self.shape

    @property
    def nnz(self):
        return self.column_indices.numel()


def second_product(h, w2, batch_sizes, combine, weights_need_grad):
    """The experts' second product h[r_e] @ w2[e] (mlp.py:523, glu.py:205) -- or, with `combine` (a `gg.CombinedRows`:
    one expert per token), the layer's weighted combine of it (dmoe.py:280), written by the product's store phase
    (`gg.gmm_scatter`).  Returns what the node returns and what its backward needs on top of that: nothing, or (the
    product itself -- kept only if the combine's weights want a gradient --, indices, bin_ids, bins, weights)."""
    if combine is None:
        return gg.backend.gmm(h, w2, batch_sizes), ()
    y, out = gg.gmm_scatter(h, w2, batch_sizes, combine, keep_product=weights_need_grad)
    return out, (y, combine.indices, combine.bin_ids, combine.bins, combine.weights)


def second_product_grad(kept, grad, weights_need_grad):
    """(gradient of the second product's rows, gradient of the combine's weights or None) from the gradient of what
    `second_product` returned; `kept`: the tensors it asked to keep."""
    if not kept:
        return grad, None
    y, indices, bin_ids, bins, weights = kept
    return gg.CombinedRows(indices, bin_ids, bins, weights).backward(y, grad, True, weights_need_grad)


class GroupedGeluMLP(torch.autograd.Function):
    """GroupedMLP.forward with the default activation (mlp.py:499-523: gmm, tanh-GELU, gmm) and the backward autograd
    derives for it, with the two element-wise passes moved into the epilogues of the products next to them: the
    first product also writes its activation (`gmm_act`), and the gradient of the activation's input comes out of
    the `ddsd_out @ w2^T` product directly (`gmm_dact`).  Saves what autograd would save: x, the first product and its
    activation."""

    @staticmethod
    @torch.amp.custom_fwd(device_type='cuda')
    def forward(ctx, x, w1, w2, batch_sizes, c_indices=None, c_bin_ids=None, c_bins=None, c_weights=None):
        # c_*: the layer's combine (`gg.CombinedRows`), when the node is to return the combined output
        if ctx._fwd_used_autocast:
            x, w1, w2 = x.to(ctx._dtype), w1.to(ctx._dtype), w2.to(ctx._dtype)
        x, w1, w2 = x.contiguous(), w1.contiguous(), w2.contiguous()
        sdd_out, activation_fn_out = gg.gmm_act(x, w1, batch_sizes)
        combine = None if c_indices is None else gg.CombinedRows(c_indices, c_bin_ids, c_bins, c_weights)
        out, kept = second_product(activation_fn_out, w2, batch_sizes, combine, ctx.needs_input_grad[7])
        ctx.save_for_backward(w1, w2, batch_sizes, x, sdd_out, activation_fn_out, *kept)
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type='cuda')
    def backward(ctx: Any, grad: torch.Tensor):
        w1, w2, batch_sizes, x, sdd_out, activation_fn_out, *kept = ctx.saved_tensors
        ddsd_out, dweights = second_product_grad(kept, grad, ctx.needs_input_grad[7])
        return (*_gelu_mlp_backward(ctx.needs_input_grad, x, w1, w2, batch_sizes, sdd_out, activation_fn_out, ddsd_out),
                None, None, None, None, dweights)


def _gelu_mlp_backward(needs, x, w1, w2, batch_sizes, sdd_out, activation_fn_out, ddsd_out):
    """(dx, dw1, dw2) of GroupedGeluMLP from what its forward saved; needs = which of (x, w1, w2) want a gradient.
    x: the experts' input rows, or a `gg.GatheredRows` that describes them (the weight gradient then reads the rows from
    the ungathered tokens)."""
    ddsd_out = ddsd_out.contiguous()
    dx = dw1 = dw2 = None
    if needs[2]:
        dw2 = gg.backend.gmm(activation_fn_out, ddsd_out, batch_sizes, trans_a=True)
    if needs[0] or needs[1]:
        dsdd_out = gg.gmm_dact(ddsd_out, w2, sdd_out, batch_sizes)
        if needs[1]:
            dw1 = x.weight_gradient(dsdd_out, batch_sizes) if isinstance(x, gg.GatheredRows) else \
                gg.backend.gmm(dsdd_out, x, batch_sizes, trans_a=True)
        if needs[0]:
            dx = gg.backend.gmm(dsdd_out, w1, batch_sizes)
    return dx, dw1, dw2


class GatheredGeluMLP(torch.autograd.Function):
    """GroupedGeluMLP on the rows ops.gather / ops.padded_gather would copy out of the tokens `x` (dmoe.py:219 / :273
    followed by mlp.py:499-523), without that copy in the forward: the first product reads its rows from `x` through
    the sorted assignments (`gg.gmm_gather`), and so does the weight gradient of w1 in the backward
    (`gg.gmm_tn_gather`), which returns the gradient of the tokens (the sum over each token's rows, which is the
    backward of the gather).  Same values as the two separate nodes."""

    @staticmethod
    @torch.amp.custom_fwd(device_type='cuda')
    def forward(ctx, x, w1, w2, batch_sizes, indices, bin_ids, bins, padded_bins, top_k, rows, combined=False,
                c_weights=None):
        # combined: the node returns the layer's combine of its output (top_k = 1; the same assignments, c_weights)
        if ctx._fwd_used_autocast:
            x, w1, w2 = x.to(ctx._dtype), w1.to(ctx._dtype), w2.to(ctx._dtype)
        x, w1, w2 = x.contiguous(), w1.contiguous(), w2.contiguous()
        src = gg.GatheredRows(x, indices, bin_ids, bins, padded_bins, top_k, rows)
        out = gg.gmm_gather(src, w1, batch_sizes, act=gg.ACT_GELU_TANH)
        if out is None:
            out = gg.gmm_act(src.materialize(), w1, batch_sizes)
        sdd_out, activation_fn_out = out
        ctx.top_k, ctx.rows = top_k, rows
        combine = gg.CombinedRows(indices, bin_ids, bins, c_weights) if combined else None
        out, kept = second_product(activation_fn_out, w2, batch_sizes, combine, ctx.needs_input_grad[11])
        ctx.save_for_backward(w1, w2, batch_sizes, x, sdd_out, activation_fn_out, indices, bin_ids, bins, padded_bins,
                              *kept)
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type='cuda')
    def backward(ctx: Any, grad: torch.Tensor):
        w1, w2, batch_sizes, x, sdd_out, activation_fn_out, indices, bin_ids, bins, padded_bins, *kept = ctx.saved_tensors
        ddsd_out, dweights = second_product_grad(kept, grad, ctx.needs_input_grad[11])
        src = gg.GatheredRows(x, indices, bin_ids, bins, padded_bins, ctx.top_k, ctx.rows)
        dx, dw1, dw2 = _gelu_mlp_backward(ctx.needs_input_grad, src, w1, w2, batch_sizes, sdd_out,
                                          activation_fn_out, ddsd_out)
        if dx is not None:
            dx = src.scatter_grad(dx)
        return dx, dw1, dw2, None, None, None, None, None, None, None, None, dweights


def grouped_gelu_mlp(x, w1, w2, batch_sizes, combine=None):
    """GroupedGeluMLP; with `combine` (a `gg.CombinedRows`) the node returns the layer's combine of its output."""
    c = (None, None, None, None) if combine is None else (combine.indices, combine.bin_ids, combine.bins, combine.weights)
    return GroupedGeluMLP.apply(x, w1, w2, batch_sizes, *c)


class MemoryOptimizedGroupedMLP(torch.autograd.Function):
    """GroupedMLP with a hand-scheduled backward that recomputes the activation and reuses
    buffers (mlp.py:397-493)."""

    @staticmethod
    @torch.amp.custom_fwd(device_type='cuda')
    def forward(ctx, x, w1, w2, batch_sizes, activation_fn):
        if ctx._fwd_used_autocast:
            x, w1, w2 = x.to(ctx._dtype), w1.to(ctx._dtype), w2.to(ctx._dtype)
        if not x.is_contiguous() or not w1.is_contiguous() or not w2.is_contiguous():
            raise ValueError("Expected contiguous 'x', 'w1' and 'w2'.")
        if activation_fn is DEFAULT_ACTIVATION_FN:
            sdd_out, activation_fn_out = gg.gmm_act(x, w1, batch_sizes)
        else:
            sdd_out = gg.backend.gmm(x, w1, batch_sizes, trans_b=True)
            activation_fn_out = activation_fn(sdd_out)
        dsd_out = gg.backend.gmm(activation_fn_out, w2, batch_sizes)
        ctx.x_shape = x.shape
        ctx.sdd_out_shape = sdd_out.shape
        ctx.dtype = x.dtype
        ctx.activation_fn = activation_fn
        ctx.save_for_backward(w1, w2, batch_sizes, x, sdd_out)
        return dsd_out

    @staticmethod
    @torch.amp.custom_bwd(device_type='cuda')
    def backward(ctx: Any, ddsd_out: torch.Tensor):
        if not ctx.needs_input_grad[0] or not ctx.needs_input_grad[1] or not ctx.needs_input_grad[2]:
            raise ValueError('Expected all MLP inputs to need grad.')
        w1, w2, batch_sizes, x, sdd_out = ctx.saved_tensors
        ddsd_out = ddsd_out.contiguous()
        activation_fn = ctx.activation_fn
        default_act = activation_fn is DEFAULT_ACTIVATION_FN

        # Recompute the activation (kept in the graph only when its gradient is taken by autograd).
        if default_act:
            activation_fn_out = activation_fn(sdd_out)
        else:
            with torch.set_grad_enabled(True):
                sdd_out = sdd_out.detach().requires_grad_(True)
                activation_fn_out = activation_fn(sdd_out)

        dw2 = gg.backend.gmm(activation_fn_out.detach(), ddsd_out, batch_sizes, trans_a=True)

        if default_act:
            # d(sdd_out) overwrites the recomputed activation: the product ddsd_out @ w2^T with the closed-form GELU
            # gradient (gelu.py:9-13) in its epilogue
            dsdd_out = gg.gmm_dact(ddsd_out, w2, sdd_out, batch_sizes, c=activation_fn_out)
        else:
            dactivation_fn_out = gg.backend.gmm(ddsd_out, w2, batch_sizes, trans_b=True)
            activation_fn_out.backward(dactivation_fn_out)
            dsdd_out = sdd_out.grad

        dw1 = gg.backend.gmm(dsdd_out, x, batch_sizes, trans_a=True)
        dx = gg.backend.gmm(dsdd_out, w1, batch_sizes, c=ddsd_out)   # reuses the incoming gradient buffer
        return dx, dw1, dw2, None, None


memory_optimized_grouped_mlp = MemoryOptimizedGroupedMLP.apply
# The block-sparse memory-optimised MLP (mlp.py:187-302) is the same schedule over padded groups.
memory_optimized_mlp = MemoryOptimizedGroupedMLP.apply


class SparseMLP(torch.nn.Module):
    """Owner of the dMoE expert weights w1, w2 : [E * ffn, hidden] (mlp.py:308-394).  Its forward
    takes the padded activations and the block-diagonal topology."""

    def __init__(self, args: Arguments):
        super().__init__()
        self.args = args
        self._num_rows_per_rank = mpu.experts_per_rank(args) * mpu.features_per_rank(args)
        self.w1 = torch.nn.Parameter(torch.empty(self._num_rows_per_rank, args.hidden_size, device=args.device,
                                                 dtype=common.dtype(args)))
        self.w2 = torch.nn.Parameter(torch.empty(self._num_rows_per_rank, args.hidden_size, device=args.device,
                                                 dtype=common.dtype(args)))
        with torch.no_grad():
            self.w1.copy_(create_dmoe_expert_weights(args, args.moe_num_experts, args.ffn_hidden_size,
                                                     args.hidden_size, args.init_method))
            self.w2.copy_(create_dmoe_expert_weights(args, args.moe_num_experts, args.ffn_hidden_size,
                                                     args.hidden_size, args.output_layer_init_method))
        self._should_set_parallelism_attribute = args.moe_expert_model_parallelism
        mpu.set_expert_model_parallel_attributes(self.w1, self._should_set_parallelism_attribute)
        mpu.set_expert_model_parallel_attributes(self.w2, self._should_set_parallelism_attribute)
        self.gradient_scale = None

    def scale_grad(self, w):
        if self.gradient_scale is None:
            return w
        return scale_gradient(w, self.gradient_scale)

    def _expert_views(self, *weights):
        ne = mpu.experts_per_rank(self.args)
        return [resolve_dtensor(self.scale_grad(w)).view(ne, -1, self.args.hidden_size) for w in weights]

    takes_combine = True   # forward / forward_tokens accept the layer's combine (`gg.CombinedRows`) and then return the combined output

    @staticmethod
    def _combined(y, combine):
        """The combine as ops.scatter (dmoe.py:280), for the paths whose second product does not write it."""
        if combine is None:
            return y
        from megablocks_amd import ops
        return ops.scatter(y, combine.indices, combine.bin_ids, combine.weights, combine.bins, 1)

    def _compute(self, x, batch_sizes, combine=None):
        w1, w2 = self._expert_views(self.w1, self.w2)
        if self.args.memory_optimized_mlp:
            return self._combined(memory_optimized_grouped_mlp(x, w1, w2, batch_sizes, self.args.activation_fn), combine)
        if self.args.activation_fn is DEFAULT_ACTIVATION_FN and x.is_cuda:
            return grouped_gelu_mlp(x, w1, w2, batch_sizes, combine)
        x = gg.ops.gmm(x, w1, batch_sizes, trans_b=True)
        x = self.args.activation_fn(x)
        return self._combined(gg.ops.gmm(x, w2, batch_sizes), combine)

    def forward(self, x, topo: Topology):
        return self._compute(x, topo.padded_tokens_per_expert)

    def forward_tokens(self, src, batch_sizes, combine=None):
        """forward on the rows of the tokens that `src` (a `gg.GatheredRows`) describes, which are then never copied
        out in the forward; None where that is not built (the caller gathers and calls forward).  combine: as for
        forward (its assignments are src's)."""
        if self.args.activation_fn is not DEFAULT_ACTIVATION_FN or not src.x.is_cuda:
            return None
        if self.args.memory_optimized_mlp and torch.is_grad_enabled():
            return None   # the memory-optimised schedule is a matter of what the backward keeps: without one, the same forward
        w1, w2 = self._expert_views(self.w1, self.w2)
        return GatheredGeluMLP.apply(src.x, w1, w2, batch_sizes, src.indices, src.bin_ids, src.bins, src.padded_bins,
                                     src.top_k, src.rows, combine is not None, None if combine is None else combine.weights)


class GroupedMLP(SparseMLP):
    """mlp.py:499-523.  `tokens_per_expert` stays on the device: the grouped GEMM reads the row
    bins there, so the reference's `.cpu()` copy (mlp.py:502) is not needed."""

    def forward(self, x, tokens_per_expert, combine=None):
        """combine (a `gg.CombinedRows`, one expert per token): return the layer's weighted combine of the experts' output
        (dmoe.py:280) instead of the output itself."""
        return self._compute(x, tokens_per_expert, combine)
