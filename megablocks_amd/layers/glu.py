"""Gated expert MLPs: megablocks/layers/glu.py.  y = (act(x @ w1.T) * (x @ v1.T)) @ w2 per expert."""
import torch

from functools import partial

import torch.nn.functional as F

from megablocks_amd import _lib
from megablocks_amd import grouped_gemm_util as gg
from megablocks_amd._lib import lib
from megablocks_amd.layers import common, mpu
from megablocks_amd.layers.arguments import DEFAULT_ACTIVATION_FN, Arguments
from megablocks_amd.layers.mlp import SparseMLP, Topology, create_dmoe_expert_weights, second_product, second_product_grad

_ACT_SILU, _ACT_GELU_TANH = 0, 1


def _activation_code(fn):
    """Code of an activation the fused gated-activation kernels implement, else None."""
    if fn is F.silu:
        return _ACT_SILU
    if fn is DEFAULT_ACTIVATION_FN:
        return _ACT_GELU_TANH
    if isinstance(fn, partial) and fn.func is F.gelu and not fn.args and fn.keywords == {'approximate': 'tanh'}:
        return _ACT_GELU_TANH
    return None


def _fusable(*tensors):
    t0 = tensors[0]
    per = 16 // t0.element_size()
    return (t0.is_cuda and t0.dtype in _lib.DTYPE and t0.numel() % per == 0 and
            all(t.is_contiguous() and t.dtype == t0.dtype and t.shape == t0.shape and t.data_ptr() % 16 == 0
                for t in tensors))


def _glu_forward(a, b, act):
    out = torch.empty_like(a)
    with _lib.device_of(a):
        _lib.check(lib.mbx_glu_forward(_lib.ptr(a), _lib.ptr(b), _lib.ptr(out), _lib.dtype_of(a), act, a.numel(),
                                       _lib.stream()), 'glu_forward')
    return out


def _glu_backward(g, a, b, act):
    da, db = torch.empty_like(a), torch.empty_like(a)
    with _lib.device_of(a):
        _lib.check(lib.mbx_glu_backward(_lib.ptr(g), _lib.ptr(a), _lib.ptr(b), _lib.ptr(da), _lib.ptr(db),
                                        _lib.dtype_of(a), act, a.numel(), _lib.stream()), 'glu_backward')
    return da, db


class GatedActivation(torch.autograd.Function):
    """`activation_fn(a) * b` (glu.py:89,204) and its gradient, one kernel each instead of two and
    three element-wise passes; same values (each intermediate is rounded as the separate ops round it)."""

    @staticmethod
    def forward(ctx, a, b, act):
        ctx.save_for_backward(a, b)
        ctx.act = act
        return _glu_forward(a, b, act)

    @staticmethod
    def backward(ctx, g):
        a, b = ctx.saved_tensors
        g = g.contiguous()
        if not _fusable(g, a, b):
            with torch.enable_grad():
                a_, b_ = a.detach().requires_grad_(True), b.detach().requires_grad_(True)
                fn = F.silu if ctx.act == _ACT_SILU else DEFAULT_ACTIVATION_FN
                (fn(a_) * b_).backward(g)
            return a_.grad, b_.grad, None
        da, db = _glu_backward(g, a, b, ctx.act)
        return da, db, None


def gated_activation(activation_fn, a, b):
    """activation_fn(a) * b, fused when the activation is SiLU or tanh-GELU and the layout allows."""
    act = _activation_code(activation_fn)
    if act is not None and _fusable(a, b):
        return GatedActivation.apply(a, b, act)
    return activation_fn(a) * b


class GLUProjection(torch.autograd.Function):
    """(x @ w1[e]^T, x @ v1[e]^T) per expert, glu.py:201-203.  Equivalent to two `gg.ops.gmm` calls, except that
    the input gradient da @ w1 + db @ v1 is one reduction over both pairs instead of two products and a sum."""

    @staticmethod
    @torch.amp.custom_fwd(device_type='cuda')
    def forward(ctx, x, w1, v1, batch_sizes):
        ctx.save_for_backward(x, w1, v1, batch_sizes)
        return (gg.backend.gmm(x, w1, batch_sizes, trans_b=True), gg.backend.gmm(x, v1, batch_sizes, trans_b=True))

    @staticmethod
    @torch.amp.custom_bwd(device_type='cuda')
    def backward(ctx, d1, d2):
        x, w1, v1, batch_sizes = ctx.saved_tensors
        d1, d2 = d1.contiguous(), d2.contiguous()
        dx = dw1 = dv1 = None
        if ctx.needs_input_grad[0]:
            dx = gg.gmm_dual(d1, w1, d2, v1, batch_sizes)
        if ctx.needs_input_grad[1]:
            dw1 = gg.backend.gmm(d1, x, batch_sizes, trans_a=True)
        if ctx.needs_input_grad[2]:
            dv1 = gg.backend.gmm(d2, x, batch_sizes, trans_a=True)
        return dx, dw1, dv1, None


class GroupedGLUExperts(torch.autograd.Function):
    """The grouped GLU experts of glu.py:201-205 as one node: the same products and element-wise steps as
    GLUProjection -> GatedActivation -> gmm, with everything they save, but the backward can then hand the product
    `ddsd_out @ w2[e]^T` and the backward of the gated activation to one launch (`gg.gmm_dglu`): the gradient of the
    activation output is never written to memory."""

    @staticmethod
    @torch.amp.custom_fwd(device_type='cuda')
    def forward(ctx, x, w1, v1, w2, batch_sizes, act, c_indices=None, c_bin_ids=None, c_bins=None, c_weights=None):
        # c_*: the layer's combine (`gg.CombinedRows`), when the node is to return the combined output
        x = x.contiguous()
        sdd_out, v1_out, activation_fn_out = gg.gmm_glu(x, w1, v1, batch_sizes, act)
        ctx.act = act
        combine = None if c_indices is None else gg.CombinedRows(c_indices, c_bin_ids, c_bins, c_weights)
        out, kept = second_product(activation_fn_out, w2, batch_sizes, combine, ctx.needs_input_grad[9])
        ctx.save_for_backward(x, w1, v1, w2, batch_sizes, sdd_out, v1_out, activation_fn_out, *kept)
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type='cuda')
    def backward(ctx, grad):
        x, w1, v1, w2, batch_sizes, sdd_out, v1_out, activation_fn_out, *kept = ctx.saved_tensors
        ddsd_out, dweights = second_product_grad(kept, grad, ctx.needs_input_grad[9])
        return (*_glu_experts_backward(ctx.needs_input_grad, x, w1, v1, w2, batch_sizes, sdd_out, v1_out,
                                       activation_fn_out, ddsd_out, ctx.act), None, None, None, None, None, dweights)


def _glu_experts_backward(needs, x, w1, v1, w2, batch_sizes, sdd_out, v1_out, activation_fn_out, ddsd_out, act):
    """(dx, dw1, dv1, dw2) of GroupedGLUExperts from what its forward saved; needs = which of (x, w1, v1, w2) want a
    gradient.  x: the experts' input rows, or a `gg.GatheredRows` that describes them (the weight gradients then read
    the rows from the ungathered tokens)."""
    ddsd_out = ddsd_out.contiguous()
    dx = dw1 = dv1 = dw2 = None
    if needs[3]:
        dw2 = gg.backend.gmm(activation_fn_out, ddsd_out, batch_sizes, trans_a=True)
    if needs[0] or needs[1] or needs[2]:
        dsdd_out, dv1_out = gg.gmm_dglu(ddsd_out, w2, sdd_out, v1_out, batch_sizes, act)
        wgrad = x.weight_gradient if isinstance(x, gg.GatheredRows) else (lambda d, sizes: gg.backend.gmm(d, x, sizes, trans_a=True))
        if needs[1]:
            dw1 = wgrad(dsdd_out, batch_sizes)
        if needs[2]:
            dv1 = wgrad(dv1_out, batch_sizes)
        if needs[0]:
            dx = gg.gmm_dual(dsdd_out, w1, dv1_out, v1, batch_sizes)
    return dx, dw1, dv1, dw2


class GatheredGLUExperts(torch.autograd.Function):
    """GroupedGLUExperts on the rows ops.gather / ops.padded_gather would copy out of the tokens `x` (dmoe.py:219 / :273
    followed by glu.py:201-205), without that copy in the forward: the launch that computes both first products and
    the gated activation reads its rows from `x` through the sorted assignments (`gg.gmm_gather`).  The weight
    gradients of w1 and v1 need the gathered rows as an operand, so the backward makes the copy then, and returns the
    gradient of the tokens (the backward of the gather).  Same values as the two separate nodes."""

    @staticmethod
    @torch.amp.custom_fwd(device_type='cuda')
    def forward(ctx, x, w1, v1, w2, batch_sizes, act, indices, bin_ids, bins, padded_bins, top_k, rows, combined=False,
                c_weights=None):
        # combined: the node returns the layer's combine of its output (top_k = 1; the same assignments, c_weights)
        x = x.contiguous()
        src = gg.GatheredRows(x, indices, bin_ids, bins, padded_bins, top_k, rows)
        out = gg.gmm_gather(src, w1, batch_sizes, b2=v1, act=act)
        if out is None:
            out = gg.gmm_glu(src.materialize(), w1, v1, batch_sizes, act)
        sdd_out, v1_out, activation_fn_out = out
        ctx.act, ctx.top_k, ctx.rows = act, top_k, rows
        combine = gg.CombinedRows(indices, bin_ids, bins, c_weights) if combined else None
        out, kept = second_product(activation_fn_out, w2, batch_sizes, combine, ctx.needs_input_grad[13])
        ctx.save_for_backward(x, w1, v1, w2, batch_sizes, sdd_out, v1_out, activation_fn_out, indices, bin_ids, bins,
                              padded_bins, *kept)
        return out

    @staticmethod
    @torch.amp.custom_bwd(device_type='cuda')
    def backward(ctx, grad):
        (x, w1, v1, w2, batch_sizes, sdd_out, v1_out, activation_fn_out, indices, bin_ids, bins,
         padded_bins, *kept) = ctx.saved_tensors
        ddsd_out, dweights = second_product_grad(kept, grad, ctx.needs_input_grad[13])
        src = gg.GatheredRows(x, indices, bin_ids, bins, padded_bins, ctx.top_k, ctx.rows)
        dx, dw1, dv1, dw2 = _glu_experts_backward(ctx.needs_input_grad, src, w1, v1, w2, batch_sizes, sdd_out,
                                                  v1_out, activation_fn_out, ddsd_out, ctx.act)
        if dx is not None:
            dx = src.scatter_grad(dx)
        return dx, dw1, dv1, dw2, None, None, None, None, None, None, None, None, None, dweights


def _one_node(x, w1, v1, w2, act):
    """Whether the experts can run as GroupedGLUExperts: an activation the library has, 16-bit operands of one type on
    the GPU, rows the element-wise kernels take."""
    return (act is not None and x.is_cuda and x.dtype in (torch.bfloat16, torch.float16) and
            w1.dtype == v1.dtype == w2.dtype == x.dtype and (w1.shape[1] * x.element_size()) % 16 == 0 and
            w1.is_contiguous() and v1.is_contiguous() and w2.is_contiguous())


class MemoryOptimizedGroupedGLU(torch.autograd.Function):
    """glu.py:66-167: saves (x, sdd_out, v1_out), recomputes the gated activation in backward."""

    @staticmethod
    @torch.amp.custom_fwd(device_type='cuda')
    def forward(ctx, x, w1, v1, w2, batch_sizes, activation_fn):
        if ctx._fwd_used_autocast:
            x, w1, v1, w2 = x.to(ctx._dtype), w1.to(ctx._dtype), v1.to(ctx._dtype), w2.to(ctx._dtype)
        if not x.is_contiguous() or not w1.is_contiguous() or not v1.is_contiguous() or not w2.is_contiguous():
            raise ValueError("Expected contiguous 'x', 'w1', 'v1' and 'w2'.")
        act = _activation_code(activation_fn)
        if act is not None and _one_node(x, w1, v1, w2, act):
            sdd_out, v1_out, activation_fn_out = gg.gmm_glu(x, w1, v1, batch_sizes, act)
        else:
            sdd_out = gg.backend.gmm(x, w1, batch_sizes, trans_b=True)
            v1_out = gg.backend.gmm(x, v1, batch_sizes, trans_b=True)
            if act is not None and _fusable(sdd_out, v1_out):
                activation_fn_out = _glu_forward(sdd_out, v1_out, act)
            else:
                activation_fn_out = activation_fn(sdd_out) * v1_out
        dsd_out = gg.backend.gmm(activation_fn_out, w2, batch_sizes)
        ctx.x_shape = x.shape
        ctx.sdd_out_shape = sdd_out.shape
        ctx.dtype = x.dtype
        ctx.activation_fn = activation_fn
        ctx.save_for_backward(w1, v1, w2, batch_sizes, x, sdd_out, v1_out)
        return dsd_out

    @staticmethod
    @torch.amp.custom_bwd(device_type='cuda')
    def backward(ctx, ddsd_out):
        if not ctx.needs_input_grad[0] or not ctx.needs_input_grad[1] or not ctx.needs_input_grad[2]:
            raise ValueError('Expected all MLP inputs to need grad.')
        w1, v1, w2, batch_sizes, x, sdd_out, v1_out = ctx.saved_tensors
        ddsd_out = ddsd_out.contiguous()
        activation_fn = ctx.activation_fn
        act = _activation_code(activation_fn)
        fused = act is not None and _fusable(sdd_out, v1_out)
        if fused:
            activation_fn_out = _glu_forward(sdd_out, v1_out, act)       # recomputed, not saved
        else:
            with torch.set_grad_enabled(True):
                sdd_out = sdd_out.detach().requires_grad_(True)
                v1_out = v1_out.detach().requires_grad_(True)
                activation_fn_out = activation_fn(sdd_out) * v1_out

        dw2 = gg.backend.gmm(activation_fn_out.detach(), ddsd_out, batch_sizes, trans_a=True)
        if fused:
            # one launch where the library has it; else the product (which then overwrites the recomputed activation,
            # glu.py:138) and the element-wise backward
            dsdd_out, dv1_out = gg.gmm_dglu(ddsd_out, w2, sdd_out, v1_out, batch_sizes, act)
        else:
            dactivation_fn_out = gg.backend.gmm(ddsd_out, w2, batch_sizes, trans_b=True)
            activation_fn_out.backward(dactivation_fn_out)
            dsdd_out, dv1_out = sdd_out.grad, v1_out.grad

        dw1 = gg.backend.gmm(dsdd_out, x, batch_sizes, trans_a=True)
        dv1 = gg.backend.gmm(dv1_out, x, batch_sizes, trans_a=True)
        dx = gg.gmm_dual(dsdd_out, w1, dv1_out, v1, batch_sizes, c=ddsd_out)   # reuses the ddsd_out allocation
        return dx, dw1, dv1, dw2, None, None


memory_optimized_grouped_glu = MemoryOptimizedGroupedGLU.apply


class SparseGLU(SparseMLP):
    """glu.py:19-63: adds the gate projection v1 : [E * ffn, hidden]."""

    def __init__(self, args: Arguments):
        super().__init__(args)
        self.v1 = torch.nn.Parameter(torch.empty(self._num_rows_per_rank, args.hidden_size, device=args.device,
                                                 dtype=common.dtype(args)))
        with torch.no_grad():
            self.v1.copy_(create_dmoe_expert_weights(args, args.moe_num_experts, args.ffn_hidden_size,
                                                     args.hidden_size, args.init_method))
        mpu.set_expert_model_parallel_attributes(self.v1, self._should_set_parallelism_attribute)

    def _compute(self, x, batch_sizes, allow_memory_optimized=True, combine=None):
        w1, v1, w2 = self._expert_views(self.w1, self.v1, self.w2)
        if self.args.memory_optimized_mlp:
            if not allow_memory_optimized:
                raise NotImplementedError(
                    'Memory optimized implementation not yet supported with GLU with sparse kernels.')
            return self._combined(memory_optimized_grouped_glu(x, w1, v1, w2, batch_sizes, self.args.activation_fn), combine)
        act = _activation_code(self.args.activation_fn)
        operands = gg.autocast_operands(x, w1, v1, w2)
        if _one_node(*operands, act):
            c = (None, None, None, None) if combine is None else (combine.indices, combine.bin_ids, combine.bins, combine.weights)
            return GroupedGLUExperts.apply(*operands, batch_sizes, act, *c)
        x1, x2 = GLUProjection.apply(*operands[:3], batch_sizes)
        x1 = gated_activation(self.args.activation_fn, x1, x2)
        return self._combined(gg.ops.gmm(x1, w2, batch_sizes), combine)

    def forward(self, x, topo: Topology):
        return self._compute(x, topo.padded_tokens_per_expert, allow_memory_optimized=False)   # glu.py:47-50

    def forward_tokens(self, src, batch_sizes, combine=None):
        """forward on the rows of the tokens that `src` (a `gg.GatheredRows`) describes, which are then never copied
        out in the forward; None where that is not built (the caller gathers and calls forward).  combine: as for
        forward (its assignments are src's)."""
        if self.args.memory_optimized_mlp and (torch.is_grad_enabled() or not isinstance(self, GroupedGLU)):
            # the memory-optimised schedule is a matter of what the backward keeps (without one, the same forward);
            # with the block-sparse experts it raises (glu.py:47-50), which is left to forward()
            return None
        act = _activation_code(self.args.activation_fn)
        w1, v1, w2 = self._expert_views(self.w1, self.v1, self.w2)
        x, w1, v1, w2 = gg.autocast_operands(src.x, w1, v1, w2)
        if not _one_node(x, w1, v1, w2, act):
            return None
        return GatheredGLUExperts.apply(x, w1, v1, w2, batch_sizes, act, src.indices, src.bin_ids, src.bins,
                                        src.padded_bins, src.top_k, src.rows, combine is not None,
                                        None if combine is None else combine.weights)


class GroupedGLU(SparseGLU):
    """glu.py:173-205."""

    def forward(self, x, tokens_per_expert, combine=None):
        return self._compute(x, tokens_per_expert, combine=combine)
