"""Gated expert MLPs: megablocks/layers/glu.py.  y = (act(x @ w1.T) * (x @ v1.T)) @ w2 per expert."""
import torch

from megablocks_amd import grouped_gemm_util as gg
from megablocks_amd.layers import common, mpu
from megablocks_amd.layers.arguments import Arguments
from megablocks_amd.layers.mlp import SparseMLP, Topology, create_dmoe_expert_weights


class MemoryOptimizedGroupedGLU(torch.autograd.Function):
    """glu.py:66-167: saves (x, sdd_out, v1_out), recomputes the gated activation in backward."""

    @staticmethod
    @torch.amp.custom_fwd(device_type='cuda')
    def forward(ctx, x, w1, v1, w2, batch_sizes, activation_fn):
        if ctx._fwd_used_autocast:
            x, w1, v1, w2 = x.to(ctx._dtype), w1.to(ctx._dtype), v1.to(ctx._dtype), w2.to(ctx._dtype)
        if not x.is_contiguous() or not w1.is_contiguous() or not v1.is_contiguous() or not w2.is_contiguous():
            raise ValueError("Expected contiguous 'x', 'w1', 'v1' and 'w2'.")
        sdd_out = gg.backend.gmm(x, w1, batch_sizes, trans_b=True)
        v1_out = gg.backend.gmm(x, v1, batch_sizes, trans_b=True)
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
        with torch.set_grad_enabled(True):
            sdd_out = sdd_out.detach().requires_grad_(True)
            v1_out = v1_out.detach().requires_grad_(True)
            activation_fn_out = activation_fn(sdd_out) * v1_out

        dw2 = gg.backend.gmm(activation_fn_out.detach(), ddsd_out, batch_sizes, trans_a=True)
        dactivation_fn_out = gg.backend.gmm(ddsd_out, w2, batch_sizes, trans_b=True)
        activation_fn_out.backward(dactivation_fn_out)
        dsdd_out, dv1_out = sdd_out.grad, v1_out.grad

        dw1 = gg.backend.gmm(dsdd_out, x, batch_sizes, trans_a=True)
        dv1 = gg.backend.gmm(dv1_out, x, batch_sizes, trans_a=True)
        dx = gg.backend.gmm(dsdd_out, w1, batch_sizes, c=ddsd_out)
        dx += gg.backend.gmm(dv1_out, v1, batch_sizes)
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

    def _compute(self, x, batch_sizes, allow_memory_optimized=True):
        w1, v1, w2 = self._expert_views(self.w1, self.v1, self.w2)
        if self.args.memory_optimized_mlp:
            if not allow_memory_optimized:
                raise NotImplementedError(
                    'Memory optimized implementation not yet supported with GLU with sparse kernels.')
            return memory_optimized_grouped_glu(x, w1, v1, w2, batch_sizes, self.args.activation_fn)
        x1 = gg.ops.gmm(x, w1, batch_sizes, trans_b=True)
        x2 = gg.ops.gmm(x, v1, batch_sizes, trans_b=True)
        x1 = self.args.activation_fn(x1) * x2
        return gg.ops.gmm(x1, w2, batch_sizes)

    def forward(self, x, topo: Topology):
        return self._compute(x, topo.padded_tokens_per_expert, allow_memory_optimized=False)   # glu.py:47-50


class GroupedGLU(SparseGLU):
    """glu.py:173-205."""

    def forward(self, x, tokens_per_expert):
        return self._compute(x, tokens_per_expert)
