"""MoE layer shell and the routing bookkeeping shared with the dropless layer:
megablocks/layers/moe.py (single GPU: no expert-parallel forward)."""
from typing import Optional, Tuple

import numpy as np
import torch

import megablocks_amd.ops as ops
from megablocks_amd.ops import routing as ops_routing
from megablocks_amd import grouped_gemm_util as gg
from megablocks_amd.layers import common, mlp, router
from megablocks_amd.layers.arguments import Arguments

_LOAD_BALANCING_LOSS = []


def save_load_balancing_loss(loss):
    _LOAD_BALANCING_LOSS.append(loss)


def get_load_balancing_loss():
    return _LOAD_BALANCING_LOSS


def clear_load_balancing_loss():
    _LOAD_BALANCING_LOSS.clear()


def batched_load_balancing_loss(args: Arguments):
    """moe.py:32-89: loss_weight * E / (layers * tokens * top_k) * <tokens_per_expert, mean scores>."""
    if args.moe_loss_weight == 0:
        return 0.0
    tokens_per_expert, expert_scores = zip(*get_load_balancing_loss())
    layers = args.num_layers // args.pipeline_model_parallel_size
    if args.num_layers_per_virtual_pipeline_stage is not None:
        layers = args.num_layers_per_virtual_pipeline_stage
    if len(tokens_per_expert) != layers:
        raise ValueError(f'Expected {layers} token_per_experts but found {len(tokens_per_expert)}.\n'
                         f'num_layers = {args.num_layers}\n'
                         f'pipeline_model_parallel_size = {args.pipeline_model_parallel_size}\n'
                         f'num_layers_per_virtual_pipeline_stage = {args.num_layers_per_virtual_pipeline_stage}')
    assert all((x.ndim == 1 and x.numel() == args.moe_num_experts for x in tokens_per_expert))
    tokens = expert_scores[0].shape[0]
    assert all(((x.ndim == 2 and x.shape[1] == args.moe_num_experts and x.shape[0] == tokens) for x in expert_scores))
    expert_scores = torch.cat(expert_scores, dim=1)
    if args.moe_lbl_in_fp32:
        expert_scores = expert_scores.float()
    expert_scores = expert_scores.mean(dim=0) if tokens != 0 else expert_scores.sum(dim=0)
    tokens_per_expert = torch.cat(tokens_per_expert).to(expert_scores.dtype)
    expected_values = layers * args.moe_num_experts
    assert tokens_per_expert.numel() == expected_values
    assert expert_scores.numel() == expected_values
    scale = (args.moe_num_experts * args.moe_loss_weight) / (args.num_layers * tokens * args.moe_top_k)
    return scale * torch.dot(tokens_per_expert, expert_scores)


class ParallelMLP(torch.nn.Module):
    """Capacity-factor expert computation (moe.py:95-437) on one GPU.  Also the base of the
    dropless layer, which replaces `mlp` and `forward_once`."""

    _builds_dense_mlp = True

    def __init__(self, args: Arguments):
        super().__init__()
        self.args = args
        self.num_experts = args.moe_num_experts
        self.top_k = self.args.moe_top_k
        # bits needed to tell the expert ids apart: the radix sort looks at no others (moe.py:110)
        self.sort_end_bit = max(int(np.ceil(np.log2(self.num_experts))), 1)
        if self._builds_dense_mlp:
            self.mlp = mlp.MLP(args)
        self.bias: Optional[torch.Tensor]
        if self.args.bias:
            self.bias = torch.nn.Parameter(torch.empty(args.hidden_size, device=args.device, dtype=common.dtype(args)))
            torch.nn.init.zeros_(self.bias)
        else:
            self.register_parameter('bias', None)
        self.forward_fn = self.forward_once

    def expert_capacity(self, tokens: int) -> int:
        tokens_per_expert = self.top_k * tokens / self.num_experts
        return int(self.args.moe_capacity_factor * tokens_per_expert)

    def load_balancing_loss(self, tokens_per_expert: torch.Tensor, expert_scores: torch.Tensor):
        assert len(expert_scores.size()) == 2
        tokens, num_experts = expert_scores.size()
        assert num_experts == self.num_experts
        assert len(tokens_per_expert.size()) == 1
        assert tokens_per_expert.size(0) == self.num_experts
        scale = self.num_experts / (tokens * self.top_k)
        return scale * torch.dot(tokens_per_expert.to(expert_scores.dtype), expert_scores.mean(dim=0))

    def indices_and_bins(self, top_expert: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        """moe.py:152-183 -> (indices, bin_ids, bins, tokens_per_expert), all int32 on the device."""
        top_expert = top_expert.int()
        if ops_routing.route_supported(top_expert, self.num_experts, self.sort_end_bit):
            indices, bin_ids, tokens_per_expert, bins, _ = ops_routing.route(top_expert, self.num_experts, self.sort_end_bit)
        else:
            bin_ids, indices = ops.sort(top_expert, self.sort_end_bit)
            tokens_per_expert = ops.histogram(top_expert, self.num_experts)
            bins = ops.inclusive_cumsum(tokens_per_expert, 0)
            bins = bins.view(1) if not len(bins.size()) else bins
        gg.note_bins(tokens_per_expert, bins)     # the grouped products of this step take these row bins
        return indices, bin_ids, bins, tokens_per_expert

    def permute_and_compute(self, x, tokens_per_expert, indices, bin_ids, expert_weights, bins, expert_capacity,
                            top_k):
        """moe.py:185-207: binned gather -> batched MLP -> binned scatter."""
        x = x.view(-1, x.shape[-1])
        x = ops.binned_gather(x, indices, bins, expert_capacity, top_k)
        x = self.mlp(x)
        return ops.binned_scatter(x, indices, expert_weights, bins, top_k)

    def forward_once(self, x, expert_weights, top_experts):
        """moe.py:209-235."""
        expert_weights = expert_weights.flatten()
        top_experts = top_experts.flatten()
        with torch.no_grad():
            indices, bin_ids, bins, tokens_per_expert = self.indices_and_bins(top_experts)
            sl, bs, _ = x.size()
            expert_capacity = self.expert_capacity(sl * bs)
            if expert_capacity == 0:
                expert_capacity = torch.max(tokens_per_expert).item()
        x = self.permute_and_compute(x, tokens_per_expert, indices, bin_ids, expert_weights, bins, expert_capacity,
                                     self.top_k)
        return x, tokens_per_expert

    def forward(self, x, scores, expert_weights, top_experts):
        """moe.py:425-437."""
        in_shape = x.size()
        x, tokens_per_expert = self.forward_fn(x, expert_weights, top_experts)
        if self.training and self.args.moe_loss_weight > 0:
            save_load_balancing_loss((tokens_per_expert, scores))
        x = x.view(in_shape)
        if self.bias is not None:
            if self.args.return_bias:
                return x, self.bias
            return x + self.bias
        return x


class MoE(torch.nn.Module):
    """moe.py:440-475."""

    def __init__(self, args: Arguments):
        super().__init__()
        self.router = router.LearnedRouter(args)
        self.experts = self._init_experts_mlp(args)
        self.shared_expert = None

    def _init_experts_mlp(self, args: Arguments):
        return ParallelMLP(args)

    def forward(self, x: torch.Tensor):
        x = common.cast_if_autocast_enabled(x)
        # Called as a module (moe.py:468), so that hooks on the router and routers that only define forward() work.
        # LearnedRouter hangs the int32 copy of its indices, which its kernel writes anyway, on the int64 tensor it
        # returns; the routing takes that copy (no cast, moe.py:160) unless something has replaced or rewritten the
        # indices on the way here.
        scores, expert_weights, top_experts = self.router(x)
        return self.experts(x, scores, expert_weights, router.int32_indices(top_experts))
