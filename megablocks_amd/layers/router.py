"""Learned top-k router: megablocks/layers/router.py:10-114.  Plain PyTorch-ROCm (a small dense
GEMM, softmax and top-k); its outputs feed the HIP routing kernels."""
from typing import Any

import torch

from megablocks_amd.layers import common
from megablocks_amd.layers.arguments import Arguments

_ROUTER_LOGITS = []


def _save_router_logits(logits: torch.Tensor, args: Arguments):
    if args.moe_zloss_weight == 0:
        return
    _ROUTER_LOGITS.append(logits)


def clear_router_zloss():
    _ROUTER_LOGITS.clear()


def batched_router_zloss(args: Arguments):
    """router.py:25-42: weight * mean(logsumexp(logits)^2) per router."""
    if args.moe_zloss_weight == 0:
        import warnings
        warnings.warn('Call to batched_router_zloss, but moe_zloss_weight=0')
        return 0
    logits_per_router = _ROUTER_LOGITS
    if args.moe_zloss_in_fp32:
        logits_per_router = [logits.float() for logits in logits_per_router]
    unscaled = torch.stack([torch.logsumexp(logits, dim=1).square().mean() for logits in logits_per_router])
    return args.moe_zloss_weight * unscaled


class _UniformExpertAssignment(torch.autograd.Function):

    @staticmethod
    def forward(ctx: Any, x: torch.Tensor, num_experts: int):
        out = torch.arange(x.numel(), dtype=x.dtype, device=x.device)
        return torch.remainder(out, num_experts).view(x.shape)


class LearnedRouter(torch.nn.Module):

    def __init__(self, args: Arguments):
        super().__init__()
        self.args = args
        self.layer = torch.nn.Linear(args.hidden_size, args.moe_num_experts, bias=False, dtype=common.dtype(args),
                                     device=args.device)
        args.init_method(self.layer.weight)

    def jitter(self, x: torch.Tensor):
        low = 1.0 - self.args.moe_jitter_eps
        high = 1.0 + self.args.moe_jitter_eps
        noise = torch.rand(x.size(), dtype=x.dtype, device=x.device)
        return low + noise * (high - low)

    def _top_k(self, scores: torch.Tensor):
        if self.args.moe_top_k == 1:
            return scores.max(dim=-1, keepdim=True)
        return torch.topk(scores, self.args.moe_top_k, dim=-1)

    def forward(self, x: torch.Tensor):
        if self.training and self.args.moe_jitter_eps is not None:
            x = x * self.jitter(x)
        logits = self.layer(x.view(-1, x.shape[-1]))
        _save_router_logits(logits, self.args)
        scores = logits.softmax(dim=-1)
        expert_weights, expert_indices = self._top_k(scores)
        if self.args.moe_normalize_expert_weights:
            expert_weights = expert_weights / torch.norm(
                expert_weights, p=self.args.moe_normalize_expert_weights, dim=-1, keepdim=True)
        if self.args.uniform_expert_assignment:
            expert_indices = _UniformExpertAssignment.apply(expert_indices, self.args.moe_num_experts)
        return scores, expert_weights, expert_indices
