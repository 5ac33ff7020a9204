"""CPU oracle: the router's auxiliary losses.  Test infrastructure only.

Restates megablocks/layers/moe.py:32-89 (`batched_load_balancing_loss`), moe.py:138-150
(`ParallelMLP.load_balancing_loss`) and megablocks/layers/router.py:25-42 (`batched_router_zloss`) as
differentiable torch-CPU code, layer by layer instead of on concatenated tensors.
"""
import torch


def load_balancing_loss(tokens_per_expert, expert_scores, *, num_experts, top_k, loss_weight, num_layers=None,
                        in_fp32=True):
    """moe.py:32-89.  `tokens_per_expert`: one int vector [E] per layer; `expert_scores`: one [tokens, E] matrix of
    router probabilities per layer (the softmax over all experts, not the selected weights).

        loss = loss_weight * E / (num_layers * tokens * top_k) * sum_layers <tokens_per_expert, mean_tokens scores>

    With no tokens the mean is replaced by a sum (moe.py:71-74).  `num_layers` defaults to the number of layers
    handed in (the reference raises when they differ, moe.py:42-60)."""
    if loss_weight == 0:
        return 0.0                                                   # moe.py:33-34
    if isinstance(tokens_per_expert, torch.Tensor):
        tokens_per_expert, expert_scores = [tokens_per_expert], [expert_scores]
    if num_layers is None:
        num_layers = len(tokens_per_expert)
    if len(tokens_per_expert) != num_layers or len(expert_scores) != num_layers:
        raise ValueError(f'Expected {num_layers} token_per_experts but found {len(tokens_per_expert)}.')
    tokens = expert_scores[0].shape[0]
    total = None
    for counts, scores in zip(tokens_per_expert, expert_scores):
        assert counts.ndim == 1 and counts.numel() == num_experts
        assert scores.ndim == 2 and scores.shape == (tokens, num_experts)
        if in_fp32:
            scores = scores.float()                                  # moe.py:69-70
        per_expert = scores.mean(dim=0) if tokens != 0 else scores.sum(dim=0)
        term = (counts.to(per_expert.dtype) * per_expert).sum()
        total = term if total is None else total + term
    scale = (num_experts * loss_weight) / (num_layers * tokens * top_k) if tokens else float('inf')
    return scale * total


def layer_load_balancing_loss(tokens_per_expert, expert_scores, *, top_k):
    """moe.py:138-150: one layer's unweighted contribution, E / (tokens * top_k) * <counts, mean scores>."""
    tokens, num_experts = expert_scores.shape
    assert tokens_per_expert.shape == (num_experts,)
    return num_experts / (tokens * top_k) * (tokens_per_expert.to(expert_scores.dtype) * expert_scores.mean(dim=0)).sum()


def router_zloss(logits_per_router, *, zloss_weight, in_fp32=True):
    """router.py:25-42: one value per router, zloss_weight * mean_tokens(logsumexp_experts(logits) ** 2)."""
    if zloss_weight == 0:
        return 0
    if isinstance(logits_per_router, torch.Tensor):
        logits_per_router = [logits_per_router]
    out = []
    for logits in logits_per_router:
        if in_fp32:
            logits = logits.float()
        m = logits.max(dim=1, keepdim=True).values
        lse = m.squeeze(1) + (logits - m).exp().sum(dim=1).log()
        out.append((lse * lse).mean())
    return zloss_weight * torch.stack(out)


def uniform_expert_assignment(shape, num_experts):
    """router.py:49-58: expert of flattened slot i is i mod num_experts."""
    numel = 1
    for s in shape:
        numel *= s
    return (torch.arange(numel, dtype=torch.int64) % num_experts).view(shape)
