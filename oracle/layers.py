"""CPU oracle: the dMoE layer (router -> permute -> expert MLP -> weighted combine).
Test infrastructure only.

A differentiable torch-CPU formulation (sort / bincount / cumsum / index_select ->
per-expert matmul loop -> weighted index_add); gradients come from autograd.  It is also
the CPU baseline that bench.py times on the host cores.
"""
import torch
import torch.nn.functional as F

from oracle import routing


def gelu_tanh_backward(g: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """megablocks/layers/gelu.py:9-13: g * d/dx gelu_tanh(x) (out of place here)."""
    t = torch.tanh(0.79788456 * x * (1 + 0.044715 * x * x))
    ff = 0.5 * x * ((1 - t * t) * (0.79788456 + 0.1070322243 * x * x)) + 0.5 * (1 + t)
    return g * ff


def router_forward(x, router_weight, top_k, normalize_p=None):
    """megablocks/layers/router.py:87-114 (no jitter, no uniform assignment).
    -> (scores [T,E], expert_weights [T,k], expert_indices [T,k] int64)."""
    logits = F.linear(x.view(-1, x.shape[-1]), router_weight)
    scores = logits.softmax(dim=-1)
    if top_k == 1:
        expert_weights, expert_indices = scores.max(dim=-1, keepdim=True)
    else:
        expert_weights, expert_indices = torch.topk(scores, top_k, dim=-1)
    if normalize_p:
        expert_weights = expert_weights / torch.norm(expert_weights, p=normalize_p, dim=-1, keepdim=True)
    return scores, expert_weights, expert_indices


def dmoe_forward(x, expert_weights, top_experts, w1, w2, v1=None, *, num_experts, top_k,
                 activation=None):
    """megablocks/layers/dmoe.py:239-280 (grouped_forward_once + grouped_permute_and_compute)
    with GroupedMLP (mlp.py:499-523) or, when ``v1`` is given, GroupedGLU (glu.py:173-205).

    x [T,h]; expert_weights/top_experts [T,k]; w1, v1, w2 [E*f, h].  Returns
    (out [T,h], tokens_per_expert int32 [E]).  The 128-padded sparse formulation
    (dmoe.py:156-193) computes the same values: pad rows are zero, the experts have no
    bias, and padded_scatter never reads a pad row.
    """
    if activation is None:
        activation = lambda t: F.gelu(t, approximate='tanh')  # arguments.py:19
    hidden = x.shape[-1]
    x = x.reshape(-1, hidden)
    flat_w = expert_weights.flatten()
    indices, bin_ids, bins, tokens_per_expert = routing.indices_and_bins(top_experts.flatten(), num_experts)
    idx = indices.long()
    token = idx // top_k
    xg = x.index_select(0, token)                       # ops.gather
    w1e = w1.view(num_experts, -1, hidden)
    w2e = w2.view(num_experts, -1, hidden)
    v1e = None if v1 is None else v1.view(num_experts, -1, hidden)
    outs, start = [], 0
    for e in range(num_experts):
        n = int(tokens_per_expert[e])
        xe = xg[start:start + n]
        hcur = activation(xe @ w1e[e].t())
        if v1e is not None:
            hcur = hcur * (xe @ v1e[e].t())
        outs.append(hcur @ w2e[e])
        start += n
    y = torch.cat(outs, 0)
    y = y * flat_w.index_select(0, idx).unsqueeze(-1)   # ops.scatter: scale by weights[indices[i]] ...
    out = torch.zeros_like(x).index_add(0, token, y)    # ... and sum the top_k rows of each token
    return out, tokens_per_expert
