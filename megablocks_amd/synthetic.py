"""Synthetic workloads for the dropless-MoE layer: the five benchmark configurations and their
seeded inputs.  Everything is drawn on the CPU in fp32 from `torch.manual_seed(seed)` so that a
CPU formulation and the GPU layer can be fed identical values.
"""
import dataclasses
from typing import Optional

import torch
import torch.nn.functional as F


@dataclasses.dataclass(frozen=True)
class Workload:
    name: str
    tokens: int
    hidden: int
    ffn: int
    experts: int
    top_k: int
    mlp_type: str          # 'mlp' (tanh-GELU) or 'glu' (SiLU-gated)
    mlp_impl: str          # 'grouped' or 'sparse' (128-padded expert groups)
    dtype: torch.dtype
    routing: str           # 'router' | 'zipf' | 'logits'
    normalize: Optional[int] = None
    description: str = ''

    @property
    def slots(self):
        return self.tokens * self.top_k

    @property
    def gemms_forward(self):
        return 3 if self.mlp_type == 'glu' else 2

    def gemm_flops(self):
        """Grouped-GEMM FLOPs of one forward+backward on the unpadded slots: G * 2 N h f, times 3."""
        return 3 * self.gemms_forward * 2 * self.slots * self.hidden * self.ffn

    def permute_bytes(self):
        """Minimum HBM traffic of the five permutation passes of one forward+backward."""
        return 5 * (self.tokens + self.slots) * self.hidden * torch.finfo(self.dtype).bits // 8

    def activation(self):
        return F.silu if self.mlp_type == 'glu' else (lambda t: F.gelu(t, approximate='tanh'))


WORKLOADS = {
    'c1': Workload('c1', 4096, 1024, 4096, 8, 2, 'mlp', 'grouped', torch.float32, 'router',
                   description='CPU plumbing: fp32, 8 experts top-2, GELU MLP'),
    'c2': Workload('c2', 16384, 1024, 4096, 64, 1, 'mlp', 'grouped', torch.bfloat16, 'router',
                   description='GPT-2-medium-scale dMoE: 64 experts top-1, GELU MLP, bf16'),
    'c3': Workload('c3', 8192, 4096, 14336, 8, 2, 'glu', 'grouped', torch.bfloat16, 'router', normalize=1,
                   description='Mixtral-8x7B-shaped dMoE layer: 8 experts top-2, SwiGLU, bf16'),
    'c4': Workload('c4', 32768, 2048, 1408, 64, 6, 'glu', 'grouped', torch.bfloat16, 'zipf',
                   description='fine-grained skewed routing: 64 experts top-6, Zipf(1.2), 4 empty experts, SwiGLU'),
    'c5': Workload('c5', 24576, 2048, 8192, 16, 4, 'mlp', 'sparse', torch.bfloat16, 'logits',
                   description='block-sparse mode: 16 experts top-4, 128-padded groups, GELU MLP'),
}


def make_inputs(w: Workload, tokens: Optional[int] = None, seed: int = 0):
    """fp32 CPU tensors: x [T,h], grad [T,h], router_weight [E,h], w1/w2 (and v1) [E*f,h], and the
    routing decision (expert_weights [T,k] fp32, top_experts [T,k] int64, scores [T,E])."""
    T = w.tokens if tokens is None else tokens
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, w.hidden, generator=g)
    router_weight = torch.randn(w.experts, w.hidden, generator=g) * 0.02
    w1 = torch.randn(w.experts * w.ffn, w.hidden, generator=g) * 0.02
    w2 = torch.randn(w.experts * w.ffn, w.hidden, generator=g) * 0.02
    v1 = torch.randn(w.experts * w.ffn, w.hidden, generator=g) * 0.02 if w.mlp_type == 'glu' else None
    grad = torch.randn(T, w.hidden, generator=g)

    if w.routing == 'router':
        scores = (x @ router_weight.t()).softmax(-1)
        if w.top_k == 1:
            expert_weights, top_experts = scores.max(-1, keepdim=True)
        else:
            expert_weights, top_experts = torch.topk(scores, w.top_k, -1)
        if w.normalize:
            expert_weights = expert_weights / torch.norm(expert_weights, p=w.normalize, dim=-1, keepdim=True)
    elif w.routing == 'zipf':
        # popularity r^-1.2 over ranks, the 4 least popular ranks get no tokens; ranks -> expert ids
        # through a seeded permutation; k distinct experts per token; gate = softmax of N(0,1)
        p = torch.arange(1, w.experts + 1, dtype=torch.float32) ** -1.2
        p[-4:] = 0
        ids = torch.randperm(w.experts, generator=g)
        ranks = torch.multinomial(p.expand(T, -1), w.top_k, replacement=False, generator=g)
        top_experts = ids[ranks]
        expert_weights = torch.randn(T, w.top_k, generator=g).softmax(-1)
        scores = torch.zeros(T, w.experts).scatter_(1, top_experts, expert_weights)
    elif w.routing == 'logits':
        scores = (2 * torch.randn(T, w.experts, generator=g)).softmax(-1)
        expert_weights, top_experts = torch.topk(scores, w.top_k, -1)
    else:
        raise ValueError(w.routing)
    return dict(x=x, grad=grad, router_weight=router_weight, w1=w1, w2=w2, v1=v1, scores=scores,
                expert_weights=expert_weights, top_experts=top_experts)


def build_layer(w: Workload, inputs, device='cuda', memory_optimized=False):
    """A dMoE layer of the workload's shape holding the given weights (bias off, no aux loss)."""
    from megablocks_amd.layers.arguments import DEFAULT_ACTIVATION_FN, Arguments
    from megablocks_amd.layers.dmoe import dMoE
    args = Arguments(
        hidden_size=w.hidden, ffn_hidden_size=w.ffn, moe_num_experts=w.experts, moe_top_k=w.top_k,
        mlp_type=w.mlp_type, mlp_impl=w.mlp_impl, bias=False, moe_loss_weight=0.0,
        moe_normalize_expert_weights=w.normalize,
        activation_fn=F.silu if w.mlp_type == 'glu' else DEFAULT_ACTIVATION_FN,
        fp16=w.dtype == torch.float16, bf16=w.dtype == torch.bfloat16, device=torch.device(device),
        memory_optimized_mlp=memory_optimized, init_method=lambda t: None, output_layer_init_method=lambda t: None)
    layer = dMoE(args)
    with torch.no_grad():
        layer.router.layer.weight.copy_(inputs['router_weight'])
        layer.experts.mlp.w1.copy_(inputs['w1'])
        layer.experts.mlp.w2.copy_(inputs['w2'])
        if w.mlp_type == 'glu':
            layer.experts.mlp.v1.copy_(inputs['v1'])
    return layer


def layer_step(layer, w: Workload, x, grad, routing=None):
    """One forward+backward of the layer.  With `routing` = (scores, expert_weights, top_experts)
    the router is bypassed (workloads whose expert assignment is prescribed)."""
    if routing is None:
        out = layer(x)
    else:
        out = layer.experts(x, *routing)
    out.backward(grad)
    return out
