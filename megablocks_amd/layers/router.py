"""Learned top-k router: megablocks/layers/router.py:10-114.  The linear layer is torch's (a small dense
GEMM), except for its weight gradient on large 16-bit batches, which goes through the grouped TN kernel;
softmax, top-k and the renormalisation of the selected weights are one HIP kernel each way.  The outputs
feed the HIP routing kernels."""
from typing import Any

import torch

from megablocks_amd import _lib
from megablocks_amd.layers import common
from megablocks_amd.layers.arguments import Arguments

_ROUTER_LOGITS = []

# softmax / top-k / renormalisation as one HIP kernel each way (False: torch's operations, as the reference)
FUSED_SOFTMAX_TOPK = True


def _save_router_logits(logits: torch.Tensor, args: Arguments, lse=None):
    """router.py:17-22.  lse: logsumexp(logits, dim=1) in fp32 where the router kernel has written it (differentiable
    through that kernel's backward), else None."""
    if args.moe_zloss_weight == 0:
        return
    _ROUTER_LOGITS.append((logits, lse))


def clear_router_zloss():
    _ROUTER_LOGITS.clear()


def batched_router_zloss(args: Arguments):
    """router.py:25-42: weight * mean(logsumexp(logits)^2) per router."""
    if args.moe_zloss_weight == 0:
        import warnings
        warnings.warn('Call to batched_router_zloss, but moe_zloss_weight=0')
        return 0
    terms = []
    for logits, lse in _ROUTER_LOGITS:
        if lse is None:
            lse = torch.logsumexp(logits.float() if args.moe_zloss_in_fp32 else logits, dim=1)
        elif not args.moe_zloss_in_fp32:
            lse = lse.to(logits.dtype)     # what torch.logsumexp returns for 16-bit logits: computed in fp32, rounded
        terms.append(lse.square().mean())
    return args.moe_zloss_weight * torch.stack(terms)


class _UniformExpertAssignment(torch.autograd.Function):

    @staticmethod
    def forward(ctx: Any, x: torch.Tensor, num_experts: int):
        out = torch.arange(x.numel(), dtype=x.dtype, device=x.device)
        return torch.remainder(out, num_experts).view(x.shape)


class _RouterLinear(torch.autograd.Function):
    """`x @ weight^T` of the router's `torch.nn.Linear` (router.py:96), with the weight gradient
    `[E, T] @ [T, h]` (a short, wide output over a reduction as long as the batch: a handful of tiles for the
    vendor GEMM) computed by the grouped TN kernel instead: the token range is cut into equal pieces, each
    piece is one group, and the partial products are summed in fp32."""

    PIECE_ROWS = 256   # tokens per piece (four K tiles of the TN kernel)
    MAX_PIECES = 64

    _sizes = {}

    @staticmethod
    def piece_sizes(tokens: int) -> torch.Tensor:
        """Rows per piece (kept per batch size: the grouped GEMM caches the device-side bins on this tensor)."""
        sizes = _RouterLinear._sizes.get(tokens)
        if sizes is None:
            pieces = max(1, min(_RouterLinear.MAX_PIECES, tokens // _RouterLinear.PIECE_ROWS))
            sizes = torch.full((pieces,), tokens // pieces, dtype=torch.int64)
            sizes[:tokens % pieces] += 1
            _RouterLinear._sizes[tokens] = sizes
        return sizes

    @staticmethod
    @torch.amp.custom_fwd(device_type='cuda')
    def forward(ctx: Any, x: torch.Tensor, weight: torch.Tensor):
        # Under autocast the product runs in x's 16-bit type, as torch's own linear would; the cast weight is
        # what the backward multiplies with, and the weight gradient goes back in the parameter's type (fp32
        # master weights).  Outside autocast mismatched types are an error, as for torch.nn.Linear.
        ctx.weight_dtype = weight.dtype
        if weight.dtype != x.dtype and torch.is_autocast_enabled():
            weight = weight.to(x.dtype)
        ctx.save_for_backward(x, weight)
        return torch.nn.functional.linear(x, weight)

    @staticmethod
    @torch.amp.custom_bwd(device_type='cuda')
    def backward(ctx: Any, grad: torch.Tensor):
        x, weight = ctx.saved_tensors
        grad = grad.to(x.dtype)
        dx = grad @ weight if ctx.needs_input_grad[0] else None
        dw = None
        if ctx.needs_input_grad[1]:
            from megablocks_amd import grouped_gemm_util as gg
            sizes = _RouterLinear.piece_sizes(x.shape[0])
            pieces = sizes.shape[0]
            parts = gg.gmm(grad.contiguous(), x.contiguous(), sizes, trans_a=True, _record_as='router_wgrad')   # [pieces, E, h]
            dw = (parts[0] if pieces == 1 else parts.sum(0, dtype=torch.float32)).to(ctx.weight_dtype)
        return dx, dw


class _SoftmaxTopK(torch.autograd.Function):
    """softmax -> top-k -> optional p-norm renormalisation (router.py:87-106) as one kernel each way.
    Returns (scores, expert_weights, expert_indices, expert_indices as int32, lse) with torch's shapes and dtypes (int64
    indices); the int32 copy, written by the same kernel, is what the layer's routing takes (moe.py:160 casts); lse
    (`want_lse`, else None) is logsumexp(logits, dim=1) in fp32, the term of the z-loss (router.py:37), which the
    backward kernel differentiates along with the rest."""

    @staticmethod
    def supported(logits: torch.Tensor, top_k: int) -> bool:
        return (logits.is_cuda and logits.ndim == 2 and logits.dtype in _lib.DTYPE and 0 < logits.shape[1] <= 512
                and 0 < top_k <= min(64, logits.shape[1]))

    @staticmethod
    def forward(ctx: Any, logits: torch.Tensor, top_k: int, norm_p: float, want_lse: bool = False):
        logits = logits.contiguous()
        tokens, experts = logits.shape
        scores = torch.empty_like(logits)
        weights = torch.empty((tokens, top_k), dtype=logits.dtype, device=logits.device)
        indices = torch.empty((tokens, top_k), dtype=torch.int64, device=logits.device)
        indices32 = torch.empty((tokens, top_k), dtype=torch.int32, device=logits.device)
        lse = torch.empty((tokens,), dtype=torch.float32, device=logits.device) if want_lse else None
        with _lib.device_of(logits):
            _lib.check(_lib.lib.mbx_router_forward(_lib.ptr(logits), _lib.dtype_of(logits), tokens, experts, top_k,
                                                   float(norm_p), _lib.ptr(scores), _lib.ptr(weights), _lib.ptr(indices),
                                                   _lib.ptr(indices32), _lib.ptr(lse), _lib.stream()), 'router_forward')
        ctx.save_for_backward(scores, indices)
        ctx.top_k, ctx.norm_p = top_k, float(norm_p)
        ctx.mark_non_differentiable(indices, indices32)
        # an output nobody differentiates (the scores without a load-balancing loss, lse without a z-loss, the indices)
        # arrives in backward as None instead of a zero-filled tensor: three fill launches less per step
        ctx.set_materialize_grads(False)
        return scores, weights, indices, indices32, lse

    @staticmethod
    def backward(ctx: Any, grad_scores, grad_weights, _grad_indices, _grad_indices32, grad_lse):
        scores, indices = ctx.saved_tensors
        tokens, experts = scores.shape
        grad_logits = torch.empty_like(scores)
        gs = None if grad_scores is None else grad_scores.to(scores.dtype).contiguous()
        gw = None if grad_weights is None else grad_weights.to(scores.dtype).contiguous()
        gl = None if grad_lse is None else grad_lse.float().contiguous()
        with _lib.device_of(scores):
            _lib.check(_lib.lib.mbx_router_backward(_lib.ptr(gw), _lib.ptr(gs), _lib.ptr(scores), _lib.ptr(indices),
                                                    _lib.dtype_of(scores), tokens, experts, ctx.top_k, ctx.norm_p,
                                                    _lib.ptr(grad_logits), _lib.ptr(gl), _lib.stream()), 'router_backward')
        return grad_logits, None, None, None


def int32_indices(expert_indices: torch.Tensor) -> torch.Tensor:
    """The int32 copy LearnedRouter.forward attached to its indices, if `expert_indices` still is that tensor with
    that content; else `expert_indices` itself (the routing then casts, as moe.py:160 does)."""
    attached = getattr(expert_indices, '_mbx_int32', None)
    if attached is not None and attached[1] == expert_indices._version and attached[0].shape == expert_indices.shape:
        return attached[0]
    return expert_indices


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
        scores, expert_weights, expert_indices, expert_indices32 = self.route(x)
        if expert_indices32 is not None:
            # out of band: the same indices as int32, valid while the int64 tensor is the one returned here, unmodified
            expert_indices._mbx_int32 = (expert_indices32, expert_indices._version)
        return scores, expert_weights, expert_indices

    def route(self, x: torch.Tensor):
        """forward's (scores, expert_weights, expert_indices) and, where the router kernel wrote them, the indices as
        int32 (else None): the layer routes with those and skips the cast of moe.py:160."""
        if self.training and self.args.moe_jitter_eps is not None:
            x = x * self.jitter(x)
        x2d = x.view(-1, x.shape[-1])
        if x2d.is_cuda and x2d.dtype in (torch.bfloat16, torch.float16) and x2d.shape[0] >= 4 * _RouterLinear.PIECE_ROWS:
            logits = _RouterLinear.apply(x2d, self.layer.weight)
        else:
            logits = self.layer(x2d)
        saved_logits, lse = logits, None
        if logits.is_cuda and logits.dtype != torch.float32 and torch.is_autocast_enabled():
            # autocast runs softmax in fp32 (router.py:98 under torch.autocast): scores and weights come out in fp32
            logits = logits.float()
        expert_indices32 = None
        if FUSED_SOFTMAX_TOPK and _SoftmaxTopK.supported(logits, self.args.moe_top_k):
            scores, expert_weights, expert_indices, expert_indices32, lse = _SoftmaxTopK.apply(
                logits, self.args.moe_top_k, self.args.moe_normalize_expert_weights or 0,
                self.args.moe_zloss_weight != 0)
        else:
            scores = logits.softmax(dim=-1)
            expert_weights, expert_indices = self._top_k(scores)
            if self.args.moe_normalize_expert_weights:
                expert_weights = expert_weights / torch.norm(
                    expert_weights, p=self.args.moe_normalize_expert_weights, dim=-1, keepdim=True)
        _save_router_logits(saved_logits, self.args, lse)
        if self.args.uniform_expert_assignment:
            expert_indices = _UniformExpertAssignment.apply(expert_indices, self.args.moe_num_experts)
            expert_indices32 = None
        return scores, expert_weights, expert_indices, expert_indices32
