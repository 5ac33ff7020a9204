"""GPU parity tests of the dMoE layer (forward and backward) against the CPU oracle, in the
manner of the reference's tests/layers/{dmoe,glu,moe}_test.py.  Tolerance: relative Frobenius
error <= 1e-2 for bf16/f16 (north-star bar), 1e-4 for fp32."""
import dataclasses
import math
from functools import partial

import pytest
import torch
import torch.nn.functional as F

import oracle

pytestmark = pytest.mark.gpu


def rel_err(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


@pytest.fixture(scope='module')
def syn():
    from megablocks_amd import synthetic
    return synthetic


def _oracle_step(w, inp, routing_given, top_experts=None):
    """fp32 forward + backward of the oracle.  With the router in the chain, `top_experts` (the layer's own choice:
    a 16-bit router breaks near-ties differently from fp32) replaces the oracle's top-k; the weights are then the
    oracle's own fp32 scores at those experts, renormalised as router.py:100-106 does."""
    x = inp['x'].clone().requires_grad_(True)
    rw = inp['router_weight'].clone().requires_grad_(True)
    w1, w2 = inp['w1'].clone().requires_grad_(True), inp['w2'].clone().requires_grad_(True)
    v1 = None if inp['v1'] is None else inp['v1'].clone().requires_grad_(True)
    if routing_given:
        ew = inp['expert_weights'].clone().requires_grad_(True)
        te = inp['top_experts']
    else:
        scores, ew, te = oracle.router_forward(x, rw, w.top_k, w.normalize)
        if top_experts is not None:
            te = top_experts
            ew = scores.gather(1, te)
            if w.normalize:
                ew = ew / torch.norm(ew, p=w.normalize, dim=-1, keepdim=True)
    out, tpe = oracle.dmoe_forward(x, ew, te, w1, w2, v1, num_experts=w.experts, top_k=w.top_k,
                                   activation=w.activation())
    out.backward(inp['grad'])
    grads = dict(x=x.grad, w1=w1.grad, w2=w2.grad)
    if v1 is not None:
        grads['v1'] = v1.grad
    if routing_given:
        grads['expert_weights'] = ew.grad
    else:
        grads['router'] = rw.grad
    return out.detach(), tpe, grads, te


CASES = [  # tokens, hidden, ffn, experts, top_k, mlp_type, mlp_impl, routing
    (256, 128, 256, 4, 1, 'mlp', 'grouped', 'router'),
    (512, 256, 512, 8, 2, 'mlp', 'grouped', 'router'),
    (512, 256, 512, 8, 2, 'glu', 'grouped', 'router'),
    (1000, 128, 384, 16, 4, 'glu', 'grouped', 'zipf'),
    (512, 256, 512, 8, 2, 'mlp', 'sparse', 'logits'),
    (512, 256, 512, 8, 2, 'glu', 'sparse', 'logits'),
    (300, 72, 136, 5, 3, 'mlp', 'grouped', 'logits'),          # sizes off the MFMA fast path
    (2048, 256, 512, 8, 2, 'glu', 'grouped', 'router'),        # enough tokens for the router's grouped weight gradient
    (1536, 128, 256, 16, 1, 'mlp', 'sparse', 'router'),
]


@pytest.mark.parametrize('tokens,hidden,ffn,experts,top_k,mlp_type,mlp_impl,routing', CASES)
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize('memopt', [False, True])
def test_dmoe_forward_backward_vs_oracle(syn, tokens, hidden, ffn, experts, top_k, mlp_type, mlp_impl, routing, dtype,
                                         memopt):
    if memopt and mlp_type == 'glu' and mlp_impl == 'sparse':
        pytest.skip('the reference rejects memory_optimized_mlp for the sparse GLU (glu.py:47-50)')
    if mlp_impl == 'sparse' and ffn % 128:
        pytest.skip('sparse mode needs ffn divisible by the 128 block size')
    w = syn.Workload('t', tokens, hidden, ffn, experts, top_k, mlp_type, mlp_impl, dtype, routing,
                     normalize=1 if routing == 'router' and top_k > 1 else None)
    inp = syn.make_inputs(w, seed=3)
    if dtype != torch.float32:   # the oracle sees the values the layer sees: rounded weights and inputs
        for k in ('x', 'grad', 'router_weight', 'w1', 'w2', 'v1', 'expert_weights'):
            if inp[k] is not None:
                inp[k] = inp[k].to(dtype).float()
    given = routing != 'router'
    layer = syn.build_layer(w, inp, memory_optimized=memopt)
    x = inp['x'].to(dtype).cuda().requires_grad_(True)
    grad = inp['grad'].to(dtype).cuda()
    if given:
        ew = inp['expert_weights'].to(dtype).cuda().requires_grad_(True)
        routing_t = (inp['scores'].to(dtype).cuda(), ew, inp['top_experts'].cuda())
        own_choice = None
    else:
        routing_t = None
        with torch.no_grad():   # the experts the layer's own router picks for these inputs
            own_choice = layer.router(x)[2].cpu()
    want, want_tpe, want_grads, te = _oracle_step(w, inp, given, own_choice)
    out = syn.layer_step(layer, w, x, grad, routing_t)

    tol = 1e-4 if dtype == torch.float32 else 1e-2                 # f16 has three more mantissa bits than bf16: same bound
    assert out.shape == (tokens, hidden) and out.dtype == dtype
    assert rel_err(out, want) < tol
    assert rel_err(x.grad, want_grads['x']) < tol
    assert rel_err(layer.experts.mlp.w1.grad, want_grads['w1']) < tol
    assert rel_err(layer.experts.mlp.w2.grad, want_grads['w2']) < tol
    if mlp_type == 'glu':
        assert rel_err(layer.experts.mlp.v1.grad, want_grads['v1']) < tol
    if given:
        assert rel_err(ew.grad, want_grads['expert_weights']) < tol
    else:
        assert rel_err(layer.router.layer.weight.grad, want_grads['router']) < 5 * tol


@pytest.mark.parametrize('mlp_type,activation', [('mlp', 'relu'), ('glu', 'gelu_exact'), ('mlp', 'silu')])
@pytest.mark.parametrize('mlp_impl,memopt', [('grouped', False), ('grouped', True), ('sparse', False)])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
def test_dmoe_with_an_activation_the_library_has_no_kernel_for(syn, mlp_type, activation, mlp_impl, memopt, dtype):
    """`activation_fn` is the user's (arguments.py:30): anything but SiLU for the gated experts or tanh-GELU takes
    torch's own forward and autograd (mlp.py:478-483 "else autograd", glu.py:120-124) around the library's grouped
    products.  Forward and every gradient against the oracle with the same callable."""
    import torch.nn.functional as F
    fn = {'relu': F.relu, 'gelu_exact': F.gelu, 'silu': F.silu}[activation]
    w = syn.Workload('t', 700, 128, 384, 4, 2, mlp_type, mlp_impl, dtype, 'logits')
    inp = syn.make_inputs(w, seed=11)
    if dtype != torch.float32:
        for k in ('x', 'grad', 'w1', 'w2', 'v1', 'expert_weights'):
            if inp[k] is not None:
                inp[k] = inp[k].to(dtype).float()
    leaves = {k: inp[k].clone().requires_grad_(True) for k in ('x', 'w1', 'w2', 'expert_weights')}
    v1 = None if inp['v1'] is None else inp['v1'].clone().requires_grad_(True)
    want, _ = oracle.dmoe_forward(leaves['x'], leaves['expert_weights'], inp['top_experts'], leaves['w1'], leaves['w2'], v1,
                                  num_experts=w.experts, top_k=w.top_k, activation=fn)
    want.backward(inp['grad'])
    layer = syn.build_layer(w, inp, memory_optimized=memopt)
    layer.experts.mlp.args.activation_fn = fn
    x = inp['x'].to(dtype).cuda().requires_grad_(True)
    ew = inp['expert_weights'].to(dtype).cuda().requires_grad_(True)
    from megablocks_amd import _lib
    _lib.profile_hook = []
    try:
        out = syn.layer_step(layer, w, x, inp['grad'].to(dtype).cuda(), (inp['scores'].to(dtype).cuda(), ew, inp['top_experts'].cuda()))
        torch.cuda.synchronize()
        launched = {name for name, *_ in _lib.profile_hook}
    finally:
        _lib.profile_hook = None
    assert not launched & {'gmm_nt_act', 'gmm_nt_dact', 'gmm_nt_glu', 'gmm_nt_dglu'}   # no epilogue was mistaken for it
    tol = 1e-4 if dtype == torch.float32 else 1e-2
    assert rel_err(out, want.detach()) < tol and rel_err(x.grad, leaves['x'].grad) < tol
    mlp = layer.experts.mlp
    assert rel_err(mlp.w1.grad, leaves['w1'].grad) < tol and rel_err(mlp.w2.grad, leaves['w2'].grad) < tol
    if v1 is not None:
        assert rel_err(mlp.v1.grad, v1.grad) < tol
    assert rel_err(ew.grad, leaves['expert_weights'].grad) < tol


@pytest.mark.parametrize('mlp_impl,memopt', [('grouped', False), ('grouped', True), ('sparse', False), ('sparse', True)])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_dmoe_mlp_with_activation_epilogues_vs_oracle(syn, monkeypatch, mlp_impl, memopt, dtype):
    """The GELU expert MLP with the activation and its gradient in the epilogues of the grouped products (a size
    threshold can switch them off; set to zero here) against the oracle, forward and backward."""
    from megablocks_amd import grouped_gemm_util as gg
    monkeypatch.setattr(gg, 'ACTIVATION_EPILOGUE_MIN_BYTES', 0)
    w = syn.Workload('t', 1500, 256, 768, 8, 2, 'mlp', mlp_impl, dtype, 'logits')
    inp = syn.make_inputs(w, seed=5)
    for k in ('x', 'grad', 'w1', 'w2', 'expert_weights'):
        inp[k] = inp[k].to(dtype).float()
    want, _, want_grads, _ = _oracle_step(w, inp, True)
    layer = syn.build_layer(w, inp, memory_optimized=memopt)
    x = inp['x'].to(dtype).cuda().requires_grad_(True)
    ew = inp['expert_weights'].to(dtype).cuda().requires_grad_(True)
    from megablocks_amd import _lib
    _lib.profile_hook = []
    try:
        out = syn.layer_step(layer, w, x, inp['grad'].to(dtype).cuda(), (inp['scores'].to(dtype).cuda(), ew, inp['top_experts'].cuda()))
        torch.cuda.synchronize()
        launched = {name for name, *_ in _lib.profile_hook}
    finally:
        _lib.profile_hook = None
    assert {'gmm_nt_act', 'gmm_nt_dact'} <= launched                      # the epilogue kernels are what ran
    assert rel_err(out, want) < 1e-2 and rel_err(x.grad, want_grads['x']) < 1e-2
    assert rel_err(layer.experts.mlp.w1.grad, want_grads['w1']) < 1e-2 and rel_err(layer.experts.mlp.w2.grad, want_grads['w2']) < 1e-2
    assert rel_err(ew.grad, want_grads['expert_weights']) < 1e-2


@pytest.mark.parametrize('mlp_impl,memopt', [('grouped', False), ('grouped', True), ('sparse', False)])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_dmoe_glu_with_the_gate_in_the_epilogues_vs_oracle(syn, monkeypatch, mlp_impl, memopt, dtype):
    """The gated experts with the gated activation in the epilogue of the launch that computes both of its products,
    and its backward in the epilogue of the product that feeds it (a size threshold can switch them off; set to zero here)
    against the oracle, forward and backward."""
    from megablocks_amd import grouped_gemm_util as gg
    monkeypatch.setattr(gg, 'ACTIVATION_EPILOGUE_MIN_BYTES', 0)
    w = syn.Workload('t', 1500, 256, 768, 8, 2, 'glu', mlp_impl, dtype, 'logits')
    inp = syn.make_inputs(w, seed=6)
    for k in ('x', 'grad', 'w1', 'v1', 'w2', 'expert_weights'):
        inp[k] = inp[k].to(dtype).float()
    want, _, want_grads, _ = _oracle_step(w, inp, True)
    layer = syn.build_layer(w, inp, memory_optimized=memopt)
    x = inp['x'].to(dtype).cuda().requires_grad_(True)
    ew = inp['expert_weights'].to(dtype).cuda().requires_grad_(True)
    from megablocks_amd import _lib
    _lib.profile_hook = []
    try:
        out = syn.layer_step(layer, w, x, inp['grad'].to(dtype).cuda(), (inp['scores'].to(dtype).cuda(), ew, inp['top_experts'].cuda()))
        torch.cuda.synchronize()
        launched = {name for name, *_ in _lib.profile_hook}
    finally:
        _lib.profile_hook = None
    assert {'gmm_nt_glu', 'gmm_nt_dglu'} <= launched                       # the epilogue kernels are what ran
    assert rel_err(out, want) < 1e-2 and rel_err(x.grad, want_grads['x']) < 1e-2
    mlp = layer.experts.mlp
    for name in ('w1', 'v1', 'w2'):
        assert rel_err(getattr(mlp, name).grad, want_grads[name]) < 1e-2, name
    assert rel_err(ew.grad, want_grads['expert_weights']) < 1e-2


@pytest.mark.parametrize('tokens,hidden,experts', [(4096, 1024, 64), (5003, 264, 8), (16384, 512, 16)])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_router_linear_gradients(tokens, hidden, experts, dtype):
    """The router's linear layer on large 16-bit batches: logits are torch's own, the weight gradient comes
    from the grouped TN kernel over equal pieces of the batch (router.py:96 and its autograd)."""
    from megablocks_amd.layers.arguments import Arguments
    from megablocks_amd.layers.router import LearnedRouter, _RouterLinear
    torch.manual_seed(tokens)
    args = Arguments(hidden_size=hidden, ffn_hidden_size=hidden, moe_num_experts=experts, moe_top_k=1, device='cuda',
                     bf16=dtype == torch.bfloat16, fp16=dtype == torch.float16)
    router = LearnedRouter(args)
    x = torch.randn(tokens, hidden, device='cuda', dtype=dtype, requires_grad=True)
    g = torch.randn(tokens, experts, device='cuda', dtype=dtype)
    assert tokens >= 4 * _RouterLinear.PIECE_ROWS
    logits = _RouterLinear.apply(x, router.layer.weight)
    assert torch.equal(logits, torch.nn.functional.linear(x, router.layer.weight))
    logits.backward(g)
    want_dw = g.float().t() @ x.detach().float()
    want_dx = g.float() @ router.layer.weight.detach().float()
    assert router.layer.weight.grad.dtype == dtype and router.layer.weight.grad.shape == (experts, hidden)
    assert rel_err(router.layer.weight.grad, want_dw) < 1e-2
    assert rel_err(x.grad, want_dx) < 1e-2
    sizes = _RouterLinear.piece_sizes(tokens)
    assert int(sizes.sum()) == tokens and sizes.shape[0] == min(64, tokens // 256) and int(sizes.max() - sizes.min()) <= 1


def _softmax_topk_reference(logits, top_k, norm_p):
    """router.py:87-106 with torch's own operations."""
    scores = logits.softmax(dim=-1)
    if top_k == 1:
        w, i = scores.max(dim=-1, keepdim=True)
    else:
        w, i = torch.topk(scores, top_k, dim=-1)
    if norm_p:
        w = w / torch.norm(w, p=norm_p, dim=-1, keepdim=True)
    return scores, w, i


@pytest.mark.parametrize('tokens,experts,top_k', [(1, 1, 1), (300, 8, 2), (257, 64, 1), (200, 65, 6), (100, 128, 8),
                                                  (50, 512, 64), (1000, 16, 4)])
@pytest.mark.parametrize('norm_p', [0, 1, 2, 3.0])
def test_router_softmax_topk_fp32_matches_oracle(tokens, experts, top_k, norm_p):
    import oracle
    from megablocks_amd.layers.router import _SoftmaxTopK
    torch.manual_seed(tokens + experts)
    logits = torch.randn(tokens, experts) * 3
    want_s, want_w, want_i = oracle.router_forward(logits, torch.eye(experts), top_k, norm_p or None)
    s, w, i, i32, _ = _SoftmaxTopK.apply(logits.cuda(), top_k, norm_p)
    assert i32.dtype == torch.int32 and torch.equal(i32.long(), i)
    assert s.dtype == torch.float32 and w.shape == (tokens, top_k) and i.dtype == torch.int64
    assert torch.allclose(s.cpu(), want_s, rtol=1e-5, atol=1e-7)
    assert torch.equal(i.cpu(), want_i)                      # fp32 scores of random logits have no ties
    assert torch.allclose(w.cpu(), want_w, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('tokens,experts,top_k,norm_p', [(4096, 8, 2, 1), (4096, 64, 1, 0), (2048, 64, 6, 1),
                                                         (1024, 200, 4, 2)])
def test_router_softmax_topk_16bit(dtype, tokens, experts, top_k, norm_p):
    """16-bit scores tie often: the selection is checked against the kernel's own scores (descending, equal
    scores in ascending expert index), the values against torch's operations in the same dtype."""
    from megablocks_amd.layers.router import _SoftmaxTopK
    torch.manual_seed(experts)
    logits = (torch.randn(tokens, experts, device='cuda') * 2).to(dtype)
    s, w, i, _, _ = _SoftmaxTopK.apply(logits, top_k, norm_p)
    ref_s, _, _ = _softmax_topk_reference(logits, top_k, norm_p)
    ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
    assert ((s.float() - ref_s.float()).abs() <= ulp * ref_s.float().abs() + 1e-30).all()   # at most one rounding step apart
    order = torch.sort(s.float().cpu(), dim=-1, descending=True, stable=True).indices[:, :top_k]
    assert torch.equal(i.cpu(), order)
    picked = s.gather(1, i)
    want_w = picked / torch.norm(picked, p=norm_p, dim=-1, keepdim=True) if norm_p else picked
    assert ((w.float() - want_w.float()).abs() <= ulp * want_w.float().abs()).all()


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('experts,top_k,norm_p,with_score_grad', [(8, 2, 1, False), (64, 1, 0, True), (64, 6, 1, True),
                                                                  (130, 4, 2, False), (16, 4, 3.0, True)])
def test_router_softmax_topk_backward(dtype, experts, top_k, norm_p, with_score_grad):
    from megablocks_amd.layers.router import _SoftmaxTopK
    tokens = 777
    torch.manual_seed(experts * top_k)
    logits = (torch.randn(tokens, experts, device='cuda') * 2).to(dtype)
    gw = torch.randn(tokens, top_k, device='cuda').to(dtype)
    gs = torch.randn(tokens, experts, device='cuda').to(dtype) if with_score_grad else None
    x = logits.clone().requires_grad_(True)
    s, w, i, _, _ = _SoftmaxTopK.apply(x, top_k, norm_p)
    loss = (w.float() * gw.float()).sum() + ((s.float() * gs.float()).sum() if with_score_grad else 0)
    loss.backward()
    # reference: autograd through torch's operations in fp32, with the kernel's selection
    xr = logits.float().clone().requires_grad_(True)
    sr = xr.softmax(dim=-1)
    wr = sr.gather(1, i)
    if norm_p:
        wr = wr / torch.norm(wr, p=norm_p, dim=-1, keepdim=True)
    ((wr * gw.float()).sum() + ((sr * gs.float()).sum() if with_score_grad else 0)).backward()
    assert x.grad.dtype == dtype
    assert rel_err(x.grad, xr.grad) < (1e-5 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('tokens,experts,top_k', [(777, 8, 2), (300, 64, 1), (100, 200, 4), (5, 1, 1)])
def test_router_logsumexp_for_the_zloss(dtype, tokens, experts, top_k):
    """The router kernel's optional fifth output: logsumexp(logits, dim=1) in fp32 (the term of router.py:37), against
    torch.logsumexp on the same logits in fp32, and its gradient through the kernel's backward together with a gradient
    of the weights, against autograd through torch's operations."""
    from megablocks_amd.layers.router import _SoftmaxTopK
    torch.manual_seed(tokens + experts)
    logits = (torch.randn(tokens, experts, device='cuda') * 4).to(dtype)
    logits[0] = 50.0 if dtype != torch.float16 else 9.0      # large equal logits: lse = value + log(experts)
    x = logits.clone().requires_grad_(True)
    s, w, i, _, lse = _SoftmaxTopK.apply(x, top_k, 0, True)
    assert lse.dtype == torch.float32 and lse.shape == (tokens,)
    want = torch.logsumexp(logits.float(), dim=1)
    assert torch.allclose(lse, want, rtol=1e-6, atol=1e-6)
    assert abs(float(lse[0].detach()) - (float(logits[0, 0]) + math.log(experts))) < 1e-4
    assert _SoftmaxTopK.apply(logits, top_k, 0)[4] is None
    gw = torch.randn(tokens, top_k, device='cuda')
    (lse.square().mean() * 3.0 + (w.float() * gw).sum()).backward()
    xr = logits.float().clone().requires_grad_(True)
    (torch.logsumexp(xr, dim=1).square().mean() * 3.0 + (xr.softmax(-1).gather(1, i) * gw).sum()).backward()
    assert rel_err(x.grad, xr.grad) < (1e-5 if dtype == torch.float32 else 1e-2)
    # -inf everywhere: -inf, as torch gives it
    dead = torch.full((2, experts), float('-inf'), device='cuda', dtype=dtype)
    assert bool((_SoftmaxTopK.apply(dead, top_k, 0, True)[4] == float('-inf')).all())


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_router_softmax_topk_with_nan_and_inf_logits(dtype):
    """A NaN or +inf logit makes its row of scores NaN (as torch's softmax does); torch.topk ranks NaN above every
    number and still returns expert indices.  The fused kernel does too: indices stay inside [0, E), distinct per
    token, and the other rows are untouched."""
    from megablocks_amd.layers.router import _SoftmaxTopK
    tokens, experts, top_k = 64, 8, 2
    torch.manual_seed(0)
    logits = torch.randn(tokens, experts, device='cuda').to(dtype)
    clean = _SoftmaxTopK.apply(logits, top_k, 1)
    bad = logits.clone()
    bad[3, 5] = float('nan')
    bad[10, 0] = float('inf')
    bad[20, :] = float('nan')
    s, w, i, i32, _ = _SoftmaxTopK.apply(bad, top_k, 1)
    assert torch.equal(i32.long(), i)
    assert int(i.min()) >= 0 and int(i.max()) < experts
    assert bool((i[:, 0] != i[:, 1]).all())
    ref_s = bad.float().softmax(-1)
    for t in (3, 10, 20):
        assert bool(torch.isnan(s[t]).all()) and bool(torch.isnan(ref_s[t]).all()) and bool(torch.isnan(w[t]).all())
        assert i[t].tolist() == [0, 1]                              # equal ranks are taken in ascending expert index
    keep = torch.ones(tokens, dtype=torch.bool, device='cuda')
    keep[[3, 10, 20]] = False
    for got, want in zip((s, w, i), clean):
        assert torch.equal(got[keep], want[keep])
    # downstream: every slot lands in a bin, so the permuted buffers have no unowned rows
    import megablocks_amd.ops as ops
    assert int(ops.histogram(i.flatten().int(), experts).sum()) == tokens * top_k


def test_router_falls_back_to_torch_for_many_experts():
    from megablocks_amd.layers.arguments import Arguments
    from megablocks_amd.layers.router import LearnedRouter
    args = Arguments(hidden_size=64, ffn_hidden_size=64, moe_num_experts=600, moe_top_k=2, device='cuda', bf16=True,
                     fp16=False, moe_normalize_expert_weights=1)
    router = LearnedRouter(args)
    x = torch.randn(33, 64, device='cuda', dtype=torch.bfloat16, requires_grad=True)
    scores, w, i = router(x)
    assert scores.shape == (33, 600) and w.shape == (33, 2) and i.dtype == torch.int64
    w.sum().backward()
    assert router.layer.weight.grad is not None and x.grad is not None


@pytest.mark.parametrize('name', ['c2', 'c3', 'c4', 'c5'])
def test_full_size_layer_properties(syn, monkeypatch, name):
    """The benchmark workloads at full size, through properties that do not need an oracle of that size:
    the backward is linear in the upstream gradient (doubling it doubles every gradient exactly: a power
    of two commutes with every rounding on the way), and sampled output rows equal the per-token definition
    sum_j w_j MLP_{e_j}(x_t) computed in fp32."""
    w = syn.WORKLOADS[name]
    inp = syn.make_inputs(w, seed=0)
    layer = syn.build_layer(w, inp)
    x = inp['x'].to(w.dtype).cuda().requires_grad_(True)
    grad = inp['grad'].to(w.dtype).cuda()
    routing_t = None
    if w.routing != 'router':
        routing_t = (inp['scores'].to(w.dtype).cuda(), inp['expert_weights'].to(w.dtype).cuda(), inp['top_experts'].cuda())
    params = [layer.experts.mlp.w1, layer.experts.mlp.w2] + ([layer.experts.mlp.v1] if w.mlp_type == 'glu' else [])
    if routing_t is None:
        params.append(layer.router.layer.weight)

    def grads(g):
        x.grad = None
        for p in params:
            p.grad = None
        out = syn.layer_step(layer, w, x, g, routing_t)
        return out.detach(), [x.grad.clone()] + [p.grad.clone() for p in params]

    out, g1 = grads(grad)
    out_again, g2 = grads(grad * 2)
    assert torch.equal(out, out_again)                                   # same kernels, same order: deterministic
    for a, b in zip(g1, g2):
        assert torch.isfinite(a).all() and torch.equal(a * 2, b)

    # the token gather as the operand load of the first product: the forward without gradients (where it is the
    # default) and the step with it switched on give the same bits
    from megablocks_amd import grouped_gemm_util as gg
    with torch.no_grad():
        assert torch.equal(layer(x) if routing_t is None else layer.experts(x, *routing_t), out)
    monkeypatch.setattr(gg, 'FUSED_GATHER', '1')
    out_fused, g_fused = grads(grad)
    monkeypatch.setattr(gg, 'FUSED_GATHER', 'auto')
    assert torch.equal(out_fused, out)
    for a, b in zip(g1, g_fused):
        assert torch.equal(a, b)

    # sampled rows against the definition
    with torch.no_grad():
        if routing_t is None:
            _, ew, te = layer.router(x)
        else:
            ew, te = routing_t[1], routing_t[2]
        ew, te = ew.view(-1, w.top_k).float(), te.view(-1, w.top_k)
        w1 = layer.experts.mlp.w1.view(w.experts, w.ffn, w.hidden)
        w2 = layer.experts.mlp.w2.view(w.experts, w.ffn, w.hidden)
        v1 = layer.experts.mlp.v1.view(w.experts, w.ffn, w.hidden) if w.mlp_type == 'glu' else None
        act = w.activation()
        rows = torch.randperm(w.tokens, generator=torch.Generator().manual_seed(1))[:48].tolist()
        want = torch.zeros(len(rows), w.hidden, device='cuda')
        for r, t in enumerate(rows):
            xt = x[t].float()
            for j in range(w.top_k):
                e = int(te[t, j])
                h = act(w1[e].float() @ xt)
                if v1 is not None:
                    h = h * (v1[e].float() @ xt)
                want[r] += ew[t, j] * (w2[e].float().t() @ h)
        assert rel_err(out[rows], want) < 2e-2

    # Reference values for the backward, in fp32 on the GPU from the definition (autograd): the weight gradients
    # of one expert that has tokens, and the input gradient of the sampled tokens (with the router's share where
    # the router is part of the step).
    g1 = dict(zip(['x', 'w1', 'w2'] + (['v1'] if v1 is not None else []) + (['router'] if routing_t is None else []), g1))
    flat_te = te.flatten()
    counts = torch.bincount(flat_te, minlength=w.experts)
    e = int(torch.nonzero(counts > 0).flatten()[w.experts // 2 % int((counts > 0).sum())])
    slots = torch.nonzero(flat_te == e).flatten()
    xe = x.detach()[slots // w.top_k].float()
    ge = grad[slots // w.top_k].float() * ew.flatten()[slots].unsqueeze(1)      # what reaches the expert's output rows
    pw = [w1[e].detach().float().requires_grad_(True), w2[e].detach().float().requires_grad_(True)]
    if v1 is not None:
        pw.append(v1[e].detach().float().requires_grad_(True))
    h = act(xe @ pw[0].t())
    if v1 is not None:
        h = h * (xe @ pw[2].t())
    ((h @ pw[1]) * ge).sum().backward()
    f0, f1 = e * w.ffn, (e + 1) * w.ffn
    assert rel_err(g1['w1'][f0:f1], pw[0].grad) < 1e-2
    assert rel_err(g1['w2'][f0:f1], pw[1].grad) < 1e-2
    if v1 is not None:
        assert rel_err(g1['v1'][f0:f1], pw[2].grad) < 1e-2

    xs = x.detach()[rows].float().requires_grad_(True)
    if routing_t is None:
        sc = (xs @ layer.router.layer.weight.detach().float().t()).softmax(-1)
        ws = sc.gather(1, te[rows])
        if w.normalize:
            ws = ws / torch.norm(ws, p=w.normalize, dim=-1, keepdim=True)
    else:
        ws = ew[rows]
    total = 0
    for r, t in enumerate(rows):
        for j in range(w.top_k):
            ex = int(te[t, j])
            hh = act(w1[ex].detach().float() @ xs[r])
            if v1 is not None:
                hh = hh * (v1[ex].detach().float() @ xs[r])
            total = total + ws[r, j] * ((w2[ex].detach().float().t() @ hh) * grad[t].float()).sum()
    total.backward()
    assert rel_err(g1['x'][rows], xs.grad) < 2e-2


def test_c1_full_size_fp32_vs_oracle(syn):
    """Workload c1 (4096 tokens, hidden 1024, ffn 4096, 8 experts, top-2, fp32) at full size against the CPU oracle:
    forward and every gradient, 1e-4."""
    w = syn.WORKLOADS['c1']
    inp = syn.make_inputs(w, seed=0)
    layer = syn.build_layer(w, inp)
    x = inp['x'].cuda().requires_grad_(True)
    with torch.no_grad():
        own_choice = layer.router(x)[2].cpu()
    want, want_tpe, want_grads, _ = _oracle_step(w, inp, False, own_choice)
    out = syn.layer_step(layer, w, x, inp['grad'].cuda(), None)
    theirs = oracle.router_forward(inp['x'], inp['router_weight'], w.top_k, w.normalize)[2]
    assert float((own_choice != theirs).float().mean()) < 1e-3      # fp32 on both sides: only exact near-ties may differ
    assert out.dtype == torch.float32 and rel_err(out, want) < 1e-4
    assert rel_err(x.grad, want_grads['x']) < 1e-4
    assert rel_err(layer.experts.mlp.w1.grad, want_grads['w1']) < 1e-4
    assert rel_err(layer.experts.mlp.w2.grad, want_grads['w2']) < 1e-4
    assert rel_err(layer.router.layer.weight.grad, want_grads['router']) < 5e-4


def test_routing_bookkeeping_is_bit_exact(syn):
    from megablocks_amd.layers.arguments import Arguments
    from megablocks_amd.layers.dmoe import ParallelDroplessMLP
    for experts, top_k, tokens in [(8, 2, 8192), (64, 1, 16384), (64, 6, 32768), (16, 4, 24576), (1, 1, 64)]:
        args = Arguments(hidden_size=128, ffn_hidden_size=128, moe_num_experts=experts, moe_top_k=top_k, bias=False,
                         fp16=False, bf16=True, device=torch.device('cuda'))
        pdm = ParallelDroplessMLP(args)
        top = torch.randint(0, experts, (tokens, top_k))
        if experts > 8:
            top[top == 3] = 4                                    # an expert with no tokens
        indices, bin_ids, bins, tpe = pdm.indices_and_bins(top.flatten().cuda())
        wi, wb, wbins, wtpe = oracle.indices_and_bins(top.flatten(), experts)
        assert torch.equal(indices.cpu(), wi) and torch.equal(bin_ids.cpu(), wb)
        assert torch.equal(bins.cpu(), wbins) and torch.equal(tpe.cpu(), wtpe)
        indices, bin_ids, bins, pbins, tpe = pdm.indices_and_padded_bins(top.flatten().cuda())
        oi, ob, obins, opbins, otpe = oracle.indices_and_padded_bins(top.flatten(), experts)
        assert torch.equal(indices.cpu(), oi) and torch.equal(pbins.cpu(), opbins) and torch.equal(bins.cpu(), obins)


def test_topology_metadata_matches_oracle():
    from megablocks_amd.layers.arguments import Arguments
    from megablocks_amd.layers.dmoe import ParallelDroplessMLP
    experts, ffn, tokens, top_k = 16, 1024, 4096, 4
    args = Arguments(hidden_size=256, ffn_hidden_size=ffn, moe_num_experts=experts, moe_top_k=top_k, bias=False,
                     mlp_impl='sparse', fp16=False, bf16=True, device=torch.device('cuda'))
    pdm = ParallelDroplessMLP(args)
    top = torch.randint(0, experts, (tokens * top_k,))
    _, _, _, pbins, _ = oracle.indices_and_padded_bins(top, experts)
    x = torch.empty(int(pbins[-1]), 256, device='cuda', dtype=torch.bfloat16)
    topo = pdm.topology(x, pbins.cuda())
    br, bpr = int(pbins[-1]) // 128, ffn // 128
    col = oracle.topology(pbins, 128, br, bpr)
    row = oracle.row_indices(br, bpr)
    col_t, off_t, boff_t = oracle.sparse_transpose((br * 128, ffn * experts), row, col, 128, pdm.transpose_sort_end_bit)
    assert topo.shape == (br * 128, ffn * experts)
    assert torch.equal(topo.column_indices.cpu(), col) and torch.equal(topo.row_indices.cpu(), row)
    assert torch.equal(topo.offsets.cpu(), torch.arange(0, br * bpr + 1, bpr, dtype=torch.int32))
    assert torch.equal(topo.column_indices_t.cpu(), col_t) and torch.equal(topo.offsets_t.cpu(), off_t)
    assert torch.equal(topo.block_offsets_t.cpu(), boff_t)


def _args(**kw):
    from megablocks_amd.layers.arguments import Arguments
    base = dict(hidden_size=128, ffn_hidden_size=256, moe_num_experts=1, moe_top_k=1, bias=False, fp16=False,
                bf16=True, device=torch.device('cuda'), moe_loss_weight=0.0)
    base.update(kw)
    return Arguments(**base)


@pytest.mark.parametrize('mlp_impl', ['grouped', 'sparse'])
@pytest.mark.parametrize('mlp_type', ['mlp', 'glu'])
def test_single_expert_dmoe_is_dense_ffn(mlp_impl, mlp_type):
    # tests/layers/dmoe_test.py:191-213 and glu_test.py:64-123
    from megablocks_amd.layers.dmoe import dMoE
    torch.manual_seed(42)
    layer = dMoE(_args(mlp_impl=mlp_impl, mlp_type=mlp_type))
    x = torch.randn(16, 8, 128, device='cuda').bfloat16()
    out = layer(x)
    m = layer.experts.mlp
    xf = x.view(-1, 128).float()
    h = F.gelu(xf @ m.w1.float().t(), approximate='tanh')
    if mlp_type == 'glu':
        h = h * (xf @ m.v1.float().t())
    want = h @ m.w2.float()
    assert out.shape == x.shape and rel_err(out.view(-1, 128), want) < 1e-2


@pytest.mark.parametrize('bs,sl,hs,ne,top_k', [(2, 64, 128, 1, 1), (2, 64, 128, 2, 1), (2, 64, 128, 4, 1),
                                              (2, 64, 128, 8, 1), (4, 32, 256, 4, 2), (4, 32, 256, 8, 4)])
@pytest.mark.parametrize('mlp_impl', ['grouped', 'sparse'])
def test_dmoe_equals_capacity_moe_without_dropping(bs, sl, hs, ne, top_k, mlp_impl):
    # tests/layers/dmoe_test.py:216-241: dMoE == MoE(capacity_factor=0) given the same weights
    from megablocks_amd.layers.dmoe import dMoE
    from megablocks_amd.layers.moe import MoE
    torch.manual_seed(42)
    kw = dict(hidden_size=hs, ffn_hidden_size=hs * 2, moe_num_experts=ne, moe_top_k=top_k, moe_capacity_factor=0)
    moe_layer, dmoe_layer = MoE(_args(**kw)), dMoE(_args(mlp_impl=mlp_impl, **kw))
    with torch.no_grad():
        moe_layer.router.layer.weight.copy_(dmoe_layer.router.layer.weight)
        w1 = dmoe_layer.experts.mlp.w1.view(ne, hs * 2, hs)
        moe_layer.experts.mlp.w1.copy_(w1.transpose(1, 2).contiguous())
        moe_layer.experts.mlp.w2.copy_(dmoe_layer.experts.mlp.w2.view(ne, hs * 2, hs))
    x = torch.randn(sl, bs, hs, device='cuda').bfloat16()
    assert rel_err(dmoe_layer(x), moe_layer(x)) < 1e-2


@pytest.mark.parametrize('bs,sl,hs', [(16, 1, 128), (1, 16, 128), (16, 16, 128), (8, 8, 256), (2, 256, 512)])
def test_single_expert_capacity_moe_is_dense_ffn(bs, sl, hs):
    # tests/layers/moe_test.py:155-199: forward, and the gradients of both weight matrices
    from megablocks_amd.layers.moe import MoE
    torch.manual_seed(42)
    layer = MoE(_args(hidden_size=hs, ffn_hidden_size=2 * hs, moe_capacity_factor=1))
    x = torch.randn(sl, bs, hs, device='cuda').bfloat16().requires_grad_(True)
    out = layer(x)
    out.sum().backward()
    m = layer.experts.mlp
    xf = x.detach().view(-1, hs).float().requires_grad_(True)
    w1, w2 = m.w1.detach().float().requires_grad_(True), m.w2.detach().float().requires_grad_(True)
    want = F.gelu(xf @ w1[0], approximate='tanh') @ w2[0]
    want.sum().backward()
    assert out.shape == x.shape and rel_err(out.view(-1, hs), want) < 1e-2
    assert rel_err(m.w1.grad, w1.grad) < 1e-2 and rel_err(m.w2.grad, w2.grad) < 1e-2
    assert rel_err(x.grad.view(-1, hs), xf.grad) < 1e-2


@pytest.mark.parametrize('tokens,hs,ne,top_k,capacity_factor', [(256, 128, 4, 1, 1.0), (512, 128, 8, 2, 0.5),
                                                                 (1024, 256, 16, 4, 1.0), (300, 64, 3, 2, 0.75)])
def test_capacity_moe_with_dropped_tokens_vs_oracle(tokens, hs, ne, top_k, capacity_factor):
    """moe.py:185-235 on the oracle's binned gather / scatter with fp32 expert products: tokens beyond an
    expert's capacity contribute nothing, the others their weighted expert output."""
    from megablocks_amd.layers.moe import MoE
    torch.manual_seed(tokens)
    layer = MoE(_args(hidden_size=hs, ffn_hidden_size=2 * hs, moe_num_experts=ne, moe_top_k=top_k,
                      moe_capacity_factor=capacity_factor))
    x = torch.randn(tokens, 1, hs, device='cuda').bfloat16()
    out = layer(x)
    with torch.no_grad():
        _, weights, top = layer.router(x)
    weights, top = weights.flatten().cpu(), top.flatten().cpu().int()
    indices, _, bins, tpe = oracle.indices_and_bins(top, ne)
    capacity = int(capacity_factor * top_k * tokens / ne)
    assert int(tpe.max()) > capacity                               # something is dropped
    xb = oracle.binned_gather(x.view(tokens, hs).cpu(), indices, None, bins, capacity, top_k).float()
    m = layer.experts.mlp
    h = F.gelu(torch.bmm(xb, m.w1.detach().float().cpu()), approximate='tanh')
    yb = torch.bmm(h, m.w2.detach().float().cpu())
    want = oracle.binned_scatter(yb, indices, weights.float(), bins, top_k)
    assert rel_err(out.view(tokens, hs), want) < 1e-2


@pytest.mark.parametrize('mlp_type,tokens,hs,ffn,ne,top_k,memory_optimized',
                         [('mlp', 2048, 1024, 4096, 64, 1, False), ('glu', 1024, 512, 1408, 8, 2, False),
                          ('glu', 1000, 256, 512, 4, 2, True)])
def test_dmoe_step_replays_from_a_captured_graph(mlp_type, tokens, hs, ffn, ne, top_k, memory_optimized):
    """The grouped dMoE step (forward + backward) has no host synchronisation and the library allocates
    nothing, so it can be captured once and replayed: every replay, with new inputs in the static buffers and
    eager work in between, gives bit for bit what the eager step gives."""
    from megablocks_amd.layers.dmoe import dMoE
    torch.manual_seed(tokens)
    layer = dMoE(_args(hidden_size=hs, ffn_hidden_size=ffn, moe_num_experts=ne, moe_top_k=top_k, mlp_type=mlp_type,
                       memory_optimized_mlp=memory_optimized, moe_normalize_expert_weights=1 if top_k > 1 else None))
    params = list(layer.parameters())
    xs = [torch.randn(tokens, 1, hs, device='cuda').bfloat16() for _ in range(3)]
    gs = [torch.randn(tokens, 1, hs, device='cuda').bfloat16() for _ in range(3)]

    def eager(x, g):
        layer.zero_grad(set_to_none=True)
        x = x.clone().requires_grad_(True)
        out = layer(x)
        out.backward(g)
        return [out.detach().clone(), x.grad.clone()] + [p.grad.clone() for p in params]

    want = [eager(x, g) for x, g in zip(xs, gs)]
    static_x, static_g = xs[0].clone().requires_grad_(True), gs[0].clone()
    layer.zero_grad(set_to_none=True)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = layer(static_x)
        static_out.backward(static_g)
    static_results = [static_out.detach(), static_x.grad] + [p.grad for p in params]
    for i in (1, 2, 0, 1, 2, 0):
        static_x.detach().copy_(xs[i])
        static_g.copy_(gs[i])
        for t in static_results:
            t.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip(static_results, want[i]):
            assert torch.equal(got, ref)
        eager(xs[(i + 1) % 3], gs[i])                               # eager work between the replays


@pytest.mark.parametrize('mlp_impl', ['grouped', 'sparse'])
@pytest.mark.parametrize('tokens', [0, 1])
def test_dmoe_with_no_tokens_and_with_one(mlp_impl, tokens):
    from megablocks_amd.layers.dmoe import dMoE
    layer = dMoE(_args(moe_num_experts=4, moe_top_k=2, mlp_impl=mlp_impl))
    x = torch.randn(tokens, 1, 128, device='cuda').bfloat16().requires_grad_(True)
    out = layer(x)
    out.sum().backward()
    assert out.shape == x.shape and x.grad.shape == x.shape
    assert all(p.grad is not None and p.grad.shape == p.shape for p in layer.parameters())
    if tokens == 0:
        assert all(torch.count_nonzero(p.grad) == 0 for p in layer.parameters())


@pytest.mark.parametrize('mlp_type,mlp_impl,memopt', [('mlp', 'grouped', False), ('mlp', 'grouped', True), ('mlp', 'sparse', False),
                                                      ('mlp', 'sparse', True), ('glu', 'grouped', False),
                                                      ('glu', 'grouped', True), ('glu', 'sparse', False)])
def test_autocast_with_fp32_parameters_equals_the_bf16_layer(mlp_type, mlp_impl, memopt):
    """fp32 master weights under torch.autocast(bf16): the products run on the bf16 casts, so the layer gives what
    the same layer with bf16 parameters gives, and its gradients arrive in fp32."""
    from megablocks_amd.layers.dmoe import dMoE
    torch.manual_seed(7)
    # every token takes all four experts: the fp32 scores of the autocast router and the bf16 scores of the bf16 layer
    # then pick the same experts (with fewer, near-ties fall differently and single tokens differ by whole experts)
    kw = dict(hidden_size=256, ffn_hidden_size=512, moe_num_experts=4, moe_top_k=4, mlp_type=mlp_type, mlp_impl=mlp_impl,
              memory_optimized_mlp=memopt)
    master = dMoE(_args(bf16=False, **kw))
    half = dMoE(_args(**kw))
    with torch.no_grad():
        for p16, p32 in zip(half.parameters(), master.parameters()):
            assert p32.dtype == torch.float32 and p16.dtype == torch.bfloat16
            p16.copy_(p32)
    x = torch.randn(512, 4, 256, device='cuda')          # 2048 tokens: the router's weight gradient takes the grouped kernel
    x32 = x.clone().requires_grad_(True)
    x16 = x.bfloat16().requires_grad_(True)
    grad = torch.randn(512, 4, 256, device='cuda').bfloat16()
    with torch.autocast('cuda', dtype=torch.bfloat16):
        scores, weights, _ = master.router(x32.detach().bfloat16())
        out = master(x32)
    out.backward(grad)
    want = half(x16)
    want.backward(grad)
    # autocast runs the router's softmax in fp32 (router.py:98 under torch.autocast), so scores and expert weights are
    # fp32 there and bf16 in the bf16 layer: equal up to that rounding, not bit for bit
    assert scores.dtype == torch.float32 and weights.dtype == torch.float32
    assert out.dtype == torch.bfloat16 and rel_err(out, want) < 1e-2
    assert x32.grad.dtype == torch.float32 and rel_err(x32.grad, x16.grad) < 1e-2
    for (name, p32), p16 in zip(master.named_parameters(), half.parameters()):
        assert p32.grad.dtype == torch.float32 and rel_err(p32.grad, p16.grad) < (2e-2 if 'router' in name else 1e-2), name
    # the forward without gradients (first product on the ungathered tokens, cast inside) and the step with the gather
    # fused: what the autocast step above gave
    from megablocks_amd import grouped_gemm_util as gg
    with torch.no_grad(), torch.autocast('cuda', dtype=torch.bfloat16):
        assert torch.equal(master(x32), out)
    grads = [x32.grad.clone()] + [p.grad.clone() for p in master.parameters()]
    x32.grad = None
    master.zero_grad(set_to_none=True)
    mode, gg.FUSED_GATHER = gg.FUSED_GATHER, '1'
    try:
        with torch.autocast('cuda', dtype=torch.bfloat16):
            fused = master(x32)
        fused.backward(grad)
    finally:
        gg.FUSED_GATHER = mode
    assert torch.equal(fused, out)
    for got, ref in zip([x32.grad] + [p.grad for p in master.parameters()], grads):
        assert got.dtype == ref.dtype and torch.equal(got, ref)


def test_parameter_names_and_shapes_are_the_reference_checkpoint_layout():
    """A state dict written by the reference's dMoE / MoE loads unchanged: `router.layer.weight [E, h]`,
    `experts.mlp.{w1, v1, w2} [E * ffn, h]` (mlp.py:315-330, glu.py:23-43), `experts.bias [h]` (moe.py:116-128); the
    capacity-factor MoE keeps `w1 [E, h, ffn]`, `w2 [E, ffn, h]` (mlp.py:99-116)."""
    from megablocks_amd.layers.dmoe import dMoE
    from megablocks_amd.layers.moe import MoE
    kw = dict(hidden_size=128, ffn_hidden_size=384, moe_num_experts=4, moe_top_k=2, bias=True)
    for mlp_impl in ('grouped', 'sparse'):
        shapes = {k: tuple(v.shape) for k, v in dMoE(_args(mlp_type='glu', mlp_impl=mlp_impl, **kw)).state_dict().items()}
        assert shapes == {'router.layer.weight': (4, 128), 'experts.bias': (128,), 'experts.mlp.w1': (4 * 384, 128),
                          'experts.mlp.w2': (4 * 384, 128), 'experts.mlp.v1': (4 * 384, 128)}
        shapes = {k: tuple(v.shape) for k, v in dMoE(_args(mlp_type='mlp', mlp_impl=mlp_impl, **kw)).state_dict().items()}
        assert shapes == {'router.layer.weight': (4, 128), 'experts.bias': (128,), 'experts.mlp.w1': (4 * 384, 128),
                          'experts.mlp.w2': (4 * 384, 128)}
    shapes = {k: tuple(v.shape) for k, v in MoE(_args(**kw)).state_dict().items()}
    assert shapes == {'router.layer.weight': (4, 128), 'experts.bias': (128,), 'experts.mlp.w1': (4, 128, 384),
                      'experts.mlp.w2': (4, 384, 128)}


def test_forward_shapes_bias_and_losses():
    # tests/layers/dmoe_test.py:103-188
    from megablocks_amd.layers import moe, router
    from megablocks_amd.layers.dmoe import dMoE
    args = _args(moe_num_experts=4, moe_top_k=2, bias=True, moe_loss_weight=0.1, moe_zloss_weight=1e-3)
    layer = dMoE(args)
    layer.train()
    x = torch.randn(8, 4, 128, device='cuda').bfloat16().requires_grad_(True)
    out, bias = layer(x)
    assert out.shape == x.shape and bias.shape == (128,)
    loss = out.sum() + moe.batched_load_balancing_loss(args) + router.batched_router_zloss(args).sum()
    loss.backward()
    assert x.grad is not None and layer.router.layer.weight.grad is not None
    assert all(p.grad is not None for p in layer.experts.mlp.parameters())
    moe.clear_load_balancing_loss()
    router.clear_router_zloss()
    layer2 = dMoE(dataclasses.replace(args, return_bias=False))
    assert layer2(x.detach()).shape == x.shape


@pytest.mark.parametrize('dtype,in_fp32', [(torch.float32, False), (torch.bfloat16, True), (torch.bfloat16, False)])
@pytest.mark.parametrize('tokens,hs,ne,top_k,layers', [(96, 128, 4, 2, 1), (2048, 256, 8, 2, 1), (300, 64, 16, 4, 2)])
def test_auxiliary_losses_match_oracle(dtype, in_fp32, tokens, hs, ne, top_k, layers):
    """batched_load_balancing_loss (moe.py:32-89), ParallelMLP.load_balancing_loss (moe.py:138-150) and
    batched_router_zloss (router.py:25-42): the values the layers report and the router weight gradient they
    produce, against the oracle fed with the same routing decision."""
    from megablocks_amd.layers import moe, router
    from megablocks_amd.layers.dmoe import dMoE
    torch.manual_seed(tokens + ne)
    lw, zw = 0.1, 1e-3
    args = _args(hidden_size=hs, ffn_hidden_size=2 * hs, moe_num_experts=ne, moe_top_k=top_k, moe_loss_weight=lw,
                 moe_zloss_weight=zw, num_layers=layers, bf16=dtype == torch.bfloat16, moe_lbl_in_fp32=in_fp32,
                 moe_zloss_in_fp32=in_fp32, moe_normalize_expert_weights=1 if top_k > 1 else None)
    moe.clear_load_balancing_loss()
    router.clear_router_zloss()
    models = [dMoE(args) for _ in range(layers)]
    for m in models:
        m.train()
    xs = [torch.randn(tokens, 1, hs, device='cuda').to(dtype) for _ in range(layers)]
    outs = [m(x) for m, x in zip(models, xs)]
    saved = moe.get_load_balancing_loss()
    assert len(saved) == layers and all(t.shape == (ne,) and sc.shape == (tokens, ne) for t, sc in saved)
    lbl = moe.batched_load_balancing_loss(args)
    zloss = router.batched_router_zloss(args)
    assert zloss.shape == (layers,)
    per_layer = models[0].experts.load_balancing_loss(saved[0][0], saved[0][1])
    (lbl + zloss.sum()).backward()

    # oracle: fp32 router on the same (rounded) inputs, counts from the layer's own expert choice
    rws = [m.router.layer.weight.detach().float().cpu().requires_grad_(True) for m in models]
    logits = [x.view(tokens, hs).float().cpu() @ rw.t() for x, rw in zip(xs, rws)]
    scores = [lg.softmax(-1) for lg in logits]
    counts = [t.cpu() for t, _ in saved]
    for c, sc, (_, got_sc) in zip(counts, scores, saved):
        assert int(c.sum()) == tokens * top_k
        assert rel_err(got_sc, sc) < (1e-5 if dtype == torch.float32 else 1e-2)
    want_lbl = oracle.load_balancing_loss(counts, scores, num_experts=ne, top_k=top_k, loss_weight=lw, num_layers=layers)
    want_z = oracle.router_zloss(logits, zloss_weight=zw)
    # 16-bit scores / logits reduced in 16 bits (the reference's default, moe_lbl_in_fp32 = moe_zloss_in_fp32 = False)
    # carry a few rounding steps of 2^-9 each
    tol = 1e-5 if dtype == torch.float32 else (1e-2 if in_fp32 else 3e-2)
    loss_dtype = torch.float32 if in_fp32 else dtype
    assert lbl.dtype == loss_dtype and abs(float(lbl) - float(want_lbl)) < tol * abs(float(want_lbl))
    assert zloss.dtype == loss_dtype and rel_err(zloss, want_z) < tol
    want_one = oracle.layer_load_balancing_loss(counts[0], scores[0], top_k=top_k)
    assert abs(float(per_layer) - float(want_one)) < tol * abs(float(want_one))
    (want_lbl + want_z.sum()).backward()
    for m, rw in zip(models, rws):
        # in 16 bits the gradient of the logits is a rounded difference of nearly equal terms (the softmax backward of
        # the almost uniform load-balancing gradient): a few percent, as with torch's own operations
        assert rel_err(m.router.layer.weight.grad, rw.grad) < (1e-4 if dtype == torch.float32 else 5e-2)
    del outs
    moe.clear_load_balancing_loss()
    router.clear_router_zloss()
    assert moe.get_load_balancing_loss() == [] and moe.batched_load_balancing_loss(_args(moe_loss_weight=0.0)) == 0.0


def test_load_balancing_loss_closed_forms_on_the_layer():
    """Evenly loaded experts give loss_weight whatever the scores (uniform_expert_assignment makes them even);
    the wrong number of saved layers raises as moe.py:42-60 does."""
    from megablocks_amd.layers import moe
    from megablocks_amd.layers.dmoe import dMoE
    moe.clear_load_balancing_loss()
    args = _args(moe_num_experts=8, moe_top_k=2, moe_loss_weight=0.25, uniform_expert_assignment=True)
    layer = dMoE(args)
    layer.train()
    layer(torch.randn(64, 4, 128, device='cuda').bfloat16())
    tpe, _ = moe.get_load_balancing_loss()[0]
    assert tpe.tolist() == [64] * 8
    assert abs(float(moe.batched_load_balancing_loss(args)) - 0.25) < 1e-3
    layer(torch.randn(64, 4, 128, device='cuda').bfloat16())
    with pytest.raises(ValueError):
        moe.batched_load_balancing_loss(args)          # two saved layers, num_layers = 1
    moe.clear_load_balancing_loss()
    layer.eval()
    layer(torch.randn(64, 4, 128, device='cuda').bfloat16())
    assert moe.get_load_balancing_loss() == []         # saved in training mode only (moe.py:430-431)


@pytest.mark.parametrize('mlp_impl', ['grouped', 'sparse'])
def test_uniform_expert_assignment_routes_round_robin(mlp_impl):
    """router.py:49-58,108-113: expert of slot i is i mod E (the weights stay the router's top-k scores); the layer
    output is the oracle's for that assignment."""
    from megablocks_amd.layers.dmoe import dMoE
    torch.manual_seed(11)
    tokens, hs, ne, top_k = 200, 128, 8, 2
    layer = dMoE(_args(hidden_size=hs, ffn_hidden_size=256, moe_num_experts=ne, moe_top_k=top_k, mlp_impl=mlp_impl,
                       uniform_expert_assignment=True))
    x = torch.randn(tokens, 1, hs, device='cuda').bfloat16()
    scores, weights, top = layer.router(x)
    assert top.dtype == torch.int64 and torch.equal(top.cpu(), oracle.uniform_expert_assignment((tokens, top_k), ne))
    assert torch.equal(weights, torch.topk(scores, top_k, dim=-1).values)
    out = layer(x)
    m = layer.experts.mlp
    want, tpe = oracle.dmoe_forward(x.view(tokens, hs).float().cpu(), weights.float().cpu(), top.cpu(),
                                    m.w1.detach().float().cpu(), m.w2.detach().float().cpu(), num_experts=ne, top_k=top_k)
    assert tpe.tolist() == [tokens * top_k // ne] * ne
    assert rel_err(out.view(tokens, hs), want) < 1e-2


def test_router_jitter():
    """router.py:81-85,93-94: in training mode the router input is multiplied element-wise by uniform noise from
    [1 - eps, 1 + eps); nothing is drawn in eval mode or when moe_jitter_eps is None."""
    from megablocks_amd.layers.router import LearnedRouter
    eps = 0.25
    args = _args(hidden_size=256, moe_num_experts=8, moe_top_k=2, moe_jitter_eps=eps, bf16=False)
    router = LearnedRouter(args)
    x = torch.randn(4096, 256, device='cuda')
    noise = router.jitter(x)
    assert noise.shape == x.shape and noise.dtype == x.dtype
    assert float(noise.min()) >= 1 - eps and float(noise.max()) <= 1 + eps
    assert abs(float(noise.mean()) - 1.0) < 2e-3 and abs(float(noise.std()) - 2 * eps / 12 ** 0.5) < 2e-3
    rw = router.layer.weight.detach().cpu()
    router.eval()
    s_eval, w_eval, i_eval = router(x)
    want_s, want_w, want_i = oracle.router_forward(x.cpu(), rw, 2)
    assert torch.allclose(s_eval.cpu(), want_s, rtol=1e-4, atol=1e-6) and torch.equal(i_eval.cpu(), want_i)
    router.train()
    torch.manual_seed(5)
    s_train, w_train, i_train = router(x)
    torch.manual_seed(5)
    jittered = x * router.jitter(x)                     # the same draw
    want_s, want_w, want_i = oracle.router_forward(jittered.cpu(), rw, 2)
    assert torch.allclose(s_train.cpu(), want_s, rtol=1e-4, atol=1e-6) and torch.equal(i_train.cpu(), want_i)
    assert torch.allclose(w_train.cpu(), want_w, rtol=1e-4, atol=1e-6)
    assert not torch.equal(s_train, s_eval)
    plain = LearnedRouter(_args(hidden_size=256, moe_num_experts=8, moe_jitter_eps=None)).train()
    state = torch.cuda.get_rng_state()
    plain(x.bfloat16())
    router.eval()(x)
    assert torch.equal(state, torch.cuda.get_rng_state())      # no draw without jitter


def test_memory_optimized_requires_all_grads():
    from megablocks_amd.layers.dmoe import dMoE
    layer = dMoE(_args(moe_num_experts=2, memory_optimized_mlp=True))
    x = torch.randn(4, 4, 128, device='cuda').bfloat16()     # x does not need grad
    with pytest.raises(ValueError):
        layer(x).sum().backward()


@pytest.mark.parametrize('mlp_type,mlp_impl', [('glu', 'grouped'), ('mlp', 'grouped'), ('glu', 'sparse'), ('mlp', 'sparse')])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_dmoe_with_the_gather_in_the_first_product(syn, monkeypatch, mlp_type, mlp_impl, dtype):
    """The layer with the token gather of dmoe.py:219 / :273 done by the operand loads of the experts' first product and,
    in the backward, of its weight gradients (gg.FUSED_GATHER).
    Output and every gradient must be the unfused layer's bit for bit (the same kernels on the same values), and the
    gather kernel must be gone from the forward."""
    from megablocks_amd import _lib
    from megablocks_amd import grouped_gemm_util as gg
    w = syn.Workload('t', 1500, 256, 768, 8, 2, mlp_type, mlp_impl, dtype, 'logits')
    inp = syn.make_inputs(w, seed=9)
    for k in ('x', 'grad', 'w1', 'v1', 'w2', 'expert_weights'):
        if inp[k] is not None:
            inp[k] = inp[k].to(dtype).float()
    oracle_out, _, oracle_grads, _ = _oracle_step(w, inp, True)
    layer = syn.build_layer(w, inp)
    routing = lambda ew: (inp['scores'].to(dtype).cuda(), ew, inp['top_experts'].cuda())
    grad = inp['grad'].to(dtype).cuda()

    def step(mode, with_grad):
        monkeypatch.setattr(gg, 'FUSED_GATHER', mode)
        layer.zero_grad(set_to_none=True)
        x = inp['x'].to(dtype).cuda().requires_grad_(with_grad)
        ew = inp['expert_weights'].to(dtype).cuda().requires_grad_(with_grad)
        _lib.profile_hook = []
        try:
            if with_grad:
                out = syn.layer_step(layer, w, x, grad, routing(ew))
            else:
                with torch.no_grad():
                    out = layer.experts(x, *routing(ew))
            torch.cuda.synchronize()
            launched = [name for name, *_ in _lib.profile_hook]
        finally:
            _lib.profile_hook = None
        mlp = layer.experts.mlp
        grads = [x.grad, ew.grad] + [getattr(mlp, n).grad for n in ('w1', 'v1', 'w2') if hasattr(mlp, n)] if with_grad else []
        return out.detach().clone(), [g.clone() for g in grads], launched

    first = 'gmm_nt_glu' if mlp_type == 'glu' else 'gmm_nt_act'
    want, _, launched = step('0', False)
    assert 'gather' in launched
    got, _, launched = step('auto', False)
    assert torch.equal(got, want) and 'gather' not in launched
    assert rel_err(got, oracle_out) < 1e-2                                    # the fused forward against the CPU oracle
    want, want_grads, launched = step('auto', True)        # top_k = 2 with gradients recorded: not fused by default
    assert launched.count('gather') == 1 and launched.index('gather') < launched.index(first)
    probe = torch.zeros(1, device='cuda', requires_grad=True)
    assert layer.experts._fuse_gather(probe, 4) and not layer.experts._fuse_gather(probe, 2)   # 'auto' with gradients
    assert layer.experts._fuse_gather(probe.detach(), 1) == (not any(p.requires_grad for p in layer.experts.mlp.parameters()))
    got, got_grads, launched = step('1', True)
    assert torch.equal(got, want)
    assert 'gather' not in launched                        # nor in the backward: the weight gradients read the tokens
    assert len(got_grads) == len(want_grads) >= 4
    for g, wg in zip(got_grads, want_grads):
        assert torch.equal(g, wg)
    # ... and the fused step against the oracle's forward and autograd
    assert rel_err(got, oracle_out) < 1e-2
    names = ['x', 'expert_weights', 'w1'] + (['v1'] if mlp_type == 'glu' else []) + ['w2']
    for name, g in zip(names, got_grads):
        assert rel_err(g, oracle_grads[name]) < 1e-2, name


@pytest.mark.parametrize('mlp_type', ['mlp', 'glu'])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('fused_gather', ['0', '1'])
def test_dmoe_with_the_combine_in_the_second_product(syn, monkeypatch, mlp_type, dtype, fused_gather):
    """One expert per token: the weighted combine of dmoe.py:280 written by the store phase of the experts' second
    product (gg.FUSED_COMBINE).  Output and every gradient -- the router weights' included, which the backward takes
    from the product the launch also keeps -- must be the unfused layer's bit for bit, the combine kernel must be gone
    from the forward, and the step must meet the oracle."""
    from megablocks_amd import _lib
    from megablocks_amd import grouped_gemm_util as gg
    w = syn.Workload('t', 1500, 256, 768, 8, 1, mlp_type, 'grouped', dtype, 'logits')
    inp = syn.make_inputs(w, seed=11)
    for k in ('x', 'grad', 'w1', 'v1', 'w2', 'expert_weights'):
        if inp[k] is not None:
            inp[k] = inp[k].to(dtype).float()
    oracle_out, _, oracle_grads, _ = _oracle_step(w, inp, True)
    layer = syn.build_layer(w, inp)
    routing = lambda ew: (inp['scores'].to(dtype).cuda(), ew, inp['top_experts'].cuda())
    grad = inp['grad'].to(dtype).cuda()
    monkeypatch.setattr(gg, 'FUSED_GATHER', fused_gather)
    monkeypatch.setattr(gg, 'GMM_WORKSPACE', False)   # no tail cut along K in the unfused second product: the combined launch has none

    def step(mode, with_grad):
        monkeypatch.setattr(gg, 'FUSED_COMBINE', mode)
        layer.zero_grad(set_to_none=True)
        x = inp['x'].to(dtype).cuda().requires_grad_(with_grad)
        ew = inp['expert_weights'].to(dtype).cuda().requires_grad_(with_grad)
        _lib.profile_hook = []
        try:
            if with_grad:
                out = syn.layer_step(layer, w, x, grad, routing(ew))
            else:
                with torch.no_grad():
                    out = layer.experts(x, *routing(ew))
            torch.cuda.synchronize()
            launched = [name for name, *_ in _lib.profile_hook]
        finally:
            _lib.profile_hook = None
        mlp = layer.experts.mlp
        grads = [x.grad, ew.grad] + [getattr(mlp, n).grad for n in ('w1', 'v1', 'w2') if hasattr(mlp, n)] if with_grad else []
        return out.detach().clone(), [g.clone() for g in grads], launched

    want, _, launched = step('0', False)
    assert 'scatter_weighted' in launched and 'gmm_nn_scatter' not in launched
    got, _, launched = step('auto', False)
    assert torch.equal(got, want) and 'scatter_weighted' not in launched and 'gmm_nn_scatter' in launched
    assert rel_err(got, oracle_out) < 1e-2
    want, want_grads, launched = step('0', True)
    assert 'scatter_weighted' in launched
    got, got_grads, launched = step('auto', True)
    assert torch.equal(got, want) and 'scatter_weighted' not in launched and launched.count('gmm_nn_scatter') == 1
    assert len(got_grads) == len(want_grads) >= 4
    for g, wg in zip(got_grads, want_grads):
        assert torch.equal(g, wg)
    assert rel_err(got, oracle_out) < 1e-2
    names = ['x', 'expert_weights', 'w1'] + (['v1'] if mlp_type == 'glu' else []) + ['w2']
    for name, g in zip(names, got_grads):
        assert rel_err(g, oracle_grads[name]) < 1e-2, name


@pytest.mark.parametrize('mlp_type,tokens,hs,ffn,ne,top_k', [('mlp', 2048, 1024, 1024, 64, 1), ('glu', 1024, 512, 1408, 8, 2)])
def test_dmoe_forward_replays_from_a_captured_graph(monkeypatch, mlp_type, tokens, hs, ffn, ne, top_k):
    """The forward pass without gradients, where the first product of the experts reads the ungathered tokens: captured
    once and replayed with new inputs and eager work in between, every replay gives bit for bit what the eager pass gives,
    fused or not."""
    from megablocks_amd import grouped_gemm_util as gg
    from megablocks_amd.layers.dmoe import dMoE
    torch.manual_seed(tokens + 1)
    layer = dMoE(_args(hidden_size=hs, ffn_hidden_size=ffn, moe_num_experts=ne, moe_top_k=top_k, mlp_type=mlp_type,
                       moe_normalize_expert_weights=1 if top_k > 1 else None))
    xs = [torch.randn(tokens, 1, hs, device='cuda').bfloat16() for _ in range(3)]
    with torch.no_grad():
        monkeypatch.setattr(gg, 'FUSED_GATHER', '0')
        want = [layer(x).clone() for x in xs]
        monkeypatch.setattr(gg, 'FUSED_GATHER', 'auto')
        for x, w in zip(xs, want):
            assert torch.equal(layer(x), w)
        static_x = xs[0].clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_out = layer(static_x)
        for i in (1, 2, 0, 1, 2, 0):
            static_x.copy_(xs[i])
            static_out.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_out, want[i])
            layer(xs[(i + 1) % 3])                                      # eager work between the replays


@pytest.mark.parametrize('mlp_type,mlp_impl', [('mlp', 'grouped'), ('glu', 'grouped'), ('mlp', 'sparse'), ('glu', 'sparse')])
@pytest.mark.parametrize('tokens', [0, 1, 3])
def test_dmoe_forward_without_gradients_on_no_tokens_and_on_a_few(monkeypatch, mlp_type, mlp_impl, tokens):
    """Empty and nearly empty batches through the forward whose first product gathers its own rows: most experts (all
    of them for an empty batch) have no rows, and the result is the unfused layer's."""
    from megablocks_amd import grouped_gemm_util as gg
    from megablocks_amd.layers.dmoe import dMoE
    torch.manual_seed(tokens)
    layer = dMoE(_args(moe_num_experts=4, moe_top_k=2, mlp_type=mlp_type, mlp_impl=mlp_impl))
    x = torch.randn(tokens, 1, 128, device='cuda').bfloat16()
    with torch.no_grad():
        monkeypatch.setattr(gg, 'FUSED_GATHER', '0')
        want = layer(x).clone()
        monkeypatch.setattr(gg, 'FUSED_GATHER', 'auto')
        got = layer(x)
    assert got.shape == x.shape and torch.equal(got, want)


@pytest.mark.parametrize('mlp_type', ['mlp', 'glu'])
def test_memory_optimized_dmoe_forward_without_gradients_gathers_in_the_first_product(syn, monkeypatch, mlp_type):
    """memory_optimized_mlp only changes what the backward keeps: without gradients the layer takes the same forward
    as the plain one, first product on the ungathered tokens included."""
    from megablocks_amd import _lib
    from megablocks_amd import grouped_gemm_util as gg
    w = syn.Workload('t', 1200, 256, 512, 8, 2, mlp_type, 'grouped', torch.bfloat16, 'logits')
    inp = syn.make_inputs(w, seed=4)
    plain, memopt = syn.build_layer(w, inp), syn.build_layer(w, inp, memory_optimized=True)
    x = inp['x'].bfloat16().cuda()
    routing = (inp['scores'].bfloat16().cuda(), inp['expert_weights'].bfloat16().cuda(), inp['top_experts'].cuda())
    with torch.no_grad():
        want = plain.experts(x, *routing)
        _lib.profile_hook = []
        try:
            got = memopt.experts(x, *routing)
            torch.cuda.synchronize()
            launched = [name for name, *_ in _lib.profile_hook]
        finally:
            _lib.profile_hook = None
    assert torch.equal(got, want) and 'gather' not in launched


def test_router_is_called_as_a_module(syn):
    """moe.py:468 calls `self.router(x)`: forward hooks on the router run, a hook may replace the routing, and a router
    that only defines forward() works.  The int32 indices the built-in router passes out of band are used only while
    the int64 tensor it returned is what arrives, unmodified."""
    from megablocks_amd.layers import router as router_mod
    w = syn.Workload('t', 512, 128, 256, 8, 2, 'mlp', 'grouped', torch.bfloat16, 'router', normalize=1)
    inp = syn.make_inputs(w, seed=13)
    layer = syn.build_layer(w, inp)
    x = inp['x'].bfloat16().cuda().view(w.tokens, 1, w.hidden)
    with torch.no_grad():
        base = layer(x)
        scores, weights, indices = layer.router(x)
        assert router_mod.int32_indices(indices).dtype == torch.int32
        assert torch.equal(router_mod.int32_indices(indices).long(), indices)
        seen = []
        handle = layer.router.register_forward_hook(lambda mod, args, out: seen.append(out[2].shape))
        assert torch.equal(layer(x), base) and seen == [indices.shape]
        handle.remove()
        # a hook that reroutes every token to experts (0, 1): the layer must follow the hook, not the stale int32 copy
        def reroute(mod, args, out):
            s, wgt, idx = out
            new = torch.zeros_like(idx)
            new[:, 1] = 1
            return s, wgt, new
        handle = layer.router.register_forward_hook(reroute)
        rerouted = layer(x)
        handle.remove()
        tpe_hooked = []
        orig = layer.experts.forward_fn
        def spy(xx, ew, te):
            out, tpe = orig(xx, ew, te)
            tpe_hooked.append(tpe.cpu())
            return out, tpe
        layer.experts.forward_fn = spy
        handle = layer.router.register_forward_hook(reroute)
        assert torch.equal(layer(x), rerouted)
        handle.remove()
        layer.experts.forward_fn = orig
        assert tpe_hooked[0].tolist() == [w.tokens, w.tokens] + [0] * (w.experts - 2)
        # in-place modification of the returned indices invalidates the attached copy
        scores, weights, indices = layer.router(x)
        indices.zero_()
        assert router_mod.int32_indices(indices) is indices

        class ForwardOnlyRouter(torch.nn.Module):
            def __init__(self, inner):
                super().__init__()
                self.layer = inner.layer
                self.inner = inner
            def forward(self, xx):
                s, wgt, idx = self.inner(xx)
                return s, wgt, idx.clone()
        layer.router = ForwardOnlyRouter(layer.router)
        assert torch.equal(layer(x), base)
