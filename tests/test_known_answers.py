"""Hand-derived known answers (tests/golden/known_answers.json) against both CPU oracles and, on a GPU, the
library.  These values were worked out on paper from the reference's documented semantics, independently of
any code in this repository."""
import json
import os

import pytest
import torch

import oracle

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'known_answers.json')) as f:
    KA = json.load(f)


def i32(v):
    return torch.tensor(v, dtype=torch.int32)


def _check_routing(mod, on_gpu):
    """`mod` offers sort / histogram / inclusive_cumsum / exclusive_cumsum / topology / replicate / round_up."""
    dev = (lambda t: t.cuda()) if on_gpu else (lambda t: t)
    back = lambda t: t.cpu()
    r = KA['route']
    te = dev(i32(r['top_expert']))
    bin_ids, indices = mod.sort(te, r['end_bit'])
    tpe = mod.histogram(te, r['num_experts'])
    bins = mod.inclusive_cumsum(tpe, 0)
    pbins = mod.inclusive_cumsum(mod.round_up(tpe, r['blocking']), 0)
    assert back(bin_ids).tolist() == r['bin_ids'] and back(indices).tolist() == r['indices']
    assert back(tpe).tolist() == r['tokens_per_expert']
    assert back(bins).view(-1).tolist() == r['bins'] and back(pbins).view(-1).tolist() == r['padded_bins']
    s = KA['sort_low_bit_only']
    k, p = mod.sort(dev(i32(s['x'])), s['end_bit'])
    assert back(k).tolist() == s['keys'] and back(p).tolist() == s['perm']
    s = KA['sort_signed_full_width']
    k, p = mod.sort(dev(torch.tensor(s['x'], dtype=torch.int16)), 16)
    assert back(k).tolist() == s['keys'] and back(p).tolist() == s['perm']
    h = KA['histogram']
    assert back(mod.histogram(dev(i32(h['x'])), h['num_bins'])).tolist() == h['out']
    c = KA['cumsum']
    assert back(mod.inclusive_cumsum(dev(i32(c['x'])), 1)).tolist() == c['inclusive']
    assert back(mod.exclusive_cumsum(dev(i32(c['x'])), 1)).tolist() == c['exclusive']
    t = KA['topology']
    assert back(mod.topology(dev(i32(t['padded_bins'])), t['block_size'], t['block_rows'], t['block_cols'])).tolist() == t['out']
    p = KA['replicate']
    assert back(mod.replicate(dev(i32(p['x'])), dev(i32(p['bins'])), p['num_outputs'])).tolist() == p['out']


def test_torch_oracle_routing():
    _check_routing(oracle, False)


def test_c_oracle():
    import shutil
    from oracle import routing_c as rc
    if not os.path.exists(rc.LIB_PATH) and shutil.which('gcc') is None:
        pytest.skip('oracle/liboracle_routing.so is not built and there is no gcc')
    r = KA['route']
    idx, ids, bins, pbins, tpe = rc.route(i32(r['top_expert']), r['num_experts'], r['end_bit'], r['blocking'])
    assert (idx.tolist(), ids.tolist(), bins.tolist(), pbins.tolist(), tpe.tolist()) == \
        (r['indices'], r['bin_ids'], r['bins'], r['padded_bins'], r['tokens_per_expert'])
    s = KA['sort_low_bit_only']
    k, p = rc.sort(i32(s['x']), s['end_bit'])
    assert k.tolist() == s['keys'] and p.tolist() == s['perm']
    s = KA['sort_signed_full_width']
    k, p = rc.sort(torch.tensor(s['x'], dtype=torch.int16), 16)
    assert k.tolist() == s['keys'] and p.tolist() == s['perm']
    h = KA['histogram']
    assert rc.histogram(i32(h['x']), h['num_bins']).tolist() == h['out']
    c = KA['cumsum']
    assert rc.cumsum(i32(c['x']), False).tolist() == c['inclusive'] and rc.cumsum(i32(c['x']), True).tolist() == c['exclusive']
    t = KA['topology']
    assert rc.topology(i32(t['padded_bins']), t['block_size'], t['block_rows'], t['block_cols']).tolist() == t['out']
    p = KA['replicate']
    assert rc.replicate(i32(p['x']), i32(p['bins']), p['num_outputs']).tolist() == p['out']


def _check_permute(k, on_gpu):
    """`k` offers gather / scatter / scatter_wgrad with the signatures of megablocks/backend/kernels.py."""
    dev = (lambda t: t.cuda()) if on_gpu else (lambda t: t)
    p = KA['permute']
    x = dev(torch.tensor(p['x']))
    indices, bin_ids, bins = dev(i32(p['indices'])), dev(i32(p['bin_ids'])), dev(i32(p['bins']))
    w = dev(torch.tensor(p['weights']))
    g = k.gather(x, indices, bin_ids, None, bins, p['top_k'])
    assert g.cpu().tolist() == p['gathered']
    assert k.scatter(g, indices, bin_ids, w, bins, p['top_k']).cpu().tolist() == p['scattered']
    assert k.scatter_wgrad(g, x, indices, bin_ids, bins, p['top_k']).cpu().tolist() == p['wgrad_with_grad_equal_to_x']


def _check_router(fn, on_gpu, ties_ascending):
    """`fn(logits, top_k, norm_p)` -> (scores, weights, indices) as LearnedRouter computes them after its linear layer.
    torch.topk leaves the order of equal scores open (the reference inherits that); the library takes them in
    ascending expert index (`ties_ascending`).  Otherwise the indices only have to point at the right scores."""
    r = KA['router']
    logits = torch.tensor(r['logits'])
    if on_gpu:
        logits = logits.cuda()
    close = lambda got, want: torch.allclose(got.cpu(), torch.tensor(want), rtol=1e-6, atol=1e-7)

    def check_indices(i, s, w_unnormalised, want):
        if ties_ascending:
            assert i.cpu().tolist() == want
        assert close(s.gather(1, i), w_unnormalised) and all(len(set(row)) == len(row) for row in i.cpu().tolist())

    s, w, i = fn(logits, 1, 0)
    assert close(s, r['scores']) and close(w, r['top1']['weights'])
    check_indices(i, s, r['top1']['weights'], r['top1']['indices'])
    s, w, i = fn(logits, 2, 0)
    assert close(s, r['scores']) and close(w, r['top2']['weights'])
    check_indices(i, s, r['top2']['weights'], r['top2']['indices'])
    assert i.cpu()[0].tolist() == r['top2']['indices'][0]                 # no tie in the first row
    assert close(fn(logits, 2, 1)[1], r['top2']['weights_p1']) and close(fn(logits, 2, 2)[1], r['top2']['weights_p2'])
    s, w, i = fn(logits, 3, 0)
    check_indices(i, s, [[0.5, 0.25, 0.125], [0.25, 0.25, 0.25]], r['top3_indices'])
    x = logits[1:2].clone().requires_grad_(True)
    _, w, i = fn(x, 1, 0)
    w.sum().backward()
    e = int(i[0, 0])
    want = [r['grad_logits_row1_top1_unit_grad'][0 if j == e else 1] for j in range(4)]   # by symmetry, whichever expert was taken
    assert close(x.grad[0], want)


def test_torch_oracle_router():
    _check_router(lambda logits, k, p: oracle.router_forward(logits, torch.eye(logits.shape[1]), k, p or None), False, False)


def test_torch_oracle_permute():
    _check_permute(oracle, False)


@pytest.mark.gpu
def test_library_routing():
    import megablocks_amd.ops as ops
    _check_routing(ops, True)


@pytest.mark.gpu
def test_library_permute():
    from megablocks_amd.backend import kernels
    _check_permute(kernels, True)


@pytest.mark.gpu
def test_library_router():
    from megablocks_amd.layers.router import _SoftmaxTopK
    _check_router(lambda logits, k, p: _SoftmaxTopK.apply(logits, k, p)[:3], True, True)
