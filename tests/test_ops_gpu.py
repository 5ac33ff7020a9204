"""GPU parity tests of the routing and permutation operators against the CPU oracle.

Shapes follow the reference's tests/ops/*_test.py.  Integer results, permutations and
unweighted copies must match bit for bit; weighted combines and dot products are held to
a relative Frobenius error of 1e-2 (and in practice match the oracle to rounding).
"""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def ops():
    import megablocks_amd.ops as ops
    return ops


@pytest.fixture(scope='module')
def kernels():
    from megablocks_amd.backend import kernels
    return kernels


def dev(t):
    return None if t is None else t.cuda()


def rel_err(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


# ------------------------------------------------------------------ histogram
@pytest.mark.parametrize('m,n', [(1, 32), (2, 32), (2, 1024), (16, 1024), (1, 16384), (3, 300000)])
@pytest.mark.parametrize('dtype', [torch.int16, torch.int32, torch.int64])
@pytest.mark.parametrize('max_val', [2, 8, 64, 128, 1000, 20000])
def test_histogram(ops, m, n, dtype, max_val):
    hi = min(max_val, 32000) if dtype == torch.int16 else max_val
    x = torch.randint(0, hi, (m, n)).to(dtype)
    got = ops.histogram(dev(x), max_val)
    assert got.dtype == torch.int32 and torch.equal(got.cpu(), oracle.histogram(x, max_val))
    got1 = ops.histogram(dev(x[0]), max_val)
    assert got1.shape == (max_val,) and torch.equal(got1.cpu(), oracle.histogram(x[0], max_val))


def test_histogram_ignores_out_of_range_and_empty(ops):
    x = torch.tensor([-1, 0, 3, 4, 7, 7, 100], dtype=torch.int32)
    assert ops.histogram(dev(x), 4).tolist() == [1, 0, 0, 1]
    assert ops.histogram(torch.empty(0, dtype=torch.int32).cuda(), 5).tolist() == [0] * 5
    assert ops.histogram(dev(x), 0).numel() == 0
    with pytest.raises(RuntimeError):
        ops.histogram(x.float().cuda(), 4)


# ------------------------------------------------------------------ sort
SORT_CASES = [(n, dt, mv) for n in (1, 7, 64, 2048, 2049, 16384, 200000)
              for dt in (torch.int16, torch.int32, torch.int64) for mv in (None, 2, 8, 128, 1024)]


@pytest.mark.parametrize('n,dtype,max_val', SORT_CASES)
def test_sort(ops, n, dtype, max_val):
    if dtype == torch.int16 and n > 32767:
        pytest.skip('an int16 payload cannot index this many elements')
    info = torch.iinfo(dtype)
    if max_val is None:
        x = torch.randint(info.min // 2, info.max // 2, (n,), dtype=torch.int64).to(dtype)
        end_bit = None
    else:
        x = torch.randint(0, max_val, (n,), dtype=torch.int64).to(dtype)
        end_bit = max(int(np.ceil(np.log2(max_val))), 1)
    keys, perm = ops.sort(dev(x), end_bit)
    want_keys, want_perm = oracle.sort(x, end_bit)
    assert keys.dtype == dtype and perm.dtype == dtype
    assert torch.equal(keys.cpu(), want_keys)
    assert torch.equal(perm.cpu(), want_perm)       # stable: ties in ascending original position


def test_sort_end_bit_ignores_high_bits(ops):
    x = torch.randint(0, 1 << 20, (5000,)).int()
    keys, perm = ops.sort(dev(x), 5)
    wk, wp = oracle.sort(x, 5)
    assert torch.equal(keys.cpu(), wk) and torch.equal(perm.cpu(), wp)
    k0, p0 = ops.sort(dev(x), 0)
    assert torch.equal(k0.cpu(), x) and torch.equal(p0.cpu(), torch.arange(5000, dtype=torch.int32))
    e = torch.empty(0, dtype=torch.int32).cuda()
    assert ops.sort(e)[0].numel() == 0


# ------------------------------------------------------------------ cumsum
@pytest.mark.parametrize('m,n', [(1, 1), (1, 8), (3, 64), (2, 257), (16, 1024), (2, 5000)])
@pytest.mark.parametrize('dtype', [torch.int16, torch.int32, torch.int64])
def test_cumsum(ops, m, n, dtype):
    x = torch.randint(0, 3, (m, n)).to(dtype)
    assert torch.equal(ops.inclusive_cumsum(dev(x), 1).cpu(), oracle.inclusive_cumsum(x, 1))
    assert torch.equal(ops.exclusive_cumsum(dev(x), 1).cpu(), oracle.exclusive_cumsum(x, 1))
    got = ops.inclusive_cumsum(dev(x[0]), 0)
    want = oracle.inclusive_cumsum(x[0], 0)
    assert got.shape == want.shape and torch.equal(got.cpu(), want)   # [1] -> 0-dim, like the reference
    with pytest.raises(RuntimeError):
        ops.inclusive_cumsum(dev(x), 0)


# ------------------------------------------------------------------ topology / replicate / round_up
@pytest.mark.parametrize('sl,hs,ne', [(1024, 1536, 2), (1024, 1536, 16), (16384, 768, 64), (16384, 768, 128),
                                      (8192, 4096, 512), (300, 256, 8)])
def test_topology(ops, sl, hs, ne):
    blocking = 128
    top = torch.randint(0, ne, (sl,)).int()
    tpe = oracle.histogram(top, ne)
    pbins = oracle.inclusive_cumsum(oracle.round_up(tpe, blocking), 0).view(-1)
    rows, cols = int(pbins[-1]) // blocking, hs // blocking
    got = ops.topology(dev(pbins), blocking, rows, cols)
    assert got.dtype == torch.int16 and torch.equal(got.cpu(), oracle.topology(pbins, blocking, rows, cols))
    assert torch.equal(ops.round_up(dev(tpe), blocking).cpu(), oracle.round_up(tpe, blocking))


@pytest.mark.parametrize('tokens,centers,top_k', [(8, 2, 1), (8, 2, 2), (64, 8, 4), (1024, 64, 2), (16384, 128, 8),
                                                  (16384, 2, 1)])
@pytest.mark.parametrize('dtype', [torch.float16, torch.int16, torch.int32])
def test_replicate(ops, tokens, centers, top_k, dtype):
    assign = torch.randint(0, centers, (tokens,)).int()
    tpe = oracle.histogram(assign, centers)
    bins = oracle.inclusive_cumsum(tpe, 0).view(-1)
    x = torch.randn(top_k, centers).half() if dtype == torch.float16 else torch.randint(-99, 99, (top_k, centers)).to(dtype)
    got = ops.replicate(dev(x), dev(bins), tokens)
    assert torch.equal(got.cpu(), oracle.replicate(x, bins, tokens))
    if dtype == torch.float16:
        from megablocks_amd.ops.routing import replicate_backward
        out = torch.empty_like(x).cuda()
        replicate_backward(got, dev(bins), out)
        want = x.float() * tpe.view(1, -1)
        assert torch.allclose(out.float().cpu(), want, rtol=1e-2, atol=1e-2)   # replicate_test.py:108
        xg = dev(x).requires_grad_(True)
        ops.replicate(xg, dev(bins), tokens).backward(torch.ones(top_k, tokens, dtype=dtype).cuda())
        assert torch.allclose(xg.grad.float().cpu(), tpe.float().expand(top_k, -1), rtol=1e-2)


# ------------------------------------------------------------------ gather / scatter
PERMUTE_CASES = [(4, 2, 2, 1), (4, 2, 2, 2), (1024, 1, 4, 1), (1024, 1, 64, 4), (1024, 1536, 4, 1), (1024, 1536, 64, 2),
                 (1024, 1536, 128, 4), (16384, 768, 4, 1), (16384, 768, 64, 2), (16384, 768, 128, 4), (16384, 1, 128, 2),
                 (2048, 4096, 8, 2), (777, 100, 5, 3)]


def _routing(sl, ne, top_k, seed=0):
    g = torch.Generator().manual_seed(seed)
    top = torch.randint(0, ne, (sl * top_k,), generator=g).int()
    bin_ids, indices = oracle.sort(top, max(int(np.ceil(np.log2(ne))), 1))
    tpe = oracle.histogram(top, ne)
    bins = oracle.inclusive_cumsum(tpe, 0).view(-1)
    pbins = oracle.inclusive_cumsum(oracle.round_up(tpe, 128), 0).view(-1)
    return indices, bin_ids, bins, pbins


@pytest.mark.parametrize('sl,hs,ne,top_k', PERMUTE_CASES)
@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16, torch.float32])
def test_gather_and_padded_gather(kernels, sl, hs, ne, top_k, dtype):
    indices, bin_ids, bins, pbins = _routing(sl, ne, top_k)
    x = torch.randn(sl, hs).to(dtype)
    w = torch.rand(sl * top_k).to(dtype)
    args = [dev(t) for t in (indices, bin_ids)]
    got = kernels.gather(dev(x), *args, None, dev(bins), top_k)
    assert torch.equal(got.cpu(), oracle.gather(x, indices, bin_ids, None, bins, top_k))
    got = kernels.padded_gather(dev(x), *args, None, dev(bins), dev(pbins), top_k)
    assert torch.equal(got.cpu(), oracle.padded_gather(x, indices, bin_ids, None, bins, pbins, top_k))
    got = kernels.gather(dev(x), *args, dev(w), dev(bins), top_k)
    assert torch.equal(got.cpu(), oracle.gather(x, indices, bin_ids, w, bins, top_k))   # one rounding, same as oracle
    got = kernels.padded_gather(dev(x), *args, dev(w), dev(bins), dev(pbins), top_k)
    assert torch.equal(got.cpu(), oracle.padded_gather(x, indices, bin_ids, w, bins, pbins, top_k))


@pytest.mark.parametrize('sl,hs,ne,top_k', PERMUTE_CASES)
@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16, torch.float32])
def test_scatter_and_padded_scatter(kernels, sl, hs, ne, top_k, dtype):
    indices, bin_ids, bins, pbins = _routing(sl, ne, top_k, seed=1)
    xt = torch.randn(sl, hs).to(dtype)
    w = torch.rand(sl * top_k).to(dtype)
    args = [dev(t) for t in (indices, bin_ids)]
    x = oracle.gather(xt, indices, bin_ids, None, bins, top_k)
    xp = oracle.padded_gather(xt, indices, bin_ids, None, bins, pbins, top_k)
    for weights in (None, w):
        got = kernels.scatter(dev(x), *args, dev(weights), dev(bins), top_k)
        want = oracle.scatter(x, indices, bin_ids, weights, bins, top_k)
        got_p = kernels.padded_scatter(dev(xp), *args, dev(weights), dev(bins), dev(pbins), top_k)
        want_p = oracle.padded_scatter(xp, indices, bin_ids, weights, bins, pbins, top_k)
        if top_k <= 2:          # one rounding per product and at most one add: bit-exact
            assert torch.equal(got.cpu(), want) and torch.equal(got_p.cpu(), want_p)
        else:                   # fp32 sum order over top_k may differ from torch's reduction
            assert rel_err(got, want) < 1e-2 and rel_err(got_p, want_p) < 1e-2
            assert torch.allclose(got.float().cpu(), want.float(), rtol=5e-3, atol=5e-3)
    if top_k == 1:              # unweighted round trip is the identity, bit for bit
        back = kernels.scatter(kernels.gather(dev(xt), *args, None, dev(bins), 1), *args, None, dev(bins), 1)
        assert torch.equal(back.cpu(), xt)


@pytest.mark.parametrize('sl,hs,ne,top_k', PERMUTE_CASES)
@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16, torch.float32])
def test_scatter_wgrad(kernels, sl, hs, ne, top_k, dtype):
    indices, bin_ids, bins, pbins = _routing(sl, ne, top_k, seed=2)
    xt = torch.randn(sl, hs).to(dtype)
    grad = torch.randn(sl, hs).to(dtype)
    args = [dev(t) for t in (indices, bin_ids)]
    x = oracle.gather(xt, indices, bin_ids, None, bins, top_k)
    xp = oracle.padded_gather(xt, indices, bin_ids, None, bins, pbins, top_k)
    got = kernels.scatter_wgrad(dev(x), dev(grad), *args, dev(bins), top_k)
    want = oracle.scatter_wgrad(x, grad, indices, bin_ids, bins, top_k)
    assert rel_err(got, want) < 1e-2
    got = kernels.padded_scatter_wgrad(dev(xp), dev(grad), *args, dev(bins), dev(pbins), top_k)
    want = oracle.padded_scatter_wgrad(xp, grad, indices, bin_ids, bins, pbins, top_k)
    assert rel_err(got, want) < 1e-2


@pytest.mark.parametrize('sl,hs,ne,top_k', [(4, 2, 2, 1), (1024, 1536, 4, 2), (1024, 1536, 64, 4), (16384, 768, 128, 1),
                                            (16384, 768, 4, 4), (1000, 50, 7, 2)])
@pytest.mark.parametrize('cap_factor', [0.5, 1.0, 2.0])
@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16, torch.float32])
def test_binned_ops(kernels, sl, hs, ne, top_k, cap_factor, dtype):
    indices, bin_ids, bins, pbins = _routing(sl, ne, top_k, seed=3)
    cap = max(int(cap_factor * sl * top_k / ne), 1)
    xt = torch.randn(sl, hs).to(dtype)
    w = torch.rand(sl * top_k).to(dtype)
    grad = torch.randn(sl, hs).to(dtype)
    got = kernels.binned_gather(dev(xt), dev(indices), None, dev(bins), cap, top_k)
    want = oracle.binned_gather(xt, indices, None, bins, cap, top_k)
    assert torch.equal(got.cpu(), want)
    got_w = kernels.binned_gather(dev(xt), dev(indices), dev(w), dev(bins), cap, top_k)
    assert torch.equal(got_w.cpu(), oracle.binned_gather(xt, indices, w, bins, cap, top_k))
    sc = kernels.binned_scatter(got, dev(indices), dev(w), dev(bins), top_k)
    want_sc = oracle.binned_scatter(want, indices, w, bins, top_k)
    # one rounding step of the storage type per addend (bf16: 2^-8) on sums of up to top_k products below one
    step = {torch.float16: 5e-3, torch.bfloat16: 4e-2, torch.float32: 1e-5}[dtype]
    assert rel_err(sc, want_sc) < 1e-2 and torch.allclose(sc.float().cpu(), want_sc.float(), rtol=step, atol=step)
    wg = kernels.binned_scatter_wgrad(got, dev(grad), dev(indices), dev(bins), top_k)
    assert rel_err(wg, oracle.binned_scatter_wgrad(want, grad, indices, bins, top_k)) < 1e-2


def test_shape_errors_are_value_errors(kernels):
    x = torch.randn(4, 8).cuda()
    idx = torch.zeros(4, dtype=torch.int32).cuda()
    bins = torch.tensor([4], dtype=torch.int32).cuda()
    with pytest.raises(ValueError):
        kernels.gather(x.view(-1), idx, idx, None, bins, 1)          # not a matrix
    with pytest.raises(ValueError):
        kernels.gather(x, idx[:3], idx, None, bins, 1)                # tokens * top_k mismatch
    with pytest.raises(ValueError):
        kernels.padded_gather(x, idx, idx, None, bins, torch.cat([bins, bins]), 1)
    with pytest.raises(ValueError):
        kernels.binned_scatter(x, idx, None, bins, 1)                 # needs a 3-tensor


# ------------------------------------------------------------------ autograd pairing
def test_autograd_pairing_matches_oracle_autograd(ops):
    sl, hs, ne, top_k = 512, 256, 8, 2
    indices, bin_ids, bins, pbins = _routing(sl, ne, top_k, seed=4)
    x = torch.randn(sl, hs)
    w = torch.rand(sl * top_k)
    gout = torch.randn(sl, hs)
    # oracle: differentiable formulation on the CPU in fp32
    xo, wo = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    tok = indices.long() // top_k
    y = xo.index_select(0, tok) * 2.0
    out = torch.zeros(sl, hs).index_add(0, tok, y * wo[indices.long()].unsqueeze(1))
    out.backward(gout)
    for padded in (False, True):
        xg, wg = dev(x).requires_grad_(True), dev(w).requires_grad_(True)
        i, b, bn, pb = dev(indices), dev(bin_ids), dev(bins), dev(pbins)
        if padded:
            yg = ops.padded_gather(xg, i, b, bn, pb, top_k) * 2.0
            og = ops.padded_scatter(yg, i, b, wg, bn, pb, top_k)
        else:
            yg = ops.gather(xg, i, b, bn, top_k) * 2.0
            og = ops.scatter(yg, i, b, wg, bn, top_k)
        og.backward(dev(gout))
        assert rel_err(og, out) < 1e-5 and rel_err(xg.grad, xo.grad) < 1e-5 and rel_err(wg.grad, wo.grad) < 1e-5


def test_full_size_round_trip_properties(ops):
    # Mixtral-shaped permutation at full size, checked through size-independent properties
    T, h, E, k = 8192, 4096, 8, 2
    x = torch.randn(T, h, device='cuda').bfloat16()
    top = torch.randint(0, E, (T * k,), device='cuda').int()
    bin_ids, indices = ops.sort(top, 3)
    tpe = ops.histogram(top, E)
    bins = ops.inclusive_cumsum(tpe, 0)
    assert int(tpe.sum()) == T * k and int(bins[-1]) == T * k
    assert bool((bin_ids[1:] >= bin_ids[:-1]).all())                               # sortedness
    assert torch.equal(torch.sort(indices.long())[0], torch.arange(T * k, device='cuda'))  # a permutation
    assert torch.equal(top[indices.long()], bin_ids)
    g = ops.gather(x, indices, bin_ids, bins, k)
    assert torch.equal(g, x[indices.long() // k])                                  # bit-exact copy
    half = torch.full((T * k,), 0.5, device='cuda').bfloat16()
    back = ops.scatter(g, indices, bin_ids, half, bins, k)                         # 0.5 x + 0.5 x == x exactly
    assert torch.equal(back, x)


def test_empty_and_degenerate_inputs(ops, kernels):
    """No tokens, no capacity, one column: shapes as the reference's wrappers give them, nothing launched wrongly."""
    from megablocks_amd import grouped_gemm_util as gg
    none = dev(torch.empty(0, dtype=torch.int32))
    bins = dev(torch.zeros(4, dtype=torch.int32))
    x = dev(torch.empty(0, 64).bfloat16())
    assert ops.gather(x, none, none, bins, 1).shape == (0, 64)
    assert ops.scatter(x, none, none, None, bins, 1).shape == (0, 64)
    assert ops.padded_gather(x, none, none, bins, bins, 1).shape == (0, 64)
    assert ops.padded_scatter(x, none, none, None, bins, bins, 1).shape == (0, 64)
    full = ops.binned_gather(x, none, bins, 8, 1)
    assert full.shape == (4, 8, 64) and torch.count_nonzero(full) == 0
    assert ops.binned_scatter(dev(torch.empty(4, 0, 64).bfloat16()), none, None, bins, 1).shape == (0, 64)
    assert kernels.scatter_wgrad(x, x, none, none, bins, 1).shape == (0,)
    assert ops.inclusive_cumsum(dev(torch.empty(3, 0, dtype=torch.int32)), 1).shape == (3, 0)
    assert ops.inclusive_cumsum(dev(torch.tensor([5], dtype=torch.int32)), 0).shape == ()     # the squeeze of ops/cumsum.py:24-48
    assert ops.replicate(dev(torch.tensor([[1, 2]], dtype=torch.int32)), dev(torch.tensor([0, 0], dtype=torch.int32)), 0).shape == (1, 0)
    assert ops.topology(dev(torch.tensor([0, 0], dtype=torch.int32)), 128, 0, 4).shape == (0,)
    one_col = dev(torch.tensor([[1.], [2.], [3.]]).bfloat16())
    got = ops.gather(one_col, dev(torch.tensor([2, 0, 1], dtype=torch.int32)), dev(torch.tensor([0, 0, 1], dtype=torch.int32)),
                     dev(torch.tensor([2, 3], dtype=torch.int32)), 1)
    assert got.view(-1).tolist() == [3.0, 1.0, 2.0]
    sizes = torch.tensor([0, 0])
    w = dev(torch.randn(2, 64, 32).bfloat16())
    assert gg.backend.gmm(x, w, sizes).shape == (0, 32)
    dw = gg.backend.gmm(x, dev(torch.empty(0, 32).bfloat16()), sizes, trans_a=True)
    assert dw.shape == (2, 64, 32) and torch.count_nonzero(dw) == 0                       # no rows: zero gradients
    no_k = gg.backend.gmm(dev(torch.empty(8, 0).bfloat16()), dev(torch.empty(2, 0, 32).bfloat16()), torch.tensor([4, 4]))
    assert no_k.shape == (8, 32) and torch.count_nonzero(no_k) == 0                       # empty reduction: zeros


@pytest.mark.parametrize('padded', [False, True])
def test_c_abi_gather_and_scatter_without_a_prebuilt_map(kernels, padded):
    """mbx_gather with slot_rows = NULL copies by output row, mbx_scatter with slot_rows = NULL builds the map in
    the caller's scratch: same results as the calls the Python wrappers make (with the shared map)."""
    from megablocks_amd import _lib
    lib = _lib.lib
    sl, hs, ne, top_k = 1000, 256, 16, 4
    indices, bin_ids, bins, pbins = (dev(t) for t in _routing(sl, ne, top_k, seed=5))
    x = dev(torch.randn(sl, hs).bfloat16())
    w = dev(torch.rand(sl * top_k).bfloat16())
    pb = pbins if padded else None
    rows = int(pbins[-1]) if padded else sl * top_k
    want = kernels.padded_gather(x, indices, bin_ids, w, bins, pbins, top_k) if padded else \
        kernels.gather(x, indices, bin_ids, w, bins, top_k)
    got = torch.full((rows, hs), 7.0, device='cuda').bfloat16()
    _lib.check(lib.mbx_gather(_lib.ptr(x), _lib.dtype_of(x), sl, hs, top_k, _lib.ptr(indices), _lib.ptr(bins), _lib.ptr(pb),
                              ne, _lib.ptr(w), _lib.dtype_of(w), _lib.ptr(got), rows, None, _lib.stream()), 'gather')
    assert torch.equal(got, want)
    want_back = kernels.padded_scatter(want, indices, bin_ids, w, bins, pbins, top_k) if padded else \
        kernels.scatter(want, indices, bin_ids, w, bins, top_k)
    back = torch.full((sl, hs), 7.0, device='cuda').bfloat16()
    scratch = torch.empty(sl * top_k, dtype=torch.int32, device='cuda')
    args = (_lib.ptr(want), _lib.dtype_of(x), sl, hs, top_k, _lib.ptr(indices), _lib.ptr(bin_ids), _lib.ptr(bins), _lib.ptr(pb),
            ne, _lib.ptr(w), _lib.dtype_of(w), _lib.ptr(back), None)
    _lib.check(lib.mbx_scatter(*args, _lib.ptr(scratch), scratch.numel() * 4, _lib.stream()), 'scatter')
    assert torch.equal(back, want_back)
    assert lib.mbx_scatter(*args, None, 0, _lib.stream()) == -2                      # neither a map nor scratch


@pytest.mark.parametrize('sl,hs,ne,top_k', [(1024, 256, 8, 1), (1000, 4096, 8, 2), (777, 264, 5, 3), (2048, 2048, 64, 6),
                                            (512, 1024, 16, 8), (300, 100, 4, 2), (256, 128, 32, 9)])
@pytest.mark.parametrize('padded', [False, True])
def test_scatter_backward_in_one_pass_equals_the_two_kernels(kernels, sl, hs, ne, top_k, padded):
    """mbx_scatter_backward against mbx_gather (weighted) + mbx_scatter_wgrad: the same values bit for bit, padding
    rows zero; shapes it does not take (rows that are not 16-byte multiples, top_k above 8) fall back to the two."""
    from megablocks_amd import _lib
    indices, bin_ids, bins, pbins = (dev(t) for t in _routing(sl, ne, top_k, seed=9))
    grad = dev(torch.randn(sl, hs).bfloat16())
    w = dev(torch.rand(sl * top_k).bfloat16())
    if padded:
        x = kernels.padded_gather(dev(torch.randn(sl, hs).bfloat16()), indices, bin_ids, None, bins, pbins, top_k)
        want = (kernels.padded_gather(grad, indices, bin_ids, w, bins, pbins, top_k),
                kernels.padded_scatter_wgrad(x, grad, indices, bin_ids, bins, pbins, top_k))
    else:
        x = kernels.gather(dev(torch.randn(sl, hs).bfloat16()), indices, bin_ids, None, bins, top_k)
        want = (kernels.gather(grad, indices, bin_ids, w, bins, top_k),
                kernels.scatter_wgrad(x, grad, indices, bin_ids, bins, top_k))
    _lib.profile_hook = []
    try:
        got = kernels.scatter_backward(x, grad, indices, bin_ids, w, bins, pbins if padded else None, top_k)
        names = [r[0] for r in _lib.profile_hook]
    finally:
        _lib.profile_hook = None
    one_pass = hs % 8 == 0 and top_k <= 8
    assert names == (['scatter_backward'] if one_pass else ['gather_weighted', 'scatter_wgrad'])
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])


def test_slot_row_map_is_rebuilt_when_the_routing_changes(kernels):
    """The map the wrappers keep on `indices` is reused only for the same, unmodified indices / bins / padded_bins."""
    sl, hs, ne, top_k = 512, 128, 8, 2
    x = torch.randn(sl, hs).bfloat16()
    ia, ba, bina, pba = _routing(sl, ne, top_k, seed=11)
    ib, bb, binb, pbb = _routing(sl, ne, top_k, seed=12)
    indices, bin_ids, bins, pbins = dev(ia), dev(ba), dev(bina), dev(pba)
    got = kernels.gather(dev(x), indices, bin_ids, None, bins, top_k)
    assert torch.equal(got.cpu(), oracle.gather(x, ia, ba, None, bina, top_k))
    first = indices._mbx_slot_rows[1]
    kernels.scatter(got, indices, bin_ids, None, bins, top_k)
    assert indices._mbx_slot_rows[1] is first                                    # same routing: the map is reused
    got = kernels.padded_gather(dev(x), indices, bin_ids, None, bins, pbins, top_k)     # other layout, same indices
    assert torch.equal(got.cpu(), oracle.padded_gather(x, ia, ba, None, bina, pba, top_k))
    indices.copy_(dev(ib)); bin_ids.copy_(dev(bb)); bins.copy_(dev(binb)); pbins.copy_(dev(pbb))   # new routing in place
    got = kernels.padded_gather(dev(x), indices, bin_ids, None, bins, pbins, top_k)
    assert torch.equal(got.cpu(), oracle.padded_gather(x, ib, bb, None, binb, pbb, top_k))
    got = kernels.gather(dev(x), indices, bin_ids, None, bins, top_k)
    assert torch.equal(got.cpu(), oracle.gather(x, ib, bb, None, binb, top_k))
    w = torch.rand(sl * top_k).bfloat16()
    back = kernels.scatter(got, indices, bin_ids, dev(w), bins, top_k)
    assert torch.equal(back.cpu(), oracle.scatter(got.cpu(), ib, bb, w, binb, top_k))


def test_permutation_of_more_than_4GiB(ops):
    """Routed rows of 2.5e9 elements (4.9 GB in bf16): element offsets pass 2^31, byte offsets 2^32.  Same
    size-independent properties, plus the padded forms and the weight gradient on a slice."""
    T, h, E, k = 300000, 2048, 16, 4
    x = torch.empty(T, h, device='cuda', dtype=torch.bfloat16).normal_()
    top = torch.randint(0, E, (T * k,), device='cuda').int()
    bin_ids, indices = ops.sort(top, 4)
    tpe = ops.histogram(top, E)
    bins = ops.inclusive_cumsum(tpe, 0)
    pbins = ops.inclusive_cumsum(ops.round_up(tpe, 128), 0)
    rows = indices.long() // k
    g = ops.gather(x, indices, bin_ids, bins, k)
    assert g.numel() > 2 ** 31
    for lo in range(0, T * k, 200000):                                             # piecewise: no second 4.9 GB copy
        assert torch.equal(g[lo:lo + 200000], x[rows[lo:lo + 200000]])
    half = torch.full((T * k,), 0.25, device='cuda').bfloat16()
    assert torch.equal(ops.scatter(g, indices, bin_ids, half, bins, k), x)         # 4 x 0.25 x == x exactly
    del g
    gp = ops.padded_gather(x, indices, bin_ids, bins, pbins, k)
    assert gp.shape[0] == int(pbins[-1])
    assert torch.equal(ops.padded_scatter(gp, indices, bin_ids, half, bins, pbins, k), x)
    # the last expert's rows sit past the 2^32-byte mark; padding rows are zero
    first, last, end = int(pbins[-2]), int(pbins[-2]) + int(tpe[-1]), int(pbins[-1])
    assert torch.equal(gp[first:last], x[rows[int(bins[-2]):]]) and torch.count_nonzero(gp[last:end]) == 0
    from megablocks_amd.backend import kernels
    wgrad = kernels.padded_scatter_wgrad(gp, x, indices, bin_ids, bins, pbins, k)   # <x_t, x_t> for every slot
    want = x.float().pow(2).sum(1).repeat_interleave(k)
    assert rel_err(wgrad, want) < 1e-2 and torch.allclose(wgrad.float(), want, rtol=2e-2)


# ------------------------------------------------------------------ the routing chain against the C oracle
@pytest.mark.parametrize('tokens,experts,top_k', [(8192, 8, 2), (16384, 64, 1), (32768, 64, 6), (24576, 16, 4), (7, 3, 2)])
def test_routing_chain_matches_the_c_restatement(ops, tokens, experts, top_k):
    """sort -> histogram -> cumsum -> round_up -> cumsum as the layer runs them (moe.py:152-183,
    dmoe.py:131-154), at the token counts of the benchmark workloads, bit for bit against oracle/routing_c.c."""
    import os
    import shutil
    from oracle import routing_c
    if not os.path.exists(routing_c.LIB_PATH) and shutil.which('gcc') is None:
        pytest.skip('oracle/liboracle_routing.so is not built and there is no gcc')
    g = torch.Generator().manual_seed(tokens + experts)
    top = torch.randint(0, experts, (tokens * top_k,), dtype=torch.int32, generator=g)
    end_bit = oracle.routing.sort_end_bit(experts)
    want_idx, want_ids, want_bins, want_pbins, want_tpe = routing_c.route(top, experts, end_bit, 128)
    t = top.cuda()
    bin_ids, indices = ops.sort(t, end_bit)
    tpe = ops.histogram(t, experts)
    bins = ops.inclusive_cumsum(tpe, 0).view(-1)
    pbins = ops.inclusive_cumsum(ops.round_up(tpe, 128), 0).view(-1)
    for got, want in ((indices, want_idx), (bin_ids, want_ids), (tpe, want_tpe), (bins, want_bins), (pbins, want_pbins)):
        assert got.dtype == torch.int32 and torch.equal(got.cpu(), want)


@pytest.mark.parametrize('n', [0, 1, 100, 2048, 2049, 16384, 100003])
@pytest.mark.parametrize('experts', [1, 2, 8, 17, 64, 200, 256])
@pytest.mark.parametrize('blocking', [0, 128])
def test_route_equals_the_separate_routing_ops(n, experts, blocking):
    """ops.route (sort + histogram + cumsums + the slot -> row map in three launches) against the oracle's
    indices_and_bins / indices_and_padded_bins chain (moe.py:152-183, dmoe.py:131-154) and against the library's own
    separate entry points, bit for bit."""
    from megablocks_amd import _lib, ops
    from megablocks_amd.backend import kernels
    from megablocks_amd.ops import routing
    g = torch.Generator().manual_seed(n * 7 + experts)
    top = torch.randint(0, experts, (n,), generator=g, dtype=torch.int32)
    if experts > 4:
        top[top == 3] = 1                                           # an expert without tokens
    end_bit = max(int(np.ceil(np.log2(experts))), 1)
    ids = top.cuda()
    assert routing.route_supported(ids, experts, end_bit)
    indices, bin_ids, tpe, bins, pbins = routing.route(ids, experts, end_bit, blocking)
    if blocking:
        wi, wb, wbins, wpbins, wtpe = oracle.indices_and_padded_bins(top.long(), experts, blocking)
        assert torch.equal(pbins.cpu(), wpbins.int())
    else:
        wi, wb, wbins, wtpe = oracle.indices_and_bins(top.long(), experts)
        assert pbins is None
    assert torch.equal(indices.cpu(), wi.int()) and torch.equal(bin_ids.cpu(), wb.int())
    assert torch.equal(bins.cpu(), wbins.int()) and torch.equal(tpe.cpu(), wtpe.int())
    assert indices.dtype == torch.int32 and tpe.dtype == torch.int32 and bins.shape == (experts,)
    # the separate entry points
    s_bin_ids, s_indices = ops.sort(ids, end_bit)
    assert torch.equal(s_bin_ids, bin_ids) and torch.equal(s_indices, indices)
    assert torch.equal(ops.histogram(ids, experts), tpe)
    # the slot -> row map that came out of the same launches, against mbx_slot_rows
    if n:
        kept = indices._mbx_slot_rows[1]
        del indices._mbx_slot_rows
        built = kernels._slot_rows(indices, bin_ids, bins, pbins)
        assert torch.equal(kept[:n], built[:n])


def test_route_falls_back_where_it_does_not_apply():
    from megablocks_amd.ops import routing
    ids = torch.zeros(8, dtype=torch.int32, device='cuda')
    assert not routing.route_supported(ids.long(), 8, 3) and not routing.route_supported(ids, 512, 9)
    assert not routing.route_supported(ids, 9, 3) and not routing.route_supported(ids.cpu(), 8, 3)


@pytest.mark.parametrize('blocking', [0, 128])
def test_route_with_ids_outside_the_experts_stays_in_range(blocking):
    """Ids outside [0, num_experts) are a caller's error for ops.route; like ops.sort it orders them by their low bits,
    and no index it writes may leave its range: positions inside [0, n), rows inside the padded buffer or -1."""
    from megablocks_amd import ops
    from megablocks_amd.ops import routing
    experts, end_bit, n = 12, 4, 5000
    g = torch.Generator().manual_seed(3)
    top = torch.randint(-3, experts + 4, (n,), generator=g, dtype=torch.int32)
    ids = top.cuda()
    indices, bin_ids, tpe, bins, pbins = routing.route(ids, experts, end_bit, blocking)
    s_bin_ids, s_indices = ops.sort(ids, end_bit)
    assert torch.equal(s_bin_ids, bin_ids) and torch.equal(s_indices, indices)
    assert torch.equal(torch.sort(indices.cpu().long())[0], torch.arange(n))
    assert int(tpe.min()) >= 0 and int(bins[-1]) <= n and bool((bins[1:] >= bins[:-1]).all())
    rows = indices._mbx_slot_rows[1][:n].cpu()
    limit = int(pbins[-1]) if blocking else n
    assert int(rows.min()) >= -1 and int(rows.max()) < max(limit, n)
    # order, counts and row map agree on the expert of such an id (its low bits): the bins cover the sorted order up to
    # the ids whose low bits name no expert, and every row inside a bin has exactly one slot or is padding, so a gather
    # through this routing leaves no row of the expert-major buffer unwritten
    low = (top & ((1 << end_bit) - 1)).long()
    assert torch.equal(tpe.cpu().long(), torch.bincount(low[low < experts], minlength=experts))
    owned = rows[rows >= 0]
    assert owned.unique().numel() == owned.numel() and owned.numel() == int((low < experts).sum()) + (0 if blocking else int((low >= experts).sum()))
    poison = torch.full((max(limit, n), 64), float('nan'), dtype=torch.bfloat16, device='cuda')
    del poison                                            # the gather's output is likely to land on this block
    for top_k in (2, 1):                                  # one wave per token with the row map / one wave per output row
        x = torch.randn(n // top_k, 64, generator=g).bfloat16().cuda()
        if blocking:
            out = ops.padded_gather(x, indices, bin_ids, bins, pbins, top_k)
        else:
            out = ops.gather(x, indices, bin_ids, bins, top_k)
        assert not bool(torch.isnan(out.float()).any())
        want = torch.zeros_like(out)
        want[owned.cuda().long()] = x[((rows >= 0).nonzero().flatten() // top_k).cuda()]
        assert torch.equal(out, want)
