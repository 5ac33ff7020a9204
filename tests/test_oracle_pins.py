"""Pins the CPU oracle with independent brute-force loops and closed forms.

The reference keeps no stored golden vectors: its tests compare each op with an in-test
loop (tests/ops/*_test.py).  The loops below follow those definitions element by element
in plain Python, on small inputs, and are written independently of the vectorised
oracle; invariants (permutation validity, linearity, adjointness, dense-matmul
equivalence) cover what the loops leave open.
"""
import itertools
import os

import numpy as np
import pytest
import torch

import oracle


def _route(n_slots, ne, seed=0):
    g = torch.Generator().manual_seed(seed)
    top = torch.randint(0, ne, (n_slots,), generator=g).int()
    bin_ids, indices = oracle.sort(top, max(int(np.ceil(np.log2(ne))), 1))
    tpe = oracle.histogram(top, ne)
    bins = oracle.inclusive_cumsum(tpe, 0).view(-1)
    pbins = oracle.inclusive_cumsum(oracle.round_up(tpe, 128), 0).view(-1)
    return top, bin_ids, indices, tpe, bins, pbins


# ---------------------------------------------------------------- histogram
@pytest.mark.parametrize('dtype', [torch.int16, torch.int32, torch.int64])
@pytest.mark.parametrize('rows,n,bins', [(1, 1, 2), (1, 64, 2), (3, 257, 7), (2, 1000, 128), (1, 50, 1)])
def test_histogram_loop(dtype, rows, n, bins):
    x = torch.randint(-2, bins + 3, (rows, n)).to(dtype)      # includes out-of-range ids
    want = torch.zeros((rows, bins), dtype=torch.int32)
    for r in range(rows):
        for v in x[r].tolist():
            if 0 <= v < bins:                                  # csrc/histogram.h:36-38
                want[r, v] += 1
    assert torch.equal(oracle.histogram(x, bins), want)
    assert torch.equal(oracle.histogram(x[0], bins), want[0])
    assert oracle.histogram(x[0], bins).dtype == torch.int32


def test_histogram_matches_histc_like_reference_test():
    # tests/ops/histogram_test.py:78-82 uses torch.histc(y, max_val, 0, max_val - 1)
    x = torch.randint(0, 64, (4, 4096)).int()
    want = torch.stack([torch.histc(r.float(), 64, 0, 63) for r in x]).int()
    assert torch.equal(oracle.histogram(x, 64), want)


# ---------------------------------------------------------------- sort
def _lsd_radix(keys, end_bit):
    """Textbook stable LSD radix sort, one bit per pass, sign bit inverted at full width."""
    bits = {np.int16: 16, np.int32: 32, np.int64: 64}[keys.dtype.type]
    order = list(range(len(keys)))
    ks = [int(k) & ((1 << bits) - 1) for k in keys]            # two's-complement pattern
    for b in range(end_bit):
        flip = 1 if b == bits - 1 else 0
        zeros = [i for i in order if ((ks[i] >> b) & 1) ^ flip == 0]
        ones = [i for i in order if ((ks[i] >> b) & 1) ^ flip == 1]
        order = zeros + ones
    return order


@pytest.mark.parametrize('dtype,end_bit,lo,hi', [
    (torch.int32, 3, 0, 8), (torch.int32, 1, 0, 2), (torch.int32, 6, 0, 64), (torch.int32, 10, 0, 1024),
    (torch.int32, 32, -1000, 1000), (torch.int16, 16, -300, 300), (torch.int16, 7, 0, 128),
    (torch.int64, 64, -2**40, 2**40), (torch.int64, 63, 0, 2**62), (torch.int32, 2, 0, 64),
])
def test_sort_against_lsd_radix(dtype, end_bit, lo, hi):
    x = torch.randint(lo, hi, (300,), dtype=torch.int64).to(dtype)
    keys, perm = oracle.sort(x, end_bit)
    order = _lsd_radix(x.numpy(), end_bit)
    assert perm.tolist() == order
    assert keys.tolist() == [int(x[i]) for i in order]
    assert keys.dtype == dtype and perm.dtype == dtype


def test_sort_default_full_width_and_reference_test_properties():
    x = torch.randint(-2**31, 2**31 - 1, (1000,), dtype=torch.int64).int()
    keys, perm = oracle.sort(x)                                # end_bit=None -> full width
    assert torch.equal(keys, torch.sort(x)[0])                 # tests/ops/sort_test.py:58-60
    back = torch.empty_like(x)
    back.scatter_(0, perm.long(), keys)                        # tests/ops/sort_test.py:62-65
    assert torch.equal(back, x)
    assert sorted(perm.tolist()) == list(range(1000))


def test_sort_is_stable_within_equal_keys():
    x = torch.randint(0, 4, (200,)).int()
    keys, perm = oracle.sort(x, 2)
    for e in range(4):
        p = perm[keys == e].tolist()
        assert p == sorted(p)


# ---------------------------------------------------------------- cumsum / round_up
@pytest.mark.parametrize('dtype', [torch.int16, torch.int32, torch.int64])
def test_cumsum_loops(dtype):
    x = torch.randint(0, 5, (3, 37)).to(dtype)
    inc = torch.zeros_like(x)
    exc = torch.zeros_like(x)
    for r in range(3):
        s = 0
        for c in range(37):
            exc[r, c] = s
            s += int(x[r, c])
            inc[r, c] = s
    assert torch.equal(oracle.inclusive_cumsum(x, 1), inc)
    assert torch.equal(oracle.exclusive_cumsum(x, 1), exc)
    assert torch.equal(oracle.inclusive_cumsum(x[0], 0), inc[0])
    assert torch.equal(oracle.exclusive_cumsum(x[0], 0), exc[0])
    ones = torch.ones((2, 9), dtype=dtype)                      # tests/ops/cumsum_test.py:31-44
    assert torch.equal(oracle.exclusive_cumsum(ones, 1), (torch.cumsum(ones, 1) - 1) * ones)


def test_cumsum_one_element_is_zero_dim_and_dim_check():
    assert oracle.inclusive_cumsum(torch.tensor([5], dtype=torch.int32), 0).ndim == 0   # ops/cumsum.py:45
    with pytest.raises(RuntimeError):
        oracle.inclusive_cumsum(torch.zeros((2, 2), dtype=torch.int32), 0)              # csrc/cumsum.h:144


def test_round_up():
    x = torch.tensor([0, 1, 127, 128, 129, 255, 256, 1000], dtype=torch.int32)
    assert oracle.round_up(x, 128).tolist() == [0, 128, 128, 128, 256, 256, 256, 1024]
    assert oracle.round_up(x, 1).tolist() == x.tolist()


# ---------------------------------------------------------------- replicate / topology
@pytest.mark.parametrize('tokens,centers,batch', [(8, 2, 1), (64, 8, 2), (257, 16, 4), (100, 128, 3)])
def test_replicate_loop(tokens, centers, batch):
    assign = torch.randint(0, centers, (tokens,)).int()
    bins = oracle.inclusive_cumsum(oracle.histogram(assign, centers), 0).view(-1)
    x = torch.randn(batch, centers).half()
    want = torch.zeros(batch, tokens).half()
    for b in range(batch):                                      # tests/ops/replicate_test.py:74-85
        start = 0
        for i, end in enumerate(bins.tolist()):
            while start < end:
                want[b, start] = x[b, i]
                start += 1
    assert torch.equal(oracle.replicate(x, bins, tokens), want)
    grad = oracle.replicate(x, bins, tokens)
    got = oracle.replicate_backward(grad, bins)                 # tests/ops/replicate_test.py:94-108
    counts = oracle.histogram(assign, centers).view(1, -1)
    assert torch.allclose(got.float(), (x.float() * counts), rtol=1e-2, atol=1e-2)
    xi = torch.randint(-50, 50, (batch, centers)).int()
    gi = oracle.replicate(xi, bins, tokens)
    for i in range(centers):
        s = 0 if i == 0 else int(bins[i - 1])
        assert (gi[:, s:int(bins[i])] == xi[:, i:i + 1]).all()


@pytest.mark.parametrize('sl,hs,ne', [(256, 128, 2), (1024, 512, 4), (2000, 1024, 16), (300, 256, 64)])
def test_topology_loop(sl, hs, ne):
    blocking = 128
    top = torch.randint(0, ne, (sl,)).int()
    pbins = oracle.inclusive_cumsum(oracle.round_up(oracle.histogram(top, ne), blocking), 0).view(-1)
    rows, cols = int(pbins[-1]) // blocking, hs // blocking
    want = np.zeros([rows * cols])                              # tests/ops/topology_test.py:51-67
    start = 0
    for i in range(ne):
        end = int(pbins[i]) // blocking
        while start < end:
            for j in range(cols):
                want[start * cols + j] = j + i * cols
            start += 1
    got = oracle.topology(pbins, blocking, rows, cols)
    assert got.dtype == torch.int16
    assert got.tolist() == want.astype(np.int16).tolist()


def test_sparse_transpose_is_the_transpose_of_the_block_pattern():
    ne, ffn, blocking = 4, 512, 128
    top = torch.randint(0, ne, (700,)).int()
    pbins = oracle.inclusive_cumsum(oracle.round_up(oracle.histogram(top, ne), blocking), 0).view(-1)
    br, bpr = int(pbins[-1]) // blocking, ffn // blocking
    col = oracle.topology(pbins, blocking, br, bpr)
    row = oracle.row_indices(br, bpr)
    end_bit = max(int(np.ceil(np.log2(ffn * ne // blocking))), 1)
    col_t, off_t, boff_t = oracle.sparse_transpose((br * blocking, ffn * ne), row, col, blocking, end_bit)
    dense = np.zeros((br, bpr * ne), dtype=np.int64) - 1
    for blk, (r, c) in enumerate(zip(row.tolist(), col.tolist())):
        dense[r, c] = blk
    want_rows, want_blk, want_off = [], [], [0]
    for c in range(bpr * ne):                                   # walk the transposed matrix row by row
        for r in range(br):
            if dense[r, c] >= 0:
                want_rows.append(r)
                want_blk.append(int(dense[r, c]))
        want_off.append(len(want_rows))
    assert col_t.tolist() == want_rows and boff_t.tolist() == want_blk and off_t.tolist() == want_off


# ---------------------------------------------------------------- gather / scatter family
@pytest.mark.parametrize('sl,hs,ne,top_k', [(4, 2, 2, 1), (4, 2, 2, 2), (64, 3, 4, 2), (200, 8, 8, 4), (130, 5, 16, 1)])
def test_padded_gather_loop(sl, hs, ne, top_k):
    x = torch.randn(sl, hs).half()
    top, bin_ids, indices, tpe, bins, pbins = _route(sl * top_k, ne)
    want = np.zeros((int(pbins[-1]), hs))                       # tests/ops/padded_gather_test.py:66-90
    in_idx = 0
    for i, end in enumerate(bins.tolist()):
        out_idx = 0 if i == 0 else int(pbins[i - 1])
        while in_idx < end:
            want[out_idx, :] = x[int(indices[in_idx]) // top_k, :].numpy()
            in_idx += 1
            out_idx += 1
    got = oracle.padded_gather(x, indices, bin_ids, None, bins, pbins, top_k)
    assert np.array_equal(got.float().numpy(), want.astype(np.float32))
    g2 = oracle.gather(x, indices, bin_ids, None, bins, top_k)  # padded_bins := bins, kernels.py:163-164
    for i in range(sl * top_k):
        assert torch.equal(g2[i], x[int(indices[i]) // top_k])
    w = torch.rand(sl * top_k).half()
    g3 = oracle.gather(x, indices, bin_ids, w, bins, top_k)
    for i in range(sl * top_k):
        s = int(indices[i])
        assert torch.equal(g3[i], (x[s // top_k].float() * w[s].float()).half())


@pytest.mark.parametrize('sl,hs,ne,top_k', [(4, 2, 2, 1), (4, 2, 2, 2), (64, 3, 4, 2), (200, 8, 8, 4), (130, 5, 16, 1)])
def test_padded_scatter_loop(sl, hs, ne, top_k):
    top, bin_ids, indices, tpe, bins, pbins = _route(sl * top_k, ne, seed=1)
    xt = torch.randn(sl, hs).half()
    x = oracle.padded_gather(xt, indices, bin_ids, None, bins, pbins, top_k)
    w = torch.rand(sl * top_k).half()
    want = np.zeros((sl, hs))                                   # tests/ops/padded_scatter_test.py:97-126
    out_idx = 0
    for i in range(ne):
        in_idx = 0 if i == 0 else int(pbins[i - 1])
        end = int(bins[i])
        while out_idx < end:
            store = int(indices[out_idx])
            want[store // top_k, :] += float(w[store]) * x[in_idx, :].float().numpy()
            out_idx += 1
            in_idx += 1
    got = oracle.padded_scatter(x, indices, bin_ids, w, bins, pbins, top_k)
    assert np.allclose(got.float().numpy(), want, rtol=5e-3, atol=1e-3)
    # unweighted, top_k == 1: scatter(gather(x)) is x bit for bit
    if top_k == 1:
        assert torch.equal(oracle.padded_scatter(x, indices, bin_ids, None, bins, pbins, 1), xt)
    xu = oracle.gather(xt, indices, bin_ids, None, bins, top_k)
    su = oracle.scatter(xu, indices, bin_ids, None, bins, top_k)
    assert torch.allclose(su.float(), xt.float() * top_k, rtol=2e-3, atol=1e-3)


def test_scatter_wgrad_is_the_weight_gradient_of_scatter():
    sl, hs, ne, top_k = 48, 6, 4, 2
    top, bin_ids, indices, tpe, bins, pbins = _route(sl * top_k, ne, seed=2)
    x = torch.randn(int(pbins[-1]), hs)
    grad = torch.randn(sl, hs)
    w = torch.rand(sl * top_k, requires_grad=True)
    out = oracle.padded_scatter(x, indices, bin_ids, w, bins, pbins, top_k)
    out.backward(grad)
    got = oracle.padded_scatter_wgrad(x, grad, indices, bin_ids, bins, pbins, top_k)
    assert torch.allclose(got, w.grad, rtol=1e-5, atol=1e-5)
    # explicit loop, kernels.py:241-276
    for i in range(sl * top_k):
        e = int(bin_ids[i])
        row = i - (0 if e == 0 else int(bins[e - 1])) + (0 if e == 0 else int(pbins[e - 1]))
        s = int(indices[i])
        assert abs(float(got[s]) - float((x[row] * grad[s // top_k]).sum())) < 1e-4


def test_gather_and_scatter_are_adjoint():
    sl, hs, ne, top_k = 32, 4, 4, 2
    top, bin_ids, indices, tpe, bins, pbins = _route(sl * top_k, ne, seed=3)
    x = torch.randn(sl, hs, dtype=torch.float64)
    y = torch.randn(sl * top_k, hs, dtype=torch.float64)
    w = torch.rand(sl * top_k, dtype=torch.float64)
    lhs = (oracle.gather(x, indices, bin_ids, w, bins, top_k) * y).sum()
    rhs = (x * oracle.scatter(y, indices, bin_ids, w, bins, top_k)).sum()
    assert abs(float(lhs - rhs)) < 1e-6   # the scaled copy multiplies in fp32 (kernels.py:100)


@pytest.mark.parametrize('sl,hs,ne,top_k,cap', [(4, 2, 2, 1, 2), (64, 3, 4, 2, 16), (200, 4, 8, 4, 50), (64, 2, 4, 1, 100)])
def test_binned_loops(sl, hs, ne, top_k, cap):
    top, bin_ids, indices, tpe, bins, pbins = _route(sl * top_k, ne, seed=4)
    x = torch.randn(sl, hs).half()
    want = np.zeros((ne, cap, hs))                              # tests/ops/binned_gather_test.py:49-67
    start = 0
    for i in range(ne):
        end = int(bins[i])
        for j in range(cap):
            if start + j >= end:
                break
            want[i, j, :] = x[int(indices[start + j]) // top_k, :].numpy()
        start = end
    got = oracle.binned_gather(x, indices, None, bins, cap, top_k)
    assert np.array_equal(got.float().numpy(), want.astype(np.float32))

    w = torch.rand(sl * top_k).half()
    want = np.zeros((sl, hs))                                   # tests/ops/binned_scatter_test.py:54-76
    start = 0
    for i in range(ne):
        end = int(bins[i])
        for j in range(cap):
            if start + j >= end:
                break
            s = int(indices[start + j])
            want[s // top_k, :] += float(w[s]) * got[i, j, :].float().numpy()
        start = end
    sc = oracle.binned_scatter(got, indices, w, bins, top_k)
    assert np.allclose(sc.float().numpy(), want, rtol=5e-3, atol=1e-3)

    grad = torch.randn(sl, hs).half()
    wg = oracle.binned_scatter_wgrad(got, grad, indices, bins, top_k)
    start = 0
    for i in range(ne):
        end = int(bins[i])
        for j in range(min(cap, end - start)):
            s = int(indices[start + j])
            ref = float((got[i, j].float() * grad[s // top_k].float()).sum())
            assert abs(float(wg[s]) - ref) <= 1e-2 * max(1.0, abs(ref))
        start = end


# ---------------------------------------------------------------- gmm / layer
def test_gmm_triple_loop_and_empty_groups():
    sizes = torch.tensor([3, 0, 5, 1])
    a = torch.randn(9, 4)
    b = torch.randn(4, 4, 6)
    got = oracle.gmm(a, b, sizes)
    start = 0
    for e, n in enumerate(sizes.tolist()):
        for r in range(start, start + n):
            for c in range(6):
                assert abs(float(got[r, c]) - sum(float(a[r, k]) * float(b[e, k, c]) for k in range(4))) < 1e-4
        start += n
    bt = b.transpose(1, 2).contiguous()
    assert torch.allclose(oracle.gmm(a, bt, sizes, trans_b=True), got, atol=1e-6)
    b2 = torch.randn(9, 6)
    ta = oracle.gmm(a, b2, sizes, trans_a=True)
    assert ta.shape == (4, 4, 6) and torch.count_nonzero(ta[1]) == 0
    assert torch.allclose(ta[2], a[3:8].t() @ b2[3:8], atol=1e-6)
    c = torch.empty(9, 6)
    assert oracle.gmm(a, b, sizes, c=c) is c and torch.equal(c, got)


def test_gmm_backward_pairing_matches_autograd():
    # d/da (a @ b[e]) = dc @ b[e].T (trans_b flipped); d/db = a.T @ dc (trans_a)
    sizes = torch.tensor([4, 2, 0, 6])
    a = torch.randn(12, 5, dtype=torch.float64, requires_grad=True)
    b = torch.randn(4, 5, 3, dtype=torch.float64, requires_grad=True)
    start, outs = 0, []
    for e, n in enumerate(sizes.tolist()):
        outs.append(a[start:start + n] @ b[e])
        start += n
    dc = torch.randn(12, 3, dtype=torch.float64)
    torch.cat(outs).backward(dc)
    assert torch.allclose(oracle.gmm(dc, b.detach(), sizes, trans_b=True), a.grad, atol=1e-9)
    assert torch.allclose(oracle.gmm(a.detach(), dc, sizes, trans_a=True), b.grad, atol=1e-9)


def test_gelu_backward_closed_form_vs_autograd():
    x = torch.randn(1000, dtype=torch.float64, requires_grad=True)
    g = torch.randn(1000, dtype=torch.float64)
    torch.nn.functional.gelu(x, approximate='tanh').backward(g)
    assert torch.allclose(oracle.gelu_tanh_backward(g, x.detach()), x.grad, atol=1e-6)


def test_router_top1_is_argmax_and_topk_renormalised():
    x = torch.randn(50, 16)
    wr = torch.randn(8, 16)
    scores, ew, ei = oracle.router_forward(x, wr, 1)
    assert torch.equal(ei.flatten(), scores.argmax(-1)) and torch.allclose(scores.sum(-1), torch.ones(50))
    scores, ew, ei = oracle.router_forward(x, wr, 2, normalize_p=1)
    assert torch.allclose(ew.sum(-1), torch.ones(50), atol=1e-6)
    for t in range(50):
        assert set(ei[t].tolist()) == set(torch.argsort(scores[t], descending=True)[:2].tolist())


@pytest.mark.parametrize('glu', [False, True])
def test_dmoe_forward_equals_per_token_definition(glu):
    # per token: sum_j w_j * MLP_{e_j}(x)   (tests/layers/dmoe_test.py:216-241 equivalence)
    T, h, f, E, k = 24, 8, 16, 4, 2
    x = torch.randn(T, h, dtype=torch.float64)
    w1, w2 = torch.randn(E * f, h, dtype=torch.float64), torch.randn(E * f, h, dtype=torch.float64)
    v1 = torch.randn(E * f, h, dtype=torch.float64) if glu else None
    _, ew, ei = oracle.router_forward(x, torch.randn(E, h, dtype=torch.float64), k)
    out, tpe = oracle.dmoe_forward(x, ew, ei, w1, w2, v1, num_experts=E, top_k=k)
    act = lambda t: torch.nn.functional.gelu(t, approximate='tanh')
    for t in range(T):
        acc = torch.zeros(h, dtype=torch.float64)
        for j in range(k):
            e = int(ei[t, j])
            hmid = act(w1[e * f:(e + 1) * f] @ x[t])
            if glu:
                hmid = hmid * (v1[e * f:(e + 1) * f] @ x[t])
            acc += ew[t, j] * (w2[e * f:(e + 1) * f].t() @ hmid)
        assert torch.allclose(out[t], acc, atol=1e-9)
    assert tpe.tolist() == torch.bincount(ei.flatten(), minlength=E).tolist()


def test_dmoe_single_expert_is_dense_ffn():
    # tests/layers/dmoe_test.py:191-213: one expert, top-1 -> weight 1 -> plain FFN
    T, h, f = 16, 8, 32
    x = torch.randn(T, h)
    w1, w2 = torch.randn(f, h), torch.randn(f, h)
    _, ew, ei = oracle.router_forward(x, torch.randn(1, h), 1)
    out, _ = oracle.dmoe_forward(x, ew, ei, w1, w2, num_experts=1, top_k=1)
    want = torch.nn.functional.gelu(x @ w1.t(), approximate='tanh') @ w2
    assert torch.allclose(out, want, atol=1e-5)


# ---------------------------------------------------------------------------------------------
# The plain-C restatement of the integer routing ops (oracle/routing_c.c) against the torch one:
# two independent restatements of the same reference lines must agree bit for bit.
@pytest.fixture(scope='module')
def rc():
    import shutil
    from oracle import routing_c
    if not os.path.exists(routing_c.LIB_PATH) and shutil.which('gcc') is None:
        pytest.skip('oracle/liboracle_routing.so is not built and there is no gcc')
    routing_c.lib()
    return routing_c


@pytest.mark.parametrize('dtype', [torch.int16, torch.int32, torch.int64])
def test_c_oracle_sort_histogram_cumsum(rc, dtype):
    g = torch.Generator().manual_seed(11)
    width = {torch.int16: 16, torch.int32: 32, torch.int64: 64}[dtype]
    for n in (0, 1, 2, 63, 64, 1000):
        x = torch.randint(-70, 70, (n,), dtype=dtype, generator=g)
        for end_bit in (None, 0, 1, 3, 7, width - 1, width):
            k1, p1 = oracle.sort(x, end_bit)
            k2, p2 = rc.sort(x, end_bit)
            assert torch.equal(k1, k2) and torch.equal(p1, p2), (n, end_bit)
    h = torch.randint(-3, 12, (5, 257), dtype=dtype, generator=g)
    for bins in (1, 9, 64):
        assert torch.equal(oracle.histogram(h, bins), rc.histogram(h, bins))
        assert torch.equal(oracle.histogram(h[0], bins), rc.histogram(h[0], bins))
    c = torch.randint(0, 100, (4, 77), dtype=dtype, generator=g)
    assert torch.equal(oracle.inclusive_cumsum(c, 1), rc.cumsum(c, False))
    assert torch.equal(oracle.exclusive_cumsum(c, 1), rc.cumsum(c, True))


def test_c_oracle_topology_replicate_route(rc):
    g = torch.Generator().manual_seed(12)
    pb = torch.tensor([256, 256, 640, 1024, 1024], dtype=torch.int32)
    for rows in (8, 10):                       # fewer / more block-rows than the bins cover
        assert torch.equal(oracle.topology(pb, 128, rows, 6), rc.topology(pb, 128, rows, 6))
    x = torch.randint(0, 9, (3, 4), dtype=torch.int32, generator=g)
    bins = torch.tensor([2, 2, 7, 9], dtype=torch.int32)
    for cols in (9, 12):
        assert torch.equal(oracle.replicate(x, bins, cols), rc.replicate(x, bins, cols))
    for experts in (1, 8, 64):
        te = torch.randint(0, experts, (777,), dtype=torch.int32, generator=g)
        want = oracle.indices_and_padded_bins(te, experts, 128)
        got = rc.route(te, experts, oracle.routing.sort_end_bit(experts), 128)
        for w, t in zip(want, got):
            assert torch.equal(w.view(-1), t.view(-1))


# ---------------------------------------------------------------- auxiliary losses
def _lbl_loop(counts_per_layer, scores_per_layer, ne, top_k, weight):
    """moe.py:32-89 element by element in Python floats."""
    layers = len(counts_per_layer)
    tokens = len(scores_per_layer[0])
    dot = 0.0
    for counts, scores in zip(counts_per_layer, scores_per_layer):
        for e in range(ne):
            col = sum(row[e] for row in scores)
            dot += counts[e] * (col / tokens if tokens else col)
    return ne * weight / (layers * tokens * top_k) * dot


@pytest.mark.parametrize('tokens,ne,top_k,layers', [(7, 3, 1, 1), (16, 4, 2, 1), (33, 8, 3, 2), (5, 2, 2, 3)])
def test_load_balancing_loss_loop(tokens, ne, top_k, layers):
    g = torch.Generator().manual_seed(tokens * ne)
    scores = [torch.randn(tokens, ne, generator=g).softmax(-1) for _ in range(layers)]
    counts = [oracle.histogram(torch.topk(s, top_k, -1).indices.flatten().int(), ne) for s in scores]
    want = _lbl_loop([c.tolist() for c in counts], [s.tolist() for s in scores], ne, top_k, 0.1)
    got = oracle.load_balancing_loss(counts, scores, num_experts=ne, top_k=top_k, loss_weight=0.1)
    assert abs(float(got) - want) <= 1e-6 * abs(want)
    if layers == 1:   # the per-layer form of moe.py:138-150 is the same quantity without the weight
        one = oracle.layer_load_balancing_loss(counts[0], scores[0], top_k=top_k)
        assert abs(float(one) * 0.1 - want) <= 1e-6 * abs(want)


def test_load_balancing_loss_closed_forms():
    ne, top_k, tokens, w = 8, 2, 64, 0.25
    g = torch.Generator().manual_seed(1)
    scores = torch.randn(tokens, ne, generator=g).softmax(-1)
    # evenly loaded experts: <counts, mean scores> = tokens * top_k / E * sum_e mean_e = tokens * top_k / E,
    # whatever the scores are (each row of a softmax sums to one) -> loss = loss_weight
    even = torch.full((ne,), tokens * top_k // ne, dtype=torch.int32)
    assert abs(float(oracle.load_balancing_loss(even, scores, num_experts=ne, top_k=top_k, loss_weight=w)) - w) < 1e-6
    # everything routed to one expert whose score is 1 for every token -> loss = E * loss_weight
    onehot = torch.zeros(tokens, ne)
    onehot[:, 3] = 1
    counts = torch.zeros(ne, dtype=torch.int32)
    counts[3] = tokens * top_k
    assert abs(float(oracle.load_balancing_loss(counts, onehot, num_experts=ne, top_k=top_k, loss_weight=w)) - ne * w) < 1e-5
    # two layers with num_layers = 2: the mean of the two single-layer losses
    s2 = torch.randn(tokens, ne, generator=g).softmax(-1)
    c1 = oracle.histogram(torch.topk(scores, top_k, -1).indices.flatten().int(), ne)
    c2 = oracle.histogram(torch.topk(s2, top_k, -1).indices.flatten().int(), ne)
    both = oracle.load_balancing_loss([c1, c2], [scores, s2], num_experts=ne, top_k=top_k, loss_weight=w)
    a = oracle.load_balancing_loss(c1, scores, num_experts=ne, top_k=top_k, loss_weight=w)
    b = oracle.load_balancing_loss(c2, s2, num_experts=ne, top_k=top_k, loss_weight=w)
    assert abs(float(both) - 0.5 * (float(a) + float(b))) < 1e-6
    assert oracle.load_balancing_loss(c1, scores, num_experts=ne, top_k=top_k, loss_weight=0) == 0.0
    with pytest.raises(ValueError):
        oracle.load_balancing_loss([c1], [scores], num_experts=ne, top_k=top_k, loss_weight=w, num_layers=2)
    # the gradient reaches the scores only: d loss / d scores[t, e] = scale * counts[e] / tokens
    s = scores.clone().requires_grad_(True)
    oracle.load_balancing_loss(c1, s, num_experts=ne, top_k=top_k, loss_weight=w).backward()
    want = (ne * w / (tokens * top_k)) * c1.float() / tokens
    assert torch.allclose(s.grad, want.expand(tokens, ne), rtol=1e-6, atol=0)


def test_router_zloss_loop_and_closed_form():
    import math
    tokens, ne, w = 9, 5, 1e-3
    g = torch.Generator().manual_seed(2)
    logits = torch.randn(tokens, ne, generator=g) * 3
    want = w * sum(math.log(sum(math.exp(v) for v in row)) ** 2 for row in logits.tolist()) / tokens
    got = oracle.router_zloss(logits, zloss_weight=w)
    assert got.shape == (1,) and abs(float(got[0]) - want) <= 1e-6 * want
    # constant logits c over E experts: logsumexp = c + ln E
    for c in (-2.0, 0.0, 3.5):
        z = oracle.router_zloss(torch.full((4, ne), c), zloss_weight=w)
        want_c = w * (c + math.log(ne)) ** 2
        assert abs(float(z[0]) - want_c) <= 1e-6 * want_c
    # one value per router; large logits do not overflow
    z = oracle.router_zloss([logits, logits + 100.0], zloss_weight=w)
    assert z.shape == (2,) and torch.isfinite(z).all() and abs(float(z[0]) - want) <= 1e-6 * want
    assert oracle.router_zloss(logits, zloss_weight=0) == 0
    # 16-bit logits are widened first (router.py:36-37)
    zb = oracle.router_zloss(logits.bfloat16(), zloss_weight=w)
    assert zb.dtype == torch.float32


def test_uniform_expert_assignment():
    got = oracle.uniform_expert_assignment((5, 2), 4)
    assert got.tolist() == [[0, 1], [2, 3], [0, 1], [2, 3], [0, 1]]
    assert oracle.histogram(oracle.uniform_expert_assignment((64, 2), 8).flatten().int(), 8).tolist() == [16] * 8
