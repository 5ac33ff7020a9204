"""GPU parity tests of the grouped GEMM: against the CPU oracle at small sizes and against an
fp32 torch formulation on the GPU at the benchmark shapes.  Tolerance: relative Frobenius
error <= 1e-2 (bf16/f16 inputs, fp32 accumulation)."""
import math

import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

TOL = 1e-2


@pytest.fixture(scope='module')
def gg():
    from megablocks_amd import grouped_gemm_util as gg
    return gg


def rel_err(a, b):
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def max_block_err(got, ref, bm=64, bn=128):
    """Largest relative error over bm x bn blocks of the last two dimensions: one wrong piece of one tile
    shows here even where the error over the whole output would hide it."""
    got, ref = got.double(), ref.double()
    r, c = ref.shape[-2:]
    pr, pc = (-r) % bm, (-c) % bn
    d = torch.nn.functional.pad(got - ref, (0, pc, 0, pr))
    b = torch.nn.functional.pad(ref, (0, pc, 0, pr))
    shape = d.shape[:-2] + ((r + pr) // bm, bm, (c + pc) // bn, bn)
    num = d.reshape(shape).pow(2).sum(dim=(-3, -1)).sqrt()
    den = b.reshape(shape).pow(2).sum(dim=(-3, -1)).sqrt()
    scale = ref.norm() / max(1, num.numel()) ** 0.5              # a typical block norm, for blocks that are almost zero
    return float((num / torch.maximum(den, scale * 0.1)).max())


def _sizes(groups, rows, seed, empty=()):
    g = torch.Generator().manual_seed(seed)
    cuts = torch.sort(torch.randint(0, rows + 1, (groups - 1,), generator=g))[0]
    sizes = torch.diff(torch.cat([torch.zeros(1, dtype=torch.int64), cuts, torch.tensor([rows])]))
    for e in empty:                      # force some empty groups, keep the total
        if e + 1 < groups:
            sizes[e + 1] += sizes[e]
            sizes[e] = 0
    return sizes


def _ref_gpu(a, b, sizes, trans_a, trans_b):
    a, b = a.float(), b.float()
    outs, start = [], 0
    for e, n in enumerate(sizes.tolist()):
        ae = a[start:start + n]
        if trans_a:
            outs.append(ae.t() @ b[start:start + n])
        else:
            outs.append(ae @ (b[e].t() if trans_b else b[e]))
        start += n
    return torch.stack(outs) if trans_a else torch.cat(outs)


SMALL = [  # groups, rows, k, n
    (1, 128, 128, 128), (4, 512, 64, 256), (8, 1000, 256, 512), (3, 777, 72, 40), (5, 300, 100, 36),
    (2, 64, 8, 8), (16, 2048, 512, 1408), (4, 50, 33, 17), (1, 1, 16, 16), (8, 4096, 1024, 256),
]


@pytest.mark.parametrize('groups,k,n', [(1, 64, 256), (59, 1440, 704), (56, 960, 1104), (174, 1344, 256), (5, 33, 17)])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('sizes_on_device', [False, True])
def test_gmm_with_no_rows_at_all(gg, groups, k, n, dtype, sizes_on_device):
    """Every expert empty: the weight gradients (trans_a) are exact zeros written over whatever the output
    buffer held, and the row products are empty."""
    sizes = torch.zeros(groups, dtype=torch.int64)
    bs = sizes.cuda() if sizes_on_device else sizes
    a = torch.empty(0, k, device='cuda', dtype=dtype)
    c = torch.full((groups, k, n), float('nan'), device='cuda', dtype=dtype)
    out = gg.backend.gmm(a, torch.empty(0, n, device='cuda', dtype=dtype), bs, trans_a=True, c=c)
    assert out.shape == (groups, k, n) and int(torch.count_nonzero(out)) == 0
    w = torch.randn(groups, k, n, device='cuda').to(dtype)
    assert gg.backend.gmm(a, w, bs).shape == (0, n)
    assert gg.backend.gmm(torch.empty(0, n, device='cuda', dtype=dtype), w, bs, trans_b=True).shape == (0, k)


@pytest.mark.parametrize('groups,rows,k,n', SMALL)
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize('mode', ['nn', 'nt', 'tn'])
def test_gmm_vs_oracle(gg, groups, rows, k, n, dtype, mode):
    sizes = _sizes(groups, rows, seed=groups * 1000 + rows, empty=(1,) if groups > 2 else ())
    a = torch.randn(rows, k).to(dtype)
    if mode == 'tn':
        b = torch.randn(rows, n).to(dtype)
    elif mode == 'nt':
        b = (torch.randn(groups, n, k) * 0.1).to(dtype)
    else:
        b = (torch.randn(groups, k, n) * 0.1).to(dtype)
    want = oracle.gmm(a, b, sizes, trans_a=mode == 'tn', trans_b=mode == 'nt')
    got = gg.backend.gmm(a.cuda(), b.cuda(), sizes, trans_a=mode == 'tn', trans_b=mode == 'nt')
    assert got.shape == want.shape and got.dtype == dtype
    assert rel_err(got.cpu(), want) < TOL
    if mode == 'tn':
        for e, s in enumerate(sizes.tolist()):
            if s == 0:
                assert torch.count_nonzero(got[e]) == 0          # unused expert: exactly zero gradient
    got_dev = gg.backend.gmm(a.cuda(), b.cuda(), sizes.cuda().int(), trans_a=mode == 'tn', trans_b=mode == 'nt')
    assert torch.equal(got_dev, got)                              # device-resident sizes: same kernel, same result


def test_gmm_c_argument_and_errors(gg):
    sizes = torch.tensor([100, 28])
    a = torch.randn(128, 64).bfloat16().cuda()
    b = torch.randn(2, 64, 32).bfloat16().cuda()
    c = torch.full((128, 32), 7.0).bfloat16().cuda()
    out = gg.backend.gmm(a, b, sizes, c=c)
    assert out is c and rel_err(c.cpu(), oracle.gmm(a.cpu(), b.cpu(), sizes)) < TOL
    with pytest.raises(ValueError):
        gg.backend.gmm(a, b, sizes, c=torch.empty(128, 31).bfloat16().cuda())
    with pytest.raises(ValueError):
        gg.backend.gmm(a, b.float(), sizes)
    with pytest.raises(ValueError):
        gg.backend.gmm(a, b, sizes, trans_b=True)
    short = torch.tensor([60, 20])
    with pytest.raises(ValueError):                               # sizes on the host are checked against the operand
        gg.backend.gmm(a, b, short)
    with pytest.raises(ValueError):
        gg.backend.gmm(a, b, torch.tensor([130, -2]))
    with pytest.raises(ValueError):
        gg.backend.gmm(a, a, short, trans_a=True)
    c2 = torch.full((128, 32), 7.0).bfloat16().cuda()             # sizes on the device cannot be: rows past the last
    gg.backend.gmm(a, b, short.cuda(), c=c2)                      # bin are left alone
    assert bool((c2[80:] == 7.0).all()) and rel_err(c2[:80].cpu(), oracle.gmm(a[:80].cpu(), b.cpu(), short)) < TOL


@pytest.mark.parametrize('dtype,k,n', [(torch.bfloat16, 256, 512), (torch.bfloat16, 72, 40), (torch.float32, 64, 64),
                                       (torch.bfloat16, 1 << 16, 64)])
@pytest.mark.parametrize('mode', ['nn', 'nt', 'tn'])
def test_gmm_bins_that_do_not_match_the_operands_stay_in_range(gg, dtype, k, n, mode):
    """Device-side sizes that add up to more rows than the operands have (a stale table), or that are negative:
    the values are then unspecified, but no kernel reads or writes outside the operands -- the rows behind the
    output and a guard region around it keep their canary."""
    if k > 4096 and mode != 'nn':
        pytest.skip('the long-k case exercises the register-staged NN fallback only')
    rows, groups = 700, 4
    a = torch.randn(rows, k, device='cuda').to(dtype)
    if mode == 'tn':
        b = torch.randn(rows, n, device='cuda').to(dtype)
        shape = (groups, k, n)
    else:
        b = torch.randn(groups, n, k, device='cuda').to(dtype) if mode == 'nt' else torch.randn(groups, k, n, device='cuda').to(dtype)
        shape = (rows, n)
    numel = shape[0] * shape[1] * (shape[2] if len(shape) == 3 else 1)
    for sizes in ([300, 300, 300, 300], [900, 0, 0, 0], [200, -50, 400, 5000], [-7, 2000, -2000, 100]):
        guard = 4096
        buf = torch.full((numel + 2 * guard,), 3.0, device='cuda', dtype=dtype)
        c = buf[guard:guard + numel].view(shape)
        gg.backend.gmm(a, b, torch.tensor(sizes, dtype=torch.int32, device='cuda'), trans_a=mode == 'tn', trans_b=mode == 'nt', c=c)
        torch.cuda.synchronize()
        assert bool((buf[:guard] == 3.0).all()) and bool((buf[guard + numel:] == 3.0).all())
    # a table that does match still gives the product
    good = torch.tensor([100, 0, 250, 350], dtype=torch.int32, device='cuda')
    got = gg.backend.gmm(a, b, good, trans_a=mode == 'tn', trans_b=mode == 'nt')
    assert rel_err(got.float(), _ref_gpu(a, b, good.cpu(), mode == 'tn', mode == 'nt')) < TOL


BIG = [  # name, groups, rows, hidden, ffn, skew
    ('gpt2-64e', 64, 16384, 1024, 4096, False),
    ('mixtral', 8, 16384, 4096, 14336, False),
    ('finegrained-zipf', 64, 32768, 2048, 1408, True),
    ('sparse-padded', 16, 12288, 2048, 8192, False),
]


@pytest.mark.parametrize('name,groups,rows,hidden,ffn,skew', BIG)
def test_gmm_benchmark_shapes_vs_fp32(gg, name, groups, rows, hidden, ffn, skew):
    torch.manual_seed(1)
    if skew:
        p = torch.arange(1, groups + 1).float() ** -1.2
        p[-4:] = 0                                               # four experts receive nothing
        sizes = torch.bincount(torch.multinomial(p, rows, replacement=True), minlength=groups)
    else:
        sizes = _sizes(groups, rows, seed=3)
    x = torch.randn(rows, hidden, device='cuda').bfloat16()
    w = (torch.randn(groups, ffn, hidden, device='cuda') * 0.02).bfloat16()
    h = gg.backend.gmm(x, w, sizes, trans_b=True)                               # NT
    ref = _ref_gpu(x, w, sizes, False, True)
    assert rel_err(h, ref) < TOL and max_block_err(h, ref) < 2 * TOL
    y = gg.backend.gmm(h, w, sizes)                                             # NN
    ref = _ref_gpu(h, w, sizes, False, False)
    assert rel_err(y, ref) < TOL and max_block_err(y, ref) < 2 * TOL
    dw = gg.backend.gmm(h, x, sizes, trans_a=True)                              # TN
    ref = _ref_gpu(h, x, sizes, True, False)
    assert rel_err(dw, ref) < TOL and max_block_err(dw, ref) < 2 * TOL
    for e, s in enumerate(sizes.tolist()):
        if s == 0:
            assert torch.count_nonzero(dw[e]) == 0


def test_gmm_autograd(gg):
    sizes = torch.tensor([300, 0, 212])
    a = torch.randn(512, 256, device='cuda').bfloat16().requires_grad_(True)
    b = (torch.randn(3, 128, 256, device='cuda') * 0.1).bfloat16().requires_grad_(True)
    gout = torch.randn(512, 128, device='cuda').bfloat16()
    gg.ops.gmm(a, b, sizes, True).backward(gout)
    af, bf = a.detach().float().requires_grad_(True), b.detach().float().requires_grad_(True)
    outs, start = [], 0
    for e, n in enumerate(sizes.tolist()):
        outs.append(af[start:start + n] @ bf[e].t())
        start += n
    torch.cat(outs).backward(gout.float())
    assert rel_err(a.grad, af.grad) < TOL and rel_err(b.grad, bf.grad) < TOL
    assert torch.count_nonzero(b.grad[1]) == 0


def test_gelu_backward_inplace():
    from megablocks_amd.layers.gelu import gelu_backward_
    for dtype in (torch.bfloat16, torch.float16, torch.float32):
        for shape in ((1000, 257), (1003,), (5,)):            # whole 16-byte vectors; a tail; less than one vector
            x = torch.randn(*shape).to(dtype)
            g = torch.randn(*shape).to(dtype)
            want = oracle.gelu_tanh_backward(g.float(), x.float())
            gd = g.cuda()
            out = gelu_backward_(gd, x.cuda())
            assert out is gd and rel_err(gd.cpu().float(), want) < (1e-5 if dtype == torch.float32 else 1e-2)
        # buffers that are not 16-byte aligned: element by element, same values
        x, g = torch.randn(4100).to(dtype), torch.randn(4100).to(dtype)
        aligned = gelu_backward_(g.cuda()[8:].clone(), x.cuda()[8:].clone())
        base = g.cuda()
        gelu_backward_(base[1:], x.cuda()[1:])
        assert torch.equal(base[8:], aligned) and torch.equal(base[:1].cpu(), g[:1])


DMA_EDGE = [  # groups, rows, k, n: shapes that take the direct-to-LDS kernels, off every tile boundary
    (3, 700, 64, 8), (5, 1030, 128, 264), (2, 255, 192, 1408), (7, 3001, 320, 520), (1, 257, 64, 248),
    (4, 513, 1024, 72), (6, 40, 64, 40),
]


@pytest.mark.parametrize('groups,rows,k,n', DMA_EDGE)
@pytest.mark.parametrize('mode', ['nn', 'nt', 'tn'])
def test_gmm_ragged_shapes_on_the_pipelined_path(gg, groups, rows, k, n, mode):
    sizes = _sizes(groups, rows, seed=rows, empty=(0,) if groups > 2 else ())
    a = torch.randn(rows, k).bfloat16()
    if mode == 'tn':
        b = torch.randn(rows, n).bfloat16()
    elif mode == 'nt':
        b = (torch.randn(groups, n, k) * 0.1).bfloat16()
    else:
        b = (torch.randn(groups, k, n) * 0.1).bfloat16()
    want = oracle.gmm(a, b, sizes, trans_a=mode == 'tn', trans_b=mode == 'nt')
    guard = torch.full((want.numel() + 4096,), 3.0).bfloat16().cuda()       # canary around the output
    c = guard[2048:2048 + want.numel()].view(want.shape)
    got = gg.backend.gmm(a.cuda(), b.cuda(), sizes, trans_a=mode == 'tn', trans_b=mode == 'nt', c=c)
    assert rel_err(got.cpu(), want) < TOL
    assert bool((guard[:2048] == 3.0).all()) and bool((guard[2048 + want.numel():] == 3.0).all())
    if mode == 'tn':
        for e, s in enumerate(sizes.tolist()):
            if s == 0:
                assert torch.count_nonzero(got[e]) == 0


SCHEDULES = [  # name, groups, rows, k, n: one case per branch of the device-side tile schedulers
    ('more than 64 experts, small tile', 80, 24000, 128, 512),
    ('more than 64 experts, big tile', 72, 28800, 128, 768),
    ('fewer tiles than compute units, cut in halves', 2, 1000, 256, 2048),
    ('last round more than half full, not cut', 4, 6400, 128, 2048),
    ('several full rounds and a cut tail', 8, 9000, 64, 2048),
    ('TN with two tiles per workgroup', 4, 3000, 512, 768),
    ('one row per expert', 64, 64, 64, 256),
    ('256 experts: four per lane of the tile table', 256, 40000, 128, 512),
    ('300 experts: five per lane, the last lanes empty', 300, 30000, 64, 264),
    ('65 experts: two per lane', 65, 9000, 192, 512),
]


@pytest.mark.parametrize('name,groups,rows,k,n', SCHEDULES)
def test_gmm_tile_schedules(gg, name, groups, rows, k, n):
    sizes = _sizes(groups, rows, seed=groups + rows, empty=(1,) if groups > 2 else ())
    torch.manual_seed(groups)
    a = torch.randn(rows, k, device='cuda').bfloat16()
    b_nt = (torch.randn(groups, n, k, device='cuda') * 0.1).bfloat16()
    b_nn = (torch.randn(groups, k, n, device='cuda') * 0.1).bfloat16()
    b_tn = torch.randn(rows, n, device='cuda').bfloat16()
    for b, ta, tb in ((b_nt, False, True), (b_nn, False, False), (b_tn, True, False)):
        got = gg.backend.gmm(a, b, sizes, trans_a=ta, trans_b=tb)
        ref = _ref_gpu(a, b, sizes, ta, tb)
        assert rel_err(got, ref) < TOL and max_block_err(got, ref) < 2 * TOL, (name, ta, tb)
        again = gg.backend.gmm(a, b, sizes.cuda().int(), trans_a=ta, trans_b=tb)
        assert torch.equal(again, got)                              # same schedule, same summation order: bit-identical


SPLIT_TAILS = [  # row tiles, column tiles, k (per operand pair): the tail of `row tiles x column tiles` tiles on 256
    # compute units is cut along the reduction into min(256 // tail, 8, K tiles // 8) parts
    (12, 1, 1024),    # 12 tiles, 16 K tiles: two parts
    (12, 1, 4096),    # eight parts
    (68, 16, 1024),   # four full rounds and 64 tiles: four parts (the shape of a Mixtral-sized second product, shorter)
    (85, 1, 768),     # three parts; with two operand pairs the middle one straddles the change of pairs
    (51, 1, 1280),    # five parts
    (36, 1, 1792),    # seven parts
    (3, 43, 640),     # 129 tiles: more than half a round, not cut
    (64, 5, 512),     # a whole round and 64 tiles, reductions too short to cut (8 K tiles): half-height tiles
]


@pytest.mark.parametrize('row_tiles,col_tiles,k', SPLIT_TAILS)
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_gmm_tail_cut_along_the_reduction(gg, row_tiles, col_tiles, k, dtype):
    """NN products whose last round of workgroups is at most half full compute its tiles in parts along K, summed through
    the workspace in a fixed order (mbx_gmm_ws): against fp32, block by block; bit-identical from run to run; the
    workspace's counters are zero again afterwards; without workspace the same values to rounding of the sums' order."""
    from megablocks_amd import _lib
    groups, n = 4, 256 * col_tiles
    per = [256 * (row_tiles // groups)] * groups
    per[0] += 256 * (row_tiles % groups) - 100                       # a ragged last row tile in one expert
    if per[2] >= 256:
        per[2] -= 256
        per[3] += 256
    sizes = torch.tensor(per, dtype=torch.int64)
    rows = int(sizes.sum())
    torch.manual_seed(row_tiles * 100 + col_tiles)
    a = torch.randn(rows, k, device='cuda').to(dtype)
    b = (torch.randn(groups, k, n, device='cuda') * 0.1).to(dtype)
    a2 = torch.randn(rows, k, device='cuda').to(dtype)
    b2 = (torch.randn(groups, k, n, device='cuda') * 0.1).to(dtype)
    ref = _ref_gpu(a, b, sizes, False, False)
    ref2 = ref + _ref_gpu(a2, b2, sizes, False, False)
    guard = torch.full((rows + 64, n), 7.0, device='cuda', dtype=dtype)
    got = gg.backend.gmm(a, b, sizes)
    assert rel_err(got, ref) < TOL and max_block_err(got, ref) < 2 * TOL
    got2 = gg.gmm_dual(a, b, a2, b2, sizes)
    assert rel_err(got2, ref2) < TOL and max_block_err(got2, ref2) < 2 * TOL
    for _ in range(3):
        assert torch.equal(gg.backend.gmm(a, b, sizes), got) and torch.equal(gg.gmm_dual(a, b, a2, b2, sizes), got2)
    ws = gg._workspaces[(torch.cuda.current_device(), _lib.stream().value)]
    assert int(ws[:4096].count_nonzero()) == 0                      # every launch leaves the counters as it found them
    assert bool((guard == 7.0).all())
    # the C ABI without a workspace: one workgroup per tile (or half tile)
    bins = torch.cumsum(sizes, 0).int().cuda()
    plain = torch.empty_like(got)
    _lib.check(_lib.lib.mbx_gmm(_lib.ptr(a), _lib.ptr(b), _lib.ptr(plain), _lib.dtype_of(a), _lib.ptr(bins), groups, rows, k, n,
                                _lib.NN, _lib.stream()))
    assert rel_err(plain, ref) < TOL and rel_err(plain.float(), got.float()) < 2e-3
    # a workspace too small for two parts per tail tile, or misaligned: ignored
    small = torch.zeros(4096 + 100, dtype=torch.uint8, device='cuda')
    out = torch.empty_like(got)
    _lib.check(_lib.lib.mbx_gmm_ws(_lib.ptr(a), _lib.ptr(b), None, None, _lib.ptr(out), _lib.dtype_of(a), _lib.ptr(bins), groups,
                                   rows, k, n, _lib.NN, _lib.ptr(small), small.numel(), _lib.stream()))
    assert torch.equal(out, plain)
    assert _lib.lib.mbx_gmm_ws(_lib.ptr(a), _lib.ptr(b), _lib.ptr(a2), None, _lib.ptr(out), _lib.dtype_of(a), _lib.ptr(bins), groups,
                               rows, k, n, _lib.NN, None, 0, _lib.stream()) == _lib.EINVAL


MIXED_ROWS = [  # per-expert row counts around the boundaries between full (256-row) and half-height (128-row) tiles
    [256, 257, 300, 384, 385, 129, 128, 1, 0, 512, 640, 127],
    [300] * 48,                       # full and half-height tiles alternate along the tile list, several rounds
    [260, 250] * 40,                  # more than 64 experts
    [130] * 64,                       # on average below the full tile: half-height tiles only
    [2048 + 37 * (i % 5) for i in range(8)] + [100, 2100, 0, 385],     # many full tiles, a few short last ones
    [(300, 0, 700, 256, 40)[i % 5] for i in range(150)],             # short last tiles with several experts per lane
]


@pytest.mark.parametrize('rows_per_expert', MIXED_ROWS, ids=lambda r: f'{len(r)}experts')
@pytest.mark.parametrize('k,n', [(256, 1024), (512, 264)])
def test_gmm_full_and_half_height_row_tiles(gg, rows_per_expert, k, n):
    sizes = torch.tensor(rows_per_expert, dtype=torch.int64)
    groups, rows = len(rows_per_expert), int(sizes.sum())
    torch.manual_seed(rows)
    a = torch.randn(rows, k, device='cuda').bfloat16()
    b_nt = (torch.randn(groups, n, k, device='cuda') * 0.1).bfloat16()
    b_nn = (torch.randn(groups, k, n, device='cuda') * 0.1).bfloat16()
    for b, tb in ((b_nt, True), (b_nn, False)):
        got = gg.backend.gmm(a, b, sizes, trans_b=tb)
        ref = _ref_gpu(a, b, sizes, False, tb)
        assert rel_err(got, ref) < TOL and max_block_err(got, ref) < 2 * TOL, tb
    a2 = torch.randn(rows, k, device='cuda').bfloat16()
    b2 = (torch.randn(groups, k, n, device='cuda') * 0.1).bfloat16()
    got = gg.gmm_dual(a, b_nn, a2, b2, sizes)
    ref = _ref_gpu(a, b_nn, sizes, False, False).float() + _ref_gpu(a2, b2, sizes, False, False).float()
    assert rel_err(got.float(), ref) < TOL


@pytest.mark.parametrize('k', [264, 384, 392, 648, 1408])      # k mod 256 = 8, 128, 136, 136, 128: the last row of tiles
@pytest.mark.parametrize('n', [256, 520])                      # is half-height up to 128 rows, full above
def test_gmm_tn_last_row_of_tiles(gg, k, n):
    sizes = torch.tensor([700, 0, 64, 3000, 1, 331])
    rows = int(sizes.sum())
    torch.manual_seed(k + n)
    a = torch.randn(rows, k, device='cuda').bfloat16()
    b = torch.randn(rows, n, device='cuda').bfloat16()
    ref = _ref_gpu(a, b, sizes, True, False)
    guard = torch.full((ref.numel() + 4096,), 3.0, device='cuda').bfloat16()
    c = guard[2048:2048 + ref.numel()].view(ref.shape)
    got = gg.backend.gmm(a, b, sizes, trans_a=True, c=c)
    assert rel_err(got, ref) < TOL and max_block_err(got, ref) < 2 * TOL
    assert torch.count_nonzero(got[1]) == 0
    assert bool((guard[:2048] == 3.0).all()) and bool((guard[2048 + ref.numel():] == 3.0).all())


# Short reductions whose experts load the XCDs alike are dealt to XCDs as whole experts (the kernel decides from the
# row counts): equal experts, equal experts next to empty ones, a count that is no multiple of eight (never balanced:
# an eighth of every expert per XCD, as for long reductions), nearly equal ones, and one XCD's worth of experts.
WHOLE_EXPERTS = [[200] * 16, [256, 0] * 8, [320] * 12, [250 + (7 * i) % 13 for i in range(64)], [192] * 8, [64] * 40 + [0] * 24]


@pytest.mark.parametrize('rows_per_expert', WHOLE_EXPERTS, ids=lambda r: f'{len(r)}x{r[0]}')
@pytest.mark.parametrize('k,n', [(1024, 512), (264, 1032), (128, 256)])
def test_gmm_tn_short_reductions_dealt_by_expert(gg, rows_per_expert, k, n):
    sizes = torch.tensor(rows_per_expert)
    rows = int(sizes.sum())
    torch.manual_seed(rows + k)
    a = torch.randn(rows, k, device='cuda').bfloat16()
    b = torch.randn(rows, n, device='cuda').bfloat16()
    ref = _ref_gpu(a, b, sizes, True, False)
    guard = torch.full((ref.numel() + 4096,), 3.0, device='cuda').bfloat16()
    c = guard[2048:2048 + ref.numel()].view(ref.shape)
    got = gg.backend.gmm(a, b, sizes.cuda(), trans_a=True, c=c)
    assert rel_err(got, ref) < TOL and max_block_err(got, ref) < 2 * TOL
    for e, r in enumerate(rows_per_expert):
        if r == 0:
            assert torch.count_nonzero(got[e]) == 0
    assert bool((guard[:2048] == 3.0).all()) and bool((guard[2048 + ref.numel():] == 3.0).all())


def _random_shapes(count, seed):
    g = torch.Generator().manual_seed(seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    shapes = []
    for i in range(count):
        groups, rows = r(1, 70), r(1, 5000)
        if i % 3 == 0:      # the pipelined kernels: k a multiple of 64
            k, n = 64 * r(1, 17), 8 * r(1, 140)
        elif i % 3 == 1:    # the register-staged kernels: multiples of 8
            k, n = 8 * r(1, 140), 8 * r(1, 140)
        else:               # anything
            k, n = r(1, 600), r(1, 600)
        shapes.append((groups, rows, k, n))
    return shapes


@pytest.mark.parametrize('groups,rows,k,n', _random_shapes(36, seed=7))
def test_gmm_random_shapes_with_canaries(gg, groups, rows, k, n):
    sizes = _sizes(groups, rows, seed=groups * 7 + rows, empty=(0,) if groups > 3 else ())
    torch.manual_seed(rows)
    a = torch.randn(rows, k, device='cuda').bfloat16()
    for mode in ('nn', 'nt', 'tn'):
        if mode == 'tn':
            b = torch.randn(rows, n, device='cuda').bfloat16()
        else:
            b = (torch.randn((groups, n, k) if mode == 'nt' else (groups, k, n), device='cuda') * 0.1).bfloat16()
        ref = _ref_gpu(a, b, sizes, mode == 'tn', mode == 'nt')
        guard = torch.full((ref.numel() + 4096,), 3.0, device='cuda').bfloat16()       # canary around the output
        c = guard[2048:2048 + ref.numel()].view(ref.shape)
        got = gg.backend.gmm(a, b, sizes, trans_a=mode == 'tn', trans_b=mode == 'nt', c=c)
        assert rel_err(got, ref) < TOL and max_block_err(got, ref) < 2 * TOL, mode
        assert bool((guard[:2048] == 3.0).all()) and bool((guard[2048 + ref.numel():] == 3.0).all()), mode


DUAL = [  # groups, rows, k, n, single launch expected
    (8, 4000, 512, 1024, True), (3, 700, 256, 264, True), (64, 16384, 1408, 2048, True), (70, 21000, 256, 512, True),
    (4, 1000, 192, 256, False), (2, 300, 100, 36, False), (1, 64, 256, 8, True),
]


@pytest.mark.parametrize('groups,rows,k,n,single', DUAL)
@pytest.mark.parametrize('trans_b', [False, True])
def test_gmm_dual_is_the_sum_of_two_products(gg, groups, rows, k, n, single, trans_b):
    from megablocks_amd import _lib
    sizes = _sizes(groups, rows, seed=rows + k, empty=(1,) if groups > 2 else ())
    torch.manual_seed(k)
    a, a2 = (torch.randn(rows, k, device='cuda').bfloat16() for _ in range(2))
    shape = (groups, n, k) if trans_b else (groups, k, n)
    b, b2 = ((torch.randn(shape, device='cuda') * 0.1).bfloat16() for _ in range(2))
    ref = _ref_gpu(a, b, sizes, False, trans_b) + _ref_gpu(a2, b2, sizes, False, trans_b)
    _lib.profile_hook = []
    try:
        got = gg.gmm_dual(a, b, a2, b2, sizes, trans_b=trans_b)
        names = [r[0] for r in _lib.profile_hook]
    finally:
        _lib.profile_hook = None
    assert (names == ['gmm_nt_dual' if trans_b else 'gmm_nn_dual']) == single   # else: two products and a sum
    assert got.dtype == torch.bfloat16 and rel_err(got, ref) < TOL and max_block_err(got, ref) < 2 * TOL
    c = torch.full((rows, n), 5.0, device='cuda').bfloat16()
    assert gg.gmm_dual(a, b, a2, b2, sizes.cuda().int(), trans_b=trans_b, c=c) is c and torch.equal(c, got)
    with pytest.raises(ValueError):
        gg.gmm_dual(a, b, a2[:, :-8], b2, sizes, trans_b=trans_b)


def _ref_in_pieces(check, a, b, sizes, trans_a, trans_b, got):
    """Compare `got` with the fp32 product expert by expert (an fp32 copy of a whole operand of several GiB
    at once is not needed then); `check(piece_of_got, reference_piece)`."""
    start = 0
    for e, n in enumerate(sizes.tolist()):
        ae = a[start:start + n].float()
        if trans_a and n:
            check(got[e], ae.t() @ b[start:start + n].float())
        elif n:
            check(got[start:start + n], ae @ (b[e].float().t() if trans_b else b[e].float()))
        start += n


LARGE = [  # name, rows per expert, k, n: the [rows, k] or the [rows, n] matrix (or one expert's share of it) of 2 .. 5 GiB
    ('rows-by-k-2.3GiB', [150000, 0, 100000, 50000], 4096, 256),
    ('rows-by-n-2.3GiB', [150000, 0, 100000, 50000], 256, 4096),
    ('one-expert-4.3GiB-of-4.6GiB', [20000, 560000, 20], 4096, 128),
]


@pytest.mark.parametrize('name,rows_per_expert,k,n', LARGE, ids=[c[0] for c in LARGE])
def test_gmm_operands_beyond_2GiB(gg, name, rows_per_expert, k, n):
    """Byte offsets inside the big matrices pass 2^31 and 2^32: same kernels, same tolerance."""
    from megablocks_amd import _lib
    sizes = torch.tensor(rows_per_expert)
    rows, groups = int(sizes.sum()), len(rows_per_expert)
    torch.manual_seed(rows % 1000)
    a = torch.empty(rows, k, device='cuda', dtype=torch.bfloat16).normal_()
    a2 = a.flip(0)
    w_nn = torch.empty(groups, k, n, device='cuda', dtype=torch.bfloat16).normal_(std=0.1)
    w_nt = torch.empty(groups, n, k, device='cuda', dtype=torch.bfloat16).normal_(std=0.1)
    b_tn = torch.empty(rows, n, device='cuda', dtype=torch.bfloat16).normal_()
    assert max(a.numel(), b_tn.numel()) * 2 >= 2 ** 31

    def check(got, ref):
        assert rel_err(got, ref) < TOL and max_block_err(got, ref, bm=256, bn=256) < 2 * TOL

    _lib.profile_hook = []
    try:
        nn = gg.backend.gmm(a, w_nn, sizes)
        nt = gg.backend.gmm(a, w_nt, sizes, trans_b=True)
        tn = gg.backend.gmm(a, b_tn, sizes, trans_a=True)
        dual = gg.gmm_dual(a, w_nn, a2, w_nn, sizes) if k >= 256 else None
        names = [r[0] for r in _lib.profile_hook]
    finally:
        _lib.profile_hook = None
    _ref_in_pieces(check, a, w_nn, sizes, False, False, nn)
    _ref_in_pieces(check, a, w_nt, sizes, False, True, nt)
    _ref_in_pieces(check, a, b_tn, sizes, True, False, tn)
    assert torch.count_nonzero(tn[[i for i, s in enumerate(rows_per_expert) if s == 0]]) == 0
    if dual is not None:
        assert names[-1] == 'gmm_nn_dual'            # one launch, not two products and a sum
        second = gg.backend.gmm(a2, w_nn, sizes)
        _ref_in_pieces(check, a2, w_nn, sizes, False, False, second)
        assert rel_err(dual, nn.float() + second.float()) < TOL


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize('act_name', ['silu', 'gelu_tanh'])
def test_fused_gated_activation_matches_the_two_step_formulation(dtype, act_name):
    import torch.nn.functional as F
    from megablocks_amd.layers.arguments import DEFAULT_ACTIVATION_FN
    from megablocks_amd.layers.glu import gated_activation
    fn = F.silu if act_name == 'silu' else DEFAULT_ACTIVATION_FN
    a = (torch.randn(777, 1408) * 2).to(dtype).cuda().requires_grad_(True)
    b = torch.randn(777, 1408).to(dtype).cuda().requires_grad_(True)
    g = torch.randn(777, 1408).to(dtype).cuda()
    out = gated_activation(fn, a, b)
    out.backward(g)
    a2, b2 = a.detach().clone().requires_grad_(True), b.detach().clone().requires_grad_(True)
    want = fn(a2) * b2                                   # the reference's two element-wise ops (glu.py:89)
    want.backward(g)
    tol = 1e-6 if dtype == torch.float32 else 1e-2
    assert rel_err(out, want) < tol and rel_err(a.grad, a2.grad) < tol and rel_err(b.grad, b2.grad) < tol
    if dtype != torch.float32:                           # forward: same roundings -> almost always the same bits
        assert float((out != want).float().mean()) < 1e-3
    wantf = fn(a.detach().float().cpu()) * b.detach().float().cpu()      # CPU fp32 check of the math itself
    assert rel_err(out.cpu(), wantf) < (1e-5 if dtype == torch.float32 else 1e-2)
    odd = torch.randn(5, 3).to(dtype).cuda()             # not a multiple of 16 bytes: plain torch ops
    assert torch.equal(gated_activation(fn, odd, odd), fn(odd) * odd)


EPILOGUE = [  # groups, rows, k, n -- full and half-height tiles, partial last column tile, shapes off the fused path
    (8, 4096, 1024, 4096), (64, 16384, 1024, 1024), (5, 1500, 320, 264), (3, 700, 128, 1408), (1, 37, 64, 8),
    (4, 1000, 72, 256), (16, 6000, 2048, 520), (72, 5000, 128, 264),
]


@pytest.mark.parametrize('groups,rows,k,n', EPILOGUE)
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16, torch.float32])
def test_gmm_with_activation_epilogues(gg, groups, rows, k, n, dtype):
    """gmm_act: (x @ w1^T, gelu_tanh of it) in one launch; gmm_dact: round(dy @ w2^T) * gelu_tanh'(pre).  Against the
    two-step formulation of mlp.py:521-522 and mlp.py:478-483 / gelu.py:9-13 in fp32 with the reference's roundings."""
    torch.manual_seed(groups * 7 + n)
    sizes = _sizes(groups, rows, seed=rows + k, empty=(1,) if groups > 2 else ())
    a = torch.randn(rows, k, device='cuda').to(dtype)
    b = (torch.randn(groups, n, k, device='cuda') * (1.5 / k ** 0.5)).to(dtype)      # pre-activations of order one
    ref = _ref_gpu(a, b, sizes, False, True)
    want_pre = ref.to(dtype)
    want_act = torch.nn.functional.gelu(want_pre.float(), approximate='tanh')
    guard = torch.full((rows + 64, n), 5.0, device='cuda', dtype=dtype)
    pre, act = gg.gmm_act(a, b, sizes, fuse=True)
    assert pre.shape == (rows, n) and act.shape == (rows, n) and pre.dtype == dtype and act.dtype == dtype
    tol = 1e-4 if dtype == torch.float32 else TOL
    assert rel_err(pre.float(), ref) < tol
    assert torch.equal(pre, gg.backend.gmm(a, b, sizes, trans_b=True))         # the product itself is the same kernel's
    # the activation is taken of the stored product: one rounding step of the output type away from the fp32 formula
    assert rel_err(act.float(), torch.nn.functional.gelu(pre.float(), approximate='tanh')) < (1e-6 if dtype == torch.float32 else 3e-3)
    assert rel_err(act.float(), want_act) < tol

    dy = torch.randn(rows, k, device='cuda').to(dtype)
    x_pre = (torch.randn(rows, n, device='cuda') * 1.5).to(dtype)
    prod = _ref_gpu(dy, b, sizes, False, True).to(dtype).float()
    want = prod * oracle.gelu_tanh_backward(torch.ones_like(prod).cpu(), x_pre.float().cpu()).cuda()
    got = gg.gmm_dact(dy, b, x_pre, sizes, fuse=True)
    assert got.shape == (rows, n) and got.dtype == dtype and rel_err(got.float(), want) < tol
    out = guard[:rows]
    assert gg.gmm_dact(dy, b, x_pre, sizes, c=out, fuse=True) is out and torch.equal(out, got)
    two_step = gg.gmm_dact(dy, b, x_pre, sizes, fuse=False)            # product, then gelu_backward_ in place
    assert rel_err(two_step.float(), want) < tol and rel_err(got.float(), two_step.float()) < (1e-6 if dtype == torch.float32 else 4e-3)
    pre2, act2 = gg.gmm_act(a, b, sizes, fuse=False)
    assert torch.equal(pre2, pre) and rel_err(act.float(), act2.float()) < (1e-6 if dtype == torch.float32 else 4e-3)
    assert bool((guard[rows:] == 5.0).all())
    with pytest.raises(ValueError):
        gg.gmm_dact(dy, b, x_pre, sizes, c=x_pre)                              # the epilogue reads pre while it writes c
    with pytest.raises(ValueError):
        gg.gmm_act(a, b[:, :, :k - 8].contiguous(), sizes)


@pytest.mark.parametrize('groups,rows,k,n', EPILOGUE)
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize('act', [0, 1], ids=['silu', 'gelu_tanh'])
def test_gmm_with_gated_activation_backward_epilogue(gg, groups, rows, k, n, dtype, act):
    """gmm_dglu: with g = round(dy @ w2^T), (round(g x2) act'(x1), g round(act(x1))) in one launch, against autograd's
    gradient of act(x1) * x2 in fp32 (glu.py:120-124,135-153) and against the product followed by the element-wise
    kernel, which it must equal to a rounding step of the output type."""
    from megablocks_amd.layers.glu import _glu_backward
    torch.manual_seed(groups * 11 + n + act)
    sizes = _sizes(groups, rows, seed=rows + k + 1, empty=(1,) if groups > 2 else ())
    dy = torch.randn(rows, k, device='cuda').to(dtype)
    b = (torch.randn(groups, n, k, device='cuda') * (1.0 / k ** 0.5)).to(dtype)
    x1 = (torch.randn(rows, n, device='cuda') * 1.5).to(dtype)
    x2 = torch.randn(rows, n, device='cuda').to(dtype)
    g = _ref_gpu(dy, b, sizes, False, True).to(dtype).float()
    fn = torch.nn.functional.silu if act == 0 else (lambda t: torch.nn.functional.gelu(t, approximate='tanh'))
    a_, b_ = x1.float().requires_grad_(True), x2.float().requires_grad_(True)
    (fn(a_) * b_).backward(g)
    d1, d2 = gg.gmm_dglu(dy, b, x1, x2, sizes, act, fuse=True)
    tol = 1e-4 if dtype == torch.float32 else TOL
    assert d1.shape == (rows, n) and d2.shape == (rows, n) and d1.dtype == dtype and d2.dtype == dtype
    assert rel_err(d1.float(), a_.grad) < tol and rel_err(d2.float(), b_.grad) < tol
    t1, t2 = _glu_backward(gg.backend.gmm(dy, b, sizes, trans_b=True), x1, x2, act)
    step = 1e-6 if dtype == torch.float32 else 4e-3
    assert rel_err(d1.float(), t1.float()) < step and rel_err(d2.float(), t2.float()) < step
    u1, u2 = gg.gmm_dglu(dy, b, x1, x2, sizes.cuda(), act, fuse=False)
    assert torch.equal(u1, t1) and torch.equal(u2, t2)
    with pytest.raises(ValueError):
        gg.gmm_dglu(dy, b, x1[:, :n - 8].contiguous(), x2, sizes, act)


@pytest.mark.parametrize('groups,rows,k,n', EPILOGUE + [(6, 2500, 256, 1416), (2, 300, 64, 136)])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize('act', [0, 1], ids=['silu', 'gelu_tanh'])
def test_gmm_with_gated_activation_epilogue(gg, groups, rows, k, n, dtype, act):
    """gmm_glu: (x @ w1^T, x @ v1^T, round(round(act(x1)) x2)) in one launch (glu.py:201-204): both products must be
    the plain kernel's bit for bit, the gated activation within a rounding step of the element-wise kernel's and of the
    fp32 formula on the stored products."""
    from megablocks_amd.layers.glu import _glu_forward
    torch.manual_seed(groups * 13 + n + act)
    sizes = _sizes(groups, rows, seed=rows + k + 2, empty=(1,) if groups > 2 else ())
    a = torch.randn(rows, k, device='cuda').to(dtype)
    w1 = (torch.randn(groups, n, k, device='cuda') * (1.5 / k ** 0.5)).to(dtype)
    v1 = (torch.randn(groups, n, k, device='cuda') * (1.0 / k ** 0.5)).to(dtype)
    guard = torch.full((3, rows + 16, n), 7.0, device='cuda', dtype=dtype)
    x1, x2, h = gg.gmm_glu(a, w1, v1, sizes, act, fuse=True)
    p1, p2 = gg.backend.gmm(a, w1, sizes, trans_b=True), gg.backend.gmm(a, v1, sizes.cuda(), trans_b=True)
    assert x1.shape == (rows, n) and h.shape == (rows, n) and h.dtype == dtype
    assert torch.equal(x1, p1) and torch.equal(x2, p2)
    fn = torch.nn.functional.silu if act == 0 else (lambda t: torch.nn.functional.gelu(t, approximate='tanh'))
    want = fn(p1.float()).to(dtype).float() * p2.float()
    step = 1e-6 if dtype == torch.float32 else 4e-3
    assert rel_err(h.float(), want) < step
    assert rel_err(h.float(), _glu_forward(p1, p2, act).float()) < step
    y1, y2, g = gg.gmm_glu(a, w1, v1, sizes, act, fuse=False)
    assert torch.equal(y1, p1) and torch.equal(y2, p2) and torch.equal(g, _glu_forward(p1, p2, act))
    assert bool((guard == 7.0).all())
    with pytest.raises(ValueError):
        gg.gmm_glu(a, w1, v1[:, :n - 8].contiguous(), sizes, act)


def _routing(tokens, experts, top_k, seed, blocking=0):
    """(indices, bin_ids, bins, padded_bins or None, tokens_per_expert) of a random assignment, from the library's ops."""
    from megablocks_amd import ops
    g = torch.Generator().manual_seed(seed)
    top = torch.randint(0, experts, (tokens * top_k,), generator=g, dtype=torch.int32)
    if experts > 2:
        top[top == 1] = 0                                   # an expert without tokens
    top = top.cuda()
    end_bit = max(int(math.ceil(math.log2(experts))), 1)
    bin_ids, indices = ops.sort(top, end_bit)
    tpe = ops.histogram(top, experts)
    bins = ops.inclusive_cumsum(tpe, 0).view(-1)
    padded_bins = None
    if blocking:
        padded_bins = ops.inclusive_cumsum(ops.round_up(tpe, blocking), 0).view(-1)
    return indices, bin_ids, bins, padded_bins, tpe


GATHERED = [  # tokens, experts, top_k, k, n, blocking
    (4096, 8, 2, 1024, 512, 0), (3000, 5, 1, 320, 264, 0), (700, 3, 4, 128, 1408, 0), (37, 1, 1, 64, 8, 0),
    (2048, 16, 4, 256, 384, 128), (1000, 72, 2, 128, 264, 128), (5000, 64, 1, 1024, 1024, 0), (9, 4, 2, 64, 136, 128),
    (3000, 12, 3, 128, 256, 0), (4000, 64, 6, 192, 1408, 0), (1111, 9, 7, 64, 128, 128), (500, 40, 33, 64, 64, 0),
]


@pytest.mark.parametrize('tokens,experts,top_k,k,n,blocking', GATHERED)
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_gmm_on_rows_gathered_on_the_fly(gg, tokens, experts, top_k, k, n, blocking, dtype):
    """gmm_gather: the first product(s) of the experts reading their rows from the ungathered tokens must equal, bit
    for bit, ops.gather / ops.padded_gather (dmoe.py:219 / :273) followed by gmm, gmm_act and gmm_glu: the same
    products over the same operand values in the same order, only fetched from other addresses."""
    torch.manual_seed(tokens + n)
    indices, bin_ids, bins, padded_bins, tpe = _routing(tokens, experts, top_k, seed=tokens + k, blocking=blocking)
    x = torch.randn(tokens, k, device='cuda').to(dtype)
    w1 = (torch.randn(experts, n, k, device='cuda') * (1.5 / k ** 0.5)).to(dtype)
    v1 = (torch.randn(experts, n, k, device='cuda') * (1.0 / k ** 0.5)).to(dtype)
    rows = tokens * top_k if padded_bins is None else int(padded_bins[-1])
    sizes = tpe if padded_bins is None else torch.diff(padded_bins, prepend=padded_bins.new_zeros(1))
    src = gg.GatheredRows(x, indices, bin_ids, bins, padded_bins, top_k, rows)
    a = src.materialize()
    assert a.shape == (rows, k)
    guard = torch.full((3, rows + 16, n), 7.0, device='cuda', dtype=dtype)
    (c,) = gg.gmm_gather(src, w1, sizes)
    assert torch.equal(c, gg.backend.gmm(a, w1, sizes, trans_b=True))
    c, h = gg.gmm_gather(src, w1, sizes, act=gg.ACT_GELU_TANH)
    want_c, want_h = gg.gmm_act(a, w1, sizes, fuse=True)
    assert torch.equal(c, want_c) and torch.equal(h, want_h)
    # ... and, directly, the CPU oracle's gather (kernels.py:107-170) and grouped product on the same inputs, with the
    # activations of mlp.py:521-522 / glu.py:201-204 applied to the product as stored
    cpu = lambda t: None if t is None else t.cpu()
    if padded_bins is None:
        o_a = oracle.gather(cpu(x), cpu(indices), cpu(bin_ids), None, cpu(bins), top_k)
    else:
        o_a = oracle.padded_gather(cpu(x), cpu(indices), cpu(bin_ids), None, cpu(bins), cpu(padded_bins), top_k)
    assert torch.equal(a.cpu(), o_a)
    o_x1 = oracle.gmm(o_a, cpu(w1), cpu(sizes), trans_b=True)
    o_x2 = oracle.gmm(o_a, cpu(v1), cpu(sizes), trans_b=True)
    gelu = lambda t: torch.nn.functional.gelu(t.float(), approximate='tanh').to(dtype)
    silu = lambda t: torch.nn.functional.silu(t.float()).to(dtype)
    if rows:
        assert rel_err(c.cpu(), o_x1) < TOL and rel_err(h.cpu(), gelu(o_x1)) < TOL
    for act in (0, 1):
        x1, x2, h = gg.gmm_gather(src, w1, sizes, b2=v1, act=act)
        w_x1, w_x2, w_h = gg.gmm_glu(a, w1, v1, sizes, act, fuse=True)
        assert torch.equal(x1, w_x1) and torch.equal(x2, w_x2) and torch.equal(h, w_h)
        if rows:
            o_h = ((silu, gelu)[act](o_x1).float() * o_x2.float()).to(dtype)
            assert rel_err(x1.cpu(), o_x1) < TOL and rel_err(x2.cpu(), o_x2) < TOL and rel_err(h.cpu(), o_h) < TOL
    assert bool((guard == 7.0).all())


COMBINED = [  # tokens (= rows: one expert per token), experts, k, n
    (4096, 8, 1024, 512), (3000, 5, 320, 264), (37, 1, 64, 8), (5000, 64, 1024, 1024), (16384, 64, 512, 1024),
    (700, 3, 128, 1408), (2600, 4, 2048, 256), (300, 40, 64, 136), (511, 2, 1024, 64), (65, 1, 1024, 512), (8192, 100, 1024, 256),
]


@pytest.mark.parametrize('tokens,experts,k,n', COMBINED)
@pytest.mark.parametrize('dtype,w_dtype', [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16),
                                           (torch.bfloat16, torch.float32), (torch.float16, torch.float32),
                                           (torch.bfloat16, None)])
def test_gmm_with_the_combine_in_the_epilogue(gg, monkeypatch, tokens, experts, k, n, dtype, w_dtype):
    """gmm_scatter: with one expert per token the experts' second product (mlp.py:523, glu.py:205) writes the layer's
    weighted combine (dmoe.py:280, kernels.py:173-207) from its store phase.  Product and combined output must equal,
    bit for bit, gmm followed by the scatter kernel (the same roundings in the same places), and meet the CPU oracle's
    product and scatter directly; rows of the output that no assignment names are left alone."""
    from megablocks_amd.backend import kernels
    torch.manual_seed(tokens + n)
    indices, bin_ids, bins, _, tpe = _routing(tokens, experts, 1, seed=tokens + k)
    h = torch.randn(tokens, k, device='cuda').to(dtype)
    w2 = (torch.randn(experts, k, n, device='cuda') * (1.5 / k ** 0.5)).to(dtype)
    weights = None if w_dtype is None else (torch.rand(tokens, device='cuda') + 0.25).to(w_dtype)
    combine = gg.CombinedRows(indices, bin_ids, bins, weights)
    monkeypatch.setattr(gg, 'GMM_WORKSPACE', False)   # the plain product without a tail cut along K, as the combined launch computes it
    want_y = gg.backend.gmm(h, w2, tpe)
    want_out = kernels.scatter(want_y, indices, bin_ids, weights, bins, 1)
    y, out = gg.gmm_scatter(h, w2, tpe, combine)
    assert torch.equal(y, want_y) and torch.equal(out, want_out)
    y2, out2 = gg.gmm_scatter(h, w2, tpe, combine, keep_product=False)
    assert torch.equal(out2, want_out) and (y2 is None or torch.equal(y2, want_y))
    cpu = lambda t: None if t is None else t.cpu()
    o_y = oracle.gmm(cpu(h), cpu(w2), cpu(tpe))
    o_out = oracle.scatter(o_y, cpu(indices), cpu(bin_ids), cpu(weights), cpu(bins), 1)
    assert rel_err(y.cpu(), o_y) < TOL and rel_err(out.cpu(), o_out) < TOL
    # assignments outside the tokens, and a token nobody names: those rows are not combined, that row is not written
    bad = indices.clone()
    bad[::5] = -3
    bad[2::7] = tokens + 11
    lib, _lib = gg.lib, gg._lib
    canvas = torch.full((tokens, n), 3.0, device='cuda', dtype=dtype)
    dbins = tpe.cumsum(0).int()
    rc = lib.mbx_gmm_scatter(_lib.ptr(h), _lib.ptr(w2), None, _lib.ptr(canvas), _lib.dtype_of(h), _lib.ptr(dbins), experts,
                             tokens, k, n, _lib.ptr(bad), _lib.ptr(weights), 0 if weights is None else _lib.dtype_of(weights),
                             tokens, _lib.stream())
    if k % 64 == 0 and n % 8 == 0:
        assert rc == 0
        keep = (bad >= 0) & (bad < tokens)
        want = torch.full_like(canvas, 3.0)
        want[bad[keep].long()] = want_out[indices[keep].long()]    # the rows that kept their assignment
        assert torch.equal(canvas, want)
    else:
        assert rc == _lib.EUNSUPPORTED


GATHERED_TN = [  # tokens, experts, top_k, hidden of the tokens (n), columns of the other operand (k), blocking
    (4096, 8, 2, 1024, 512, 0), (3000, 5, 1, 320, 264, 0), (700, 3, 4, 128, 1408, 0), (2048, 16, 4, 256, 384, 128),
    (1000, 72, 2, 128, 264, 128), (5000, 64, 1, 1024, 1024, 0), (9, 4, 2, 64, 136, 128), (4000, 64, 6, 192, 1408, 0),
    (1111, 9, 7, 64, 256, 128), (500, 40, 33, 64, 192, 0), (2500, 4, 2, 2048, 320, 0),
]


@pytest.mark.parametrize('tokens,experts,top_k,n,k,blocking', GATHERED_TN)
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
def test_gmm_weight_gradient_on_rows_gathered_on_the_fly(gg, tokens, experts, top_k, n, k, blocking, dtype):
    """gmm_tn_gather: the weight gradient d^T @ x_gathered of the experts' first product (mlp.py:485-491, glu.py:154-159)
    reading the rows of x through the sorted assignments must equal, bit for bit, ops.gather / ops.padded_gather
    (dmoe.py:219 / :273) followed by gmm(trans_a=True), and the CPU oracle's gather and product to 1e-2."""
    torch.manual_seed(tokens + k)
    indices, bin_ids, bins, padded_bins, tpe = _routing(tokens, experts, top_k, seed=tokens + n, blocking=blocking)
    x = torch.randn(tokens, n, device='cuda').to(dtype)
    rows = tokens * top_k if padded_bins is None else int(padded_bins[-1])
    sizes = tpe if padded_bins is None else torch.diff(padded_bins, prepend=padded_bins.new_zeros(1))
    d = torch.randn(rows, k, device='cuda').to(dtype)
    src = gg.GatheredRows(x, indices, bin_ids, bins, padded_bins, top_k, rows)
    guard = torch.full((experts + 2, k, n), 7.0, device='cuda', dtype=dtype)
    got = gg.gmm_tn_gather(d, src, sizes)
    assert got is not None and got.shape == (experts, k, n)
    copy = src.materialize()
    assert torch.equal(got, gg.backend.gmm(d, copy, sizes, trans_a=True))
    again = gg.gmm_tn_gather(d, src, sizes)                       # with the row table the first call left on src
    assert torch.equal(again, got) and getattr(src, '_row_table', None) is not None
    assert torch.equal(src.weight_gradient(d, sizes), got)
    cpu = lambda t: None if t is None else t.cpu()
    if padded_bins is None:
        o_x = oracle.gather(cpu(x), cpu(indices), cpu(bin_ids), None, cpu(bins), top_k)
    else:
        o_x = oracle.padded_gather(cpu(x), cpu(indices), cpu(bin_ids), None, cpu(bins), cpu(padded_bins), top_k)
    want = oracle.gmm(cpu(d), o_x, cpu(sizes), trans_a=True)
    assert rel_err(got.cpu(), want) < TOL
    for e, cnt in enumerate(tpe.tolist()):
        if cnt == 0:
            assert int(torch.count_nonzero(got[e])) == 0          # an expert without tokens: exactly zero
    assert bool((guard == 7.0).all())


def test_gmm_weight_gradient_on_gathered_rows_edge_cases(gg):
    """Assignments outside [0, tokens * top_k) read as rows of zeros; shapes the kernel does not take come back as None
    and `weight_gradient` then gathers once and multiplies."""
    tokens, experts, top_k, n, k = 600, 4, 2, 128, 256
    indices, bin_ids, bins, _, tpe = _routing(tokens, experts, top_k, seed=5)
    x = torch.randn(tokens, n, device='cuda').bfloat16()
    d = torch.randn(tokens * top_k, k, device='cuda').bfloat16()
    bad = indices.clone()
    bad[::7] = -1
    bad[3::11] = tokens * top_k + 5
    got = gg.gmm_tn_gather(d, gg.GatheredRows(x, bad, bin_ids, bins, None, top_k, tokens * top_k), tpe)
    rows_of_x = x[(indices.long() // top_k)].clone()
    rows_of_x[::7] = 0
    rows_of_x[3::11] = 0
    assert torch.equal(got, gg.backend.gmm(d, rows_of_x, tpe, trans_a=True))
    src = gg.GatheredRows(x, indices, bin_ids, bins, None, top_k, tokens * top_k)
    narrow = d[:, :128].contiguous()                               # at most 128 columns: the half-height tile, no gathered form
    assert gg.gmm_tn_gather(narrow, src, tpe) is None
    assert torch.equal(src.weight_gradient(narrow, tpe), gg.backend.gmm(narrow, src.materialize(), tpe, trans_a=True))
    assert gg.gmm_tn_gather(d.float(), gg.GatheredRows(x.float(), indices, bin_ids, bins, None, top_k, tokens * top_k), tpe) is None
    # no tokens at all: every expert's gradient is zero
    none = gg.GatheredRows(x[:0], indices[:0], bin_ids[:0], torch.zeros_like(bins), None, top_k, 0)
    got = gg.gmm_tn_gather(d[:0], none, torch.zeros_like(tpe))
    assert got.shape == (experts, k, n) and not got.any()


def test_gmm_on_gathered_rows_with_assignments_out_of_range(gg):
    """An assignment outside [0, tokens * top_k) reads as a row of zeros (nothing outside x is fetched), and what the
    library has no kernel for comes back as None (the caller gathers first)."""
    tokens, experts, top_k, k, n = 600, 4, 2, 128, 256
    indices, bin_ids, bins, _, tpe = _routing(tokens, experts, top_k, seed=5)
    x = torch.randn(tokens, k, device='cuda').to(torch.bfloat16)
    w1 = (torch.randn(experts, n, k, device='cuda') / k ** 0.5).to(torch.bfloat16)
    bad = indices.clone()
    bad[::7] = -1
    bad[3::11] = tokens * top_k + 5
    src = gg.GatheredRows(x, bad, bin_ids, bins, None, top_k, tokens * top_k)
    (c,) = gg.gmm_gather(src, w1, tpe)
    a = x[(indices.long() // top_k)].clone()
    a[::7] = 0
    a[3::11] = 0
    assert torch.equal(c, gg.backend.gmm(a, w1, tpe, trans_b=True))
    # fp32, a reduction that is not whole K tiles, 64-bit assignments: no kernel
    assert gg.gmm_gather(gg.GatheredRows(x.float(), indices, bin_ids, bins, None, top_k, tokens * top_k), w1.float(), tpe) is None
    assert gg.gmm_gather(gg.GatheredRows(x[:, :72].contiguous(), indices, bin_ids, bins, None, top_k, tokens * top_k),
                         w1[:, :, :72].contiguous(), tpe) is None
    assert gg.gmm_gather(gg.GatheredRows(x, indices.long(), bin_ids, bins, None, top_k, tokens * top_k), w1, tpe) is None
