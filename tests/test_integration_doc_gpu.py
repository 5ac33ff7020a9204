"""Executes the reference-side binding that the integration guide at the repository root documents: its
`megablocks_ops.py` stand-in and its `gmm` are cut out of the guide's python blocks, loaded as a module, and held to the
oracle.  What the guide shows a maintainer of the reference therefore cannot drift from include/mbx.h."""
import os
import re
import types

import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GUIDE = 'INTEGRATION.md'


@pytest.fixture(scope='module')
def documented():
    from megablocks_amd import _lib
    text = open(os.path.join(ROOT, GUIDE)).read()
    blocks = re.findall(r'```python\n(.*?)```', text, flags=re.S)
    ops_src = next(b for b in blocks if b.lstrip().startswith('# megablocks_ops.py'))
    gmm_src = next(b for b in blocks if 'def gmm(' in b)
    assert "ctypes.CDLL('libmbx.so')" in ops_src
    mod = types.ModuleType('megablocks_ops')
    exec(compile(ops_src.replace("'libmbx.so'", repr(_lib.LIB_PATH)), GUIDE + '#ops', 'exec'), mod.__dict__)
    exec(compile(gmm_src, GUIDE + '#gmm', 'exec'), mod.__dict__)      # uses the helpers of the first block
    return mod


def test_documented_megablocks_ops_names(documented):
    # the seven functions the pybind module exports (csrc/ops.cu:11-19)
    for name in ('histogram', 'sort', 'inclusive_cumsum', 'exclusive_cumsum', 'indices', 'replicate_forward',
                 'replicate_backward'):
        assert callable(getattr(documented, name))


@pytest.mark.parametrize('dtype', [torch.int16, torch.int32, torch.int64])
def test_documented_histogram_sort_cumsum(documented, dtype):
    g = torch.Generator().manual_seed(0)
    x = torch.randint(0, 61, (3, 5000), generator=g).to(dtype)
    assert torch.equal(documented.histogram(x.cuda(), 64).cpu(), oracle.histogram(x, 64))
    assert torch.equal(documented.histogram(x[0].cuda(), 64).cpu(), oracle.histogram(x[0], 64))
    keys = x[1].contiguous()
    for end_bit in (6, 16):
        k_out, p_out = torch.empty_like(keys).cuda(), torch.empty_like(keys).cuda()
        documented.sort(keys.cuda(), end_bit, k_out, p_out)
        want_k, want_p = oracle.sort(keys, end_bit)
        assert torch.equal(k_out.cpu(), want_k) and torch.equal(p_out.cpu(), want_p)
    small = torch.randint(0, 5, (4, 300), generator=g).to(dtype)
    out = torch.empty_like(small).cuda()
    documented.inclusive_cumsum(small.cuda(), 1, out)
    assert torch.equal(out.cpu(), oracle.inclusive_cumsum(small, 1))
    documented.exclusive_cumsum(small.cuda(), 1, out)
    assert torch.equal(out.cpu(), oracle.exclusive_cumsum(small, 1))


def test_documented_indices_and_replicate(documented):
    g = torch.Generator().manual_seed(1)
    tpe = torch.randint(0, 700, (16,), generator=g).int()
    pbins = oracle.inclusive_cumsum(oracle.round_up(tpe, 128), 0).view(-1)
    block_rows, block_cols = int(pbins[-1]) // 128, 8
    out = torch.empty(block_rows * block_cols, dtype=torch.int16, device='cuda')
    documented.indices(pbins.cuda(), 128, block_rows, block_cols, out)
    assert torch.equal(out.cpu(), oracle.topology(pbins, 128, block_rows, block_cols))

    bins = oracle.inclusive_cumsum(tpe, 0).view(-1)
    x = torch.randn(3, 16, generator=g).half()
    rep = torch.empty(3, int(bins[-1]), dtype=torch.float16, device='cuda')
    documented.replicate_forward(x.cuda(), bins.cuda(), rep)
    assert torch.equal(rep.cpu(), oracle.replicate(x, bins, int(bins[-1])))
    grad = torch.randn(3, int(bins[-1]), generator=g).half()
    back = torch.empty(3, 16, dtype=torch.float16, device='cuda')
    documented.replicate_backward(grad.cuda(), bins.cuda(), back)
    want = oracle.replicate_backward(grad, bins)
    assert torch.allclose(back.float().cpu(), want.float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize('mode', ['nn', 'nt', 'tn'])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
def test_documented_gmm(documented, mode, dtype):
    g = torch.Generator().manual_seed(2)
    sizes = torch.tensor([300, 0, 212, 512])
    rows, k, n = int(sizes.sum()), 256, 384
    a = torch.randn(rows, k, generator=g).to(dtype)
    if mode == 'tn':
        b = torch.randn(rows, n, generator=g).to(dtype)
    else:
        b = (torch.randn(4, n, k, generator=g) if mode == 'nt' else torch.randn(4, k, n, generator=g)).mul(0.1).to(dtype)
    want = oracle.gmm(a, b, sizes, trans_a=mode == 'tn', trans_b=mode == 'nt')
    got = documented.gmm(a.cuda(), b.cuda(), sizes, trans_a=mode == 'tn', trans_b=mode == 'nt')
    assert got.shape == want.shape and got.dtype == dtype
    err = float((got.cpu().double() - want.double()).norm() / want.double().norm())
    assert err < 1e-2
    c = torch.empty_like(got)
    assert documented.gmm(a.cuda(), b.cuda(), sizes, trans_a=mode == 'tn', trans_b=mode == 'nt', c=c) is c
    assert torch.equal(c, got)
