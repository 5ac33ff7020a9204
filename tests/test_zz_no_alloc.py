"""mbx_scatter_static — the variant of mbx_scatter that allocates nothing (its slot -> row map lives in a
buffer inside the library image) — against mbx_scatter itself, both called through the C ABI: bit-identical
outputs on two calls in a row, the second on a smaller input, so that what the first call left in the shared
buffer would show.  Collected last (file name) so that it also runs after every other test has used the GPU."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _routing(tokens, top_k, experts, padded, seed):
    g = torch.Generator().manual_seed(seed)
    top = torch.randint(0, experts, (tokens * top_k,), generator=g).int()
    bin_ids, indices = torch.sort(top, stable=True)
    counts = torch.bincount(top.long(), minlength=experts)
    bins = torch.cumsum(counts, 0).int()
    pbins = torch.cumsum((counts + 127) // 128 * 128, 0).int() if padded else None
    return indices.int(), bin_ids.int(), bins, pbins


def _both(lib, _lib, tokens, hidden, top_k, experts, padded, dtype, weighted, seed):
    """(out of mbx_scatter with caller scratch, out of mbx_scatter_static) on the same inputs."""
    indices, bin_ids, bins, pbins = _routing(tokens, top_k, experts, padded, seed)
    rows = int(pbins[-1]) if padded else tokens * top_k
    g = torch.Generator().manual_seed(seed + 1)
    x = torch.randn(rows, hidden, generator=g).to(dtype).cuda()
    w = torch.rand(tokens * top_k, generator=g).to(dtype).cuda() if weighted else None
    indices, bin_ids, bins = indices.cuda(), bin_ids.cuda(), bins.cuda()
    pbins = None if pbins is None else pbins.cuda()
    want = torch.full((tokens, hidden), 7.0, dtype=dtype, device='cuda')
    got = torch.full((tokens, hidden), -7.0, dtype=dtype, device='cuda')
    scratch = torch.empty(tokens * top_k, dtype=torch.int32, device='cuda')
    common = (_lib.ptr(x), _lib.DTYPE[dtype], tokens, hidden, top_k, _lib.ptr(indices), _lib.ptr(bin_ids), _lib.ptr(bins),
              _lib.ptr(pbins), experts, _lib.ptr(w), _lib.DTYPE[dtype])
    s = _lib.stream()
    print(f'scatter_static case tokens={tokens} hidden={hidden} top_k={top_k} experts={experts} padded={padded} '
          f'dtype={dtype} weighted={weighted}', flush=True)
    assert lib.mbx_scatter(*common, _lib.ptr(want), None, _lib.ptr(scratch), scratch.numel() * 4, s) == 0
    assert lib.mbx_scatter_static(*common, _lib.ptr(got), s) == 0
    torch.cuda.synchronize()
    return want, got


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
@pytest.mark.parametrize('padded', [False, True])
def test_scatter_static_equals_scatter_on_two_calls_in_a_row(dtype, padded):
    from megablocks_amd import _lib
    lib = _lib.lib
    # a large call, then a smaller one whose map occupies the start of what the first call wrote
    want, got = _both(lib, _lib, 8192, 1024, 2, 8, padded, dtype, True, seed=1)
    assert torch.equal(want, got)
    want, got = _both(lib, _lib, 1000, 264, 4, 16, padded, dtype, True, seed=2)
    assert torch.equal(want, got)
    want, got = _both(lib, _lib, 333, 72, 1, 5, padded, dtype, False, seed=3)        # unweighted, rows off the vector path
    assert torch.equal(want, got)
    want, got = _both(lib, _lib, 8192, 1024, 2, 8, padded, dtype, True, seed=1)      # and the first one again
    assert torch.equal(want, got)


def test_scatter_static_limits_and_argument_errors():
    from megablocks_amd import _lib
    lib = _lib.lib
    limit = 1 << 20
    x = torch.zeros(8, 8, dtype=torch.bfloat16, device='cuda')
    idx = torch.zeros(8, dtype=torch.int32, device='cuda')
    args = lambda tokens, top_k: (_lib.ptr(x), _lib.BF16, tokens, 8, top_k, _lib.ptr(idx), _lib.ptr(idx), _lib.ptr(idx), None, 1,
                                  None, 0, _lib.ptr(x), _lib.stream())
    assert lib.mbx_scatter_static(*args(limit // 2 + 1, 2)) == _lib.ERANGE          # more slots than the static map holds
    assert b'beyond' in lib.mbx_error_string(_lib.ERANGE) or lib.mbx_error_string(_lib.ERANGE)
    assert lib.mbx_scatter_static(*args(0, 2)) == 0                                  # nothing to do
    assert lib.mbx_scatter_static(*args(8, 0)) == _lib.EINVAL
    bad = list(args(8, 1))
    bad[5] = None                                                                    # no indices
    assert lib.mbx_scatter_static(*bad) == _lib.EINVAL
    torch.cuda.synchronize()


def test_scatter_static_at_the_limit():
    """The largest call the static map takes (2^20 slots)."""
    from megablocks_amd import _lib
    want, got = _both(_lib.lib, _lib, (1 << 20) // 4, 64, 4, 64, False, torch.bfloat16, True, seed=4)
    assert torch.equal(want, got)
