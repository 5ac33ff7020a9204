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
    assert lib.mbx_error_string(_lib.ERANGE) == b'mbx: size out of the supported range'
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


_CAPTURE_SCRIPT = r"""
import sys, torch
from megablocks_amd import _lib
lib = _lib.lib
tokens, hidden, top_k, experts = 512, 128, 2, 4
g = torch.Generator().manual_seed(5)
top = torch.randint(0, experts, (tokens * top_k,), generator=g).int()
bin_ids, indices = torch.sort(top, stable=True)
bins = torch.cumsum(torch.bincount(top.long(), minlength=experts), 0).int().cuda()
indices, bin_ids = indices.int().cuda(), bin_ids.int().cuda()
x = torch.randn(tokens * top_k, hidden, generator=g).bfloat16().cuda()
w = torch.rand(tokens * top_k, generator=g).bfloat16().cuda()
want = torch.empty(tokens, hidden, dtype=torch.bfloat16, device='cuda')
got = torch.zeros_like(want)
scratch = torch.empty(tokens * top_k, dtype=torch.int32, device='cuda')
common = (_lib.ptr(x), _lib.BF16, tokens, hidden, top_k, _lib.ptr(indices), _lib.ptr(bin_ids), _lib.ptr(bins), None, experts,
          _lib.ptr(w), _lib.BF16)
assert lib.mbx_scatter(*common, _lib.ptr(want), None, _lib.ptr(scratch), scratch.numel() * 4, _lib.stream()) == 0
torch.cuda.synchronize()
# first call on this device inside a capture: refused, nothing recorded
graph = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph):
    rc_first = lib.mbx_scatter_static(*common, _lib.ptr(got), _lib.stream())
assert rc_first == _lib.ECAPTURE, rc_first
assert b'mbx_init' in lib.mbx_error_string(rc_first)
assert lib.mbx_init() == 0 and lib.mbx_init() == 0
graph = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph):
    rc = lib.mbx_scatter_static(*common, _lib.ptr(got), _lib.stream())
assert rc == 0, rc
for _ in range(3):
    got.zero_()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(got, want)
print('capture-ok')
"""


def test_scatter_static_first_call_under_capture_is_refused_until_init():
    """The lookup of the static buffer's address cannot run while a stream records a graph: a first call on a device
    under capture returns MBX_ECAPTURE and records nothing; after mbx_init() the call captures and replays.  In a
    process of its own (this one has long made its first call)."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    print('scatter_static capture case: child process', flush=True)
    proc = subprocess.run([sys.executable, '-c', _CAPTURE_SCRIPT], cwd=root, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0 and 'capture-ok' in proc.stdout, proc.stdout + proc.stderr
