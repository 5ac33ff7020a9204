"""ctypes binding of oracle/routing_c.c, the plain-C restatement of the integer routing ops.

Test infrastructure only (see oracle/__init__.py).  `build()` compiles the C file with gcc into
oracle/liboracle_routing.so; the wrappers take and return torch CPU tensors like oracle/routing.py.
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
SOURCE = os.path.join(_HERE, 'routing_c.c')
LIB_PATH = os.path.join(_HERE, 'liboracle_routing.so')
_BITS = {torch.int16: 16, torch.int32: 32, torch.int64: 64}
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(LIB_PATH) or os.path.getmtime(LIB_PATH) < os.path.getmtime(SOURCE):
        subprocess.run(['gcc', '-O2', '-Wall', '-Wextra', '-shared', '-fPIC', '-o', LIB_PATH, SOURCE], check=True)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        _lib.mbxo_sort.restype = ctypes.c_int
        _lib.mbxo_route.restype = ctypes.c_int
    return _lib


def _i64(t):
    return t.to(torch.int64).contiguous()


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _n(v):
    return ctypes.c_int64(int(v))


def histogram(x: torch.Tensor, num_bins: int) -> torch.Tensor:
    rows = x.view(1, -1) if x.ndim == 1 else x
    xi = _i64(rows)
    out = torch.empty((rows.shape[0], num_bins), dtype=torch.int32)
    lib().mbxo_histogram(_p(xi), _n(rows.shape[0]), _n(rows.shape[1]), _n(num_bins), _p(out))
    return out.flatten() if x.ndim == 1 else out


def sort(x: torch.Tensor, end_bit=None):
    width = _BITS[x.dtype]
    end_bit = width if end_bit is None else min(int(end_bit), width)
    xi = _i64(x)
    keys, perm = torch.empty_like(xi), torch.empty_like(xi)
    if lib().mbxo_sort(_p(xi), _n(x.numel()), ctypes.c_int(end_bit), ctypes.c_int(width), _p(keys), _p(perm)):
        raise MemoryError('mbxo_sort')
    return keys.to(x.dtype), perm.to(x.dtype)


def cumsum(x: torch.Tensor, exclusive: bool) -> torch.Tensor:
    """Scan of every row of a 2-D tensor (a 1-D tensor is one row)."""
    rows = x.view(1, -1) if x.ndim == 1 else x
    xi = _i64(rows)
    out = torch.empty_like(xi)
    lib().mbxo_cumsum(_p(xi), _n(rows.shape[0]), _n(rows.shape[1]), ctypes.c_int(int(exclusive)),
                      ctypes.c_int(_BITS[x.dtype]), _p(out))
    return out.to(x.dtype).view(x.shape)


def topology(padded_bins: torch.Tensor, block_size: int, block_rows: int, block_cols: int) -> torch.Tensor:
    pb = padded_bins.to(torch.int32).contiguous()
    out = torch.empty(block_rows * block_cols, dtype=torch.int16)
    lib().mbxo_topology(_p(pb), _n(pb.numel()), _n(block_size), _n(block_rows), _n(block_cols), _p(out))
    return out


def replicate(x: torch.Tensor, bins: torch.Tensor, num_outputs: int) -> torch.Tensor:
    xi, b = _i64(x), bins.to(torch.int32).contiguous()
    out = torch.empty((x.shape[0], num_outputs), dtype=torch.int64)
    lib().mbxo_replicate(_p(xi), _n(x.shape[0]), _n(b.numel()), _p(b), _n(num_outputs), _p(out))
    return out.to(x.dtype)


def route(top_expert: torch.Tensor, num_experts: int, end_bit: int, blocking: int = 0):
    """(indices, bin_ids, bins, padded_bins or None, tokens_per_expert), all int32."""
    te = _i64(top_expert)
    n = te.numel()
    bin_ids, indices = torch.empty(n, dtype=torch.int64), torch.empty(n, dtype=torch.int64)
    tpe, bins, pbins = (torch.empty(num_experts, dtype=torch.int32) for _ in range(3))
    if lib().mbxo_route(_p(te), _n(n), _n(num_experts), ctypes.c_int(end_bit), _n(blocking), _p(bin_ids), _p(indices),
                        _p(tpe), _p(bins), _p(pbins)):
        raise MemoryError('mbxo_route')
    return indices.int(), bin_ids.int(), bins, (pbins if blocking > 0 else None), tpe
