"""CPU oracle: routing / bookkeeping ops (integer, exact).  Test infrastructure only.

Restates megablocks/ops/{histogram,sort,cumsum,round_up,replicate,topology}.py and the
kernels they call in csrc/*.h, plus the bookkeeping of megablocks/layers/{moe,dmoe}.py.
"""
import numpy as np
import torch

_BITS = {torch.int16: 16, torch.int32: 32, torch.int64: 64}


def _check_int(x):
    if x.dtype not in _BITS:
        raise RuntimeError(f'expected int16/int32/int64, got {x.dtype}')


def histogram(x: torch.Tensor, num_bins: int) -> torch.Tensor:
    """csrc/histogram.h:20-81 (cub HistogramEven over [0,num_bins), one row at a time).

    Samples outside [0, num_bins) fall in no bin.  1-D in -> int32 [num_bins];
    2-D in -> int32 [rows, num_bins].
    """
    _check_int(x)
    if x.ndim not in (1, 2):
        raise RuntimeError('histogram expects a 1-D or 2-D tensor')
    rows = x.view(1, -1) if x.ndim == 1 else x
    out = torch.zeros((rows.shape[0], num_bins), dtype=torch.int32)
    for r in range(rows.shape[0]):
        v = rows[r].to(torch.int64)
        v = v[(v >= 0) & (v < num_bins)]
        if v.numel() and num_bins > 0:
            out[r] = torch.bincount(v, minlength=num_bins).to(torch.int32)
    return out.flatten() if x.ndim == 1 else out


def sort(x: torch.Tensor, end_bit=None):
    """megablocks/ops/sort.py:26-38 + csrc/sort.h:20-86 (cub DeviceRadixSort::SortPairs).

    Stable least-significant-digit radix sort of the keys on bits [0, end_bit) with an
    ``arange`` payload of the key dtype.  Only those bits take part in the comparison;
    with the full width the order is the signed order.  Returns (sorted keys,
    permutation), i.e. ``keys_out[i] == x[perm[i]]``.
    """
    _check_int(x)
    if x.ndim != 1:
        raise RuntimeError('sort expects a 1-D tensor')
    bits = _BITS[x.dtype]
    if end_bit is None:
        end_bit = bits
    if end_bit >= bits:
        cmp_key = x.to(torch.int64)
    else:
        cmp_key = x.to(torch.int64) & ((1 << end_bit) - 1)
    _, perm = torch.sort(cmp_key, stable=True)
    return x[perm], perm.to(x.dtype)


def _cumsum(x, dim, exclusive):
    _check_int(x)
    if x.ndim == 1:
        # megablocks/ops/cumsum.py:24-29,40-45: 1-D is viewed [1, n] and the result squeezed,
        # so a one-element result is 0-dim.
        y = torch.cumsum(x.view(1, -1), 1, dtype=x.dtype)
        if exclusive:
            y = y - x.view(1, -1)
        return y.squeeze()
    if x.ndim != 2 or dim != 1:
        raise RuntimeError('cumsum expects a 2-D tensor scanned along dim 1')  # csrc/cumsum.h:117,144
    y = torch.cumsum(x, 1, dtype=x.dtype)
    return y - x if exclusive else y


def inclusive_cumsum(x, dim):
    """megablocks/ops/cumsum.py:37-51 + csrc/cumsum.h:131-156."""
    return _cumsum(x, dim, False)


def exclusive_cumsum(x, dim):
    """megablocks/ops/cumsum.py:20-34 + csrc/cumsum.h:104-129."""
    return _cumsum(x, dim, True)


def round_up(x: torch.Tensor, value: int) -> torch.Tensor:
    """megablocks/ops/round_up.py:7-14."""
    assert isinstance(value, int)
    assert x.dtype == torch.int32
    return torch.div(x + (value - 1), value, rounding_mode='trunc') * value


def replicate(x: torch.Tensor, bins: torch.Tensor, num_outputs: int) -> torch.Tensor:
    """megablocks/ops/replicate.py:22-27 + csrc/replicate.h:21-61.

    out[b, bins[i-1]:bins[i]] = x[b, i].  Columns at or beyond bins[-1] are left
    unwritten by the reference (torch.empty); here they are zero.
    """
    counts = torch.diff(bins.to(torch.int64), prepend=torch.zeros(1, dtype=torch.int64))
    body = torch.repeat_interleave(x, counts, dim=1)
    out = torch.zeros((x.shape[0], num_outputs), dtype=x.dtype)
    n = min(num_outputs, body.shape[1])
    out[:, :n] = body[:, :n]
    return out


def replicate_backward(grad: torch.Tensor, bins: torch.Tensor) -> torch.Tensor:
    """megablocks/ops/replicate.py:29-33 + csrc/replicate.h:80-126 (segmented sum per bin)."""
    b = [0] + [int(v) for v in bins]
    out = torch.zeros((grad.shape[0], len(b) - 1), dtype=torch.float32)
    for i in range(len(b) - 1):
        out[:, i] = grad[:, b[i]:b[i + 1]].float().sum(1)
    return out.to(grad.dtype)


def topology(padded_bins: torch.Tensor, block_size: int, block_rows: int, block_cols: int) -> torch.Tensor:
    """megablocks/ops/topology.py:23-42 + csrc/indices.h:21-49.

    Column indices of the block-diagonal sparse matrix: every block-row owned by
    expert e lists block-columns e*C .. e*C+C-1.
    """
    assert padded_bins.dtype == torch.int32
    out = torch.zeros(block_rows * block_cols, dtype=torch.int16)
    pb = [0] + [int(v) // block_size for v in padded_bins]
    cols = torch.arange(block_cols, dtype=torch.int64)
    for e in range(len(pb) - 1):
        n = pb[e + 1] - pb[e]
        if n > 0:
            out[pb[e] * block_cols:pb[e + 1] * block_cols] = (cols + e * block_cols).repeat(n).to(torch.int16)
    return out


def sort_end_bit(num_experts: int) -> int:
    """megablocks/layers/moe.py:110."""
    return max(int(np.ceil(np.log2(num_experts))), 1)


def _promote_scalar(x):
    return x.view(1) if x.ndim == 0 else x  # megablocks/layers/dmoe.py:14-15


def indices_and_bins(top_expert: torch.Tensor, num_experts: int):
    """megablocks/layers/moe.py:152-183 -> (indices, bin_ids, bins, tokens_per_expert)."""
    top_expert = top_expert.int()
    bin_ids, indices = sort(top_expert, sort_end_bit(num_experts))
    tokens_per_expert = histogram(top_expert, num_experts)
    bins = _promote_scalar(inclusive_cumsum(tokens_per_expert, 0))
    return indices, bin_ids, bins, tokens_per_expert


def indices_and_padded_bins(top_expert: torch.Tensor, num_experts: int, blocking: int = 128):
    """megablocks/layers/dmoe.py:131-154 -> (indices, bin_ids, bins, padded_bins, tokens_per_expert)."""
    top_expert = top_expert.int()
    bin_ids, indices = sort(top_expert, sort_end_bit(num_experts))
    tokens_per_expert = histogram(top_expert, num_experts)
    padded = round_up(tokens_per_expert, blocking)
    padded_bins = _promote_scalar(inclusive_cumsum(padded, 0))
    bins = _promote_scalar(inclusive_cumsum(tokens_per_expert, 0))
    return indices, bin_ids, bins, padded_bins, tokens_per_expert


def row_indices(block_rows: int, blocks_per_row: int) -> torch.Tensor:
    """Row index of every nonzero block of a matrix with a constant number of blocks per
    block-row (what stk.ops.row_indices yields for the offsets built at
    megablocks/layers/dmoe.py:80-88), int16."""
    return torch.arange(block_rows, dtype=torch.int64).repeat_interleave(blocks_per_row).to(torch.int16)


def sparse_transpose(shape, row_idx, column_indices, blocking, transpose_sort_end_bit):
    """megablocks/layers/dmoe.py:35-66 -> (column_indices_t, offsets_t, block_offsets_t)."""
    block_columns = shape[1] // blocking
    _, gather_indices = sort(column_indices.int(), transpose_sort_end_bit)
    column_indices_t = row_idx.gather(0, gather_indices.long())
    block_offsets_t = gather_indices.int()
    zero = torch.zeros((1,), dtype=torch.int32)
    nnz_per_column = histogram(column_indices, block_columns)
    nnz_per_column = inclusive_cumsum(nnz_per_column, 0)
    if nnz_per_column.dim() == 0:
        nnz_per_column = nnz_per_column.unsqueeze(0)
    offsets_t = torch.cat([zero, nnz_per_column])
    return column_indices_t, offsets_t, block_offsets_t
