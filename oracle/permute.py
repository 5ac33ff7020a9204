"""CPU oracle: token permutation ops.  Test infrastructure only.

Restates megablocks/backend/kernels.py (the Triton row-copy kernels and their launch
wrappers).  ``indices[i]`` is a slot id in [0, tokens*top_k): its token is
``indices[i] // top_k`` and its router weight ``weights[indices[i]]``.  ``bins`` and
``padded_bins`` are inclusive cumulative sums; bin ``e`` starts at ``bins[e-1]``.
"""
import torch


def _dst_rows(bin_ids, bins, padded_bins):
    """Row in the expert-major buffer of each sorted slot i (kernels.py:60-76):
    i - bins[e-1] + padded_bins[e-1] with e = bin_ids[i]."""
    e = bin_ids.long()
    start = torch.cat([torch.zeros(1, dtype=torch.int64), bins.long()])[e]
    pstart = torch.cat([torch.zeros(1, dtype=torch.int64), padded_bins.long()])[e]
    return torch.arange(e.numel(), dtype=torch.int64) - start + pstart


def _scaled(rows, scale):
    """kernels.py:100-102: product in fp32, rounded to the storage dtype."""
    if scale is None:
        return rows
    return (rows.float() * scale.float().unsqueeze(-1)).to(rows.dtype)


def padded_gather(x, indices, bin_ids, weights, bins, padded_bins, top_k):
    """kernels.py:107-138.  out = zeros [padded_bins[-1], h]; out[dst(i)] = x[indices[i]//k] (*w)."""
    if x.ndim != 2:
        raise ValueError(f'Expected 2-tensor but got {x.ndim}-tensor')
    rows = int(padded_bins[-1]) if padded_bins.numel() else 0
    out = torch.zeros((rows, x.shape[1]), dtype=x.dtype)
    idx = indices.long()
    src = x[idx // top_k]
    out[_dst_rows(bin_ids, bins, padded_bins)] = _scaled(src, None if weights is None else weights[idx])
    return out


def gather(x, indices, bin_ids, weights, bins, top_k):
    """kernels.py:141-170: the padded form with padded_bins := bins, output [tokens*top_k, h]."""
    if x.ndim != 2:
        raise ValueError(f'Expected 2-tensor but got {x.ndim}-tensor')
    out = torch.zeros((x.shape[0] * top_k, x.shape[1]), dtype=x.dtype)
    idx = indices.long()
    src = x[idx // top_k]
    out[_dst_rows(bin_ids, bins, bins)] = _scaled(src, None if weights is None else weights[idx])
    return out


def padded_scatter(x, indices, bin_ids, weights, bins, padded_bins, top_k):
    """kernels.py:173-203.  tmp[T, k, h] (flat row = slot id) receives the scaled row of
    every sorted slot, then tmp.sum(1) if k > 1 (kernels.py:203)."""
    if x.ndim != 2:
        raise ValueError(f'Expected 2-tensor but got {x.ndim}-tensor')
    tokens = indices.shape[0] // top_k
    idx = indices.long()
    tmp = torch.zeros((tokens * top_k, x.shape[1]), dtype=x.dtype)
    src = x[_dst_rows(bin_ids, bins, padded_bins)]
    tmp[idx] = _scaled(src, None if weights is None else weights[idx])
    tmp = tmp.view(tokens, top_k, x.shape[1])
    return tmp.sum(dim=1) if top_k > 1 else tmp.view(tokens, x.shape[1])


def scatter(x, indices, bin_ids, weights, bins, top_k):
    """kernels.py:206-207."""
    return padded_scatter(x, indices, bin_ids, weights, bins, bins, top_k)


def padded_scatter_wgrad(x, grad, indices, bin_ids, bins, padded_bins, top_k):
    """kernels.py:217-303: wgrad[indices[i]] = sum_c x[src(i), c] * grad[indices[i]//k, c],
    accumulated in fp32, stored in x.dtype."""
    idx = indices.long()
    src = x[_dst_rows(bin_ids, bins, padded_bins)].float()
    g = grad[idx // top_k].float()
    out = torch.zeros(indices.shape[0], dtype=x.dtype)
    out[idx] = (src * g).sum(1).to(x.dtype)
    return out


def scatter_wgrad(x, grad, indices, bin_ids, bins, top_k):
    """kernels.py:306-307."""
    return padded_scatter_wgrad(x, grad, indices, bin_ids, bins, bins, top_k)


def _binned_map(indices, bins, capacity):
    """(expert, entry, slot id) of every kept slot: entry j of expert e holds sorted slot
    bins[e-1] + j for j < min(count_e, capacity) (kernels.py:341-358)."""
    b = [0] + [int(v) for v in bins]
    es, js, ss = [], [], []
    for e in range(len(b) - 1):
        n = min(b[e + 1] - b[e], capacity)
        if n > 0:
            es.append(torch.full((n,), e, dtype=torch.int64))
            js.append(torch.arange(n, dtype=torch.int64))
            ss.append(indices[b[e]:b[e] + n].long())
    if not es:
        z = torch.zeros(0, dtype=torch.int64)
        return z, z, z
    return torch.cat(es), torch.cat(js), torch.cat(ss)


def binned_gather(x, indices, weights, bins, expert_capacity, top_k):
    """kernels.py:392-418: out = zeros [E, capacity, h]; slots beyond the capacity are dropped."""
    if x.ndim != 2:
        raise ValueError(f'Expected 2-tensor but got {x.ndim}-tensor')
    out = torch.zeros((bins.shape[0], expert_capacity, x.shape[1]), dtype=x.dtype)
    e, j, s = _binned_map(indices, bins, expert_capacity)
    out[e, j] = _scaled(x[s // top_k], None if weights is None else weights[s])
    return out


def binned_scatter(x, indices, weights, bins, top_k):
    """kernels.py:421-449: tmp = zeros [T, k, h]; tmp[slot] = x[e, j] (*w); sum over k if k > 1."""
    if x.ndim != 3:
        raise ValueError(f'Expected 3-tensor but got {x.ndim}-tensor')
    num_experts, capacity, hidden = x.shape
    tokens = indices.shape[0] // top_k
    tmp = torch.zeros((tokens * top_k, hidden), dtype=x.dtype)
    e, j, s = _binned_map(indices, bins, capacity)
    tmp[s] = _scaled(x[e, j], None if weights is None else weights[s])
    tmp = tmp.view(tokens, top_k, hidden)
    return tmp.sum(dim=1) if top_k > 1 else tmp.view(tokens, hidden)


def binned_scatter_wgrad(x, grad, indices, bins, top_k):
    """kernels.py:457-543: out = zeros [T*k]; out[slot] = <x[e, j], grad[slot//k]> in fp32."""
    num_experts, capacity, hidden = x.shape
    out = torch.zeros(indices.shape[0], dtype=x.dtype)
    e, j, s = _binned_map(indices, bins, capacity)
    out[s] = (x[e, j].float() * grad[s // top_k].float()).sum(1).to(x.dtype)
    return out
