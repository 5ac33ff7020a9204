"""Token permutation kernels (host side), mirroring megablocks/backend/kernels.py.

Same function names, argument order, shape checks (ValueError) and results as the
reference's Triton launch wrappers; the work is done by the HIP kernels of libmbx.so on
the current stream.  `weights=None` means an unscaled copy.
"""
import torch

from megablocks_amd import _lib
from megablocks_amd._lib import lib


def assert_is_tensor(x, ndim):
    if x.ndim != ndim:
        raise ValueError(f'Expected {ndim}-tensor but got {x.ndim}-tensor')


def assert_is_matrix(x):
    assert_is_tensor(x, 2)


def assert_is_vector(x):
    if x.ndim != 1:
        raise ValueError(f'Expected 1-tensor but got {x.ndim}-tensor')


def assert_equal(a, b):
    if a != b:
        raise ValueError(f'Expected dimensions to be equal but got {a} and {b}.',)


def _w(weights):
    """(pointer, dtype code) of the optional router weights."""
    if weights is None:
        return None, 0, None
    weights = weights.contiguous()
    return _lib.ptr(weights), _lib.dtype_of(weights), weights


def _scratch(n_slots, device):
    return torch.empty(max(n_slots, 1), dtype=torch.int32, device=device)


def _slot_rows_key(indices, bins, padded_bins):
    return (indices._version, bins.data_ptr(), bins._version,
            None if padded_bins is None else (padded_bins.data_ptr(), padded_bins._version))


def remember_slot_rows(indices, bins, padded_bins, rows):
    """Leaves a slot -> row map that was built together with `indices` (ops.route) where _slot_rows looks for it.
    Not under stream capture, where nothing is kept (see _slot_rows)."""
    if torch.cuda.is_current_stream_capturing():
        return
    try:
        indices._mbx_slot_rows = (_slot_rows_key(indices, bins, padded_bins), rows, bins, padded_bins)
    except AttributeError:
        pass


def forget_slot_rows(indices):
    """Drops the slot -> row map kept on `indices` (see _slot_rows): for callers that rewrite `indices`, `bins` or
    `padded_bins` in ways torch does not see (raw pointers, a graph replay into them).  The next permutation call
    builds a new map.  A map that is stale all the same cannot take the kernels out of range: they read it with the
    row count of the expert-major buffer as a bound."""
    try:
        del indices._mbx_slot_rows
    except AttributeError:
        pass


def _slot_rows(indices, bin_ids, bins, padded_bins):
    """int32 [n_slots]: the row of the expert-major (optionally padded) buffer that holds each slot.  One map
    serves all gathers and scatters of a routing decision, forward and backward, so it is kept on the `indices`
    tensor and reused while `indices`, `bins` and `padded_bins` are the same unmodified tensors ("unmodified" as
    torch sees it, by `_version`: a caller that rewrites them through raw pointers or by replaying a captured graph
    into them must pass new tensors, or delete the `_mbx_slot_rows` attribute).  A caller that builds a new `indices` tensor for every
    call gets a new map for every call.  Under stream capture nothing is reused or kept: a captured graph has to
    contain the kernels that build its map."""
    capturing = torch.cuda.is_current_stream_capturing()
    key = _slot_rows_key(indices, bins, padded_bins)
    cached = getattr(indices, '_mbx_slot_rows', None)
    if not capturing and cached is not None and cached[0] == key:
        return cached[1]
    n_slots = indices.shape[0]
    rows = _scratch(n_slots, indices.device)
    with _lib.device_of(indices):
        _lib.check(lib.mbx_slot_rows(_lib.ptr(indices), _lib.ptr(bin_ids), _lib.ptr(bins), _lib.ptr(padded_bins),
                                     bins.shape[0], n_slots, _lib.ptr(rows), _lib.stream()), 'slot_rows')
    if not capturing:
        try:
            indices._mbx_slot_rows = (key, rows, bins, padded_bins)   # the references keep the data pointers of the key alive
        except AttributeError:   # a tensor type without instance attributes: the map is built on every call
            pass
    return rows


def _gather(x, indices, bin_ids, weights, bins, padded_bins, top_k, output_rows, what):
    _lib.require_cuda(x, indices, bin_ids, bins, padded_bins, weights)
    x = x.contiguous()
    indices, bins, padded_bins = _lib.as_i32(indices), _lib.as_i32(bins), _lib.as_i32(padded_bins)
    wp, wdt, weights = _w(weights)
    out = torch.empty((output_rows, x.shape[1]), dtype=x.dtype, device=x.device)
    # top_k = 1: every row of x is read once either way, the kernel with one wave per output row needs no map
    rows = _slot_rows(indices, _lib.as_i32(bin_ids), bins, padded_bins) if top_k > 1 and indices.shape[0] else None
    with _lib.device_of(x), _lib.record('gather_weighted' if weights is not None else 'gather',
                                              rows_in=x.shape[0], rows_out=output_rows, hidden=x.shape[1],
                                              elem=x.element_size()):
        _lib.check(lib.mbx_gather(_lib.ptr(x), _lib.dtype_of(x), x.shape[0], x.shape[1], top_k, _lib.ptr(indices),
                                  _lib.ptr(bins), _lib.ptr(padded_bins), bins.shape[0], wp, wdt, _lib.ptr(out),
                                  output_rows, _lib.ptr(rows), _lib.stream()), what)
    return out


def padded_gather(x, indices, bin_ids, weights, bins, padded_bins, top_k):
    """megablocks/backend/kernels.py:107-138."""
    assert_is_matrix(x)
    assert_is_vector(indices)
    assert_is_vector(bin_ids)
    assert_is_vector(bins)
    assert_is_vector(padded_bins)
    assert_equal(indices.shape[0], x.shape[0] * top_k)
    assert_equal(bin_ids.shape[0], x.shape[0] * top_k)
    assert_equal(bins.size(), padded_bins.size())
    if weights is not None:
        assert_equal(weights.shape[0], x.shape[0] * top_k)
    # The output size depends on the routing: one host read of the last padded bin bound,
    # as in the reference (kernels.py:123).  Padding rows are zeroed by the kernel itself.
    output_rows = int(padded_bins[-1].item()) if padded_bins.numel() else 0
    return _gather(x, indices, bin_ids, weights, bins, padded_bins, top_k, output_rows, 'padded_gather')


def gather(x, indices, bin_ids, weights, bins, top_k):
    """megablocks/backend/kernels.py:141-170."""
    assert_is_matrix(x)
    assert_is_vector(indices)
    assert_is_vector(bin_ids)
    assert_is_vector(bins)
    assert_equal(indices.shape[0], x.shape[0] * top_k)
    assert_equal(bin_ids.shape[0], x.shape[0] * top_k)
    if weights is not None:
        assert_equal(weights.shape[0], x.shape[0] * top_k)
    return _gather(x, indices, bin_ids, weights, bins, None, top_k, x.shape[0] * top_k, 'gather')


def padded_scatter(x, indices, bin_ids, weights, bins, padded_bins, top_k):
    """megablocks/backend/kernels.py:173-203 (the copy and the sum over top_k in one pass)."""
    assert_is_matrix(x)
    assert_is_vector(indices)
    assert_is_vector(bin_ids)
    assert_is_vector(bins)
    assert_is_vector(padded_bins)
    assert_equal(indices.shape[0], bin_ids.shape[0])
    assert_equal(bins.size(), padded_bins.size())
    if weights is not None:
        assert_equal(indices.shape[0], weights.shape[0])
    return _scatter(x, indices, bin_ids, weights, bins, padded_bins, top_k)


def scatter(x, indices, bin_ids, weights, bins, top_k):
    """megablocks/backend/kernels.py:206-207."""
    assert_is_matrix(x)
    assert_is_vector(indices)
    assert_is_vector(bin_ids)
    assert_is_vector(bins)
    assert_equal(indices.shape[0], bin_ids.shape[0])
    if weights is not None:
        assert_equal(indices.shape[0], weights.shape[0])
    return _scatter(x, indices, bin_ids, weights, bins, None, top_k)


def _scatter(x, indices, bin_ids, weights, bins, padded_bins, top_k):
    _lib.require_cuda(x, indices, bin_ids, bins, padded_bins, weights)
    x = x.contiguous()
    n_slots = indices.shape[0]
    tokens = n_slots // top_k
    if padded_bins is None:
        assert_equal(x.shape[0], n_slots)
    indices, bin_ids = _lib.as_i32(indices), _lib.as_i32(bin_ids)
    bins, padded_bins = _lib.as_i32(bins), _lib.as_i32(padded_bins)
    wp, wdt, weights = _w(weights)
    out = torch.empty((tokens, x.shape[1]), dtype=x.dtype, device=x.device)
    rows = _slot_rows(indices, bin_ids, bins, padded_bins) if n_slots else None
    with _lib.device_of(x), _lib.record('scatter_weighted' if weights is not None else 'scatter',
                                              rows_in=n_slots, rows_out=tokens, hidden=x.shape[1],
                                              elem=x.element_size()):
        _lib.check(lib.mbx_scatter(_lib.ptr(x), _lib.dtype_of(x), tokens, x.shape[1], top_k, _lib.ptr(indices),
                                   _lib.ptr(bin_ids), _lib.ptr(bins), _lib.ptr(padded_bins), bins.shape[0], wp, wdt,
                                   _lib.ptr(out), _lib.ptr(rows), None, 0, _lib.stream()), 'scatter')
    return out


def scatter_backward(x, grad, indices, bin_ids, weights, bins, padded_bins, top_k):
    """Both gradients of the weighted `scatter` / `padded_scatter` (padded_bins None: unpadded) of `x`:
    (gather of `grad` weighted, scatter_wgrad), as megablocks/ops/scatter.py:34-62 and
    megablocks/ops/padded_scatter.py:49-80 compute them with two kernels, in one pass over `grad` where the
    library has a kernel for the shape, else by those two calls."""
    _lib.require_cuda(x, grad, indices, bin_ids, weights, bins, padded_bins)
    xc = x.contiguous()
    gc = grad.contiguous().to(xc.dtype)
    n_slots = indices.shape[0]
    tokens = n_slots // top_k
    if n_slots and tuple(gc.shape) == (tokens, xc.shape[1]) and indices.dtype == torch.int32:
        idx, bi = indices.contiguous(), _lib.as_i32(bin_ids)
        b, pb = _lib.as_i32(bins), _lib.as_i32(padded_bins)
        wp, wdt, wc = _w(weights)
        rows = _slot_rows(idx, bi, b, pb)
        dgrad = torch.empty_like(xc)
        wgrad = torch.empty((n_slots,), dtype=xc.dtype, device=xc.device)
        with _lib.device_of(xc), _lib.record('scatter_backward', rows_in=tokens, rows_out=xc.shape[0],
                                                   hidden=xc.shape[1], elem=xc.element_size()) as rec:
            rc = lib.mbx_scatter_backward(_lib.ptr(gc), _lib.ptr(xc), _lib.dtype_of(xc), tokens, xc.shape[1], top_k,
                                          _lib.ptr(idx), _lib.ptr(b), _lib.ptr(pb), b.shape[0], wp, wdt, _lib.ptr(rows),
                                          _lib.ptr(dgrad), xc.shape[0], _lib.ptr(wgrad), _lib.stream())
            if rc == _lib.EUNSUPPORTED:
                rec.cancel()
        if rc != _lib.EUNSUPPORTED:
            _lib.check(rc, 'scatter_backward')
            return dgrad, wgrad
    if padded_bins is None:
        return (gather(grad, indices, bin_ids, weights, bins, top_k),
                scatter_wgrad(x, grad, indices, bin_ids, bins, top_k))
    return (padded_gather(grad, indices, bin_ids, weights, bins, padded_bins, top_k),
            padded_scatter_wgrad(x, grad, indices, bin_ids, bins, padded_bins, top_k))


def padded_scatter_wgrad(x, grad, indices, bin_ids, bins, padded_bins, top_k):
    """megablocks/backend/kernels.py:279-303."""
    assert_is_matrix(x)
    assert_is_matrix(grad)
    assert_is_vector(indices)
    assert_is_vector(bin_ids)
    assert_is_vector(bins)
    assert_is_vector(padded_bins)
    assert_equal(indices.shape[0], bin_ids.shape[0])
    assert_equal(bins.size(), padded_bins.size())
    return _scatter_wgrad(x, grad, indices, bin_ids, bins, padded_bins, top_k)


def scatter_wgrad(x, grad, indices, bin_ids, bins, top_k):
    """megablocks/backend/kernels.py:306-307."""
    assert_is_matrix(x)
    assert_is_matrix(grad)
    assert_is_vector(indices)
    assert_is_vector(bin_ids)
    assert_is_vector(bins)
    assert_equal(indices.shape[0], bin_ids.shape[0])
    return _scatter_wgrad(x, grad, indices, bin_ids, bins, None, top_k)


def _scatter_wgrad(x, grad, indices, bin_ids, bins, padded_bins, top_k):
    _lib.require_cuda(x, grad, indices, bin_ids, bins, padded_bins)
    x = x.contiguous()
    grad = grad.contiguous().to(x.dtype)
    assert_equal(x.shape[1], grad.shape[1])
    n_slots = indices.shape[0]
    tokens = n_slots // top_k
    assert_equal(grad.shape[0], tokens)
    indices, bin_ids = _lib.as_i32(indices), _lib.as_i32(bin_ids)
    bins, padded_bins = _lib.as_i32(bins), _lib.as_i32(padded_bins)
    out = torch.empty((n_slots,), dtype=x.dtype, device=x.device)
    with _lib.device_of(x), _lib.record('scatter_wgrad', rows_in=n_slots, rows_out=tokens, hidden=x.shape[1],
                                              elem=x.element_size()):
        _lib.check(lib.mbx_scatter_wgrad(_lib.ptr(x), _lib.ptr(grad), _lib.dtype_of(x), tokens, x.shape[1], top_k,
                                         _lib.ptr(indices), _lib.ptr(bin_ids), _lib.ptr(bins), _lib.ptr(padded_bins),
                                         bins.shape[0], _lib.ptr(out), _lib.stream()), 'scatter_wgrad')
    return out


def binned_gather(x, indices, weights, bins, expert_capacity, top_k):
    """megablocks/backend/kernels.py:392-418."""
    assert_is_matrix(x)
    assert_is_vector(indices)
    assert_is_vector(bins)
    assert_equal(indices.shape[0], x.shape[0] * top_k)
    if weights is not None:
        assert_equal(weights.shape[0], x.shape[0] * top_k)
    _lib.require_cuda(x, indices, bins, weights)
    x = x.contiguous()
    indices, bins = _lib.as_i32(indices), _lib.as_i32(bins)
    wp, wdt, weights = _w(weights)
    num_experts = bins.shape[0]
    out = torch.empty((num_experts, expert_capacity, x.shape[1]), dtype=x.dtype, device=x.device)
    with _lib.device_of(x):
        _lib.check(lib.mbx_binned_gather(_lib.ptr(x), _lib.dtype_of(x), x.shape[0], x.shape[1], top_k, _lib.ptr(indices),
                                         _lib.ptr(bins), num_experts, expert_capacity, wp, wdt, _lib.ptr(out),
                                         _lib.stream()), 'binned_gather')
    return out


def binned_scatter(x, indices, weights, bins, top_k):
    """megablocks/backend/kernels.py:421-449."""
    assert_is_tensor(x, 3)
    assert_is_vector(indices)
    assert_is_vector(bins)
    assert_equal(bins.shape[0], x.shape[0])
    if weights is not None:
        assert_equal(indices.shape[0], weights.shape[0])
    _lib.require_cuda(x, indices, bins, weights)
    x = x.contiguous()
    num_experts, expert_capacity, hidden_size = x.shape
    n_slots = indices.shape[0]
    tokens = n_slots // top_k
    indices, bins = _lib.as_i32(indices), _lib.as_i32(bins)
    wp, wdt, weights = _w(weights)
    out = torch.empty((tokens, hidden_size), dtype=x.dtype, device=x.device)
    scratch = _scratch(n_slots, x.device)
    with _lib.device_of(x):
        _lib.check(lib.mbx_binned_scatter(_lib.ptr(x), _lib.dtype_of(x), tokens, hidden_size, top_k, _lib.ptr(indices),
                                          _lib.ptr(bins), num_experts, expert_capacity, wp, wdt, _lib.ptr(out),
                                          _lib.ptr(scratch), scratch.numel() * 4, _lib.stream()), 'binned_scatter')
    return out


def binned_scatter_wgrad(x, grad, indices, bins, top_k):
    """megablocks/backend/kernels.py:521-543."""
    assert_is_tensor(x, 3)
    assert_is_matrix(grad)
    assert_is_vector(indices)
    assert_is_vector(bins)
    assert_equal(bins.shape[0], x.shape[0])
    _lib.require_cuda(x, grad, indices, bins)
    x = x.contiguous()
    grad = grad.contiguous().to(x.dtype)
    num_experts, expert_capacity, hidden_size = x.shape
    assert_equal(grad.shape[1], hidden_size)
    n_slots = indices.shape[0]
    tokens = n_slots // top_k
    assert_equal(grad.shape[0], tokens)
    indices, bins = _lib.as_i32(indices), _lib.as_i32(bins)
    out = torch.empty((n_slots,), dtype=x.dtype, device=x.device)
    with _lib.device_of(x):
        _lib.check(lib.mbx_binned_scatter_wgrad(_lib.ptr(x), _lib.ptr(grad), _lib.dtype_of(x), tokens, hidden_size, top_k,
                                                _lib.ptr(indices), _lib.ptr(bins), num_experts, expert_capacity,
                                                _lib.ptr(out), _lib.stream()), 'binned_scatter_wgrad')
    return out
