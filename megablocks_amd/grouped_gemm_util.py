"""Grouped GEMM entry points with the interface the reference reaches through
megablocks/grouped_gemm_util.py:25-26 (`gg.backend.gmm`, `gg.ops.gmm`), served by the
bf16/f16 MFMA kernels of libmbx.so.

`batch_sizes` may be the host int64 tensor the reference passes (mlp.py:502) or, to avoid
the device-to-host copy, a device tensor of per-expert row counts.
"""
import os
import types

import torch

from megablocks_amd import _lib
from megablocks_amd._lib import lib


def grouped_gemm_is_available():
    return True


def assert_grouped_gemm_is_available():
    assert grouped_gemm_is_available()


def _device_bins(batch_sizes: torch.Tensor, device, rows: int) -> torch.Tensor:
    """Inclusive int32 row bins on the device for a vector of group sizes that must add up to `rows`.

    Sizes on the host (what the reference passes, mlp.py:502) are checked here, as grouped_gemm checks them: negative
    sizes or a sum other than `rows` raise ValueError.  Sizes on the device cannot be checked without a
    synchronisation; the kernels keep every bin bound inside [0, rows], so a table that does not match the operands
    gives wrong values, never an access out of range.

    The bins are kept on the `batch_sizes` tensor and reused while its `_version` is unchanged, i.e. while no torch
    operation has written to it.  A write torch does not see (a kernel launched on its raw pointer, the replay of
    a captured graph into it) does not invalidate them: hand such a tensor to `forget_bins` first, or pass a new
    one.  Nothing is kept or reused under stream capture, where a graph must contain the kernel that computes
    the bins it uses."""
    if batch_sizes.ndim != 1:
        raise ValueError('batch_sizes must be a vector')
    capturing = batch_sizes.is_cuda and torch.cuda.is_current_stream_capturing()
    cached = getattr(batch_sizes, '_mbx_bins', None)
    if not capturing and cached is not None and cached[1] == batch_sizes._version and cached[0].device == device:
        if cached[2] is not None and cached[2] != rows:
            raise ValueError(f'gmm: batch_sizes add up to {cached[2]} rows but the operand has {rows}')
        return cached[0]
    total = None
    if batch_sizes.is_cuda:
        from megablocks_amd.ops.routing import inclusive_cumsum
        bins = inclusive_cumsum(batch_sizes.to(torch.int32), 0).view(-1)
    else:
        total = int(batch_sizes.sum()) if batch_sizes.numel() else 0
        if batch_sizes.numel() and int(batch_sizes.min()) < 0:
            raise ValueError('gmm: batch_sizes must not be negative')
        if total != rows:
            raise ValueError(f'gmm: batch_sizes add up to {total} rows but the operand has {rows}')
        bins = torch.cumsum(batch_sizes, 0).to(torch.int32).to(device)
    if not capturing:
        _remember(batch_sizes, (bins, batch_sizes._version, total))
    return bins


def _remember(batch_sizes: torch.Tensor, entry):
    try:
        batch_sizes._mbx_bins = entry
    except AttributeError:   # a tensor type without instance attributes: the bins are computed on every call
        pass


def forget_bins(batch_sizes: torch.Tensor):
    """Drops the bins kept for `batch_sizes` (for a tensor whose contents were changed behind torch's back)."""
    if getattr(batch_sizes, '_mbx_bins', None) is not None:
        batch_sizes._mbx_bins = None


def note_bins(batch_sizes: torch.Tensor, bins: torch.Tensor):
    """A caller that has already computed the inclusive cumsum of `batch_sizes` (int32, on the same device) hands
    it over, and the products of this step do not compute it again."""
    if batch_sizes.is_cuda and bins.dtype == torch.int32 and bins.device == batch_sizes.device \
            and bins.numel() == batch_sizes.numel() and not torch.cuda.is_current_stream_capturing():
        _remember(batch_sizes, (bins.view(-1), batch_sizes._version, None))


# Device memory the NN products lend the library for the parts of the tiles of their last round of workgroups
# (`mbx_gmm_ws`): one buffer per device and stream, made at the first product on that stream and kept.  Launches on
# one stream run one after the other, so they can share it; launches on different streams may overlap, so they do not.
# A stream that is being captured gets its buffer from the capture's memory pool like any tensor made during a capture
# (its zero-fill is a kernel of the graph; the buffer stays with this module, so later captures on a stream with the
# same handle reuse it).  MBX_GMM_WORKSPACE=0: none (every tile is computed by one workgroup; results differ in the
# last bits).
GMM_WORKSPACE = os.environ.get('MBX_GMM_WORKSPACE', '1') != '0'
_workspaces = {}


def _workspace(device):
    """(pointer, bytes) of the current stream's workspace on `device`; (None, 0) if switched off."""
    if not GMM_WORKSPACE:
        return None, 0
    key = (device.index if device.index is not None else torch.cuda.current_device(), _lib.stream().value)
    ws = _workspaces.get(key)
    if ws is None:
        ws = torch.zeros(lib.mbx_gmm_workspace_bytes(), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return _lib.ptr(ws), ws.numel()


def gmm(a, b, batch_sizes, trans_a=False, trans_b=False, c=None, _record_as=None):
    """out[r_e] = a[r_e] @ b[e] (`trans_b`: @ b[e].T); `trans_a`: out[e] = a[r_e].T @ b[r_e].

    a is [rows, k]; b is [E, k, n] ([E, n, k] with trans_b) or, with trans_a, [rows, n].
    fp32 accumulation, output in a.dtype, written to `c` when given.  `_record_as` names the launch in the
    optional per-launch timing (callers other than the expert MLPs keep out of their statistics).
    """
    _lib.require_cuda(a, b, c)
    if a.ndim != 2:
        raise ValueError('gmm: a must be a matrix')
    if a.dtype != b.dtype:
        raise ValueError('gmm: a and b must share a dtype')
    if trans_a and trans_b:
        raise ValueError('gmm: trans_a and trans_b cannot both be set')
    dt = _lib.dtype_of(a)
    a, b = a.contiguous(), b.contiguous()
    rows = a.shape[0]
    bins = _device_bins(batch_sizes, a.device, rows)
    groups = bins.shape[0]
    if trans_a:
        if b.ndim != 2 or b.shape[0] != rows:
            raise ValueError('gmm(trans_a): b must be [rows, n]')
        k, n, layout = a.shape[1], b.shape[1], _lib.TN
        shape = (groups, k, n)
    else:
        if b.ndim != 3 or b.shape[0] != groups:
            raise ValueError('gmm: b must be [num_groups, ., .]')
        k = a.shape[1]
        if trans_b:
            n, layout = b.shape[1], _lib.NT
            if b.shape[2] != k:
                raise ValueError('gmm(trans_b): inner dimensions differ')
        else:
            n, layout = b.shape[2], _lib.NN
            if b.shape[1] != k:
                raise ValueError('gmm: inner dimensions differ')
        shape = (rows, n)
    if c is None:
        c = torch.empty(shape, dtype=a.dtype, device=a.device)
    else:
        if tuple(c.shape) != shape or c.dtype != a.dtype or not c.is_contiguous():
            raise ValueError('gmm: c has the wrong shape, dtype or layout')
    with _lib.device_of(a), _lib.record(_record_as or ('gmm_nn', 'gmm_nt', 'gmm_tn')[layout], rows=rows, k=k, n=n,
                                              elem=a.element_size(), groups=groups):
        ws, ws_bytes = _workspace(a.device) if layout == _lib.NN else (None, 0)
        _lib.check(lib.mbx_gmm_ws(_lib.ptr(a), _lib.ptr(b), None, None, _lib.ptr(c), dt, _lib.ptr(bins), groups, rows, k, n,
                                  layout, ws, ws_bytes, _lib.stream()), 'gmm')
    return c


def gmm_dual(a, b, a2, b2, batch_sizes, trans_b=False, c=None):
    """out[r_e] = a[r_e] @ b[e] + a2[r_e] @ b2[e] (`trans_b`: both weights transposed), a2 / b2 shaped like a / b:
    the input gradient of the GLU experts (glu.py:160-166) as one reduction over both pairs.  Shapes the
    single-launch kernel does not take are computed as two `gmm` calls and an addition."""
    _lib.require_cuda(a, b, a2, b2, c)
    if a.shape != a2.shape or b.shape != b2.shape or a.dtype != a2.dtype or b.dtype != b2.dtype:
        raise ValueError('gmm_dual: the two operand pairs must have the same shapes and dtypes')
    if a.ndim != 2 or b.ndim != 3 or a.dtype != b.dtype:
        raise ValueError('gmm_dual: a must be [rows, k] and b [num_groups, ., .] of the same dtype')
    a, b, a2, b2 = a.contiguous(), b.contiguous(), a2.contiguous(), b2.contiguous()
    bins = _device_bins(batch_sizes, a.device, a.shape[0])
    groups, rows, k = bins.shape[0], a.shape[0], a.shape[1]
    n, layout = (b.shape[1], _lib.NT) if trans_b else (b.shape[2], _lib.NN)
    if b.shape[0] != groups or (b.shape[2] if trans_b else b.shape[1]) != k:
        raise ValueError('gmm_dual: b does not match a and batch_sizes')
    if c is None:
        c = torch.empty((rows, n), dtype=a.dtype, device=a.device)
    elif tuple(c.shape) != (rows, n) or c.dtype != a.dtype or not c.is_contiguous():
        raise ValueError('gmm_dual: c has the wrong shape, dtype or layout')
    with _lib.device_of(a), _lib.record('gmm_nt_dual' if trans_b else 'gmm_nn_dual', rows=rows, k=2 * k, n=n,
                                              elem=a.element_size(), groups=groups) as rec:
        ws, ws_bytes = _workspace(a.device) if layout == _lib.NN else (None, 0)
        rc = lib.mbx_gmm_ws(_lib.ptr(a), _lib.ptr(b), _lib.ptr(a2), _lib.ptr(b2), _lib.ptr(c), _lib.dtype_of(a),
                            _lib.ptr(bins), groups, rows, k, n, layout, ws, ws_bytes, _lib.stream())
        if rc == _lib.EUNSUPPORTED:
            rec.cancel()
    if rc == _lib.EUNSUPPORTED:
        gmm(a, b, batch_sizes, trans_b=trans_b, c=c)
        c += gmm(a2, b2, batch_sizes, trans_b=trans_b)
        return c
    _lib.check(rc, 'gmm_dual')
    return c


ACT_GELU_TANH = 1   # mbx_activation of include/mbx.h
# False: gmm_act / gmm_dact run the product and the element-wise pass as two launches (what they do anyway for shapes
# the epilogue kernels do not take); a switch for measurements
ACTIVATION_EPILOGUES = os.environ.get('MBX_ACTIVATION_EPILOGUES', '1') != '0'
# The epilogue's arithmetic is exposed (the matrix cores idle meanwhile), the separate pass it replaces costs a launch
# and a trip of the [rows, n] tensor through memory or, for tensors that fit it, the 256 MiB Infinity Cache.  With the
# epilogue's inputs fetched ahead the epilogues win at every size measured (c2's 128 MiB intermediate: layer step
# -1.3 %; c5's 1.5 GiB: -4.5 %; c3 / c4, gated: -2.6 % / -5.9 %), so the threshold is zero; it stays as a switch for
# measurements.
ACTIVATION_EPILOGUE_MIN_BYTES = int(os.environ.get('MBX_ACTIVATION_EPILOGUE_MIN_BYTES', 0))


def _use_epilogue(fuse, a, rows, n):
    if a.dtype not in (torch.bfloat16, torch.float16):
        return False
    if fuse is None:
        return ACTIVATION_EPILOGUES and rows * n * a.element_size() >= ACTIVATION_EPILOGUE_MIN_BYTES
    return bool(fuse)


def _nt_operands(a, b, batch_sizes, what):
    _lib.require_cuda(a, b)
    if a.ndim != 2 or b.ndim != 3 or a.dtype != b.dtype:
        raise ValueError(f'{what}: a must be [rows, k] and b [num_groups, n, k] of the same dtype')
    a, b = a.contiguous(), b.contiguous()
    bins = _device_bins(batch_sizes, a.device, a.shape[0])
    if b.shape[0] != bins.shape[0] or b.shape[2] != a.shape[1]:
        raise ValueError(f'{what}: b does not match a and batch_sizes')
    return a, b, bins


def gmm_act(a, b, batch_sizes, fuse=None):
    """(c, gelu_tanh(c)) with c[r_e] = a[r_e] @ b[e].T: the first product of the expert MLP and its activation
    (mlp.py:521-522), the activation applied in the product's epilogue where the library has a kernel for the shape
    (16-bit types, k a multiple of 64, n of 8) and the output is large enough for that to pay (`fuse` None; True /
    False force the choice), else as a separate element-wise pass."""
    a, b, bins = _nt_operands(a, b, batch_sizes, 'gmm_act')
    rows, k, n, groups = a.shape[0], a.shape[1], b.shape[1], bins.shape[0]
    c = torch.empty((rows, n), dtype=a.dtype, device=a.device)
    c_act = torch.empty_like(c)
    rc = _lib.EUNSUPPORTED
    if _use_epilogue(fuse, a, rows, n):
        with _lib.device_of(a), _lib.record('gmm_nt_act', rows=rows, k=k, n=n, elem=a.element_size(), groups=groups) as rec:
            rc = lib.mbx_gmm_act(_lib.ptr(a), _lib.ptr(b), _lib.ptr(c), _lib.ptr(c_act), _lib.dtype_of(a), _lib.ptr(bins),
                                 groups, rows, k, n, ACT_GELU_TANH, _lib.stream())
            if rc == _lib.EUNSUPPORTED:
                rec.cancel()
    if rc == _lib.EUNSUPPORTED:
        gmm(a, b, batch_sizes, trans_b=True, c=c)
        return c, torch.nn.functional.gelu(c, approximate='tanh')
    _lib.check(rc, 'gmm_act')
    return c, c_act


def gmm_dact(a, b, pre, batch_sizes, c=None, fuse=None):
    """round(a[r_e] @ b[e].T) * d/dx gelu_tanh(pre[r_e]): the activation gradient of the expert MLP's backward
    (mlp.py:478-483 with gelu.py:9-13) with the multiplication in the product's epilogue where the library has a
    kernel for the shape, else as `gmm` and `gelu_backward_`.  Written to `c` when given (which may not be `pre`)."""
    a, b, bins = _nt_operands(a, b, batch_sizes, 'gmm_dact')
    rows, k, n, groups = a.shape[0], a.shape[1], b.shape[1], bins.shape[0]
    _lib.require_cuda(pre, c)
    if tuple(pre.shape) != (rows, n) or pre.dtype != a.dtype or not pre.is_contiguous():
        raise ValueError('gmm_dact: pre has the wrong shape, dtype or layout')
    if c is None:
        c = torch.empty((rows, n), dtype=a.dtype, device=a.device)
    elif tuple(c.shape) != (rows, n) or c.dtype != a.dtype or not c.is_contiguous() or c.data_ptr() == pre.data_ptr():
        raise ValueError('gmm_dact: c has the wrong shape, dtype or layout')
    rc = _lib.EUNSUPPORTED
    if _use_epilogue(fuse, a, rows, n):
        with _lib.device_of(a), _lib.record('gmm_nt_dact', rows=rows, k=k, n=n, elem=a.element_size(), groups=groups) as rec:
            rc = lib.mbx_gmm_dact(_lib.ptr(a), _lib.ptr(b), _lib.ptr(pre), _lib.ptr(c), _lib.dtype_of(a), _lib.ptr(bins),
                                  groups, rows, k, n, ACT_GELU_TANH, _lib.stream())
            if rc == _lib.EUNSUPPORTED:
                rec.cancel()
    if rc == _lib.EUNSUPPORTED:
        from megablocks_amd.layers.gelu import gelu_backward_
        gmm(a, b, batch_sizes, trans_b=True, c=c)
        return gelu_backward_(c, pre)
    _lib.check(rc, 'gmm_dact')
    return c


def gmm_glu(a, b1, b2, batch_sizes, act, fuse=None):
    """(x1, x2, h) with x1 = a[r_e] @ b1[e].T, x2 = a[r_e] @ b2[e].T and h = activation(x1) * x2: the two first
    products of the GLU experts and their gated activation (glu.py:201-204) in one launch where the library has a
    kernel for the shape, else as two `gmm` and the element-wise pass.  act: 0 = SiLU, 1 = tanh-GELU."""
    a, b1, bins = _nt_operands(a, b1, batch_sizes, 'gmm_glu')
    _lib.require_cuda(b2)
    if b2.shape != b1.shape or b2.dtype != b1.dtype:
        raise ValueError('gmm_glu: b2 must be shaped and typed like b1')
    b2 = b2.contiguous()
    rows, k, n, groups = a.shape[0], a.shape[1], b1.shape[1], bins.shape[0]
    rc = _lib.EUNSUPPORTED
    if _use_epilogue(fuse, a, rows, n):
        x1, x2, h = (torch.empty((rows, n), dtype=a.dtype, device=a.device) for _ in range(3))
        with _lib.device_of(a), _lib.record('gmm_nt_glu', rows=rows, k=k, n=2 * n, elem=a.element_size(), groups=groups) as rec:
            rc = lib.mbx_gmm_glu(_lib.ptr(a), _lib.ptr(b1), _lib.ptr(b2), _lib.ptr(x1), _lib.ptr(x2), _lib.ptr(h),
                                 _lib.dtype_of(a), _lib.ptr(bins), groups, rows, k, n, act, _lib.stream())
            if rc == _lib.EUNSUPPORTED:
                rec.cancel()
    if rc == _lib.EUNSUPPORTED:
        from megablocks_amd.layers.glu import _glu_forward
        x1 = gmm(a, b1, batch_sizes, trans_b=True)
        x2 = gmm(a, b2, batch_sizes, trans_b=True)
        return x1, x2, _glu_forward(x1, x2, act)
    _lib.check(rc, 'gmm_glu')
    return x1, x2, h


# Whether the dMoE layer hands the experts the ungathered tokens (`gmm_gather`) instead of calling ops.gather /
# ops.padded_gather first: 'auto' = where no gradient is recorded and, with gradients, from top_k = 4 on (the weight
# gradients then read the tokens through a row table, `gmm_tn_gather`; no gathered copy is written or kept), '1' =
# always, '0' = never.  Where a weight gradient's shape is outside what the indexed kernel takes, the copy is made in the
# backward and exists only there.
FUSED_GATHER = os.environ.get('MBX_FUSED_GATHER', 'auto')


class GatheredRows:
    """The matrix ops.gather / ops.padded_gather (dmoe.py:219 / :273) would make of `x`, as a description: the rows of
    x in the order of the sorted assignments `indices`, each expert's rows padded with zero rows up to its padded bin
    when `padded_bins` is given.  `rows` is the row count of that matrix."""

    def __init__(self, x, indices, bin_ids, bins, padded_bins, top_k, rows):
        self.x, self.indices, self.bin_ids, self.bins, self.padded_bins = x, indices, bin_ids, bins, padded_bins
        self.top_k, self.rows = int(top_k), int(rows)

    def materialize(self):
        from megablocks_amd.backend import kernels
        if self.padded_bins is None:
            return kernels.gather(self.x, self.indices, self.bin_ids, None, self.bins, self.top_k)
        return kernels.padded_gather(self.x, self.indices, self.bin_ids, None, self.bins, self.padded_bins, self.top_k)

    def weight_gradient(self, d, batch_sizes):
        """gmm(d, self.materialize(), batch_sizes, trans_a=True): the weight gradient of a product whose operand these
        rows were (mlp.py:485-491, glu.py:154-159), read from the ungathered tokens where the library has a kernel for
        the shapes (`gmm_tn_gather`), else from the copy, which is then made once and kept for the next call."""
        out = gmm_tn_gather(d, self, batch_sizes)
        if out is None:
            if getattr(self, '_copy', None) is None:
                self._copy = self.materialize()
            out = gmm(d, self._copy, batch_sizes, trans_a=True)
        return out

    def scatter_grad(self, grad):
        """The gradient of x from the gradient of the gathered matrix (gather.py:28-35, padded_gather.py:36-52)."""
        from megablocks_amd.backend import kernels
        if self.padded_bins is None:
            return kernels.scatter(grad, self.indices, self.bin_ids, None, self.bins, self.top_k)
        return kernels.padded_scatter(grad, self.indices, self.bin_ids, None, self.bins, self.padded_bins, self.top_k)


def gmm_gather(src: GatheredRows, b1, batch_sizes, b2=None, act=None):
    """The first product(s) of the experts on the rows `src` describes, read from the ungathered tokens (one launch,
    `mbx_gmm_gather`): bit-identical to `src.materialize()` followed by
        b2 None, act None:  (gmm(a, b1, trans_b=True),)
        b2 None, act ACT_GELU_TANH:  gmm_act(a, b1)  -> (c, gelu_tanh(c))
        b2 given:  gmm_glu(a, b1, b2, act)  -> (x1, x2, h)
    Returns None where the library has no kernel for the operands: the caller then gathers and multiplies."""
    x = src.x
    if not (x.is_cuda and x.ndim == 2 and x.dtype in (torch.bfloat16, torch.float16) and b1.ndim == 3 and
            b1.dtype == x.dtype and b1.shape[2] == x.shape[1] and src.indices.dtype == torch.int32 and
            src.bins.dtype == torch.int32 and ACTIVATION_EPILOGUES):
        return None
    if b2 is not None and (b2.shape != b1.shape or b2.dtype != b1.dtype or act is None):
        return None
    if src.padded_bins is not None and src.padded_bins.dtype != torch.int32:
        return None
    if src.indices.ndim != 1 or src.indices.shape[0] != x.shape[0] * src.top_k:
        raise ValueError('gmm_gather: one assignment per token and top_k choice')
    _lib.require_cuda(b1, b2, src.indices, src.bins, src.padded_bins)
    x, b1 = x.contiguous(), b1.contiguous()
    b2 = None if b2 is None else b2.contiguous()
    rows, k, n = src.rows, x.shape[1], b1.shape[1]
    bins = _device_bins(batch_sizes, x.device, rows)
    groups = bins.shape[0]
    if b1.shape[0] != groups or src.bins.numel() != groups:
        return None
    x_bins = None if src.padded_bins is None else src.bins.contiguous()
    c = torch.empty((rows, n), dtype=x.dtype, device=x.device)
    c2 = None if b2 is None else torch.empty_like(c)
    h = None if act is None else torch.empty_like(c)
    name = 'gmm_nt_glu' if b2 is not None else 'gmm_nt_act' if act is not None else 'gmm_nt'
    with _lib.device_of(x), _lib.record(name, rows=rows, k=k, n=n * (2 if b2 is not None else 1), elem=x.element_size(),
                                        groups=groups) as rec:
        rc = lib.mbx_gmm_gather(_lib.ptr(x), x.shape[0], _lib.ptr(src.indices.contiguous()), src.top_k, _lib.ptr(x_bins),
                                _lib.ptr(b1), _lib.ptr(b2), _lib.ptr(c), _lib.ptr(c2), _lib.ptr(h), _lib.dtype_of(x),
                                _lib.ptr(bins), groups, rows, k, n, 0 if act is None else act, _lib.stream())
        if rc == _lib.EUNSUPPORTED:
            rec.cancel()
    if rc == _lib.EUNSUPPORTED:
        return None
    _lib.check(rc, 'gmm_gather')
    return (c,) if act is None else (c, h) if b2 is None else (c, c2, h)


def gmm_tn_gather(a, src: GatheredRows, batch_sizes, c=None):
    """out[e] = a[r_e].T @ X[r_e] with X the rows `src` describes, read from the ungathered tokens (one launch,
    `mbx_gmm_tn_gather`; bit-identical to `gmm(a, src.materialize(), batch_sizes, trans_a=True)`).  The table of row
    offsets the kernel reads is built by the first call for a `src` and kept on it (the weight gradients of w1 and v1
    share it).  Returns None where the library has no kernel for the operands: the caller gathers first."""
    x = src.x
    if not (x.is_cuda and x.ndim == 2 and x.dtype in (torch.bfloat16, torch.float16) and a.ndim == 2 and a.dtype == x.dtype
            and a.is_cuda and a.shape[0] == src.rows and src.indices.dtype == torch.int32 and src.bins.dtype == torch.int32):
        return None
    if src.padded_bins is not None and src.padded_bins.dtype != torch.int32:
        return None
    if src.indices.ndim != 1 or src.indices.shape[0] != x.shape[0] * src.top_k:
        raise ValueError('gmm_tn_gather: one assignment per token and top_k choice')
    _lib.require_cuda(src.indices, src.bins, src.padded_bins, c)
    a, x = a.contiguous(), x.contiguous()
    rows, k, n = a.shape[0], a.shape[1], x.shape[1]
    bins = _device_bins(batch_sizes, a.device, rows)
    groups = bins.shape[0]
    if src.bins.numel() != groups:
        return None
    x_bins = None if src.padded_bins is None else src.bins.contiguous()
    if c is None:
        c = torch.empty((groups, k, n), dtype=a.dtype, device=a.device)
    elif tuple(c.shape) != (groups, k, n) or c.dtype != a.dtype or not c.is_contiguous():
        raise ValueError('gmm_tn_gather: c has the wrong shape, dtype or layout')
    table = getattr(src, '_row_table', None)
    ready = table is not None and table[1] == n
    if not ready:
        table = (torch.empty(max(lib.mbx_gmm_tn_gather_table_bytes(x.shape[0], src.top_k, groups) // 4, 4), dtype=torch.int32,
                             device=x.device), n)
    with _lib.device_of(a), _lib.record('gmm_tn', rows=rows, k=k, n=n, elem=a.element_size(), groups=groups) as rec:
        rc = lib.mbx_gmm_tn_gather(_lib.ptr(a), _lib.ptr(x), x.shape[0], _lib.ptr(src.indices.contiguous()), src.top_k,
                                   _lib.ptr(x_bins), _lib.ptr(c), _lib.dtype_of(a), _lib.ptr(bins), groups, rows, k, n,
                                   _lib.ptr(table[0]), table[0].numel() * 4, 1 if ready else 0, _lib.stream())
        if rc == _lib.EUNSUPPORTED:
            rec.cancel()
    if rc == _lib.EUNSUPPORTED:
        return None
    _lib.check(rc, 'gmm_tn_gather')
    if not torch.cuda.is_current_stream_capturing():
        src._row_table = table
    return c


# Whether, with one expert per token, the dMoE layer has the experts' second product write the weighted combine of
# ops.scatter (dmoe.py:280) from its store phase (`gmm_scatter`): 'auto' / '1' = where the experts support it, '0' =
# never.  top_k > 1 always combines in a pass of its own (a token's row is then a sum over products of several tiles).
FUSED_COMBINE = os.environ.get('MBX_FUSED_COMBINE', 'auto')


class CombinedRows:
    """Where ops.scatter (dmoe.py:280, kernels.py:173-207) puts the rows of the experts' output when every token has one
    expert (top_k = 1), as a description: row r goes to row indices[r] of the output, times weights[indices[r]]."""

    def __init__(self, indices, bin_ids, bins, weights):
        self.indices, self.bin_ids, self.bins, self.weights = indices, bin_ids, bins, weights
        self.tokens = indices.shape[0]

    def scatter(self, y):
        """The combine as a pass of its own (what the fused launch replaces)."""
        from megablocks_amd.backend import kernels
        return kernels.scatter(y, self.indices, self.bin_ids, self.weights, self.bins, 1)

    def backward(self, y, grad, need_rows=True, need_weights=True):
        """(gradient of the rows y, gradient of the weights or None) of `scatter`, as ops/scatter.py:34-62."""
        from megablocks_amd.backend import kernels
        grad = grad.contiguous()
        if need_rows and need_weights and self.weights is not None:
            return kernels.scatter_backward(y, grad, self.indices, self.bin_ids, self.weights, self.bins, None, 1)
        rows = kernels.gather(grad, self.indices, self.bin_ids, self.weights, self.bins, 1) if need_rows else None
        wgrad = kernels.scatter_wgrad(y, grad, self.indices, self.bin_ids, self.bins, 1) \
            if need_weights and self.weights is not None else None
        return rows, wgrad


def gmm_scatter(a, b, batch_sizes, combine: CombinedRows, keep_product=True):
    """(y, out): y[r_e] = a[r_e] @ b[e], the experts' second product (mlp.py:523, glu.py:205), and out =
    ops.scatter(y, indices, bin_ids, weights, bins, top_k = 1) (dmoe.py:280), the combine written by the product's
    store phase (`mbx_gmm_scatter`; bit-identical to the two steps).  y is None when `keep_product` is False and the
    launch did not have to write it (nothing will differentiate).  Shapes the kernel does not take: two steps."""
    _lib.require_cuda(a, b, combine.indices, combine.weights)
    if a.ndim != 2 or b.ndim != 3 or a.dtype != b.dtype or b.shape[1] != a.shape[1]:
        raise ValueError('gmm_scatter: a must be [rows, k] and b [num_groups, k, n] of the same dtype')
    a, b = a.contiguous(), b.contiguous()
    rows, k, n = a.shape[0], a.shape[1], b.shape[2]
    bins = _device_bins(batch_sizes, a.device, rows)
    groups = bins.shape[0]
    indices, weights = combine.indices, combine.weights
    if b.shape[0] != groups or indices.shape[0] != rows:
        raise ValueError('gmm_scatter: b, batch_sizes and the assignments do not match a')
    rc = _lib.EUNSUPPORTED
    if indices.dtype == torch.int32 and a.dtype in (torch.bfloat16, torch.float16) and rows > 0 and \
            (weights is None or (weights.dtype in _lib.DTYPE and weights.numel() == combine.tokens)):
        y = torch.empty((rows, n), dtype=a.dtype, device=a.device) if keep_product else None
        out = torch.empty((combine.tokens, n), dtype=a.dtype, device=a.device)
        w = None if weights is None else weights.contiguous()
        with _lib.device_of(a), _lib.record('gmm_nn_scatter', rows=rows, k=k, n=n, elem=a.element_size(), groups=groups) as rec:
            rc = lib.mbx_gmm_scatter(_lib.ptr(a), _lib.ptr(b), _lib.ptr(y), _lib.ptr(out), _lib.dtype_of(a), _lib.ptr(bins),
                                     groups, rows, k, n, _lib.ptr(indices.contiguous()), _lib.ptr(w),
                                     0 if w is None else _lib.dtype_of(w), combine.tokens, _lib.stream())
            if rc == _lib.EUNSUPPORTED:
                rec.cancel()
    if rc == _lib.EUNSUPPORTED:
        y = gmm(a, b, batch_sizes)
        return y, combine.scatter(y)
    _lib.check(rc, 'gmm_scatter')
    return y, out


def gmm_dglu(a, b, x1, x2, batch_sizes, act, fuse=None):
    """The gradients (d x1, d x2) of `activation(x1) * x2` where the incoming gradient is g = a[r_e] @ b[e].T: the
    `gmm(ddsd_out, w2, trans_b=True)` of the GLU experts' backward and the backward of their gated activation
    (glu.py:135-153) in one launch where the library has a kernel for the shape, else as `gmm` and the element-wise
    pass.  act: 0 = SiLU, 1 = tanh-GELU."""
    a, b, bins = _nt_operands(a, b, batch_sizes, 'gmm_dglu')
    rows, k, n, groups = a.shape[0], a.shape[1], b.shape[1], bins.shape[0]
    _lib.require_cuda(x1, x2)
    for t in (x1, x2):
        if tuple(t.shape) != (rows, n) or t.dtype != a.dtype or not t.is_contiguous():
            raise ValueError('gmm_dglu: x1 / x2 have the wrong shape, dtype or layout')
    rc = _lib.EUNSUPPORTED
    if _use_epilogue(fuse, a, rows, n):
        d1 = torch.empty((rows, n), dtype=a.dtype, device=a.device)
        d2 = torch.empty((rows, n), dtype=a.dtype, device=a.device)
        with _lib.device_of(a), _lib.record('gmm_nt_dglu', rows=rows, k=k, n=n, elem=a.element_size(), groups=groups) as rec:
            rc = lib.mbx_gmm_dglu(_lib.ptr(a), _lib.ptr(b), _lib.ptr(x1), _lib.ptr(x2), _lib.ptr(d1), _lib.ptr(d2),
                                  _lib.dtype_of(a), _lib.ptr(bins), groups, rows, k, n, act, _lib.stream())
            if rc == _lib.EUNSUPPORTED:
                rec.cancel()
    if rc == _lib.EUNSUPPORTED:
        from megablocks_amd.layers.glu import _glu_backward
        return _glu_backward(gmm(a, b, batch_sizes, trans_b=True), x1, x2, act)
    _lib.check(rc, 'gmm_dglu')
    return d1, d2


class GroupedGemm(torch.autograd.Function):
    """Differentiable gmm(a, b, batch_sizes, trans_b): da = gmm(dc, b, trans_b flipped),
    db = the per-group outer product (trans_a)."""

    @staticmethod
    def forward(ctx, a, b, batch_sizes, trans_b):
        ctx.save_for_backward(a, b, batch_sizes)
        ctx.trans_b = trans_b
        return gmm(a, b, batch_sizes, trans_a=False, trans_b=trans_b)

    @staticmethod
    def backward(ctx, grad):
        grad = grad.contiguous()
        a, b, batch_sizes = ctx.saved_tensors
        trans_b = ctx.trans_b
        agrad = bgrad = None
        if ctx.needs_input_grad[0]:
            agrad = gmm(grad, b, batch_sizes, trans_a=False, trans_b=not trans_b)
        if ctx.needs_input_grad[1]:
            lhs, rhs = (grad, a) if trans_b else (a, grad)
            bgrad = gmm(lhs, rhs, batch_sizes, trans_a=True, trans_b=False)
        return agrad, bgrad, None, None


def autocast_operands(*tensors):
    """Under autocast the operands of a product are taken in the autocast type, as torch's own matmul does: with
    fp32 master weights the grouped experts then work like the block-sparse ones, whose stk products are
    autocast-aware in the reference.  The casts are ordinary autograd nodes (a weight's gradient comes back in the
    weight's type)."""
    if tensors[0].is_cuda and torch.is_autocast_enabled():
        dt = _lib.autocast_gpu_dtype()
        return tuple(t.to(dt) for t in tensors)
    return tensors


def _ops_gmm(a, b, batch_sizes, trans_b=False):
    a, b = autocast_operands(a, b)
    return GroupedGemm.apply(a, b, batch_sizes, trans_b)


backend = types.SimpleNamespace(gmm=gmm)
ops = types.SimpleNamespace(gmm=_ops_gmm)
