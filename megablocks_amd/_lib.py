"""ctypes binding of libmbx.so (declared in include/mbx.h).

The library is required: importing this module raises if it has not been built, and no
operator has a PyTorch or CPU fallback.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# MBX_LIBRARY: another build of the library to load instead (measurements: libmbx_ticks.so)
LIB_PATH = os.environ.get('MBX_LIBRARY') or os.path.join(_HERE, 'libmbx.so')

I16, I32, I64 = 0, 1, 2
BF16, F16, F32 = 0, 1, 2
NN, NT, TN = 0, 1, 2
EINVAL, ESCRATCH, ERANGE, EUNSUPPORTED, ECAPTURE = -1, -2, -3, -4, -5

ITYPE = {torch.int16: I16, torch.int32: I32, torch.int64: I64}
DTYPE = {torch.bfloat16: BF16, torch.float16: F16, torch.float32: F32}

_vp, _i, _i64, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t

_SIGNATURES = {
    'mbx_version': (ctypes.c_int, []),
    'mbx_error_string': (ctypes.c_char_p, [_i]),
    'mbx_init': (_i, []),
    'mbx_histogram': (_i, [_vp, _i, _i64, _i64, _i, _vp, _vp]),
    'mbx_sort_scratch_bytes': (_sz, [_i64, _i, _i]),
    'mbx_sort': (_i, [_vp, _i, _i64, _i, _vp, _vp, _vp, _sz, _vp]),
    'mbx_route': (_i, [_vp, _i64, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    'mbx_cumsum': (_i, [_vp, _i, _i64, _i64, _i, _vp, _vp]),
    'mbx_topology': (_i, [_vp, _i, _i, _i, _i, _vp, _vp]),
    'mbx_replicate_forward': (_i, [_vp, _i, _i64, _i, _vp, _vp, _i64, _vp]),
    'mbx_replicate_backward': (_i, [_vp, _i, _i64, _i64, _vp, _i, _vp, _vp]),
    'mbx_gather': (_i, [_vp, _i, _i64, _i, _i, _vp, _vp, _vp, _i, _vp, _i, _vp, _i64, _vp, _vp]),
    'mbx_slot_rows': (_i, [_vp, _vp, _vp, _vp, _i, _i64, _vp, _vp]),
    'mbx_scatter': (_i, [_vp, _i, _i64, _i, _i, _vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp, _vp, _sz, _vp]),
    'mbx_scatter_static': (_i, [_vp, _i, _i64, _i, _i, _vp, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp]),
    'mbx_scatter_wgrad': (_i, [_vp, _vp, _i, _i64, _i, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp]),
    'mbx_scatter_backward': (_i, [_vp, _vp, _i, _i64, _i, _i, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp, _i64, _vp, _vp]),
    'mbx_binned_gather': (_i, [_vp, _i, _i64, _i, _i, _vp, _vp, _i, _i, _vp, _i, _vp, _vp]),
    'mbx_binned_scatter': (_i, [_vp, _i, _i64, _i, _i, _vp, _vp, _i, _i, _vp, _i, _vp, _vp, _sz, _vp]),
    'mbx_binned_scatter_wgrad': (_i, [_vp, _vp, _i, _i64, _i, _i, _vp, _vp, _i, _i, _vp, _vp]),
    'mbx_gmm': (_i, [_vp, _vp, _vp, _i, _vp, _i, _i64, _i, _i, _i, _vp]),
    'mbx_gmm_dual': (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i64, _i, _i, _i, _vp]),
    'mbx_gmm_workspace_bytes': (_sz, []),
    'mbx_gmm_ws': (_i, [_vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i64, _i, _i, _i, _vp, _sz, _vp]),
    'mbx_gmm_act': (_i, [_vp, _vp, _vp, _vp, _i, _vp, _i, _i64, _i, _i, _i, _vp]),
    'mbx_gmm_dact': (_i, [_vp, _vp, _vp, _vp, _i, _vp, _i, _i64, _i, _i, _i, _vp]),
    'mbx_gmm_glu': (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i64, _i, _i, _i, _vp]),
    'mbx_gmm_scatter': (_i, [_vp, _vp, _vp, _vp, _i, _vp, _i, _i64, _i, _i, _vp, _vp, _i, _i64, _vp]),
    'mbx_gmm_tn_gather_table_bytes': (_sz, [_i64, _i, _i]),
    'mbx_gmm_tn_gather': (_i, [_vp, _vp, _i64, _vp, _i, _vp, _vp, _i, _vp, _i, _i64, _i, _i, _vp, _sz, _i, _vp]),
    'mbx_gmm_dglu': (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i64, _i, _i, _i, _vp]),
    'mbx_gmm_gather': (_i, [_vp, _i64, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _i, _i64, _i, _i, _i, _vp]),
    'mbx_gelu_backward_inplace': (_i, [_vp, _vp, _i, _i64, _vp]),
    'mbx_glu_forward': (_i, [_vp, _vp, _vp, _i, _i, _i64, _vp]),
    'mbx_glu_backward': (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i64, _vp]),
    'mbx_router_forward': (_i, [_vp, _i, _i64, _i, _i, ctypes.c_float, _vp, _vp, _vp, _vp, _vp, _vp]),
    'mbx_router_backward': (_i, [_vp, _vp, _vp, _vp, _i, _i64, _i, _i, ctypes.c_float, _vp, _vp, _vp]),
}


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f'{LIB_PATH} is missing: build the HIP kernels first with `python megablocks_amd/build.py` '
            '(needs hipcc; cross-compiles for gfx950 without a GPU).')
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)   # AttributeError if the library lacks a declared symbol
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def check(code: int, what: str = 'mbx'):
    if code != 0:
        raise RuntimeError(f'{what} failed: {lib.mbx_error_string(code).decode()} (code {code})')


def ptr(t):
    """Device address of a tensor (None -> NULL)."""
    return None if t is None else ctypes.c_void_p(t.data_ptr())


_raw_stream = getattr(torch._C, '_cuda_getCurrentRawStream', None)


def stream():
    """The current stream of the current device as the ABI takes it.  Called once per launch: the raw handle
    straight from the binding where torch has one (several times cheaper than building a Stream object)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class device_of:
    """`with device_of(tensor):` makes the tensor's device current for the launch (and restores the previous one);
    nothing to do, and nearly free, when it already is."""
    __slots__ = ('idx', 'prev')

    def __init__(self, t):
        self.idx, self.prev = t.device.index, -1

    def __enter__(self):
        cur = torch.cuda.current_device()
        if self.idx is not None and cur != self.idx:
            self.prev = cur
            torch.cuda.set_device(self.idx)
        return self

    def __exit__(self, *exc):
        if self.prev >= 0:
            torch.cuda.set_device(self.prev)
        return False


def autocast_gpu_dtype():
    get = getattr(torch, 'get_autocast_dtype', None)
    return get('cuda') if get is not None else torch.get_autocast_gpu_dtype()


def require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError('expected a tensor on the GPU')  # TORCH_CHECK(x.is_cuda()) in csrc/*.h


def itype_of(t):
    if t.dtype not in ITYPE:
        raise RuntimeError(f'expected an int16/int32/int64 tensor but got {t.dtype}')
    return ITYPE[t.dtype]


def dtype_of(t):
    if t.dtype not in DTYPE:
        raise RuntimeError(f'expected a bfloat16/float16/float32 tensor but got {t.dtype}')
    return DTYPE[t.dtype]


def as_i32(t):
    """Index tensors cross the ABI as contiguous int32."""
    if t is None:
        return None
    if t.dtype != torch.int32:
        t = t.to(torch.int32)
    return t.contiguous()


# ---- optional per-launch timing (used by bench.py; off by default) -----------------------
# When `profile_hook` is a list, every operator appends (name, meta, start_event, end_event)
# for each launch, the events recorded on the stream the kernel was enqueued on.
profile_hook = None


class record:
    """`with record('gmm_nt', rows=..., k=..., n=...):` around a launch."""
    __slots__ = ('name', 'meta', 'ev0')

    def __init__(self, name, **meta):
        self.name, self.meta, self.ev0 = name, meta, None

    def __enter__(self):
        if profile_hook is not None:
            self.ev0 = torch.cuda.Event(enable_timing=True)
            self.ev0.record()
        return self

    def cancel(self):
        """Drop this launch from the profile (the call turned out not to launch the kernel it names)."""
        self.ev0 = None

    def __exit__(self, *exc):
        if self.ev0 is not None:
            ev1 = torch.cuda.Event(enable_timing=True)
            ev1.record()
            profile_hook.append((self.name, self.meta, self.ev0, ev1))
        return False
