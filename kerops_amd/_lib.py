"""ctypes binding of libkerops_hip.so (the C ABI declared in include/kerops_hip.h).

There is no fallback: if the library has not been built, or a call returns an
error code, a RuntimeError is raised.  `python -m kerops_amd.build` builds it.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, '_C', 'libkerops_hip.so')

KEROPS_OK = 0
KEROPS_E_BADARG = -1
KEROPS_E_UNSUPPORTED_C = -2
KEROPS_E_WORKSPACE = -3
KEROPS_E_LAUNCH = -4

# KEROPS_HIP_VERSION of include/kerops_hip.h that SIGNATURES below mirrors
HEADER_VERSION = 210

DTYPE_TAGS = {torch.float16: 0, torch.float32: 1, torch.bfloat16: 2}
# result types the gradient reduction kernels write themselves (the *_f16_out entry points)
GW_DTYPES = {torch.float16: 0, torch.float32: 1}

_p = ctypes.c_void_p
_i32 = ctypes.c_int32
_i64 = ctypes.c_int64
_f32 = ctypes.c_float

# name -> (restype, argtypes); mirrors include/kerops_hip.h one to one
SIGNATURES = {
    'kerops_hip_version': (ctypes.c_int, []),
    'kerops_last_error_string': (ctypes.c_char_p, []),
    'kerops_dwconv_fwd_f16': (ctypes.c_int, [_p, _p, _p, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _p]),
    'kerops_dwconv_stats_workspace_bytes': (_i64, [_i32, _i32, _i32, _i32, _i32]),
    'kerops_dwconv_stats_f16': (ctypes.c_int, [_p, _p, _p, _p, _p, _p, _i64, _i32, _i32, _i32, _i32, _i32, _p]),
    'kerops_dwconv_bwd_workspace_bytes': (_i64, [_i32, _i32, _i32, _i32, _i32, _i32]),
    'kerops_dwconv_bwd_f16': (ctypes.c_int, [_p, _p, _p, _p, _p, _p, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _p]),
    'kerops_dwconv_bwd_f16_out': (ctypes.c_int, [_p, _p, _p, _p, _p, _i32, _p, _i64, _i32, _i32, _i32, _i32, _i32, _i32,
                                                 _p]),
    'kerops_dwconv_wgrad_workspace_bytes': (_i64, [_i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32]),
    'kerops_dwconv_wgrad_f16': (ctypes.c_int, [_p, _p, _p, _p, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32,
                                               _i32, _p]),
    'kerops_dwconv_wgrad_f16_out': (ctypes.c_int, [_p, _p, _p, _i32, _p, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _i32,
                                                   _i32, _i32, _p]),
    'kerops_dwconv_wgrad_noalloc_f16': (ctypes.c_int, [_p, _p, _p, _i32, _i32, _i32, _i32, _i32, _p]),
    'kerops_stats_workspace_bytes': (_i64, [_i64, _i32, _i32]),
    'kerops_stats_f16': (ctypes.c_int, [_p, _p, _p, _i64, _i32, _p, _i64, _i32, _i32, _i32, _p]),
    'kerops_stats_bwd_f16': (ctypes.c_int, [_p, _p, _p, _p, _i64, _i32, _i32, _i32, _i32, _p]),
    'kerops_add_stats_f16': (ctypes.c_int, [_p, _p, _p, _p, _p, _i64, _i32, _p, _i64, _i32, _i32, _i32, _p]),
    'kerops_add_stats_bwd_f16': (ctypes.c_int, [_p, _p, _p, _p, _p, _i64, _i32, _i32, _i32, _i32, _p]),
    'kerops_bnrelu_fwd_f16': (ctypes.c_int, [_p, _p, _p, _p, _i64, _i32, _i32, _i32, _i32, _p]),
    'kerops_bnrelu_bwd_f16': (ctypes.c_int, [_p, _p, _p, _p, _p, _p, _p, _i64, _i32, _p, _i64, _i32, _i32, _i32,
                                             _p]),
    'kerops_avgpool_ceil_stats_workspace_bytes': (_i64, [_i32, _i32, _i32, _i32, _i32, _i32]),
    'kerops_avgpool_ceil_stats_f16': (ctypes.c_int, [_p, _p, _p, _p, _i32, _i32, _i32, _i32, _i32, _p, _i64, _i32,
                                                     _i32, _i32, _p]),
    'kerops_bnrelu_avgpool_ceil_stats_f16': (ctypes.c_int, [_p, _p, _p, _p, _p, _p, _i32, _i32, _i32, _i32, _i32, _p,
                                                            _i64, _i32, _i32, _i32, _p]),
    'kerops_avgpool_ceil_stats_bwd_f16': (ctypes.c_int, [_p, _p, _p, _p, _p, _i32, _i32, _i32, _i32, _i32, _i32, _i32,
                                                         _i32, _p]),
    'kerops_quant_u8_window': (ctypes.c_int, [_p, _i32, _p, _i64, _f32, _i32, _i32, _i32, _p]),
    'kerops_dequant_u8_window': (ctypes.c_int, [_p, _p, _i32, _i64, _f32, _i32, _i32, _i32, _p]),
    'kerops_absmax_workspace_bytes': (_i64, [_i32]),
    'kerops_absmax_f16': (ctypes.c_int, [_p, _p, _i64, _p, _i64, _i32, _p]),
    'kerops_quant_i8_sym_f16': (ctypes.c_int, [_p, _p, _p, _p, _i64, _i32, _i32, _i32, _p]),
    'kerops_pointwise_f16': (ctypes.c_int, [_p, _p, _p, _p, _i64, _i32, _i32, _i32, _p]),
    'kerops_bnrelu_pointwise_f16': (ctypes.c_int, [_p, _p, _p, _p, _p, _p, _i64, _i32, _i32, _p]),
    'kerops_lin_brelu_lin_add_f16': (ctypes.c_int, [_p, _p, _p, _p, _p, _p, _i64, _i32, _p]),
    'kerops_lin_brelu_lin_bwd_workspace_bytes': (_i64, [_i64, _i32]),
    'kerops_lin_brelu_lin_bwd_f16': (ctypes.c_int, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i32, _p]),
    'kerops_lin_brelu_lin_bwd_f16_out': (ctypes.c_int, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i32, _p, _i64, _i64, _i32,
                                                        _p]),
    'kerops_relu_linear_bwd_workspace_bytes': (_i64, [_i64, _i32, _i32]),
    'kerops_relu_linear_bwd_f16': (ctypes.c_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _i32, _i32, _p]),
    'kerops_relu_linear_bwd_f16_out': (ctypes.c_int, [_p, _p, _p, _p, _p, _i32, _p, _i64, _i64, _i32, _i32, _p]),
    'kerops_dwsep_block_workspace_bytes': (_i64, [_i32, _i32, _i32, _i32, _i32, _i32]),
    'kerops_dwsep_block_f16': (ctypes.c_int, [_p, _p, _p, _p, _p, _p, _p, _i32, _i32, _i32, _i32, _i32, _i32, _p,
                                              _i64, _p]),
}

_lib = None


class KeropsHipError(RuntimeError):
    def __init__(self, name, code, text):
        super().__init__(f'{name} failed with code {code}: {text}')
        self.code = code


def load():
    """Load the library once; raise if it is missing (no CPU or eager fallback exists)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f'{LIB_PATH} is missing: build the HIP extension first (python -m kerops_amd.build); '
                'kerops_amd has no fallback path'
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        built = lib.kerops_hip_version()
        if built != HEADER_VERSION:
            raise RuntimeError(
                f'{LIB_PATH} reports interface version {built}, this binding was written for {HEADER_VERSION}: '
                'rebuild the library (python -m kerops_amd.build)'
            )
        _lib = lib
    return _lib


def last_error():
    return load().kerops_last_error_string().decode('utf-8', 'replace')


def call(name, *args):
    """Call an int-returning entry point and turn error codes into exceptions."""
    rc = getattr(load(), name)(*args)
    if rc != KEROPS_OK:
        raise KeropsHipError(name, rc, last_error())
    return rc


def query(name, *args):
    """Call a *_workspace_bytes function (negative result = error)."""
    n = getattr(load(), name)(*args)
    if n < 0:
        raise KeropsHipError(name, int(n), last_error())
    return int(n)


def ptr(t):
    return t.data_ptr() if t is not None else None


_raw_stream = getattr(torch._C, '_cuda_getCurrentRawStream', None)


def stream_of(t):
    """Raw hipStream_t of torch's current stream on the tensor's device."""
    if _raw_stream is not None:  # one C call instead of building a torch.cuda.Stream object (4 us)
        index = t.device.index
        return _raw_stream(index if index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


def workspace(nbytes, device):
    """Scratch buffer owned by the caller side of the ABI (torch's caching allocator)."""
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=device)
