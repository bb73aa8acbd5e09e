"""ctypes binding of libbsp_hip.so (C ABI declared in include/bsp.h).

The library is the only compute path of this package: there is no CPU or eager fallback.  If it has not
been built, importing the package still works (so that layouts and configuration objects can be used), but
every operator raises at its first call.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), 'lib', 'libbsp_hip.so')

F16, BF16, F32 = 0, 1, 2
DTYPES = {torch.float16: F16, torch.bfloat16: BF16, torch.float32: F32}

FLAG_GENERAL_ONLY, FLAG_NO_GROUPS, FLAG_NO_WIDE, FLAG_PLAN_ROWPAIR = 1, 2, 4, 8   # bsp_launch_flags

OK = 0
OK_WHOLE_LAYOUT = 1   # bsp_sdd_matmul: the group plan was used, every block of the layout is written
NEEDS_TABLE = 2       # bsp_sdd_matmul called with the plan alone: nothing launched, the sdd table is needed
ERR_UNSUPPORTED = -2
ERR_CAPACITY = -3
ERR_EMPTY_HEAD = -4
ERR_ROW_TOO_LONG = -6
ERR_K_MULTIPLE = -7
ERR_SCRATCH_LIMIT = -8

_c = ctypes
_vp, _i, _i64, _f = _c.c_void_p, _c.c_int, _c.c_int64, _c.c_float
_pi, _pi64 = _c.POINTER(_c.c_int), _c.POINTER(_c.c_int64)

# name -> (restype, argtypes); must list every symbol of include/bsp.h
SIGNATURES = {
    'bsp_version': (_i, []),
    'bsp_strerror': (_c.c_char_p, [_i]),
    'bsp_lut_workspace_bytes': (_i64, [_i, _i, _i]),
    'bsp_layout_nnz': (_i, [_vp, _i, _i, _i, _vp, _i64, _pi64, _vp]),
    'bsp_softmax_lut_build': (_i, [_vp, _i, _i, _i, _vp, _i64, _vp, _i64, _pi64, _pi, _vp]),
    'bsp_dxx_lut_cap': (_i64, [_i, _i, _i, _i64, _i, _i, _i]),
    'bsp_dxx_plan_cap': (_i64, [_i, _i, _i, _i64, _i]),
    'bsp_dxx_plan_pairs_offset': (_i64, [_i]),
    'bsp_dxx_lut_build': (_i, [_vp, _i, _i, _i, _i, _i, _i, _vp, _i64, _vp, _vp, _i64, _pi64, _pi, _pi, _vp]),
    'bsp_sdd_lut_build': (_i, [_vp, _i, _i, _i, _i, _vp, _vp, _i64, _vp, _i64, _pi, _pi, _pi64, _pi64, _pi, _vp]),
    'bsp_group_plan_cap': (_i64, [_i, _i, _i, _i64, _i]),
    'bsp_group_plan_build': (_i, [_vp, _i, _i, _i, _i, _i, _i, _i, _vp, _i64, _vp, _i64, _pi, _pi, _pi64, _vp]),
    'bsp_xsd_workspace_bytes': (_i64, [_i, _i, _i]),
    'bsp_sdd_matmul': (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _i, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i, _i, _vp, _vp,
                            _i64, _vp, _i, _i, _i, _vp]),
    'bsp_sdd_splitk_workspace_bytes': (_i64, [_i, _i64, _i]),
    'bsp_sdd_matmul_splitk': (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _i, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i, _vp, _vp,
                                   _i64, _i, _vp, _i64, _i, _vp]),
    'bsp_dsd_matmul': (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i, _vp, _vp,
                            _i, _vp, _i, _i, _i, _vp, _i64, _i, _vp]),
    'bsp_dsd_matmul_noalloc': (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i, _vp, _vp,
                                    _i, _vp, _i, _i, _i, _i, _vp]),
    'bsp_dds_matmul': (_i, [_i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i, _vp, _vp,
                            _i, _vp, _i, _i, _i, _vp, _i64, _i, _vp]),
    'bsp_softmax_fwd': (_i, [_i, _vp, _f, _vp, _i, _vp, _i64, _i64, _i64, _vp, _i64, _i, _vp, _i64, _i, _i, _i, _i, _i,
                             _i64, _vp]),
    'bsp_softmax_bwd': (_i, [_i, _vp, _vp, _f, _vp, _i, _i, _i, _i, _i, _i64, _i64, _vp]),
    'bsp_softmax_dropout_fwd': (_i, [_i, _vp, _vp, _f, _vp, _i, _vp, _i64, _i64, _i64, _vp, _i64, _i, _vp, _i64, _i, _i, _i, _i, _i,
                                     _i64, _i64, _f, _c.c_uint64, _c.c_uint64, _vp]),
    'bsp_softmax_dropout_bwd': (_i, [_i, _vp, _vp, _f, _vp, _i, _i, _i, _i, _i, _i64, _i64, _f, _c.c_uint64, _c.c_uint64, _vp]),
    'bsp_attention_fwd': (_i, [_i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i] + [_i64] * 13 + [_i, _f, _vp, _i, _vp, _i64, _i64, _i64,
                                _vp, _i64, _i, _vp, _i64, _i, _vp]),
    'bsp_attention_bwd': (_i, [_i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i] + [_i64] * 17 + [_i, _f, _vp, _i, _vp, _i64, _vp]),
    'bsp_attention_bwd_kv': (_i, [_i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i] + [_i64] * 17 + [_i, _f, _vp, _i, _vp, _i, _vp, _i, _vp]),
    'bsp_layout_fixed': (_i, [_vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    'bsp_layout_sparse_transformer': (_i, [_vp, _i, _i, _i, _i, _i, _vp]),
    'bsp_layout_bigbird': (_i, [_vp, _i, _i, _i, _i, _i, _vp, _i, _vp]),
    'bsp_relu_workspace_bytes': (_i64, []),
    'bsp_relu_fwd': (_i, [_i, _vp, _vp, _vp, _vp, _vp, _i64, _vp]),
    'bsp_relu_bwd': (_i, [_i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    'bsp_transpose': (_i, [_i, _vp, _vp, _i64, _i64, _vp]),
}

_lib = None


class BlocksparseLibraryError(RuntimeError):
    pass


def load():
    """Load the HIP library (once).  Raises if it is missing: there is nothing to fall back to."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise BlocksparseLibraryError(
            'torch_blocksparse: %s not found. Build it with `python torch-blocksparse_amd/build.py` '
            '(needs hipcc); this package has no fallback implementation.' % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def strerror(code):
    return load().bsp_strerror(code).decode()


def check(code, what):
    if code != OK:
        raise BlocksparseLibraryError('%s failed: %s (status %d)' % (what, strerror(code), code))


def stream_ptr(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def require_gpu_tensor(t, what):
    if not t.is_cuda:
        raise BlocksparseLibraryError('torch_blocksparse: %s must live on the GPU (got device %s); '
                                      'the operators run only as HIP kernels' % (what, t.device))


def layout_to_device(layout, device):
    """int32 copy of a [H, R, C] layout on `device`."""
    if layout.dim() != 3:
        raise ValueError('layout must have shape [heads, block-rows, block-cols]')
    return layout.to(device=device, dtype=torch.int32).contiguous()


def workspace(layout, device):
    H, R, C = layout.shape
    n = load().bsp_lut_workspace_bytes(H, R, C)
    return torch.empty(n, dtype=torch.uint8, device=device), n
