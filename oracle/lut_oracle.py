"""TEST INFRASTRUCTURE ONLY: ctypes front-end for the plain-C look-up-table oracle (lut_oracle.c).

Only tests, the smoke check and the benchmark's CPU-baseline leg may import this module.  It never
touches a GPU and is never imported by the shipped package.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

i32p = ctypes.POINTER(ctypes.c_int32)
i64p = ctypes.POINTER(ctypes.c_int64)


def build():
    """Compile lut_oracle.c with gcc (a second or two)."""
    subprocess.check_call(['make', '-s', '-C', _HERE, 'liblut_oracle.so'])


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, 'liblut_oracle.so')
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
    return _LIB


def _layout_i32(layout):
    a = np.ascontiguousarray(np.asarray(layout), dtype=np.int32)
    assert a.ndim == 3
    return a


def _p32(a):
    return a.ctypes.data_as(i32p)


def _p64(a):
    return a.ctypes.data_as(i64p)


def _check(rc, what):
    if rc == -2:
        raise RuntimeError('%s: layout has a head without nonzero blocks (the reference raises here too)' % what)
    if rc != 0:
        raise RuntimeError('%s failed with code %d' % (what, rc))


def sdd_segment(layout, start_width):
    """-> list of (pack, int32 array [rows, 4]) like torch_blocksparse_cpp_utils.sdd_segment (utils.cpp:95-120)."""
    lay = _layout_i32(layout).copy()
    H, R, C = lay.shape
    nnz = int((lay != 0).sum())
    # the reference can emit more rows than nonzeros (rows for already-retained or empty positions), so size for
    # the worst case: every visit at level w emits at most w*w rows
    cap = 21 * max(nnz, 1) + 16
    out = np.zeros((cap * 4,), dtype=np.int32)
    packs = np.zeros((64,), dtype=np.int32)
    rows = np.zeros((64,), dtype=np.int64)
    nlev = ctypes.c_int(0)
    rc = lib().orc_sdd_segment(_p32(lay), H, R, C, int(start_width), _p32(out), ctypes.c_int64(cap),
                               _p32(packs), _p64(rows), ctypes.byref(nlev))
    _check(rc, 'sdd_segment')
    res, done = [], 0
    for k in range(nlev.value):
        r = int(rows[k])
        res.append((int(packs[k]), out[done * 4:(done + r) * 4].reshape(r, 4).copy()))
        done += r
    return res


def make_sdd_lut(layout, block):
    """-> (luts, widths, packs) like _sparse_matmul.make_sdd_lut (matmul.py:281-297)."""
    seg = sdd_segment(layout, 64 // block)
    luts = [t.reshape(-1) for _, t in seg]
    widths = [t.shape[0] // (p * p) for p, t in seg]
    packs = [p for p, _ in seg]
    return luts, widths, packs


def load_balance(sizes):
    """-> segments, column, lockid, maxid, offsets (int64 arrays), matmul.py:221-267."""
    s = np.ascontiguousarray(np.asarray(sizes), dtype=np.int64)
    cap = 2 * len(s) + 2
    arrs = [np.zeros((cap,), dtype=np.int64) for _ in range(5)]
    w = ctypes.c_int(0)
    rc = lib().orc_load_balance(_p64(s), len(s), *[_p64(a) for a in arrs], cap, ctypes.byref(w))
    _check(rc, 'load_balance')
    return tuple(a[:w.value].copy() for a in arrs)


def make_dxx_lut(layout, block, step, trans):
    """-> (lut int32 array, num_locks, width), matmul.py:372-458."""
    lay = _layout_i32(layout)
    H, R, C = lay.shape
    nnz = int((lay != 0).sum())
    div = max(block // step, 1)
    cap = 6 * (2 * H * max(R, C) + 2) + 2 * nnz * div + 2
    lut = np.zeros((cap,), dtype=np.int32)
    n = ctypes.c_int64(0)
    w = ctypes.c_int(0)
    nl = ctypes.c_int(0)
    rc = lib().orc_dxx_lut(_p32(lay), H, R, C, int(block), int(step), int(bool(trans)), _p32(lut), ctypes.c_int64(cap),
                           ctypes.byref(n), ctypes.byref(w), ctypes.byref(nl))
    _check(rc, 'make_dxx_lut')
    return lut[:n.value].copy(), nl.value, w.value


def make_softmax_lut(layout):
    """-> (lut int32 array, maxlut), softmax.py:201-221."""
    lay = _layout_i32(layout)
    H, R, C = lay.shape
    cap = 2 * H * R + 4 * int(lay.sum()) + 4
    lut = np.zeros((cap,), dtype=np.int32)
    n = ctypes.c_int64(0)
    mx = ctypes.c_int(0)
    rc = lib().orc_softmax_lut(_p32(lay), H, R, C, _p32(lut), ctypes.c_int64(cap), ctypes.byref(n), ctypes.byref(mx))
    _check(rc, 'make_softmax_lut')
    return lut[:n.value].copy(), mx.value


def _make_layout(fn, num_heads, num_blocks, mode, block_stride, unidirectional, numverts, vertsize):
    out = np.zeros((num_heads, num_blocks, num_blocks), dtype=np.int64)
    fn.restype = None
    fn(int(num_heads), int(num_blocks), int(mode == 'dense'), int(block_stride), int(bool(unidirectional)), int(numverts),
       int(vertsize), _p64(out))
    return out


def make_layout_cpp(num_heads, num_blocks, mode, block_stride, unidirectional, numverts, vertsize):
    """csrc/utils.cpp:123-148."""
    return _make_layout(lib().orc_make_layout_cpp, num_heads, num_blocks, mode, block_stride, unidirectional, numverts, vertsize)


def make_layout_py(num_heads, num_blocks, mode, block_stride, attention, numverts, vertsize):
    """deepspeedsparseselfattention.py:31-65 (`attention` is 'unidirectional' or 'bidirectional')."""
    return _make_layout(lib().orc_make_layout_py, num_heads, num_blocks, mode, block_stride, attention == 'unidirectional',
                        numverts, vertsize)
