"""GPU: the allocation-free variant of bsp_dsd_matmul (static scratch inside the library) against bsp_dsd_matmul itself,
through the C ABI, on two calls in a row, the second with a smaller input."""
import ctypes

import pytest
import torch

import torch_blocksparse as tb
from torch_blocksparse import _lib
from torch_blocksparse.matmul import GroupPlan
from helpers import random_layout

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def dsd_args(a, b, c, trans_a, block, lut, width):
    return [_lib.DTYPES[b.dtype], _lib.ptr(a), _lib.ptr(b), _lib.ptr(c), int(trans_a), 0, 0, b.size(0), b.size(3),
            a.stride(0), b.stride(0), b.stride(1), b.stride(2), c.stride(0), c.stride(1), c.stride(2), block,
            _lib.ptr(lut), _lib.ptr(lut.planbuf), width]


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_noalloc_entry_point_matches_the_workspace_one(dtype):
    lib = _lib.load()
    n, block = 300, 64
    lay = random_layout((2, n, 4), 0.15, 99)
    lay[:, :, 1] = 1                                       # one chain of 300 blocks per head: 5 parts each
    op = tb.MatMul(lay, block, 'dsd', trans_a=True)
    lut, _, width, _ = op.make_lut(dtype, torch.device(DEV))[:4]
    plan = lut.gplan
    assert plan.n_split == 2
    nnz = int(lay.sum())
    g = torch.Generator().manual_seed(3)
    a_full = (0.1 * torch.randn(3, nnz, block, block, generator=g)).to(dtype).to(DEV)
    b_full = torch.randn(3, 2, n * block, 128, generator=g).to(dtype).to(DEV)
    stream = _lib.stream_ptr(torch.device(DEV))
    # first call: batch 3, two tiles of the free dimension (12 slots); second call, right after it: batch 2, one tile
    for a, b in ((a_full, b_full), (a_full[:2].contiguous(), b_full[:2, :, :, :64].contiguous())):
        Z, N = b.size(0), b.size(3)
        want = torch.empty(Z, 2, 4 * block, N, dtype=dtype, device=DEV)
        got = torch.full_like(want, float('nan'))
        ws, ws_bytes = plan.workspace(N, Z)
        rc = lib.bsp_dsd_matmul(*dsd_args(a, b, want, True, block, lut, width), *GroupPlan.args(plan), plan.n_split, ws, ws_bytes, 0, stream)
        assert rc == 0
        before = torch.cuda.memory_allocated()
        rc = lib.bsp_dsd_matmul_noalloc(*dsd_args(a, b, got, True, block, lut, width), *GroupPlan.args(plan), plan.n_split, 0, stream)
        assert rc == 0, _lib.strerror(rc)
        assert torch.cuda.memory_allocated() == before
        torch.cuda.synchronize()
        assert torch.equal(got, want)                     # the parts are added in a fixed order: bit for bit
    # the same operator through the Python layer, against the dense oracle's answer for good measure
    ref = op(a_full, b_full)
    out = torch.empty_like(ref)
    rc = lib.bsp_dsd_matmul_noalloc(*dsd_args(a_full, b_full, out, True, block, lut, width), *GroupPlan.args(plan), plan.n_split, 0, stream)
    assert rc == 0 and torch.equal(out, ref)


def test_noalloc_entry_point_refuses_what_does_not_fit():
    lib = _lib.load()
    n, block = 200, 64
    lay = random_layout((3, n, 8), 0.05, 5)
    lay[:, :, 0] = 1
    lay[:, :, 2] = 1                                       # 6 split chains
    op = tb.MatMul(lay, block, 'dsd', trans_a=True)
    lut, _, width, _ = op.make_lut(torch.float16, torch.device(DEV))[:4]
    plan = lut.gplan
    assert plan.n_split == 6
    Z, N = 4, 192                                          # 6 chains x 3 tiles x 4 batches = 72 slots > 64
    a = torch.zeros(Z, int(lay.sum()), block, block, dtype=torch.float16, device=DEV)
    b = torch.zeros(Z, 3, n * block, N, dtype=torch.float16, device=DEV)
    c = torch.zeros(Z, 3, 8 * block, N, dtype=torch.float16, device=DEV)
    rc = lib.bsp_dsd_matmul_noalloc(*dsd_args(a, b, c, True, block, lut, width), *GroupPlan.args(plan), plan.n_split, 0,
                                    _lib.stream_ptr(torch.device(DEV)))
    assert rc == _lib.ERR_SCRATCH_LIMIT and 'static scratch' in _lib.strerror(rc)
