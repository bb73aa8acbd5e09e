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
    lay[:, :, 1] = 1                                       # one chain of 300 blocks per head, cut into 3 parts (split length 128)
    op = tb.MatMul(lay, block, 'dsd', trans_a=True)
    lut, _, width, _ = op.make_lut(dtype, torch.device(DEV))[:4]
    plan = lut.gplan
    assert plan.n_split == 2
    nnz = int(lay.sum())
    g = torch.Generator().manual_seed(3)
    a_full = (0.1 * torch.randn(3, nnz, block, block, generator=g)).to(dtype).to(DEV)
    b_full = torch.randn(3, 2, n * block, 128, generator=g).to(dtype).to(DEV)
    stream = _lib.stream_ptr(torch.device(DEV))
    # Set-up: the first call on a device looks up the address of the library's static buffer, which makes the runtime
    # load the code object that holds it (its 8 MiB then appear in the driver's free-memory figure, once per process).
    # That is the one-time set-up, to be done outside a graph capture; the calls after it are the ones measured below.
    warm = torch.empty(3, 2, 4 * block, 128, dtype=dtype, device=DEV)
    assert lib.bsp_dsd_matmul_noalloc(*dsd_args(a_full, b_full, warm, True, block, lut, width), *GroupPlan.args(plan), plan.n_split, 0, stream) == 0
    torch.cuda.synchronize()
    # first call: batch 3, two tiles of the free dimension (12 slots); second call, right after it: batch 2, one tile
    for a, b in ((a_full, b_full), (a_full[:2].contiguous(), b_full[:2, :, :, :64].contiguous())):
        Z, N = b.size(0), b.size(3)
        want = torch.empty(Z, 2, 4 * block, N, dtype=dtype, device=DEV)
        got = torch.full_like(want, float('nan'))
        ws, ws_bytes = plan.workspace(N, Z)
        rc = lib.bsp_dsd_matmul(*dsd_args(a, b, want, True, block, lut, width), *GroupPlan.args(plan), plan.n_split, ws, ws_bytes, 0, stream)
        assert rc == 0
        # "allocates nothing": torch's own counter sees only torch's allocator, the driver's free-memory figure sees a
        # hipMalloc made anywhere in the process (the first use of the library's static buffer maps no new memory either:
        # it is part of the loaded code object)
        torch.cuda.synchronize()
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        rc = lib.bsp_dsd_matmul_noalloc(*dsd_args(a, b, got, True, block, lut, width), *GroupPlan.args(plan), plan.n_split, 0, stream)
        assert rc == 0, _lib.strerror(rc)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.cuda.mem_get_info()[0] >= free_before, 'device memory was allocated during the call'
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
    # the limit applies only where split chains run: a free dimension of 256 or more goes to the wide kernel, a
    # reduction-contiguous dense operand or a forced kernel family to kernels without chains; none of them needs scratch
    # memory, so the same slot count is accepted, and the result is that of the workspace entry point
    g = torch.Generator().manual_seed(8)
    a = (0.1 * torch.randn(Z, int(lay.sum()), block, block, generator=g)).half().to(DEV)
    for N, trans_b, flags in ((256, False, 0), (192, True, 0), (192, False, _lib.FLAG_NO_GROUPS), (192, False, _lib.FLAG_GENERAL_ONLY)):
        b = torch.randn((Z, 3, N, n * block) if trans_b else (Z, 3, n * block, N), generator=g).half().to(DEV)
        want = torch.empty(Z, 3, 8 * block, N, dtype=torch.float16, device=DEV)
        got = torch.full_like(want, float('nan'))
        ws, ws_bytes = plan.workspace(N, Z)
        args = lambda c: [_lib.F16, _lib.ptr(a), _lib.ptr(b), _lib.ptr(c), 1, int(trans_b), 0, Z, N, a.stride(0), b.stride(0), b.stride(1),
                          b.stride(2), c.stride(0), c.stride(1), c.stride(2), block, _lib.ptr(lut), _lib.ptr(lut.planbuf), width]
        rc = lib.bsp_dsd_matmul(*args(want), *GroupPlan.args(plan), plan.n_split, ws, ws_bytes, flags, _lib.stream_ptr(torch.device(DEV)))
        assert rc == 0
        rc = lib.bsp_dsd_matmul_noalloc(*args(got), *GroupPlan.args(plan), plan.n_split, flags, _lib.stream_ptr(torch.device(DEV)))
        assert rc == 0, (N, trans_b, flags, _lib.strerror(rc))
        torch.cuda.synchronize()
        assert torch.equal(got, want), (N, trans_b, flags)
