"""Layout permutation between NCHW and CHWN.

Drop-in for the reference's torch_blocksparse/permute.py: `_permute.apply(x, in_order, out_order)`,
`_permute.strides(N, C, H, W, order)`, `Permute(in_order, out_order)`.  The tensor keeps its logical shape
[N, C, H, W]; only its strides (memory order) change (permute.py:33-40, 89).  NCHW <-> CHWN is the transposition
of an [N, C*H*W] matrix, done by one HIP kernel reached through the C ABI in include/bsp.h.
"""
import torch

from . import _lib


class _permute(torch.autograd.Function):

    @staticmethod
    def strides(N, C, H, W, order):
        return {
            'CHWN': [1, N * W * H, N * W, N],
            'NCHW': [W * H * C, W * H, W, 1]
        }[order]                                                   # permute.py:35-40 (KeyError for other orders)

    @staticmethod
    def do_work(x, in_order, out_order):
        lib = _lib.load()
        _lib.require_gpu_tensor(x, 'x')
        if x.dim() != 4:
            raise ValueError('Permute expects a 4-D tensor [N, C, H, W]')
        N, C, H, W = x.shape
        sx, sy = _permute.strides(N, C, H, W, in_order), _permute.strides(N, C, H, W, out_order)
        if x.dtype not in _lib.DTYPES:
            raise ValueError('Permute supports float16, bfloat16 and float32 (got %s)' % x.dtype)
        if list(x.stride()) != sx:
            xx = torch.empty_strided(x.shape, sx, device=x.device, dtype=x.dtype)   # bring x into the order it is said to have
            xx.copy_(x)
            x = xx
        y = torch.empty_strided(x.shape, sy, device=x.device, dtype=x.dtype)        # permute.py:89
        if in_order == out_order:
            y.copy_(x)
            return y
        rows, cols = (N, C * H * W) if in_order == 'NCHW' else (C * H * W, N)
        rc = lib.bsp_transpose(_lib.DTYPES[x.dtype], _lib.ptr(x), _lib.ptr(y), rows, cols, _lib.stream_ptr(x.device))
        _lib.check(rc, 'bsp_transpose')
        return y

    @staticmethod
    def forward(ctx, x, in_order, out_order):
        y = _permute.do_work(x, in_order, out_order)
        ctx.in_order = in_order
        ctx.out_order = out_order
        return y

    @staticmethod
    def backward(ctx, dy):
        dx = _permute.do_work(dy, ctx.out_order, ctx.in_order)     # permute.py:104-107
        return dx, None, None


class Permute(torch.nn.Module):

    def __init__(self, in_order, out_order):
        super(Permute, self).__init__()
        self.in_order = in_order
        self.out_order = out_order

    def forward(self, x):
        return _permute.apply(x, self.in_order, self.out_order)
