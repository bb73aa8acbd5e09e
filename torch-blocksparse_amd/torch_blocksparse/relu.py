"""Fused scale-bias-residual ReLU: y = relu(x * scale + bias + residual).

Drop-in for the reference's torch_blocksparse/relu.py (`ReLU().forward(x, scale, bias, residual)`, relu.py:95-103):
same arguments (scale and bias are one-element tensors that receive gradients), same four gradients
(relu.py:74-91).  The kernels are HIP kernels reached through the C ABI in include/bsp.h; scale and bias are read on
the device, so unlike the reference's `.item()` calls nothing waits for the GPU.
"""
import torch

from . import _lib


def _dense_like(x):
    """x itself if its elements fill one block of memory without gaps (any dimension order), else a contiguous copy."""
    if x.is_contiguous():
        return x
    order = sorted(range(x.dim()), key=lambda d: x.stride(d), reverse=True)
    if x.permute(order).is_contiguous():
        return x
    return x.contiguous()


class _relu(torch.autograd.Function):

    @staticmethod
    def forward(ctx, x, scale, bias, res):
        lib = _lib.load()
        _lib.require_gpu_tensor(x, 'x')
        if x.dtype not in _lib.DTYPES:
            raise ValueError('ReLU supports float16, bfloat16 and float32 (got %s)' % x.dtype)
        x = _dense_like(x)
        if res.stride() != x.stride() or res.shape != x.shape:       # the kernels walk memory, not indices
            r = torch.empty_strided(x.shape, x.stride(), device=x.device, dtype=x.dtype)
            r.copy_(res)
            res = r
        scale = scale.to(device=x.device, dtype=x.dtype).reshape(1)
        bias = bias.to(device=x.device, dtype=x.dtype).reshape(1)
        y = torch.empty_strided(x.shape, x.stride(), device=x.device, dtype=x.dtype)   # relu.py:68
        rc = lib.bsp_relu_fwd(_lib.DTYPES[x.dtype], _lib.ptr(x), _lib.ptr(res), _lib.ptr(y), _lib.ptr(scale), _lib.ptr(bias),
                              x.numel(), _lib.stream_ptr(x.device))
        _lib.check(rc, 'bsp_relu_fwd')
        ctx.save_for_backward(x, y, scale)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, y, scale = ctx.saved_tensors
        lib = _lib.load()
        if dy.stride() != x.stride():
            d = torch.empty_strided(x.shape, x.stride(), device=x.device, dtype=x.dtype)
            d.copy_(dy)
            dy = d
        dx = torch.empty_strided(x.shape, x.stride(), device=x.device, dtype=x.dtype)       # relu.py:82-85
        dres = torch.empty_strided(x.shape, x.stride(), device=x.device, dtype=x.dtype)
        sums = torch.empty((2,), device=x.device, dtype=torch.float32)                        # dscale, dbias
        ws_bytes = lib.bsp_relu_workspace_bytes()
        ws = torch.empty((ws_bytes,), device=x.device, dtype=torch.uint8)
        rc = lib.bsp_relu_bwd(_lib.DTYPES[x.dtype], _lib.ptr(x), _lib.ptr(y), _lib.ptr(dy), _lib.ptr(dx), _lib.ptr(dres),
                              _lib.ptr(scale), _lib.ptr(sums[0:1]), _lib.ptr(sums[1:2]), _lib.ptr(ws), ws_bytes, x.numel(),
                              _lib.stream_ptr(x.device))
        _lib.check(rc, 'bsp_relu_bwd')
        return dx, sums[0:1].to(x.dtype), sums[1:2].to(x.dtype), dres                         # relu.py:91


relu = _relu.apply


class ReLU(torch.nn.Module):

    def __init__(self):
        super(ReLU, self).__init__()

    def forward(self, x, scale, bias, residual):
        return relu(x, scale, bias, residual)
