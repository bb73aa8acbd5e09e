"""GPU: the package's two dense utility ops, ReLU (scale-bias-residual) and Permute (NCHW <-> CHWN), against plain
PyTorch on the CPU -- the same checks as the reference's tests/test_relu.py:10-69 and tests/test_permute.py:10-46."""
import pytest
import torch

import torch_blocksparse as tb
from helpers import assert_close

pytestmark = pytest.mark.gpu
DEV = 'cuda'


@pytest.mark.parametrize('dtype', [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize('shape', [(4, 64, 15, 15), (3, 5, 7, 1), (2, 8, 16, 16)])   # reference case; odd sizes (tail); vector-only
def test_relu(dtype, shape):
    torch.manual_seed(sum(shape))
    x, res, dy = [torch.randn(shape).to(dtype) for _ in range(3)]
    scale, bias = torch.randn(1).to(dtype), torch.randn(1).to(dtype)
    ref = [t.detach().clone().float().requires_grad_(True) for t in (x, scale, bias, res)]
    ry = torch.relu(ref[0] * ref[1] + ref[2] + ref[3])
    ry.backward(dy.float())
    got = [t.detach().to(DEV).requires_grad_(True) for t in (x, scale, bias, res)]
    y = tb.ReLU()(*got)
    y.backward(dy.to(DEV))
    assert y.stride() == got[0].stride()
    assert_close(y, ry.detach(), dtype, 'relu y')
    # where the pre-activation rounds to exactly 0 in the narrow type the two sides may disagree on y > 0; none here
    for g, r, name in zip(got, ref, ('dx', 'dscale', 'dbias', 'dres')):
        assert g.grad.dtype == dtype and g.grad.shape == r.grad.shape
        if name in ('dscale', 'dbias'):       # sums of thousands of terms: compare relative to the sum of magnitudes
            mag = (dy.float().abs() * (x.float().abs() if name == 'dscale' else 1)).sum()
            tol = {torch.float32: 1e-5, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}[dtype]
            assert abs(float(g.grad.float().cpu()) - float(r.grad)) <= tol * float(mag) + tol, name
        else:
            assert_close(g.grad, r.grad, dtype, 'relu ' + name)


def test_relu_unaligned_views_and_channels_last():
    torch.manual_seed(3)
    base = torch.randn(4 * 6 * 5 * 5 + 3)
    x = base[3:].reshape(4, 6, 5, 5)                          # 12-byte offset: the scalar variant
    res = torch.randn(4, 6, 5, 5).to(memory_format=torch.channels_last)
    scale, bias = torch.tensor([0.7]), torch.tensor([-0.1])
    ry = torch.relu(x * scale + bias + res)
    xg = base.to(DEV)[3:].reshape(4, 6, 5, 5)
    y = tb.ReLU()(xg, scale.to(DEV), bias.to(DEV), res.to(DEV))
    assert_close(y, ry, torch.float32, 'relu unaligned')
    xc = x.contiguous(memory_format=torch.channels_last)
    y = tb.ReLU()(xc.to(DEV), scale.to(DEV), bias.to(DEV), res.to(DEV))
    assert y.stride() == xc.stride()
    assert_close(y, ry, torch.float32, 'relu channels_last')


@pytest.mark.parametrize('dtype', [torch.float16, torch.float32, torch.bfloat16])
@pytest.mark.parametrize('orders', [('NCHW', 'CHWN'), ('CHWN', 'NCHW'), ('NCHW', 'NCHW')])
@pytest.mark.parametrize('shape', [(32, 32, 4, 4), (5, 3, 7, 9), (130, 2, 1, 67)])    # reference case; ragged tiles
def test_permute(dtype, orders, shape):
    torch.manual_seed(1)
    in_order, out_order = orders
    N, C, H, W = shape
    sx = tb._permute.strides(N, C, H, W, in_order)
    sy = tb._permute.strides(N, C, H, W, out_order)
    x = torch.rand(N * C * H * W).as_strided(shape, sx).to(dtype)
    xg = torch.empty_strided(shape, sx, dtype=dtype, device=DEV)
    xg.copy_(x)
    xg.requires_grad_(True)
    y = tb.Permute(in_order, out_order)(xg)
    assert list(y.stride()) == sy and y.shape == x.shape
    assert torch.equal(y.cpu(), x)                              # same values at the same indices
    dy = torch.empty_strided(shape, sy, dtype=dtype, device=DEV)
    dy.copy_(torch.rand(shape).to(dtype))
    y.backward(dy)
    assert list(xg.grad.stride()) == sx and torch.equal(xg.grad.cpu(), dy.cpu())


def test_permute_brings_its_input_into_the_stated_order():
    x = torch.rand(6, 4, 3, 5)                                  # NCHW memory, declared CHWN
    y = tb._permute.apply(x.to(DEV), 'CHWN', 'NCHW')
    assert y.is_contiguous() and torch.equal(y.cpu(), x)
    with pytest.raises(KeyError):
        tb._permute.apply(x.to(DEV), 'NHWC', 'NCHW')
