"""GPU: block-sparse softmax forward/backward against the fp32 dense-masked oracle (through the C ABI)."""
import pytest
import torch

import torch_blocksparse as tb
from oracle import dense_oracle as D
from helpers import Guarded, assert_close, guard_allocations, random_layout, softmax_dx_magnitude

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def run_case(Z, H, R, C, block, dtype, density, seed, scale=0.4, rpe=False, kpm=None, attn=None, layout=None):
    torch.manual_seed(seed)
    lay = layout if layout is not None else random_layout((H, R, C), density, seed, at_least_one_per_row=True)
    nnz = int(lay.sum())
    M, N = R * block, C * block
    x = torch.rand((Z, nnz, block, block), dtype=torch.float32).to(dtype)
    dy = torch.rand((Z, nnz, block, block), dtype=torch.float32).to(dtype)
    kw = {}
    if rpe:
        kw['rpe'] = (0.5 * torch.randn(Z, H, M, N)).to(dtype)
    if kpm == 'add':            # the reference's test: 0 / -inf, at least one key kept per row is not guaranteed there
        m = torch.zeros(Z, N)
        m[torch.rand(Z, N) < 0.3] = float('-inf')
        m[:, ::block] = 0       # keep one key per block so that no row is fully masked
        kw['key_padding_mask'] = m.to(dtype)
        kw['key_padding_mask_mode'] = 'add'
    elif kpm == 'mul':
        m = (torch.rand(Z, N) > 0.3).float()
        m[:, ::block] = 1
        kw['key_padding_mask'] = m.to(dtype)
        kw['key_padding_mask_mode'] = 'mul'
    if attn == 'mul':
        a = (torch.rand(M, N) > 0.4).float()
        a[:, 1::block] = 1
        kw['attn_mask'] = a.to(dtype)
        kw['attn_mask_mode'] = 'mul'
    elif attn == 'add':
        kw['attn_mask'] = torch.randn(M, N).to(dtype)
        kw['attn_mask_mode'] = 'add'
    ry, rdx = D.softmax(x, lay, block, scale=scale, dy=dy, **kw)
    op = tb.Softmax(lay, block)
    xg = x.to(DEV).requires_grad_(True)
    gkw = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in kw.items()}
    # the op works in place: feed it a temporary, here the interior of a sentinel-filled buffer (as is the gradient
    # tensor the backward pass makes): the kernels take their addresses from the table and must stay inside
    guard = Guarded(tuple(x.shape), dtype)
    xin = guard.t
    xin.copy_(xg)
    with guard_allocations('softmax'):
        y = op(xin, scale=scale, **gkw)
        y.backward(dy.to(DEV))
    guard.check('softmax x')
    assert_close(y, ry, dtype, 'softmax y', no_cancellation=True)     # a softmax's output: positive terms only
    assert_close(xg.grad, rdx, dtype, 'softmax dx', mag=softmax_dx_magnitude(ry, dy, lay, block, scale))


# the reference's own cases (tests/test_softmax.py:80-90): block 16, widths 256 / 576, fp16 / fp32
@pytest.mark.parametrize('width', [256, 576])
@pytest.mark.parametrize('dtype', [torch.float16, torch.float32])
def test_reference_cases(width, dtype):
    run_case(2, 4, width // 16, width // 16, 16, dtype, 0.6, width, scale=0.4, kpm='add', attn='mul')


@pytest.mark.parametrize('block', [16, 32, 64, 128])
@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16, torch.float32])
def test_blocks_and_dtypes(block, dtype):
    run_case(2, 2, 6, 5, block, dtype, 0.5, block, scale=0.7)


@pytest.mark.parametrize('dtype', [torch.float16, torch.float32])
def test_rpe_and_mask_modes(dtype):
    run_case(2, 3, 4, 6, 32, dtype, 0.6, 11, scale=0.3, rpe=True, kpm='mul', attn='add')
    run_case(2, 3, 4, 6, 16, dtype, 0.6, 12, scale=1.0, rpe=True)
    run_case(1, 2, 3, 3, 64, dtype, 0.7, 13, scale=0.125, kpm='add')


@pytest.mark.parametrize('block,cols', [(16, 70), (64, 20), (128, 9), (32, 40)])
def test_long_rows_streaming_variant(block, cols):
    # more blocks per row than the register variant holds
    run_case(1, 1, 2, cols, block, torch.float16, 0.95, cols, scale=0.5, kpm='add')
    run_case(1, 1, 2, cols, block, torch.float32, 0.95, cols + 1, scale=0.5)


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize('block,cols', [(16, 70), (16, 200), (32, 70), (32, 140), (64, 20), (64, 40), (64, 100), (128, 20), (128, 60)])
def test_long_rows_one_wavefront_per_row(block, cols, dtype):
    # rows of more blocks than the register variants hold: one wavefront per row with 4, 8 or 16 sixteen-byte pieces per
    # lane (every step count for every block size); rows of ragged lengths in one launch (a full row, a short one, an
    # empty one, a single block); every mask at once in both modes; batch 2, 2 heads.  The longest rows of fp32 at
    # block 128 (60 blocks = 7680 elements, more than 16 steps hold) fall back to the variant that re-reads x.
    lay = random_layout((2, 4, cols), 0.7, cols + block)
    lay[0, 0, :] = 1
    lay[0, 1, :] = 0
    lay[0, 1, cols // 2] = 1
    lay[1, 2, :] = 0
    lay[1, 3, :3] = 1
    run_case(2, 2, 4, cols, block, dtype, 0, 400 + cols, scale=0.3, layout=lay)
    run_case(1, 2, 4, cols, block, dtype, 0, 500 + cols, scale=0.5, rpe=True, kpm='add', attn='mul', layout=lay)
    run_case(1, 2, 4, cols, block, dtype, 0, 600 + cols, scale=0.5, kpm='mul', attn='add', layout=lay)


@pytest.mark.parametrize('longest', [1, 2, 3, 4, 5, 6, 7, 8, 9, 16, 17, 18, 19, 22, 27, 30, 32, 33])
def test_every_row_length_bucket(longest):
    # one kernel instantiation per bucket of "blocks kept in registers": the longest row decides which one runs, the
    # other rows (1 block, longest - 1 blocks, none) exercise its partially filled and empty paths
    C = longest + 1
    lay = torch.zeros(2, 4, C, dtype=torch.int64)
    lay[0, 0, :longest] = 1
    lay[0, 1, C - 1] = 1
    lay[0, 3, 1:longest] = 1
    lay[1, 2, 1:1 + longest] = 1
    lay[1, 0, 0] = 1
    run_case(2, 2, 4, C, 64, torch.float16, 0, 100 + longest, scale=0.3, kpm='add', layout=lay)
    run_case(1, 2, 4, C, 16, torch.bfloat16, 0, 200 + longest, scale=0.3, kpm='mul', attn='add', layout=lay)
    run_case(1, 2, 4, C, 32, torch.float32, 0, 300 + longest, scale=0.3, rpe=True, kpm='add', layout=lay)


def test_rows_without_blocks_and_single_block():
    lay = torch.zeros(2, 4, 4, dtype=torch.int64)
    lay[0, 0, 1] = 1
    lay[0, 2, :] = 1
    lay[1, 3, 3] = 1
    run_case(2, 2, 4, 4, 32, torch.float16, 0, 21, layout=lay)


def test_attention_config_shape_small_batch():
    # the benchmark configuration (block 64, seq 4096, fixed layout, additive key padding mask) at batch 1, 2 heads
    lay = tb.sparse_transformer_layout(2, 64, 4, 16, True)
    run_case(1, 2, 64, 64, 64, torch.float16, 0, 31, scale=0.125, kpm='add', layout=lay)


def test_fully_masked_row_gives_nan_like_the_dense_oracle():
    lay = torch.ones(1, 2, 2, dtype=torch.int64)
    x = torch.rand(1, 4, 16, 16, dtype=torch.float16)
    m = torch.zeros(1, 32, dtype=torch.float16)
    m[:] = float('-inf')
    ry = D.softmax(x, lay, 16, key_padding_mask=m)
    y = tb.Softmax(lay, 16)(x.to(DEV), key_padding_mask=m.to(DEV))
    assert torch.isnan(ry).all() and torch.isnan(y).all()


def test_in_place_and_row_too_long():
    lay = torch.ones(1, 1, 2, dtype=torch.int64)
    x = torch.rand(1, 2, 16, 16, dtype=torch.float16, device=DEV)
    y = tb.Softmax(lay, 16)(x)
    assert y.data_ptr() == x.data_ptr()
    big = torch.ones(1, 1, 512, dtype=torch.int64)
    with pytest.raises(NotImplementedError):
        tb.Softmax(big, 64)(torch.zeros(1, 512, 64, 64, dtype=torch.float16, device=DEV))


def run_dropout_case(Z, H, R, C, block, dtype, density, seed, p, masks=False, layout=None):
    # forward and backward with dropout against the oracle with the mask re-created from the same counter
    from oracle.philox_oracle import keep_mask
    torch.manual_seed(seed)
    lay = layout if layout is not None else random_layout((H, R, C), density, seed, at_least_one_per_row=True)
    nnz = int(lay.sum())
    x = torch.rand((Z, nnz, block, block)).to(dtype)
    dy = torch.rand((Z, nnz, block, block)).to(dtype)
    kw = {}
    if masks:
        kw['rpe'] = (0.5 * torch.randn(Z, H, R * block, C * block)).to(dtype)
        kw['attn_mask'] = torch.randn(R * block, C * block).to(dtype)
    drop_seed, drop_off = 0x1234567 + seed, 3 * seed
    keep = torch.from_numpy(keep_mask(x.numel(), p, drop_seed, drop_off)).reshape(x.shape)
    m = keep.float() / (1.0 - p)
    ry, rdx = D.softmax(x, lay, block, scale=0.4, dy=dy.float() * m, **kw)
    xg = x.to(DEV).requires_grad_(True)
    xin = xg * 1.0
    y = tb.Softmax(lay, block)(xin, scale=0.4, dropout_p=p, dropout_seed=drop_seed, dropout_offset=drop_off,
                               **{k: v.to(DEV) for k, v in kw.items()})
    assert y.data_ptr() != xin.data_ptr()
    assert_close(xin, ry, dtype, 'softmax kept for the backward pass', no_cancellation=True)
    assert_close(y, ry * m, dtype, 'dropped softmax', no_cancellation=True)
    assert torch.equal(y.cpu() == 0, ~keep | (ry == 0)), 'mask differs from the oracle\'s'
    y.backward(dy.to(DEV))
    assert_close(xg.grad, rdx, dtype, 'softmax + dropout dx', mag=softmax_dx_magnitude(ry, dy.float() * m, lay, block, 0.4))


@pytest.mark.parametrize('block', [16, 32, 64, 128])
@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16, torch.float32])
def test_dropout_matches_the_counter_based_oracle(block, dtype):
    run_dropout_case(2, 2, 5, 6, block, dtype, 0.5, block, 0.3)
    run_dropout_case(1, 2, 3, 4, block, dtype, 0.7, block + 1, 0.1, masks=True)


def test_dropout_in_every_kernel_variant():
    # long rows: the 32-block bucket (block 16), the streaming variant (more blocks than registers hold), 16-block bucket
    for block, cols, dtype in ((16, 28, torch.float16), (64, 20, torch.float16), (32, 14, torch.bfloat16), (16, 70, torch.float32)):
        run_dropout_case(2, 1, 2, cols, block, dtype, 0.95, cols, 0.25)
        run_dropout_case(1, 1, 2, cols, block, dtype, 0.95, cols + 1, 0.5, masks=True)


def test_dropout_rate_and_repeatability():
    lay = tb.sparse_transformer_layout(2, 16, 4, 8, True)
    nnz = int(lay.sum())
    x = torch.randn(4, nnz, 64, 64, dtype=torch.float16, device=DEV)
    sm = tb.Softmax(lay, 64)
    for p in (0.1, 0.5):
        y = sm(x.clone(), dropout_p=p, dropout_seed=99)
        kept = (y != 0).float().mean().item()
        n = y.numel()
        assert abs(kept - (1 - p)) < 5 * (p * (1 - p) / n) ** 0.5 + 1e-4      # (softmax values that round to 0 in fp16 are rare)
        assert torch.equal(y, sm(x.clone(), dropout_p=p, dropout_seed=99))
        assert not torch.equal(y, sm(x.clone(), dropout_p=p, dropout_seed=100))
        assert not torch.equal(y, sm(x.clone(), dropout_p=p, dropout_seed=99, dropout_offset=1))
    torch.manual_seed(5)
    a = sm(x.clone(), dropout_p=0.2)
    torch.manual_seed(5)
    b = sm(x.clone(), dropout_p=0.2)
    assert torch.equal(a, b)                               # the seed comes from torch's generator when not given
    assert torch.equal(sm(x.clone(), dropout_p=0.0), sm(x.clone()))


def test_backward_overwrites_only_a_private_gradient():
    # The reference runs its backward kernel in place on whatever gradient comes in (softmax.py:316-325).  This one does so
    # only when nobody else holds that tensor: (1) the tensor a user hands to backward() stays as it was; (2) a gradient
    # that an addition passes on to a second branch reaches that branch unchanged; (3) inside the attention chain, where
    # the gradient is a fresh result of the next operator's backward, the in-place path is the one taken.
    from torch_blocksparse.softmax import _sparse_softmax
    lay = random_layout((2, 4, 4), 0.6, 3)
    nnz = int(lay.sum())
    torch.manual_seed(0)
    x = torch.rand(2, nnz, 32, 32, dtype=torch.float16)
    dy = torch.rand(2, nnz, 32, 32, dtype=torch.float16)
    _, rdx = D.softmax(x, lay, 32, scale=0.7, dy=dy)
    op = tb.Softmax(lay, 32)
    xg = x.to(DEV).requires_grad_(True)
    g = dy.to(DEV)
    op(xg * 1.0, scale=0.7).backward(g)
    assert torch.equal(g.cpu(), dy), 'the gradient passed to backward() was modified'
    assert_close(xg.grad, rdx, torch.float16, 'softmax dx')
    xg = x.to(DEV).requires_grad_(True)
    w = torch.zeros_like(xg, requires_grad=True)
    (op(xg * 1.0, scale=0.7) + w).backward(g)
    assert torch.equal(w.grad.cpu(), dy), 'the other branch of an addition saw the softmax gradient instead of its own'
    assert_close(xg.grad, rdx, torch.float16, 'softmax dx-with-a-shared-gradient')
    before = _sparse_softmax.in_place_backwards
    H, L, dh = 2, 128, 64
    sdd, dsd = tb.MatMul(lay, 32, 'sdd', trans_b=True), tb.MatMul(lay, 32, 'dsd')
    q, k, v = [torch.randn(2, H, L, dh, device=DEV, dtype=torch.float16, requires_grad=True) for _ in range(3)]
    o = dsd(op(sdd(q, k), scale=0.125), v)
    o.backward(torch.randn_like(o))
    assert _sparse_softmax.in_place_backwards == before + 1, 'the chain did not take the in-place path'
