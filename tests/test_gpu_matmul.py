"""GPU: block-sparse matmul sdd / dsd / dds, forward and backward, against the fp32 dense-masked oracle."""
import pytest
import torch

import torch_blocksparse as tb
from oracle import dense_oracle as D
from helpers import assert_close, operand_shapes, random_layout, run_matmul_case as run_case

pytestmark = pytest.mark.gpu
DEV = 'cuda'


# the reference's 21 cases (tests/test_matmul.py:87-103): fp16, Z=3 H=2 M=256 N=512 K=384, half of the blocks kept
@pytest.mark.parametrize('mode', ['sdd', 'dsd', 'dds'])
@pytest.mark.parametrize('trans_a', [False, True])
@pytest.mark.parametrize('trans_b', [False, True])
def test_reference_trans_cases(mode, trans_a, trans_b):
    run_case(mode, trans_a, trans_b, 32, torch.float16)


@pytest.mark.parametrize('mode', ['sdd', 'dsd', 'dds'])
@pytest.mark.parametrize('block', [16, 32, 64, 128])
def test_reference_block_cases(mode, block):
    run_case(mode, False, False, block, torch.float16)


@pytest.mark.parametrize('mode', ['sdd', 'dsd', 'dds'])
@pytest.mark.parametrize('block', [16, 32, 64, 128])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_other_dtypes(mode, block, dtype):
    run_case(mode, False, True, block, dtype, Z=2, seed=block)
    run_case(mode, True, False, block, dtype, Z=1, seed=block + 1)


def test_readme_configuration():
    # README of the reference: fp32, Z=4 H=2 M=256 N=512 K=384, block 16, sdd with trans_a, layout randint(0, 2)
    torch.manual_seed(0)
    lay = torch.randint(0, 2, (2, 16, 32))
    run_case('sdd', True, False, 16, torch.float32, Z=4, layout=lay)


def test_normal_inputs_with_cancellation():
    run_case('dsd', False, False, 32, torch.float16, dist='randn', scale=0.05, seed=7)
    run_case('dds', False, True, 64, torch.float16, dist='randn', scale=0.05, seed=8)
    run_case('sdd', False, True, 64, torch.float32, dist='randn', scale=1.0, seed=9)


@pytest.mark.parametrize('mode,trans_a,trans_b', [('dsd', False, False), ('dsd', True, False), ('dds', False, False), ('dds', True, True)])
@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_long_lines_become_chains(mode, trans_a, trans_b, dtype):
    # block 64: lines far longer than the average leave their group and are reduced by the four wavefronts of a
    # workgroup in parallel.  A full column, a full row, a 19-block line (19 = 4*4 + 3: wavefronts with unequal shares)
    # and ordinary lines around them, including a group whose four lines are all chains.
    R = C = 40
    lay = torch.zeros(2, R, C, dtype=torch.int64)
    for i in range(R):
        lay[:, i, max(0, i - 1):i + 1] = 1           # two-block diagonal band
    lay[0, :, 5] = 1                                  # global column
    lay[0, 9, :] = 1                                  # global row
    lay[1, 12:16, :] = 1                              # a whole group of long rows
    lay[1, :, 20:24] = 1                              # a whole group of long columns
    lay[1, 30, :19] = 1
    lay[1, :19, 33] = 1
    from torch_blocksparse.matmul import GroupPlan
    assert GroupPlan.thin_min(lay, True) == 16 and GroupPlan.thin_min(lay, False) == 16
    Z, H = 2, 2
    F = 128                                           # dense free dimension: two 64-wide tiles
    if mode == 'dsd':
        run_case(mode, trans_a, trans_b, 64, dtype, Z=Z, H=H, M=64 * R, N=F, K=64 * C, layout=lay, seed=5, dist='randn', scale=0.25)
    else:
        run_case(mode, trans_a, trans_b, 64, dtype, Z=Z, H=H, M=F, N=64 * C, K=64 * R, layout=lay, seed=5, dist='randn', scale=0.25)


@pytest.mark.parametrize('Z', [1, 4])
def test_block128_sdd_one_or_four_workgroups_per_block(Z):
    # 128 blocks: with Z = 4 there are 512 block products and each gets one workgroup; with Z = 1 every block is split
    # into four 64 x 64 workgroups so that the chip is not left half empty
    lay = torch.ones(2, 8, 8, dtype=torch.int64)
    run_case('sdd', True, False, 128, torch.float16, Z=Z, H=2, M=1024, N=1024, K=64, layout=lay, seed=9, backward=False)
    run_case('sdd', False, True, 128, torch.bfloat16, Z=Z, H=2, M=1024, N=1024, K=48, layout=lay, seed=10, backward=False)


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_block128_sdd_long_reduction_cut_into_parts(dtype, monkeypatch):
    # few blocks of 128 and a long reduction (the weight gradient of a sparse linear layer): the reduction is cut into
    # parts whose fp32 partial blocks a second kernel adds in part order.  All four orientations; reductions of 1056
    # (33 steps over 4 parts: the last part is shorter), 544 (2 parts) and 4096 (16 parts); batch 2; a layout with an empty
    # row; repeated launches agree bit for bit; the workspace is reused by a smaller launch; and the same products
    # with the parts switched off (one workgroup per block writes the block directly)
    from torch_blocksparse.matmul import _sparse_matmul
    lay = random_layout((2, 3, 4), 0.5, 128)
    lay[0, 1, :] = 0
    for ta, tb_ in ((False, True), (True, False), (False, False), (True, True)):
        run_case('sdd', ta, tb_, 128, dtype, Z=2, H=2, M=384, N=512, K=1056, layout=lay, seed=50 + ta + 2 * tb_, dist='randn', scale=0.2, backward=False)
    run_case('sdd', True, False, 128, dtype, Z=1, H=2, M=384, N=512, K=544, layout=lay, seed=54, dist='randn', scale=0.2, backward=False)
    run_case('sdd', True, False, 128, dtype, Z=1, H=2, M=384, N=512, K=4096, layout=lay, seed=55, dist='randn', scale=0.05, backward=False)
    op = tb.MatMul(lay, 128, 'sdd', trans_a=True)
    g = torch.Generator().manual_seed(56)
    a = (0.1 * torch.randn(2, 2, 2048, 384, generator=g)).to(dtype).to(DEV)
    b = torch.randn(2, 2, 2048, 512, generator=g).to(dtype).to(DEV)
    c1, c2 = op(a, b), op(a, b)
    c3 = op(a[:1], b[:1])
    assert torch.equal(c1, c2) and torch.equal(c3, c1[:1])
    monkeypatch.setattr(_sparse_matmul, 'SPLITK_TARGET_WORKGROUPS', 1)        # no parts: the general path
    c4 = tb.MatMul(lay, 128, 'sdd', trans_a=True)(a, b)
    assert_close(c1, c4.float(), dtype, 'sdd in parts vs in one piece')


@pytest.mark.parametrize('block', [16, 32, 64, 128])
@pytest.mark.parametrize('mode,trans_a,trans_b', [('dsd', False, False), ('dsd', True, True), ('dds', False, True), ('dds', True, False)])
def test_narrow_free_dimension(block, mode, trans_a, trans_b):
    # free dimension of at most 64 (the head dimension of an attention product): the kernels use a 64-wide tile
    # instead of their wide one; 48 leaves part of that tile empty
    for free, dtype in ((64, torch.float16), (48, torch.float32)):
        if mode == 'dsd':
            run_case(mode, trans_a, trans_b, block, dtype, Z=2, H=2, M=256, N=free, K=384, seed=block + free, backward=False)
        else:
            run_case(mode, trans_a, trans_b, block, dtype, Z=2, H=2, M=free, N=256, K=384, seed=block + free, backward=False)


@pytest.mark.parametrize('block', [16, 32])
@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_small_block_row_groups(block, dtype):
    # blocks of 16 and 32 with a free dimension of 64 or 128 (attention shapes) run on row-group kernels with one
    # wavefront per member.  22 lines: the last group has two members; one empty block-row, one full block-column,
    # one full block-row; forward and backward reach the plain and the transposed variant of dsd and of dds.
    n = 22
    lay = random_layout((3, n, n), 0.3, 77 + block)
    lay[:, 5, :] = 0
    lay[:, :, 7] = 1
    lay[1, 9, :] = 1
    lay[:, 5, :] = 0
    for free in (64, 128):
        run_case('dsd', False, False, block, dtype, Z=2, H=3, M=n * block, K=n * block, N=free, layout=lay, seed=block + free, dist='randn', scale=0.25)
        run_case('dsd', True, False, block, dtype, Z=2, H=3, M=n * block, K=n * block, N=free, layout=lay, seed=block + free + 1, dist='randn', scale=0.25)
        run_case('sdd', False, True, block, dtype, Z=2, H=3, M=n * block, N=n * block, K=free, layout=lay, seed=block + free + 2, dist='randn', scale=0.25)
    # lines of 128 blocks and more become chains (split over the wavefronts): a full block-column of 132 and, seen from
    # the transposed product, a full block-row
    tall = random_layout((2, 132, 6), 0.2, 5 + block)
    tall[:, :, 2] = 1
    run_case('dsd', True, False, block, dtype, Z=2, H=2, M=6 * block, K=132 * block, N=64, layout=tall, seed=block + 3, dist='randn', scale=0.1)
    wide = tall.transpose(1, 2).contiguous()
    run_case('dsd', False, False, block, dtype, Z=2, H=2, M=6 * block, K=132 * block, N=64, layout=wide, seed=block + 4, dist='randn', scale=0.1)


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_block16_products_on_64x64_tiles(dtype):
    # a block-16 layout whose sides divide by 4: sdd / dsd / dds run the block-64 row-group kernels on 64 x 64 tiles
    # gathered from (scattered to) 4 x 4 small blocks (absent ones read as zeros, are not written).  Sparse tiles with 1 .. 16 blocks, an empty tile row, a full
    # tile column and a full tile row (20 tiles: a chain), free dimension 64, 128 and 192; forward and backward reach
    # the plain and the transposed product of dsd and, through sdd's backward, of dds (written transposed).
    n = 80                                                           # 20 x 20 tiles
    lay = random_layout((2, n, n), 0.12, 4242)
    lay[:, 8:12, :] = 0                                              # tile row 2 empty
    lay[:, :, 28:32] = (torch.rand(2, n, 4) < 0.5).long()            # tile column 7: present in every tile row ...
    lay[:, ::4, 28] = 1
    lay[:, 8:12, :] = 0                                              # ... but the empty one
    lay[1, 36:40, :] = (torch.rand(n) < 0.6).long()                  # tile row 9 of head 1: every tile, partly filled
    lay[1, 36, ::4] = 1
    lay[0, 0:4, 0:4] = 1                                             # one full tile
    for free in (64, 128, 192):
        run_case('dsd', False, False, 16, dtype, Z=2, H=2, M=n * 16, K=n * 16, N=free, layout=lay, seed=free, dist='randn', scale=0.25)
        run_case('dsd', True, False, 16, dtype, Z=2, H=2, M=n * 16, K=n * 16, N=free, layout=lay, seed=free + 1, dist='randn', scale=0.25)
    # sdd scatters its 64 x 64 result tiles to the blocks present (reduction 64 and 128)
    run_case('sdd', False, True, 16, dtype, Z=2, H=2, M=n * 16, N=n * 16, K=64, layout=lay, seed=9, dist='randn', scale=0.25)
    run_case('sdd', False, True, 16, dtype, Z=2, H=2, M=n * 16, N=n * 16, K=128, layout=lay, seed=12, dist='randn', scale=0.25)
    run_case('dds', False, False, 16, dtype, Z=2, H=2, M=64, K=n * 16, N=n * 16, layout=lay, seed=10, dist='randn', scale=0.25)
    run_case('dds', False, True, 16, dtype, Z=2, H=2, M=128, K=n * 16, N=n * 16, layout=lay, seed=11, dist='randn', scale=0.25)


def test_degenerate_layouts():
    # rows / columns without blocks must come out as zeros (the output buffer is uninitialised memory)
    lay = torch.zeros(2, 4, 6, dtype=torch.int64)
    lay[0, 1, 2] = 1
    lay[0, 1, 5] = 1
    lay[1, 3, 0] = 1
    run_case('dsd', False, False, 32, torch.float16, M=128, K=192, N=64, layout=lay)
    run_case('dsd', True, False, 32, torch.float16, M=192, K=128, N=64, layout=lay)
    run_case('dds', False, False, 32, torch.float16, M=64, K=128, N=192, layout=lay)
    run_case('sdd', False, False, 32, torch.float16, M=128, N=192, K=64, layout=lay)
    one = torch.ones(1, 1, 1, dtype=torch.int64)
    run_case('sdd', False, True, 64, torch.float16, Z=1, H=1, M=64, N=64, K=16, layout=one)


def test_dense_layout_with_pack4_rows_outside_the_layout():
    # at 90% density the reference's packing emits rows for absent / repeated blocks; results must still be right
    lay = random_layout((1, 24, 24), 0.9, 1234)
    run_case('sdd', False, False, 16, torch.float16, Z=1, H=1, M=384, N=384, K=64, layout=lay)


def test_free_dimension_not_a_multiple_of_the_tile():
    # multiples of 16 that do not fill a 64-wide tile: forward and backward
    run_case('dsd', False, False, 32, torch.float16, Z=1, H=2, M=128, K=128, N=80)
    run_case('dds', False, True, 32, torch.float32, Z=1, H=2, M=48, K=128, N=128)
    # any size works forward; the backward's sdd keeps the reference's rule (reduction % 16, matmul.py:318-319)
    run_case('dsd', False, False, 32, torch.float16, Z=1, H=2, M=128, K=128, N=72, backward=False)
    run_case('dsd', False, False, 32, torch.float32, Z=1, H=2, M=128, K=128, N=20, backward=False)
    run_case('dds', False, False, 32, torch.float16, Z=1, H=2, M=40, K=128, N=128, backward=False)
    run_case('dsd', False, True, 16, torch.float16, Z=1, H=1, M=64, K=64, N=10, backward=False)
    run_case('dsd', False, True, 16, torch.bfloat16, Z=1, H=1, M=64, K=64, N=3, backward=False)


def test_sdd_reduction_multiple_of_16():
    lay = torch.ones(1, 2, 2, dtype=torch.int64)
    a = torch.zeros(1, 1, 32, 24, dtype=torch.float16, device=DEV)
    b = torch.zeros(1, 1, 24, 32, dtype=torch.float16, device=DEV)
    with pytest.raises(ValueError):
        tb.MatMul(lay, 16, 'sdd')(a, b)


def test_dsd_dds_round_trip_config_reduced():
    # config 2 (fp16, block 32, 2048^3, quarter of the blocks kept), all four transpositions, at Z=1 H=2
    lay = random_layout((2, 64, 64), 0.25, 2, at_least_one_per_row=True)
    for ta in (False, True):
        for tb_ in (False, True):
            run_case('dsd', ta, tb_, 32, torch.float16, Z=1, H=2, M=2048, N=256, K=2048, layout=lay, dist='randn', scale=2048 ** -0.25)
            run_case('dds', ta, tb_, 32, torch.float16, Z=1, H=2, M=256, N=2048, K=2048, layout=lay, dist='randn', scale=2048 ** -0.25)


def test_sparse_linear_layer_config_reduced():
    # config 5: dds with trans_b, block 128, tenth of the blocks kept, weight 4096x4096, 1024 tokens; backward dsd + sdd
    torch.manual_seed(5)
    lay = random_layout((1, 32, 32), 0.1, 5)
    run_case('dds', False, True, 128, torch.float16, Z=1, H=1, M=1024, N=4096, K=4096, layout=lay, dist='randn', scale=0.14)


@pytest.mark.parametrize('tokens', [(5, 7), (3, 16)])
def test_linear_module(tokens):
    # y, dx and the weight gradient against dense fp32; 35 tokens are padded to a multiple of 16 inside the module (the
    # weight gradient is an sdd product over the tokens), 48 are not
    torch.manual_seed(3)
    lay = random_layout((1, 4, 6), 0.5, 3)
    lin = tb.Linear(256, 384, 64, lay).to(DEV).half()
    x = torch.randn(*tokens, 256, device=DEV, dtype=torch.float16, requires_grad=True)
    dy = torch.randn(*tokens, 384, device=DEV, dtype=torch.float16)
    y = lin(x)
    wd = D.sparse_to_dense(lin.weight.detach().cpu().float()[None], lay, 64)[0, 0]
    ref = x.detach().cpu().float() @ wd
    assert_close(y, ref, torch.float16, 'linear y')
    y.backward(dy)
    assert_close(x.grad, dy.cpu().float() @ wd.t(), torch.float16, 'linear dx')
    dw = x.detach().cpu().float().reshape(-1, 256).t() @ dy.cpu().float().reshape(-1, 384)
    assert_close(lin.weight.grad, D.dense_to_sparse(dw[None, None], lay, 64)[0], torch.float16, 'linear dw')


@pytest.mark.parametrize('mode,trans_a,trans_b', [('dsd', False, False), ('dsd', True, False), ('dds', False, False), ('dds', False, True)])
@pytest.mark.parametrize('block', [32, 64])
def test_sparse_operand_shared_by_the_batch(mode, trans_a, trans_b, block):
    # a 3-D sparse operand [nnz, block, block] with a dense batch of 3: every batch multiplies the same blocks and the
    # gradient of the sparse operand is the sum over the batch
    torch.manual_seed(17)
    Z, H, M, N, K = 3, 2, 128, 192, 256
    ashape, bshape, sp = operand_shapes(mode, trans_a, trans_b, M, N, K)
    lay = random_layout((H, sp[0] // block, sp[1] // block), 0.5, 17)
    a = (0.25 * torch.randn((Z, H) + ashape)).half()
    b = (0.25 * torch.randn((Z, H) + bshape)).half()
    dc = torch.randn(Z, H, M, N).half()
    if mode == 'dsd':
        a = D.dense_to_sparse(a[:1], lay, block)[0]                       # [nnz, block, block]
        full = (a[None].expand(Z, -1, -1, -1).contiguous(), b)
    else:
        b = D.dense_to_sparse(b[:1], lay, block)[0]
        full = (a, b[None].expand(Z, -1, -1, -1).contiguous())
    rc, rda, rdb = D.matmul(full[0], full[1], mode, trans_a, trans_b, lay, block, dc=dc)
    ag, bg = a.to(DEV).requires_grad_(True), b.to(DEV).requires_grad_(True)
    c = tb.MatMul(lay, block, mode, trans_a=trans_a, trans_b=trans_b)(ag, bg)
    c.backward(dc.to(DEV))
    assert_close(c, rc, torch.float16, 'c')
    if mode == 'dsd':
        assert_close(ag.grad, rda.sum(0), torch.float16, 'da summed over the batch')
        assert_close(bg.grad, rdb, torch.float16, 'db')
    else:
        assert_close(ag.grad, rda, torch.float16, 'da')
        assert_close(bg.grad, rdb.sum(0), torch.float16, 'db summed over the batch')


def test_random_attention_shapes_specialised_against_general(monkeypatch):
    # 60 random layouts / block sizes / head dimensions / dtypes: the row-group kernels (blocks 16, 32, 64) must agree
    # with the general kernels on the same inputs; covers ragged groups, empty and full lines, chains, one to three batches
    import random
    from torch_blocksparse import _lib, matmul
    rnd = random.Random(7)
    for it in range(60):
        block = rnd.choice([16, 32, 64])
        H, R, C = rnd.randint(1, 4), rnd.randint(1, 30), rnd.randint(1, 30)
        lay = random_layout((H, R, C), rnd.choice([0.05, 0.2, 0.5, 0.9, 1.0]), it)
        if rnd.random() < 0.3 and R > 2:
            lay[:, rnd.randrange(R), :] = 1
        if rnd.random() < 0.3 and C > 2:
            lay[:, :, rnd.randrange(C)] = 1
        lay[:, 0, 0] = 1                                  # no empty head
        Z, free = rnd.randint(1, 3), rnd.choice([64, 128])
        dtype = rnd.choice([torch.float16, torch.bfloat16])
        mode = rnd.choice(['dsd', 'dsd_t', 'sdd', 'sdd_bwd'])
        nnz = int(lay.sum())
        g = torch.Generator().manual_seed(it)
        mk = lambda *shape: torch.randn(*shape, generator=g).to(dtype).to(DEV)
        if mode == 'dsd':
            ops = (mk(Z, nnz, block, block), mk(Z, H, C * block, free))
            f = lambda a, b: tb.MatMul(lay, block, 'dsd')(a, b)
        elif mode == 'dsd_t':
            ops = (mk(Z, nnz, block, block), mk(Z, H, R * block, free))
            f = lambda a, b: tb.MatMul(lay, block, 'dsd', trans_a=True)(a, b)
        else:
            ops = (mk(Z, H, R * block, free), mk(Z, H, C * block, free), mk(Z, nnz, block, block))

            def f(a, b, dc=None, bwd=(mode == 'sdd_bwd')):
                a, b = a.clone().requires_grad_(bwd), b.clone().requires_grad_(bwd)
                c = tb.MatMul(lay, block, 'sdd', trans_b=True)(a, b)
                if not bwd:
                    return c
                c.backward(ops[2])
                return torch.cat([a.grad.flatten(), b.grad.flatten()])
        monkeypatch.setattr(matmul, 'KERNEL_FLAGS', 0)
        x = f(*ops[:2]).float()
        monkeypatch.setattr(matmul, 'KERNEL_FLAGS', _lib.FLAG_GENERAL_ONLY)
        y = f(*ops[:2]).float()
        monkeypatch.setattr(matmul, 'KERNEL_FLAGS', 0)
        tol = (2e-2 if dtype == torch.bfloat16 else 4e-3) * (float(y.abs().max()) + 1e-6)
        assert torch.isfinite(x).all() and float((x - y).abs().max()) <= tol, (it, mode, block, H, R, C, Z, free, dtype)


@pytest.mark.parametrize('block', [32, 64, 128])
@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_wide_free_dimension_kernels(block, dtype):
    # dsd / dds with 256 dense rows or more take the kernels that load straight into LDS (blocks 64 and 128; block 32
    # through row groups that share the dense tiles): every orientation, a free dimension that does not fill its last
    # 256-wide tile (328) and one of exactly two tiles, an empty line, a full line, a number of lines that is not a
    # multiple of the group size
    n = 9 if block == 128 else 11
    lay = random_layout((2, n, n), 0.35, 900 + block)
    lay[:, 3, :] = 0
    lay[:, :, 4] = 0
    lay[0, 5, :] = 1
    lay[1, :, 6] = 1
    lay[:, 3, :] = 0
    lay[:, :, 4] = 0
    lay[:, 0, 0] = 1
    for free in (328, 512):
        for ta in (False, True):
            for tb_ in (False, True):
                run_case('dsd', ta, tb_, block, dtype, Z=2, H=2, M=n * block, K=n * block, N=free, layout=lay, seed=free + block, dist='randn',
                         scale=0.2, backward=False)
                run_case('dds', ta, tb_, block, dtype, Z=2, H=2, M=free, K=n * block, N=n * block, layout=lay, seed=free + block + 1,
                         dist='randn', scale=0.2, backward=False)
    # forward and backward once (the backward products are dsd / dds / sdd calls of their own, written transposed)
    run_case('dsd', False, False, block, dtype, Z=2, H=2, M=n * block, K=n * block, N=320, layout=lay, seed=block, dist='randn', scale=0.2)
    run_case('dds', False, True, block, dtype, Z=2, H=2, M=320, K=n * block, N=n * block, layout=lay, seed=block + 5, dist='randn', scale=0.2)


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_sdd_with_a_long_reduction_at_block_32(dtype):
    # reductions of 256 and more at blocks of 32 run dense 128 x 256 tiles over a row group and eight of its block-columns
    # and write only the blocks that exist: 22 block-rows (the last group has two lines), 19 block-columns (three chunks,
    # the last one ragged), an empty row, an empty column, a full row; all four operand orientations
    lay = random_layout((3, 22, 19), 0.3, 3232)
    lay[:, 7, :] = 0
    lay[:, :, 11] = 0
    lay[1, 20, :] = 1
    lay[:, 7, :] = 0
    lay[:, :, 11] = 0
    lay[:, 0, 0] = 1
    for K in (256, 352):
        for ta in (False, True):
            for tb_ in (False, True):
                run_case('sdd', ta, tb_, 32, dtype, Z=2, H=3, M=22 * 32, N=19 * 32, K=K, layout=lay, seed=K, dist='randn', scale=0.2, backward=False)
    run_case('sdd', False, True, 32, dtype, Z=2, H=3, M=22 * 32, N=19 * 32, K=320, layout=lay, seed=7, dist='randn', scale=0.2)


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_sdd_with_a_long_reduction_at_block_16(dtype):
    # blocks of 16, reduction >= 256 and a multiple of 32: the same 128 x 256 products from a plan over pairs of
    # block-rows, sixteen gathered block-columns per workgroup; every orientation, batch 2, layouts with an empty
    # column, members with one of their two block-rows absent, a ragged last group (10 block-rows: 5 pairs) and
    # more block-columns than one chunk (24 > 16); also the stripe layout of the reference's own benchmark
    # (tests/test_matmul.py:105-122: 'fixed', one dense column in four, local windows of four blocks)
    lay = random_layout((2, 10, 24), 0.3, 31)
    lay[:, :, 5] = 0
    lay[0, 3, :] = 0
    lay[1, 8:, :] = 0
    lay[1, 9, 2] = 1
    for ta, tb_ in ((False, True), (True, False), (False, False), (True, True)):
        run_case('sdd', ta, tb_, 16, dtype, Z=2, H=2, M=160, N=384, K=320, layout=lay, seed=40 + ta + 2 * tb_, dist='randn', scale=0.25)
    stripes = tb.make_layout(3, 16, 'fixed', 4, False, 4, 1)
    run_case('sdd', False, False, 16, dtype, Z=1, H=3, M=256, N=256, K=512, layout=stripes, seed=44, dist='randn', scale=0.25)
    # reductions the kernel leaves to the others: not a multiple of 32, or short; and an odd number of block-rows
    run_case('sdd', False, True, 16, dtype, Z=1, H=2, M=160, N=384, K=272, layout=lay, seed=45, dist='randn', scale=0.25)
    run_case('sdd', False, True, 16, dtype, Z=1, H=2, M=160, N=384, K=64, layout=lay, seed=46, dist='randn', scale=0.25)
    odd = random_layout((1, 7, 9), 0.5, 33)
    run_case('sdd', False, True, 16, dtype, Z=1, H=1, M=112, N=144, K=256, layout=odd, seed=47, dist='randn', scale=0.25)


def test_wide_kernels_agree_with_the_general_ones(monkeypatch):
    # the same launches with and without the wide-free-dimension / long-reduction kernels (a launch flag of the C ABI)
    from torch_blocksparse import _lib, matmul
    torch.manual_seed(77)
    for block in (16, 32, 64, 128):
        lay = random_layout((2, 6, 7), 0.4, 70 + block)
        nnz = int(lay.sum())
        sp = torch.randn(2, nnz, block, block, device=DEV, dtype=torch.float16)
        dn = torch.randn(2, 2, 7 * block, 512, device=DEV, dtype=torch.float16)
        a, b = torch.randn(2, 2, 6 * block, 512, device=DEV, dtype=torch.float16), torch.randn(2, 2, 7 * block, 512, device=DEV, dtype=torch.float16)
        outs = []
        for flags in (0, _lib.FLAG_NO_WIDE):
            monkeypatch.setattr(matmul, 'KERNEL_FLAGS', flags)
            outs.append((tb.MatMul(lay, block, 'dsd')(sp, dn), tb.MatMul(lay, block, 'sdd', trans_b=True)(a, b)))
        monkeypatch.setattr(matmul, 'KERNEL_FLAGS', 0)
        for x, y in zip(*outs):
            tol = 4e-3 * (float(y.float().abs().max()) + 1e-6)
            assert float((x.float() - y.float()).abs().max()) <= tol
