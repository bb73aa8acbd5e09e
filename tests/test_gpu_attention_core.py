"""GPU: the fused attention chain (bsp_attention_fwd / bsp_attention_bwd behind attention_chain) against the dense fp32
oracle, against the three-operator chain it stands for, and at the points where it must hand over to that chain."""
import ctypes

import pytest
import torch

import torch_blocksparse as tb
from torch_blocksparse import _lib, attention_core as ac
from oracle import dense_oracle as D
from helpers import assert_close, guard_allocations

pytestmark = pytest.mark.gpu
DEV = 'cuda'


@pytest.fixture(autouse=True)
def fused_on():
    old = ac.FUSED
    ac.FUSED = True
    yield
    ac.FUSED = old


def _ops(layout):
    return (tb.MatMul(layout, 64, 'sdd', trans_a=False, trans_b=True), tb.Softmax(layout, 64), tb.MatMul(layout, 64, 'dsd'))


def _causal_window_layout(H, R, window=3, stride=4):
    """causal: `window` blocks before the diagonal plus every stride-th block-column: rows of 1 .. window + R / stride blocks"""
    lay = torch.zeros(H, R, R, dtype=torch.int64)
    for h in range(H):
        for r in range(R):
            lay[h, r, max(0, r - window + 1):r + 1] = 1
            lay[h, r, [c for c in range(0, r + 1) if c % stride == (h % stride)]] = 1
    return lay


def _run(ops, q, k, v, do, fused, **kw):
    ac.FUSED = fused
    qg, kg, vg = [t.detach().clone().requires_grad_(True) for t in (q, k, v)]
    before = ac.fused_calls
    o = ac.attention_chain(ops[0], ops[1], ops[2], qg, kg, vg, **kw)
    assert (ac.fused_calls > before) == fused
    o.backward(do)
    torch.cuda.synchronize()
    return o.detach(), qg.grad, kg.grad, vg.grad


# differences between the fused kernels and the three operators, relative to the largest value of the tensor: the
# forward pass computes the same roundings (scores to the storage type, softmax in fp32) and differs by the order of
# the sums; the backward pass replaces sum(p dp) by sum(do o), equal in exact arithmetic
CHAIN_TOL = {torch.float16: (1.5e-3, 4e-3), torch.bfloat16: (1.2e-2, 3e-2)}


@pytest.mark.parametrize('dtype,dh,masks', [
    (torch.float16, 64, ()),
    (torch.float16, 64, ('kpm_add',)),
    (torch.float16, 64, ('kpm_mul', 'attn_mul')),
    (torch.float16, 64, ('rpe', 'attn_add')),
    (torch.bfloat16, 64, ('kpm_add', 'rpe')),
    (torch.float16, 128, ('kpm_add',)),
    (torch.bfloat16, 128, ('rpe', 'attn_mul', 'kpm_mul')),
])
def test_fused_chain_against_dense_oracle_and_three_operators(dtype, dh, masks):
    torch.manual_seed(len(masks) * 7 + dh)
    Z, H, R = 2, 3, 16
    L = R * 64
    layout = _causal_window_layout(H, R)
    assert 4 < int(layout.sum(2).max()) <= 8
    ops = _ops(layout)
    q, k, v, do = [torch.randn(Z, H, L, dh, device=DEV).to(dtype) for _ in range(4)]
    kw = dict(scale=dh ** -0.5)
    okw = {}
    if 'kpm_add' in masks:
        m = torch.zeros(Z, L)
        m[0, L - 100:] = float('-inf')
        kw.update(key_padding_mask=m.to(DEV).to(dtype), key_padding_mask_mode='add')
    if 'kpm_mul' in masks:
        m = torch.ones(Z, L)
        m[1, L - 77:] = 0
        kw.update(key_padding_mask=m.to(DEV).to(dtype), key_padding_mask_mode='mul')
    if 'attn_mul' in masks:
        kw.update(attn_mask=torch.tril(torch.ones(L, L)).to(DEV).to(dtype), attn_mask_mode='mul')
    if 'attn_add' in masks:
        kw.update(attn_mask=(0.5 * torch.randn(L, L)).to(DEV).to(dtype), attn_mask_mode='add')
    if 'rpe' in masks:
        kw.update(rpe=(0.3 * torch.randn(H, L, L)).to(DEV).to(dtype))
    okw = {n: kw[n] for n in ('rpe', 'key_padding_mask', 'attn_mask', 'key_padding_mask_mode') if n in kw}
    okw['attn_mask_mode'] = kw.get('attn_mask_mode', 'add')
    with guard_allocations('fused attention'):
        got = _run(ops, q, k, v, do, True, **kw)
    ref = D.attention(q, k, v, layout, 64, kw['scale'], do=do, **okw)
    chain = _run(ops, q, k, v, do, False, **kw)
    for name, g, r, c in zip(('o', 'dq', 'dk', 'dv'), got, ref, chain):
        assert_close(g, r, dtype, 'fused ' + name)
        tol = CHAIN_TOL[dtype][0 if name in ('o', 'dv') else 1] * float(c.float().abs().max())
        assert float((g.float() - c.float()).abs().max()) <= tol, name


def test_rows_of_zero_one_and_eight_blocks_and_rectangular_layout():
    # keys longer than queries (C > R), an empty block-row (its rows of o and dq are zero), rows of 1 and of 8 blocks
    torch.manual_seed(3)
    Z, H, R, C, dh = 2, 2, 6, 10, 64
    layout = torch.zeros(H, R, C, dtype=torch.int64)
    layout[:, 0, 3] = 1
    layout[:, 1, :8] = 1
    layout[0, 3, [0, 9]] = 1
    layout[1, 3, [2, 4, 5]] = 1
    layout[:, 4, 1:9] = 1
    layout[:, 5, 9] = 1                     # block-row 2 stays empty
    ops = _ops(layout)
    q, do = [torch.randn(Z, H, R * 64, dh, device=DEV).half() for _ in range(2)]
    k, v = [torch.randn(Z, H, C * 64, dh, device=DEV).half() for _ in range(2)]
    with guard_allocations('fused attention, ragged layout'):
        got = _run(ops, q, k, v, do, True, scale=0.125)
    chain = _run(ops, q, k, v, do, False, scale=0.125)
    assert not bool(got[0][:, :, 128:192].any()) and not bool(got[1][:, :, 128:192].any())
    for name, g, c in zip(('o', 'dq', 'dk', 'dv'), got, chain):
        assert float((g.float() - c.float()).abs().max()) <= 4e-3 * float(c.float().abs().max()), name
    live = torch.ones(R, dtype=torch.bool)
    live[2] = False
    rows = live.repeat_interleave(64)
    ref = D.attention(q[:, :, rows], k, v, layout[:, live], 64, 0.125, do=do[:, :, rows], attn_mask_mode='add')
    assert_close(got[0][:, :, rows], ref[0], torch.float16, 'o')
    assert_close(got[1][:, :, rows], ref[1], torch.float16, 'dq')
    assert_close(got[2], ref[2], torch.float16, 'dk')
    assert_close(got[3], ref[3], torch.float16, 'dv')


def test_strided_operands_and_gradient_subsets():
    torch.manual_seed(5)
    Z, H, R, dh = 2, 4, 8, 64
    L = R * 64
    layout = _causal_window_layout(H, R, window=2, stride=3)
    ops = _ops(layout)
    # [Z, L, H, dh] storage seen as [Z, H, L, dh]: unit stride along the head dimension, the rest strided
    q, k, v, do = [torch.randn(Z, L, H, dh, device=DEV).half().permute(0, 2, 1, 3) for _ in range(4)]
    got = _run(ops, q, k, v, do, True, scale=0.125)
    chain = _run(ops, q.contiguous(), k.contiguous(), v.contiguous(), do.contiguous(), False, scale=0.125)
    for name, g, c in zip(('o', 'dq', 'dk', 'dv'), got, chain):
        assert g.shape == c.shape
        assert float((g.float() - c.float()).abs().max()) <= 4e-3 * float(c.float().abs().max()), name
    # only some inputs need a gradient
    for need in ((True, False, False), (False, True, False), (False, False, True), (False, True, True)):
        ts = [t.detach().clone().requires_grad_(n) for t, n in zip((q, k, v), need)]
        o = ac.attention_chain(ops[0], ops[1], ops[2], ts[0], ts[1], ts[2], scale=0.125)
        o.backward(do)
        for t, n, c in zip(ts, need, chain[1:]):
            assert (t.grad is not None) == n
            if n:
                assert float((t.grad.float() - c.float()).abs().max()) <= 4e-3 * float(c.float().abs().max())


def test_backward_is_reproducible_at_full_occupancy():
    """BigBird layout at 16384 positions: 6144 workgroups, four per compute unit.  The kernels' tile ring relies on every
    LDS read of a stage having returned before the barrier that lets the stage be refilled; with that wait missing, one
    block in about 150000 came out with another tile's values.  Identical inputs must give identical bits."""
    torch.manual_seed(0)
    layout = tb.bigbird_layout(12, 256, 3, 2, 3, seed=0, causal=True)
    B, H, L, dh = 2, 12, 16384, 64
    q, k, v, do = [torch.randn(B, H, L, dh, device=DEV, dtype=torch.float16) for _ in range(4)]
    core = ac.AttentionCore(layout, 64)
    first = None
    for rep in range(6):
        qg, kg = q.clone().requires_grad_(True), k.clone().requires_grad_(True)
        o = core(qg, kg, v, scale=0.125)
        o.backward(do)
        torch.cuda.synchronize()
        if first is None:
            first = (o.detach().clone(), qg.grad.clone(), kg.grad.clone())
        else:
            assert torch.equal(o, first[0]) and torch.equal(qg.grad, first[1]) and torch.equal(kg.grad, first[2]), rep
    # and right: one (batch, head) slice against the dense oracle
    z, h = 1, 3
    ref = D.attention(q[z:z + 1, h:h + 1], k[z:z + 1, h:h + 1], v[z:z + 1, h:h + 1], layout[h:h + 1], 64, 0.125,
                      do=do[z:z + 1, h:h + 1], attn_mask_mode='add')
    assert_close(first[0][z:z + 1, h:h + 1], ref[0], torch.float16, 'o')
    assert_close(first[1][z:z + 1, h:h + 1], ref[1], torch.float16, 'dq')
    assert_close(first[2][z:z + 1, h:h + 1], ref[2], torch.float16, 'dk')


def test_modules_take_the_fused_kernels_and_agree_with_the_operators():
    torch.manual_seed(6)
    cfg = tb.SparsityConfig(mode='fixed', block=64, stride=256, attention='unidirectional')
    mod = tb.SparseSelfAttention(cfg)
    B, H, L, dh = 2, 4, 1024, 64
    q, k, v, do = [torch.randn(B, H, L, dh, device=DEV).half() for _ in range(4)]
    kpm = torch.zeros(B, L, device=DEV).half()
    kpm[1, 900:] = float('-inf')
    res = {}
    for fused in (True, False):
        ac.FUSED = fused
        ts = [t.clone().requires_grad_(True) for t in (q, k, v)]
        n0 = ac.fused_calls
        o = mod(ts[0], ts[1], ts[2], key_padding_mask=kpm)
        assert (ac.fused_calls - n0) == int(fused)
        o.backward(do)
        res[fused] = [o.detach()] + [t.grad for t in ts]
    for g, c in zip(res[True], res[False]):
        assert float((g.float() - c.float()).abs().max()) <= 4e-3 * float(c.float().abs().max())
    # nn.MultiheadAttention drop-in: block 64, head dimension 64
    E, heads, Lm = 256, 4, 512
    layout = torch.tril(torch.ones(heads, Lm // 64, Lm // 64)).long()
    torch.manual_seed(0)
    mha = tb.MultiheadAttention(E, heads, layout, 64).to(DEV).half()
    x = torch.rand(Lm, 2, E, device=DEV).half()
    outs = {}
    for fused in (True, False):
        ac.FUSED = fused
        n0 = ac.fused_calls
        xg = x.clone().requires_grad_(True)
        y, _ = mha(xg, xg, xg, need_weights=False)
        assert (ac.fused_calls - n0) == int(fused)
        y.float().sum().backward()
        outs[fused] = (y.detach(), xg.grad)
    for g, c in zip(outs[True], outs[False]):
        assert float((g.float() - c.float()).abs().max()) <= 6e-3 * float(c.float().abs().max()) + 1e-3


def test_cases_left_to_the_three_operators():
    torch.manual_seed(7)
    Z, H, dh = 1, 2, 64
    q = torch.randn(Z, H, 640, dh, device=DEV).half()
    n0 = ac.fused_calls
    # a row of 32768 elements: the softmax operator's own bound (softmax.py:225-227)
    layout = torch.ones(1, 1, 512, dtype=torch.int64)
    ops = _ops(layout)
    k = torch.randn(1, 1, 32768, dh, device=DEV).half()
    with pytest.raises(NotImplementedError):
        ac.attention_chain(ops[0], ops[1], ops[2], q[:, :1, :64], k, k, scale=0.125)
    assert ac.fused_calls == n0
    # dropout, fp32, a head dimension the kernels do not have, blocks of 128
    lay = torch.tril(torch.ones(H, 4, 4)).long()
    ops = _ops(lay)
    q, k, v = [torch.randn(Z, H, 256, dh, device=DEV).half() for _ in range(3)]
    for args, kw in (((q, k, v), dict(dropout_p=0.5)), ((q.float(), k.float(), v.float()), {}),
                     ((q[..., :32].contiguous(), k[..., :32].contiguous(), v[..., :32].contiguous()), {})):
        n0 = ac.fused_calls
        ac.attention_chain(ops[0], ops[1], ops[2], *args, scale=0.125, **kw)
        assert ac.fused_calls == n0
    lay128 = torch.ones(H, 2, 2).long()                        # blocks of 128 have no fused kernel
    ops128 = (tb.MatMul(lay128, 128, 'sdd', trans_b=True), tb.Softmax(lay128, 128), tb.MatMul(lay128, 128, 'dsd'))
    n0 = ac.fused_calls
    ac.attention_chain(ops128[0], ops128[1], ops128[2], q, k, v, scale=0.125)
    assert ac.fused_calls == n0
    # operators built on different layouts are not a chain the fused kernels can stand for
    other = lay.clone()
    other[:, 3, 0] = 0
    mixed = (tb.MatMul(lay, 64, 'sdd', trans_b=True), tb.Softmax(lay, 64), tb.MatMul(other, 64, 'dsd'))
    assert ac._core_for(*mixed) is None
    # the reference's dtype check on the masks (softmax.py:348-353) comes before any launch
    with pytest.raises(ValueError):
        ac.attention_chain(ops[0], ops[1], ops[2], q, k, v, key_padding_mask=torch.zeros(Z, 256, device=DEV))


@pytest.mark.parametrize('block,dtype,dh,R,C,density,masks', [
    (32, torch.float16, 64, 8, 8, 0.5, ()),
    (16, torch.float16, 64, 16, 16, 0.4, ('kpm',)),
    (16, torch.float16, 64, 32, 32, 0.3, ('kpm', 'attn')),
    (32, torch.bfloat16, 128, 16, 12, 0.4, ('kpm', 'rpe')),
    (16, torch.float16, 128, 24, 32, 0.25, ('rpe',)),
    (16, torch.bfloat16, 64, 12, 20, 0.15, ()),
])
def test_blocks_of_16_and_32_on_gathered_tiles(block, dtype, dh, R, C, density, masks):
    """Small blocks: the kernels work on 64 x 64 tiles of the layout; blocks absent from a present tile take no part in
    the softmax and are not stored, a row of small blocks without any block (inside a tile-row that its neighbours
    keep alive) gives zero rows of o and dq, rectangular layouts, every mask."""
    torch.manual_seed(R * C + block)
    Z, H = 2, 2
    lay = (torch.rand(H, R, C) < density).long()
    lay[:, :, 0] = 1
    lay[:, 4:8, :] = 0                # rows of small blocks without any block ...
    lay[:, 5, 3] = 1                  # ... one of which is kept (so at block 16 its tile-row exists)
    ops = (tb.MatMul(lay, block, 'sdd', trans_b=True), tb.Softmax(lay, block), tb.MatMul(lay, block, 'dsd'))
    q, do = [torch.randn(Z, H, R * block, dh, device=DEV).to(dtype) for _ in range(2)]
    k, v = [torch.randn(Z, H, C * block, dh, device=DEV).to(dtype) for _ in range(2)]
    kw = dict(scale=dh ** -0.5)
    if 'kpm' in masks:
        m = torch.zeros(Z, C * block)
        m[0, -37:] = float('-inf')
        kw['key_padding_mask'] = m.to(DEV).to(dtype)
    if 'rpe' in masks:
        kw['rpe'] = (0.3 * torch.randn(R * block, C * block)).to(DEV).to(dtype)
    if 'attn' in masks:
        kw.update(attn_mask=(torch.rand(R * block, C * block) < 0.8).to(DEV).to(dtype), attn_mask_mode='mul')
        kw['attn_mask'][:, 0] = 1      # (no row loses all its columns)
    with guard_allocations('fused attention, block %d' % block):
        got = _run(ops, q, k, v, do, True, **kw)
    chain = _run(ops, q, k, v, do, False, **kw)
    live = lay.sum(2).ne(0).all(0)                    # rows of small blocks that hold a block in every head
    rows = live.repeat_interleave(block)
    dead = ~lay.sum(2).ne(0).any(0).repeat_interleave(block)
    assert not bool(got[0][:, :, dead.to(DEV)].any()) and not bool(got[1][:, :, dead.to(DEV)].any())
    tol = CHAIN_TOL[dtype][1]
    for name, g, c in zip(('o', 'dq', 'dk', 'dv'), got, chain):
        assert not bool(torch.isnan(g).any()), name
        assert float((g.float() - c.float()).abs().max()) <= tol * float(c.float().abs().max()), name
    okw = {n: kw[n] for n in ('key_padding_mask', 'attn_mask') if n in kw}
    if 'rpe' in kw:
        okw['rpe'] = kw['rpe'][rows.to(DEV)]
    if 'attn_mask' in okw:
        okw['attn_mask'] = okw['attn_mask'][rows.to(DEV)]
    ref = D.attention(q[:, :, rows.to(DEV)], k, v, lay[:, live], block, kw['scale'], do=do[:, :, rows.to(DEV)],
                      attn_mask_mode=kw.get('attn_mask_mode', 'add'), **okw)
    assert_close(got[0][:, :, rows.to(DEV)], ref[0], dtype, 'o')
    assert_close(got[1][:, :, rows.to(DEV)], ref[1], dtype, 'dq')
    # dk and dv collect contributions from every row: against the oracle when the rows left out above (empty in some
    # head) are empty in every head, against the three operators (above) in any case
    if bool((lay.sum(2).ne(0).all(0) | ~lay.sum(2).ne(0).any(0)).all()):
        assert_close(got[2], ref[2], dtype, 'dk')
        assert_close(got[3], ref[3], dtype, 'dv')


def test_small_blocks_that_the_tiles_do_not_fit_go_to_the_operators():
    torch.manual_seed(9)
    Z, H, dh = 1, 2, 64
    q, k, v = [torch.randn(Z, H, 18 * 16, dh, device=DEV).half() for _ in range(3)]
    lay = torch.tril(torch.ones(H, 18, 18)).long()            # 18 rows of blocks of 16: not a whole number of tiles
    ops = (tb.MatMul(lay, 16, 'sdd', trans_b=True), tb.Softmax(lay, 16), tb.MatMul(lay, 16, 'dsd'))
    n0 = ac.fused_calls
    o = ac.attention_chain(ops[0], ops[1], ops[2], q, k, v, scale=0.125)
    assert ac.fused_calls == n0
    assert_close(o, D.attention(q, k, v, lay, 16, 0.125, attn_mask_mode='add'), torch.float16, 'o')
    # blocks scattered one per 64 x 64 area: the tiles gather them (four block-columns of a line of tiles into one tile)
    lay = torch.zeros(H, 16, 16, dtype=torch.int64)
    lay[:, torch.arange(0, 16, 2), torch.arange(0, 16, 2)] = 1
    ops = (tb.MatMul(lay, 16, 'sdd', trans_b=True), tb.Softmax(lay, 16), tb.MatMul(lay, 16, 'dsd'))
    q, k, v = [torch.randn(Z, H, 256, dh, device=DEV).half() for _ in range(3)]
    n0 = ac.fused_calls
    o = ac.attention_chain(ops[0], ops[1], ops[2], q, k, v, scale=0.125)
    assert ac.fused_calls == n0 + 1
    assert ac._core_for(*ops).tables(torch.device(DEV))[1] == 1          # one tile per line
    live = lay.sum(2).ne(0).all(0).repeat_interleave(16)
    assert_close(o[:, :, live], D.attention(q[:, :, live], k, v, lay[:, lay.sum(2).ne(0).all(0)], 16, 0.125, attn_mask_mode='add'), torch.float16, 'o')
    assert not bool(o[:, :, ~live].any())
    # the default block of the sparse self-attention module is 16: it takes the fused kernels
    mod = tb.SparseSelfAttention(tb.SparsityConfig(mode='fixed', block=16, stride=64, attention='unidirectional'))
    q, k, v = [torch.randn(2, 4, 512, dh, device=DEV).half() for _ in range(3)]
    n0 = ac.fused_calls
    mod(q, k, v)
    assert ac.fused_calls == n0 + 1


@pytest.mark.parametrize('block,dtype,dh,R,C,kpm,extra', [
    (64, torch.float16, 64, 12, 20, None, ()),
    (64, torch.float16, 64, 16, 16, 'add', ()),
    (64, torch.bfloat16, 128, 10, 24, 'mul', ()),
    (64, torch.float16, 128, 9, 9, None, ()),
    (32, torch.float16, 64, 16, 40, 'add', ()),
    (16, torch.bfloat16, 64, 24, 80, 'mul', ()),
    (16, torch.float16, 128, 16, 48, None, ()),
    (64, torch.float16, 64, 12, 20, None, ('rpe',)),
    (64, torch.float16, 64, 16, 16, 'add', ('attn_mul',)),
    (64, torch.bfloat16, 128, 10, 24, 'mul', ('rpe', 'attn_add')),
    (64, torch.float16, 128, 12, 12, 'add', ('rpe', 'attn_mul')),
    (32, torch.float16, 64, 16, 40, None, ('attn_add',)),
    (16, torch.bfloat16, 64, 24, 80, 'add', ('rpe', 'attn_mul')),
])
def test_rows_longer_than_eight_tiles_are_streamed(block, dtype, dh, R, C, kpm, extra):
    """Rows of 9 .. 24 tiles beside short and empty ones: two-sweep forward, block-by-block backward; key-padding masks
    in both modes, among them a whole masked tile in the middle of a row (its maximum so far stays where it was) and
    one at the start (the running maximum starts at -inf)."""
    torch.manual_seed(R + C + block)
    Z, H = 2, 2
    lay = (torch.rand(H, R, C) < 0.7).long()
    lay[:, 0, :] = 1                       # the longest row the layout allows
    lay[:, 1, :] = 0
    lay[:, 1, C - 1] = 1                   # a row of one block (which the masks below leave alone)
    lay[0, 2, :] = 0                       # an empty row in one head
    S = 64 // block
    assert int(lay.view(H, R // S, S, C // S, S).sum((2, 4)).ne(0).sum(2).max()) > 8
    ops = (tb.MatMul(lay, block, 'sdd', trans_b=True), tb.Softmax(lay, block), tb.MatMul(lay, block, 'dsd'))
    q, do = [torch.randn(Z, H, R * block, dh, device=DEV).to(dtype) for _ in range(2)]
    k, v = [torch.randn(Z, H, C * block, dh, device=DEV).to(dtype) for _ in range(2)]
    kw = dict(scale=dh ** -0.5)
    if kpm == 'add':
        m = 0.5 * torch.randn(Z, C * block)
        m[0, 128:200] = float('-inf')
        m[1, :70] = float('-inf')
        kw.update(key_padding_mask=m.to(DEV).to(dtype), key_padding_mask_mode='add')
    if kpm == 'mul':
        m = torch.ones(Z, C * block)
        m[0, :64] = 0
        m[1, 190:330] = 0
        kw.update(key_padding_mask=m.to(DEV).to(dtype), key_padding_mask_mode='mul')
    Lq, Lk = R * block, C * block
    if 'rpe' in extra:
        kw['rpe'] = (0.3 * torch.randn(H, Lq, Lk)).to(DEV).to(dtype)
    if 'attn_add' in extra:
        kw.update(attn_mask=(0.5 * torch.randn(Lq, Lk)).to(DEV).to(dtype), attn_mask_mode='add')
    if 'attn_mul' in extra:
        m = (torch.rand(Lq, Lk) < 0.7).float()
        m[:, Lk - block:] = 1              # (no row loses all its columns: the last block-column is in every row with a block)
        kw.update(attn_mask=m.to(DEV).to(dtype), attn_mask_mode='mul')
    with guard_allocations('fused attention, long rows'):
        got = _run(ops, q, k, v, do, True, **kw)
    chain = _run(ops, q, k, v, do, False, **kw)
    tol = CHAIN_TOL[dtype]
    for name, g, c in zip(('o', 'dq', 'dk', 'dv'), got, chain):
        assert not bool(torch.isnan(g).any()), name
        assert float((g.float() - c.float()).abs().max()) <= tol[0 if name in ('o', 'dv') else 1] * float(c.float().abs().max()), name
    live = lay.sum(2).ne(0).all(0)
    rows = live.repeat_interleave(block).to(DEV)
    okw = {n: kw[n] for n in ('key_padding_mask', 'key_padding_mask_mode') if n in kw}
    if 'rpe' in kw:
        okw['rpe'] = kw['rpe'][:, rows]
    if 'attn_mask' in kw:
        okw['attn_mask'] = kw['attn_mask'][rows]
    ref = D.attention(q[:, :, rows], k, v, lay[:, live], block, kw['scale'], do=do[:, :, rows], attn_mask_mode=kw.get('attn_mask_mode', 'add'), **okw)
    assert_close(got[0][:, :, rows], ref[0], dtype, 'o')
    assert_close(got[1][:, :, rows], ref[1], dtype, 'dq')


def test_streamed_rows_that_are_masked_everywhere_give_nan_like_the_operators():
    torch.manual_seed(11)
    Z, H, R, C, dh = 1, 1, 2, 12, 64
    lay = torch.ones(H, R, C, dtype=torch.int64)
    ops = _ops(lay)
    q = torch.randn(Z, H, R * 64, dh, device=DEV).half()
    k, v = [torch.randn(Z, H, C * 64, dh, device=DEV).half() for _ in range(2)]
    m = torch.full((Z, C * 64), float('-inf'), device=DEV).half()
    ac.FUSED = True
    n0 = ac.fused_calls
    o = ac.attention_chain(ops[0], ops[1], ops[2], q, k, v, scale=0.125, key_padding_mask=m)
    assert ac.fused_calls == n0 + 1
    ac.FUSED = False
    c = ac.attention_chain(ops[0], ops[1], ops[2], q, k, v, scale=0.125, key_padding_mask=m)
    assert bool(torch.isnan(o).all()) and bool(torch.isnan(c).all())


def test_streamed_backward_is_reproducible_at_full_occupancy():
    """Dense attention over 2048 keys (32 tiles a row), enough workgroups to fill every compute unit several times: the
    tile ring is reused under load; the same inputs give the same bits."""
    torch.manual_seed(13)
    Z, H, R, dh = 4, 8, 32, 64
    lay = torch.ones(H, R, R, dtype=torch.int64)
    ops = _ops(lay)
    q, k, v, do = [torch.randn(Z, H, R * 64, dh, device=DEV).half() for _ in range(4)]
    first = _run(ops, q, k, v, do, True, scale=0.125)
    for _ in range(4):
        again = _run(ops, q, k, v, do, True, scale=0.125)
        for a, b in zip(first, again):
            assert torch.equal(a, b)
    chain = _run(ops, q, k, v, do, False, scale=0.125)
    for name, g, c in zip(('o', 'dq', 'dk', 'dv'), first, chain):
        assert float((g.float() - c.float()).abs().max()) <= CHAIN_TOL[torch.float16][1] * float(c.float().abs().max()), name


@pytest.mark.parametrize('block,dh,dtype', [(64, 64, torch.float16), (64, 128, torch.bfloat16), (16, 64, torch.float16), (32, 128, torch.float16)])
def test_backward_through_the_column_kernel_and_through_the_two_operators(block, dh, dtype):
    """dk and dv from the column kernel (the default) against the stored softmax gradient and the two transposed dsd
    operators; a layout whose global columns are cut into parts (every size of part from 1 block on) beside short and
    empty columns, keys longer than queries."""
    torch.manual_seed(block + dh)
    Z, H = 2, 3
    S = 64 // block
    R, C = 40 * S, 44 * S
    lay = torch.zeros(H, R, C, dtype=torch.int64)
    for r in range(R):
        lay[:, r, max(0, r - 2 * S):r + 1] = 1            # a band
    lay[:, :, 0] = 1                                     # a global column: 40 tiles
    lay[1, 3 * S:, 5 * S] = 1                            # 37 tiles in one head
    lay[:, :, C - 2 * S:] = 0                            # columns without blocks
    lay[2, 17 * S:, :] = 0                               # a head whose later rows are empty
    if S > 1:
        lay[:, 1::2, 1::3] = 0                           # holes inside the tiles
        lay[:, :, 0] = 1
    ops = (tb.MatMul(lay, block, 'sdd', trans_b=True), tb.Softmax(lay, block), tb.MatMul(lay, block, 'dsd'))
    core = ac._core_for(*ops)
    ct = core.tables(torch.device(DEV))[5]
    assert ct.n_split >= H and ct.n_slots > ct.n_split
    q, do = [torch.randn(Z, H, R * block, dh, device=DEV).to(dtype) for _ in range(2)]
    k, v = [torch.randn(Z, H, C * block, dh, device=DEV).to(dtype) for _ in range(2)]
    kpm = torch.zeros(Z, C * block)
    kpm[1, 100:180] = float('-inf')
    kw = dict(scale=dh ** -0.5, key_padding_mask=kpm.to(DEV).to(dtype))
    old = ac.FUSED_KV
    try:
        ac.FUSED_KV = True
        with guard_allocations('fused attention, column kernel'):
            got = _run(ops, q, k, v, do, True, **kw)
        again = _run(ops, q, k, v, do, True, **kw)
        ac.FUSED_KV = False
        stored = _run(ops, q, k, v, do, True, **kw)
    finally:
        ac.FUSED_KV = old
    chain = _run(ops, q, k, v, do, False, **kw)
    tol = CHAIN_TOL[dtype]
    for name, g, a2, s2, c in zip(('o', 'dq', 'dk', 'dv'), got, again, stored, chain):
        assert torch.equal(g, a2), name                  # parts are summed in a fixed order
        assert not bool(torch.isnan(g).any()), name
        ref = float(c.float().abs().max())
        assert float((g.float() - s2.float()).abs().max()) <= tol[0] * ref, name
        assert float((g.float() - c.float()).abs().max()) <= tol[0 if name in ('o', 'dv') else 1] * ref, name
    assert torch.equal(got[0], stored[0]) and torch.equal(got[1], stored[1])      # o and dq do not depend on the choice
    assert not bool(got[2][:, :, (C - 2 * S) * block:].any()) and not bool(got[3][:, :, (C - 2 * S) * block:].any())
    live = lay.sum(2).ne(0).all(0)
    if bool(live.all()):
        ref = D.attention(q, k, v, lay, block, kw['scale'], do=do, key_padding_mask=kw['key_padding_mask'], attn_mask_mode='add')
        for name, g, r in zip(('o', 'dq', 'dk', 'dv'), got, ref):
            assert_close(g, r, dtype, name)


def _fwd_tables(core, device, keep_p=True):
    lut, maxlut, _, rows = core.tables(device)[:4]
    return lut, maxlut, keep_p, rows


class _FakeCtx:
    """stand-in for the autograd context: the kernels of the backward pass called one by one"""
    needs_input_grad = (True, True, True)

    def save_for_backward(self, *t):
        self.saved_tensors = t


@pytest.mark.parametrize('R,block', [(6, 64), (12, 64), (8, 32)])
def test_rows_kernel_outputs_in_every_combination(R, block):
    """bsp_attention_bwd writes dq always, ds and the rows' delta each only when asked: the same bits in every
    combination, delta = sum_d do . o, and the column kernel fed with that delta reproduces ds^T . q and p^T . do.
    R = 12 block-rows of 64: rows of up to 12 tiles, the streaming kernels."""
    torch.manual_seed(R)
    Z, H, dh = 2, 2, 64
    lay = torch.tril(torch.ones(H, R, R, dtype=torch.int64))
    lay[1, :, 1] = 0
    core = ac.AttentionCore(lay, block)
    L = R * block
    q, k, v, do = [torch.randn(Z, H, L, dh, device=DEV).half() for _ in range(4)]
    ctx = _FakeCtx()
    with torch.no_grad():
        o = ac._attention_core.forward(ctx, q, k, v, 0.125, None, None, None, 'add', 'add', core, *_fwd_tables(core, q.device))
        p = ctx.saved_tensors[3]
        outs = {}
        for want_ds in (False, True):
            for want_delta in (False, True):
                ds = torch.full_like(p, 7.0) if want_ds else None
                delta = torch.full((Z, H, ctx.rows * 64), 7.0, device=DEV) if want_delta else None
                outs[(want_ds, want_delta)] = (ac._attention_core.rows_kernel(ctx, do, ds, delta), ds, delta)
        dq, ds, delta = outs[(True, True)]
        for key, (dq2, ds2, delta2) in outs.items():
            assert torch.equal(dq2, dq), key
            assert ds2 is None or torch.equal(ds2, ds), key
            assert delta2 is None or torch.equal(delta2, delta), key
        ref_delta = (do.float() * o.float()).sum(-1)
        assert float((delta - ref_delta).abs().max()) <= 1e-3 * float(ref_delta.abs().max())
        dk, dv = ac._attention_core.columns_kernel(ctx, do, delta)
        dk_ops, dv_ops = core.dsd_tn(ds, q), core.dsd_tn(p, do)
    for name, g, c in (('dk', dk, dk_ops), ('dv', dv, dv_ops)):
        assert float((g.float() - c.float()).abs().max()) <= 1.5e-3 * float(c.float().abs().max()), name


@pytest.mark.parametrize('seed', list(range(32)) + [-s for s in range(1, 9)])
def test_seeded_random_sweep_against_the_three_operators(seed):
    """Random layouts (square and rectangular, rows and columns from empty to long, tiles from full to mostly holes),
    block sizes, head dimensions, types and mask combinations: every kernel variant (rows in registers / streamed, with
    and without per-element masks, columns whole / in parts) against the three-operator chain."""
    stored_gradient = seed < 0                             # negative seeds: dk and dv from the stored gradient and the two operators
    seed = abs(seed) + (100 if stored_gradient else 0)
    g = torch.Generator().manual_seed(1000 + seed)
    rnd = lambda n: int(torch.randint(0, n, (1,), generator=g))
    block = (64, 32, 16)[rnd(3)]
    S = 64 // block
    dh = (64, 128)[rnd(2)]
    dtype = (torch.float16, torch.bfloat16)[rnd(2)]
    Z, H = 1 + rnd(2), 1 + rnd(3)
    Rt, Ct = 1 + rnd(20), 1 + rnd(20)                     # tiles of 64
    if seed % 4 == 0:
        Rt, Ct = 9 + rnd(12), 9 + rnd(12)                  # long rows more often
    R, C = Rt * S, Ct * S
    density = (0.15, 0.4, 0.7, 1.0)[rnd(4)]
    lay = (torch.rand(H, R, C, generator=g) < density).long()
    lay[:, :, rnd(C)] = 1                                  # a full column (long when R is), so no row is empty ...
    if R > 2:
        lay[rnd(H), rnd(R), :] = 0                         # ... except one
    torch.manual_seed(seed)
    ops = (tb.MatMul(lay, block, 'sdd', trans_b=True), tb.Softmax(lay, block), tb.MatMul(lay, block, 'dsd'))
    Lq, Lk = R * block, C * block
    q, do = [torch.randn(Z, H, Lq, dh, device=DEV).to(dtype) for _ in range(2)]
    k, v = [torch.randn(Z, H, Lk, dh, device=DEV).to(dtype) for _ in range(2)]
    kw = dict(scale=dh ** -0.5)
    choice = rnd(8)
    if choice & 1:
        kw['key_padding_mask'] = (0.5 * torch.randn(Z, Lk, generator=g)).to(DEV).to(dtype)
    if choice & 2:
        kw['rpe'] = (0.3 * torch.randn(H, Lq, Lk, generator=g)).to(DEV).to(dtype)
    if choice & 4:
        kw.update(attn_mask=(0.5 * torch.randn(Lq, Lk, generator=g)).to(DEV).to(dtype), attn_mask_mode='add')
    old_kv = ac.FUSED_KV
    try:
        ac.FUSED_KV = not stored_gradient
        got = _run(ops, q, k, v, do, True, **kw)
    finally:
        ac.FUSED_KV = old_kv
    chain = _run(ops, q, k, v, do, False, **kw)
    tol = CHAIN_TOL[dtype]
    for name, a, c in zip(('o', 'dq', 'dk', 'dv'), got, chain):
        assert not bool(torch.isnan(a).any()), name
        ref = float(c.float().abs().max())
        assert float((a.float() - c.float()).abs().max()) <= tol[0 if name in ('o', 'dv') else 1] * ref, (name, block, dh, dtype, Rt, Ct, density, choice)


@pytest.mark.parametrize('cfg', [dict(), dict(attention='bidirectional'), dict(stride=128), dict(numverts=4, vertsize=1), dict(block=32, stride=128)])
def test_fixed_layouts_of_the_module_at_small_blocks(cfg):
    """The 'fixed' layouts of the sparse self-attention module (local windows plus single global block-columns): the tiles
    gather the global columns, rows view and columns view; against the dense oracle and the three operators."""
    torch.manual_seed(17)
    conf = tb.SparsityConfig(mode='fixed', **cfg)
    mod = tb.SparseSelfAttention(conf)
    Z, H, L, dh = 2, 4, 1024, 64
    q, k, v, do = [torch.randn(Z, H, L, dh, device=DEV).half() for _ in range(4)]
    sdd, dsd, sm = mod.get_ops(H, L, q.device)
    lay = sm.layout.cpu()
    t = ac._core_for(sdd, sm, dsd).tables(q.device)
    aligned = int(lay.reshape(H, L // 64, 64 // conf.block, L // 64, 64 // conf.block).sum((2, 4)).ne(0).sum(2).max())
    assert t[1] < aligned                                   # fewer tiles a line than a fixed grid would give
    res = {}
    for fused in (True, False):
        ac.FUSED = fused
        ts = [x.clone().requires_grad_(True) for x in (q, k, v)]
        n0 = ac.fused_calls
        o = mod(*ts)
        assert (ac.fused_calls - n0) == int(fused)
        o.backward(do)
        res[fused] = [o.detach()] + [x.grad for x in ts]
    ref = D.attention(q, k, v, lay, conf.block, dh ** -0.5, do=do, attn_mask_mode='add')
    for name, g, c, r in zip(('o', 'dq', 'dk', 'dv'), res[True], res[False], ref):
        assert float((g.float() - c.float()).abs().max()) <= CHAIN_TOL[torch.float16][1] * float(c.float().abs().max()), name
        assert_close(g, r, torch.float16, name)


@pytest.mark.parametrize('block,R', [(64, 6), (64, 12), (16, 24)])
def test_forward_without_a_backward_pass_does_not_store_p(block, R):
    """Under no_grad, or when no operand asks for a gradient, the forward kernel gets no tensor for p (and allocates
    none): the same o to the bit."""
    torch.manual_seed(R)
    Z, H, dh = 2, 2, 64
    lay = torch.tril(torch.ones(H, R, R, dtype=torch.int64))
    ops = (tb.MatMul(lay, block, 'sdd', trans_b=True), tb.Softmax(lay, block), tb.MatMul(lay, block, 'dsd'))
    q, k, v = [torch.randn(Z, H, R * block, dh, device=DEV).half() for _ in range(3)]
    kpm = (0.5 * torch.randn(Z, R * block, device=DEV)).half()
    with_grad = ac.attention_chain(ops[0], ops[1], ops[2], q.clone().requires_grad_(True), k, v, scale=0.125, key_padding_mask=kpm)
    assert with_grad.requires_grad
    torch.cuda.synchronize()
    nnz_bytes = Z * int(lay.sum()) * block * block * 2
    before = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    with torch.no_grad():
        o1 = ac.attention_chain(ops[0], ops[1], ops[2], q.clone().requires_grad_(True), k, v, scale=0.125, key_padding_mask=kpm)
    o2 = ac.attention_chain(ops[0], ops[1], ops[2], q, k, v, scale=0.125, key_padding_mask=kpm)       # nothing requires a gradient
    torch.cuda.synchronize()
    assert torch.cuda.max_memory_allocated() - before < nnz_bytes        # o and the clone of q, but no tensor of p's size
    assert torch.equal(o1, with_grad.detach()) and torch.equal(o2, o1)


def test_c_abi_argument_checks():
    lib = _lib.load()
    t = torch.zeros(1, 1, 64, 64, device=DEV, dtype=torch.float16)
    p = torch.zeros(1, 1, 64, 64, device=DEV, dtype=torch.float16)
    lut, maxlut = tb.Softmax(torch.ones(1, 1, 1, dtype=torch.int64), 64).make_lut(torch.device(DEV))
    null = ctypes.c_void_p(0)
    st = (t.stride(0), t.stride(1), t.stride(2))

    def fwd(dtype=0, q=t, D=64, block=64, maxlut=maxlut, ldq=64, rpe=null):
        return lib.bsp_attention_fwd(dtype, _lib.ptr(q), _lib.ptr(t), _lib.ptr(t), _lib.ptr(p), _lib.ptr(t.clone()), 1, 1, 1, D,
                                     st[0], st[1], ldq, *st, *st, *st, p.stride(0), block, 1.0, _lib.ptr(lut), maxlut,
                                     rpe, 0, 0, 64, null, 0, 0, null, 0, 0, _lib.stream_ptr(torch.device(DEV)))
    assert fwd() == _lib.OK
    assert fwd(dtype=_lib.F32) == _lib.ERR_UNSUPPORTED
    assert fwd(block=128) == _lib.ERR_UNSUPPORTED
    assert fwd(D=96) == _lib.ERR_UNSUPPORTED
    assert fwd(maxlut=9) == _lib.OK                     # (the streaming kernels; the table's rows hold one block)
    assert fwd(maxlut=9, rpe=_lib.ptr(t)) == _lib.OK
    assert fwd(maxlut=512) == _lib.ERR_ROW_TOO_LONG
    assert fwd(ldq=60) != _lib.OK                       # a row stride that is not a multiple of 8 elements
    assert fwd(q=None) != _lib.OK
    # the column kernel of the backward pass
    ct = ac._ColumnTable(torch.ones(1, 1, 1, dtype=torch.int64), torch.device(DEV))
    delta = torch.zeros(1, 1, 64, device=DEV)
    dk, dv = t.clone(), t.clone()

    def kv(dtype=0, D=64, block=64, n_items=ct.n_items, lddk=64, delta=delta, n_slots=0, partial=null):
        return lib.bsp_attention_bwd_kv(dtype, _lib.ptr(t), _lib.ptr(t), _lib.ptr(t), _lib.ptr(p), _lib.ptr(delta), _lib.ptr(dk), _lib.ptr(dv),
                                        1, 1, 1, D, *st, *st, *st, st[0], st[1], lddk, *st, p.stride(0), 64, block, 1.0, _lib.ptr(ct.items), n_items,
                                        partial, n_slots, null, 0, _lib.stream_ptr(torch.device(DEV)))
    assert kv() == _lib.OK
    assert kv(dtype=_lib.F32) == _lib.ERR_UNSUPPORTED
    assert kv(D=96) == _lib.ERR_UNSUPPORTED
    assert kv(block=128) == _lib.ERR_UNSUPPORTED
    assert kv(n_items=0) != _lib.OK                     # fewer work items than columns
    assert kv(lddk=60) != _lib.OK
    assert kv(delta=None) != _lib.OK
    assert kv(n_slots=2) != _lib.OK                     # slots without a place for them and without the list of their columns
    torch.cuda.synchronize()
