"""GPU: the device-built look-up tables are bit-identical to the oracle's (and so to the reference's)."""
import numpy as np
import pytest
import torch

import torch_blocksparse as tb
from torch_blocksparse.matmul import _sparse_matmul
from torch_blocksparse.softmax import _sparse_softmax
from oracle import lut_oracle as O
from helpers import random_layout

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def check_all_tables(lay, blocks=((16, 16), (16, 8), (32, 16), (64, 16), (128, 8))):
    lay = torch.as_tensor(lay, dtype=torch.int64)
    layn = lay.numpy()
    lut, maxlut = _sparse_softmax.make_lut(lay, 16, DEV)
    elut, emax = O.make_softmax_lut(layn)
    assert lut.cpu().tolist() == elut.tolist() and maxlut == emax
    for block, step in blocks:
        for trans in (False, True):
            lut, num_locks, width, _ = _sparse_matmul.make_dxx_lut(lay, block, step, trans, DEV)
            elut, enl, ewidth = O.make_dxx_lut(layn, block, step, trans)
            assert lut.cpu().tolist() == elut.tolist(), (block, step, trans)
            assert (num_locks, width) == (enl, ewidth)
            # the per-block positions are what the increments are differences of
            nz = lay.nonzero() if trans else lay.transpose(1, 2).nonzero()
            assert lut.plan[:len(nz), 0].cpu().tolist() == (nz[:, 2] * block).tolist()
            # dispatch order of the segments (ours): head by head, the longest first inside a head, ties in table order
            hdr = elut[:6 * ewidth].reshape(ewidth, 6)
            exp_order = sorted(range(ewidth), key=lambda i: (hdr[i, 3], -hdr[i, 1], i))
            assert lut.planbuf[:width].cpu().tolist() == exp_order
    for block in (16, 32, 64, 128):
        luts, _, widths, packs = _sparse_matmul.make_sdd_lut(lay, block, torch.float16, DEV)
        exp = O.sdd_segment(layn, max(1, 64 // block))
        assert packs == [p for p, _ in exp]
        seen = set()
        for t, w, (p, e) in zip(luts, widths, exp):
            assert t.cpu().tolist() == e.reshape(-1).tolist(), (block, p)
            assert w == e.shape[0] // (p * p)
            valid = [1] * e.shape[0] if t.valid is None else t.valid.cpu().tolist()
            for (h, i, j, b), v in zip(e.tolist(), valid):      # a row is valid iff it is the first for a real block
                assert bool(v) == (layn[h, i, j] != 0 and (h, i, j) not in seen)
                seen.add((h, i, j))


def test_golden_layouts(golden):
    for name, lay in golden['layouts'].items():
        check_all_tables(lay)


@pytest.mark.parametrize('seed', range(6))
def test_random_layouts(seed):
    g = torch.Generator().manual_seed(seed)
    shape = tuple(int(torch.randint(lo, hi, (1,), generator=g)) for lo, hi in ((1, 5), (1, 40), (1, 80)))
    check_all_tables(random_layout(shape, [0.05, 0.3, 0.5, 0.8, 0.97, 0.15][seed], seed), blocks=((16, 16), (32, 8)))


def test_benchmark_config_layouts():
    check_all_tables(tb.sparse_transformer_layout(16, 64, 4, 16, True), blocks=((64, 16),))          # attention, seq 4096
    check_all_tables(tb.bigbird_layout(12, 256, 3, 2, 3, seed=0, causal=True), blocks=((64, 16),))   # long context
    check_all_tables(random_layout((1, 32, 32), 0.1, 5), blocks=((128, 16),))                        # sparse linear layer
    check_all_tables(tb.fixed_layout(4, 64, 'fixed', 4, 'bidirectional', 4, 1), blocks=((16, 16),))


def test_empty_head_raises():
    lay = torch.zeros(2, 4, 4, dtype=torch.int64)
    lay[0, 1, 2] = 1
    with pytest.raises(RuntimeError):
        _sparse_matmul.make_dxx_lut(lay, 16, 16, True, DEV)


@pytest.mark.parametrize('by_rows', [True, False])
@pytest.mark.parametrize('thin_min', [0, 6])
def test_group_plan(by_rows, thin_min):
    # our own work list for the row-group kernels: 4 consecutive lines per group, one entry per position where any
    # member has a block (positions ascending for row groups, descending for column groups); lines with at least
    # thin_min blocks leave their group (bit 24 + member of its index field) and become chains (index field
    # -(line + 1)); header sorted by decreasing number of entries (exactly, or in eighths of the largest group),
    # groups before chains at equal length
    from torch_blocksparse.matmul import GroupPlan
    import itertools
    lays = (tb.sparse_transformer_layout(3, 18, 4, 8, True), random_layout((2, 9, 13), 0.4, 77), torch.ones(1, 4, 4, dtype=torch.int64),
            torch.ones(2, 7, 9, dtype=torch.int64))
    for lay, buckets in itertools.product(lays, (0, 8)):            # exact order, coarse order
        plan = GroupPlan.build(lay, by_rows, DEV, thin_min=thin_min, order_buckets=buckets)
        t = plan.table.cpu().tolist()
        H, R, C = lay.shape
        L, B = (R, C) if by_rows else (C, R)
        NG = (L + 3) // 4
        linecnt = lay.sum(2 if by_rows else 1)                      # [H, L]
        thin = (linecnt >= thin_min) if thin_min else torch.zeros_like(linecnt, dtype=torch.bool)
        rank = (torch.cumsum(lay.reshape(-1), 0) - 1).reshape(lay.shape)
        order = range(B) if by_rows else range(B - 1, -1, -1)

        def entries(h, lines):                                      # lines: 4 line indices or None
            out = []
            for b in order:
                bids = []
                for line in lines:
                    if line is None:
                        bids.append(-1)
                    else:
                        r, c = (line, b) if by_rows else (b, line)
                        bids.append(int(rank[h, r, c]) if lay[h, r, c] else -1)
                if any(x >= 0 for x in bids):
                    out.append([b] + bids)
            return out

        slots = []                                                  # (slot order, code, head, expected entries)
        for h in range(H):
            for lg in range(NG):
                lines, skip = [], 0
                for m in range(4):
                    line = lg * 4 + m
                    if line < L and thin[h, line]:
                        skip |= 1 << m
                    lines.append(line if line < L and not thin[h, line] else None)
                slots.append((lg | (skip << 24), h, entries(h, lines)))
        for h in range(H):
            for line in range(L):
                if thin[h, line]:
                    slots.append((-(line + 1), h, entries(h, [line, None, None, None])))
        # bit 28 of every group's index field: at most 2.5 group entries per dense tile (streaming hint)
        in_groups = sum(len(e) for code, h, e in slots if code >= 0)
        hint = 1 if 2 * in_groups <= 5 * H * B else 0
        slots = [(code | (hint << 28) if code >= 0 else code, h, e) for code, h, e in slots]
        mx = max([len(e) for code, h, e in slots if code >= 0] + [0])   # the largest group (chains do not count)
        key = (lambda n: n * buckets // (mx + 1)) if buckets else (lambda n: n)
        slots.sort(key=lambda s: -key(len(s[2])))                   # stable: ties stay in slot order
        ng = len(slots)
        assert plan.n_groups == ng and plan.lines == L
        total = 0
        for i, (code, h, exp) in enumerate(slots):
            start, count, gh, gcode = t[4 * i:4 * i + 4]
            assert (count, gh, gcode) == (len(exp), h, code)
            got = [t[4 * ng + 5 * (start + k):4 * ng + 5 * (start + k + 1)] for k in range(count)]
            assert got == exp
            total += count
        assert len(t) == 4 * ng + 5 * total


@pytest.mark.parametrize('by_rows', [True, False])
def test_group_plan_over_tiles(by_rows):
    # plan of a block-16 layout over 64 x 64 tiles: header and (position, tile ids) of the plan of the coarsened layout,
    # every entry followed by the ids of the 4 x 4 small blocks of each member's tile (-1 where absent)
    from torch_blocksparse.matmul import GroupPlan
    lay = random_layout((2, 24, 36), 0.15, 99)
    lay[:, 4:8, :] = 0
    lay[1, :, 8] = 1
    S, G = 4, 4
    H, R, C = lay.shape
    coarse = lay.view(H, R // S, S, C // S, S).amax((2, 4))
    ref = GroupPlan.build(coarse, by_rows, DEV, thin_min=GroupPlan.thin_min(coarse, by_rows, 64),
                          order_buckets=GroupPlan.order_buckets(coarse, by_rows, 64))
    plan = GroupPlan.build_coarse(lay, 16, by_rows, DEV)
    assert plan.coarse and plan.n_groups == ref.n_groups and plan.lines == ref.lines
    ng = ref.n_groups
    t, r = plan.table.cpu(), ref.table.cpu()
    assert t[:4 * ng].tolist() == r[:4 * ng].tolist()
    ent, rent = t[4 * ng:].view(-1, 1 + G + G * S * S), r[4 * ng:].view(-1, 1 + G)
    assert ent[:, :1 + G].tolist() == rent.tolist()
    rank = (torch.cumsum(lay.reshape(-1), 0) - 1).reshape(lay.shape)
    fine = torch.where(lay != 0, rank, torch.full_like(rank, -1))
    tiles = coarse.nonzero()                                         # tile id -> (head, tile row, tile column)
    for e in range(ent.shape[0]):
        for m in range(G):
            tid = int(ent[e, 1 + m])
            got = ent[e, 1 + G + m * S * S:1 + G + (m + 1) * S * S].view(S, S)
            if tid < 0:
                assert bool((got == -1).all())
            else:
                h, tr, tc = tiles[tid].tolist()
                assert got.tolist() == fine[h, tr * S:(tr + 1) * S, tc * S:(tc + 1) * S].tolist()
    assert GroupPlan.build_coarse(random_layout((1, 6, 9), 0.5, 1), 16, by_rows, DEV) is None   # sides must divide by 4


def test_layouts_built_on_the_device_equal_the_host_generators(golden):
    # every generator with device='cuda' against its host form and against the vectors written by the reference's own
    # generators (C++ make_layout and Python _make_layout)
    for c in golden['make_layout_cpp']:
        assert tb.make_layout(*c['args'], device=DEV).cpu().tolist() == c['layout']
    for c in golden['make_layout_py']:
        assert tb.fixed_layout(*c['args'], device=DEV).cpu().tolist() == c['layout']
    for args in [(3, 48, 'fixed', 12, 'unidirectional', 3, 4), (5, 64, 'fixed', 16, 'bidirectional', 4, 2), (2, 7, 'dense', 7, 'unidirectional', 1, 1),
                 (16, 256, 'fixed', 4, 'unidirectional', 1, 1)]:
        dev = tb.fixed_layout(*args, device=DEV)
        assert dev.dtype == torch.int32 and dev.is_cuda
        assert torch.equal(dev.cpu().long(), tb.fixed_layout(*args))
        uni = args[4] == 'unidirectional'
        assert torch.equal(tb.make_layout(*args[:4], uni, *args[5:], device=DEV).cpu().long(), tb.make_layout(*args[:4], uni, *args[5:]))
    for args in [(16, 64, 4, 16, True), (3, 30, 5, 6, False), (2, 8, 2, 3, True), (3, 18, 4, 8, True)]:
        assert torch.equal(tb.sparse_transformer_layout(*args, device=DEV).cpu().long(), tb.sparse_transformer_layout(*args))
    for kw in [dict(seed=0, causal=True), dict(seed=3, causal=False), dict(window=5, num_global=1, num_random=0, seed=1, causal=True)]:
        assert torch.equal(tb.bigbird_layout(4, 64, device=DEV, **kw).cpu().long(), tb.bigbird_layout(4, 64, **kw))
    big = tb.bigbird_layout(12, 256, 3, 2, 3, seed=0, causal=True, device=DEV)
    assert torch.equal(big.cpu().long(), tb.bigbird_layout(12, 256, 3, 2, 3, seed=0, causal=True))


def test_operators_take_a_layout_that_lives_on_the_device():
    # tables built from a device layout are the tables built from its host copy, and the operators give the same results
    from torch_blocksparse.softmax import _sparse_softmax
    from torch_blocksparse.matmul import _sparse_matmul
    lay_d = tb.sparse_transformer_layout(2, 16, 4, 8, True, device=DEV)
    lay_h = lay_d.cpu().long()
    a, _ = _sparse_softmax.make_lut(lay_d, 64, DEV)
    b, _ = _sparse_softmax.make_lut(lay_h, 64, DEV)
    assert torch.equal(a, b)
    for trans in (False, True):
        assert torch.equal(_sparse_matmul.make_dxx_lut(lay_d, 64, 16, trans, DEV)[0], _sparse_matmul.make_dxx_lut(lay_h, 64, 16, trans, DEV)[0])
    q, k, v = [torch.randn(2, 2, 1024, 64, device=DEV, dtype=torch.float16) for _ in range(3)]
    outs = []
    for lay in (lay_d, lay_h):
        sdd, dsd, sm = tb.MatMul(lay, 64, 'sdd', trans_b=True), tb.MatMul(lay, 64, 'dsd'), tb.Softmax(lay, 64)
        outs.append(dsd(sm(sdd(q, k), scale=0.125), v))
    assert torch.equal(outs[0], outs[1])
    # block 16: the plan over 64 x 64 tiles is assembled from the device layout as well
    lay16 = tb.fixed_layout(2, 64, 'fixed', 16, 'unidirectional', 1, 1, device=DEV)
    x = torch.randn(1, int(lay16.sum()), 16, 16, device=DEV, dtype=torch.float16)
    y = torch.randn(1, 2, 1024, 64, device=DEV, dtype=torch.float16)
    assert torch.equal(tb.MatMul(lay16, 16, 'dsd')(x, y), tb.MatMul(lay16.cpu().long(), 16, 'dsd')(x, y))
