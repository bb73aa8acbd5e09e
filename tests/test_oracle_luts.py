"""CPU tests that pin the look-up-table oracle (oracle/lut_oracle.c) before anything is compared with it:
golden vectors produced by the reference itself, hand-derived known answers, closed forms and invariants."""
import os
import sys

import numpy as np
import pytest
import torch

from oracle import lut_oracle as O
from helpers import random_layout

REF_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), 'oracle', '_ref')


def test_sdd_segment_golden(golden):
    for c in golden['sdd_segment']:
        got = O.sdd_segment(golden['layouts'][c['layout']], c['start_width'])
        assert [p for p, _ in got] == [e[0] for e in c['tables']], c['layout']
        for (p, t), e in zip(got, c['tables']):
            assert t.reshape(-1).tolist() == e[1], (c['layout'], c['start_width'], p)


def test_dxx_lut_golden(golden):
    for c in golden['dxx_lut']:
        lut, num_locks, width = O.make_dxx_lut(golden['layouts'][c['layout']], c['block'], c['step'], c['trans'])
        assert (lut.tolist(), num_locks, width) == (c['lut'], c['num_locks'], c['width']), (c['layout'], c['block'], c['step'], c['trans'])


def test_load_balance_golden(golden):
    for c in golden['load_balance']:
        got = O.load_balance(c['sizes'])
        for a, k in zip(got, ['segments', 'column', 'lockid', 'maxid', 'offsets']):
            assert a.tolist() == c[k], (c['sizes'], k)


def test_make_layout_golden(golden):
    for c in golden['make_layout_cpp']:
        assert O.make_layout_cpp(*c['args']).tolist() == c['layout'], c['args']


def test_hand_derived_known_answers():
    lower = np.array([[[1, 0], [1, 1]]])
    full = np.array([[[1, 1], [1, 1]]])
    # softmax table: header (size, offset) per block-row, then (blockid, col, row, head) per block
    lut, maxlut = O.make_softmax_lut(lower)
    assert lut.tolist() == [1, 4, 2, 8, 0, 0, 0, 0, 1, 0, 1, 0, 2, 1, 1, 0] and maxlut == 2
    # dsd table, block 16, step 16, trans: note the zero-length third segment (max row population < 4)
    lut, num_locks, width = O.make_dxx_lut(lower, 16, 16, True)
    assert lut.tolist() == [18, 16, 0, 0, 0, 0, 20, 32, 1, 0, 0, 0, 22, 0, 1, 0, 0, 0, 0, 0, 0, 1, 16, 256, 0, 0]
    assert (num_locks, width) == (1, 3)
    # sdd tables at block 32 (start width 2)
    assert [(p, t.tolist()) for p, t in O.sdd_segment(lower, 2)] == [(1, [[0, 0, 0, 0], [0, 1, 0, 1], [0, 1, 1, 2]])]
    assert [(p, t.tolist()) for p, t in O.sdd_segment(full, 2)] == [(2, [[0, 0, 0, 0], [0, 0, 1, 1], [0, 1, 0, 2], [0, 1, 1, 3]])]


@pytest.mark.parametrize('seed', range(4))
def test_sdd_width1_closed_form(seed):
    # at start width 1 (block 64) the table is layout.nonzero() with its running index
    lay = random_layout((3, 9, 11), 0.4, seed)
    (p, t), = O.sdd_segment(lay.numpy(), 1)
    nz = lay.nonzero()
    assert p == 1 and t[:, :3].tolist() == nz.tolist() and t[:, 3].tolist() == list(range(len(nz)))


@pytest.mark.parametrize('seed', range(6))
def test_sdd_segment_invariants(seed):
    # sparse enough that the reference's packing emits every block exactly once; groups are row x col products
    lay = random_layout((2, 12, 14), 0.35, 100 + seed)
    rank = (torch.cumsum(lay.reshape(-1), 0) - 1).reshape(lay.shape)
    seen = set()
    for p, t in O.sdd_segment(lay.numpy(), 4):
        assert t.shape[0] % (p * p) == 0
        for g in t.reshape(-1, p * p, 4):
            rows, cols = g[:, 1].reshape(p, p), g[:, 2].reshape(p, p)
            assert (rows == rows[:, :1]).all() and (cols == cols[:1, :]).all()
        for h, i, j, b in t.tolist():
            if lay[h, i, j] != 0 and (h, i, j) not in seen:
                assert rank[h, i, j] == b
            seen.add((h, i, j))
    assert {tuple(x) for x in lay.nonzero().tolist()} <= seen


@pytest.mark.parametrize('seed', range(4))
def test_softmax_lut_closed_form(seed):
    lay = random_layout((3, 7, 10), 0.5, 200 + seed)
    lut, maxlut = O.make_softmax_lut(lay.numpy())
    sizes = lay.sum(-1).reshape(-1)
    offs = torch.cumsum(sizes, 0) - sizes
    nz = lay.nonzero()
    header = torch.stack((sizes, offs * 4 + 2 * sizes.numel()), 1).reshape(-1)
    core = torch.stack((torch.arange(len(nz)), nz[:, 2], nz[:, 1], nz[:, 0]), 1).reshape(-1)
    assert lut.tolist() == torch.cat((header, core)).tolist() and maxlut == int(sizes.max())


@pytest.mark.parametrize('block,step', [(16, 16), (32, 8), (64, 16), (128, 16)])
@pytest.mark.parametrize('trans', [False, True])
def test_dxx_lut_walk_invariants(block, step, trans):
    # Walking the table the way the reference kernel does (matmul.py:57-79, 135-148) must visit, for every
    # row/column of the layout, exactly its nonzero blocks in order.
    lay = random_layout((3, 6, 9), 0.45, 300 + block + trans)
    lut, num_locks, width = O.make_dxx_lut(lay.numpy(), block, step, trans)
    div = block // step
    wstep = step if trans else step * block
    nz = lay.nonzero() if trans else lay.transpose(1, 2).nonzero()
    rank = (torch.cumsum(lay.reshape(-1), 0) - 1).reshape(lay.shape)
    visited = {}
    total_len = 0
    for s in range(width):
        off, seglen, col, head, lockid, maxid = lut[6 * s:6 * s + 6].tolist()
        assert lockid == 0 and maxid == 0
        total_len += seglen
        pinc = off
        x, w = None, None
        for k in range(seglen // step):
            dx, dw = int(lut[pinc]), int(lut[pinc + 1])
            if k == 0:
                x, w = dx, dw * block * block         # first pair is absolute (the kernel scales the block index)
            else:
                x, w = x + dx, w + dw
            if k % div == 0:
                visited.setdefault((head, col), []).append((x // block, w // (block * block)))
                assert x % block == 0
            else:
                assert dx == step and dw == wstep
            pinc += 2
    assert total_len == int(lay.sum()) * block
    for h in range(lay.shape[0]):
        lines = lay.shape[1] if trans else lay.shape[2]
        for line in range(lines):
            if trans:
                exp = [(c, int(rank[h, line, c])) for c in range(lay.shape[2]) if lay[h, line, c]]
            else:
                exp = [(r, int(rank[h, r, line])) for r in range(lay.shape[1]) if lay[h, r, line]]
            assert visited.get((h, line), []) == exp
    assert num_locks == 1 and lut[-2:].tolist() == [0, 0]


def test_layout_generators_brute_force():
    # deepspeed-style generator against its definition, written out as loops on a small case
    H, nb, stride, nv, vs = 3, 12, 4, 2, 2
    for attention in ('unidirectional', 'bidirectional'):
        exp = np.zeros((H, nb, nb), dtype=np.int64)
        for h in range(H):
            for i in range(0, nb, stride):
                for j in range(i, i + stride):
                    for k in range(i, (j + 1) if attention == 'unidirectional' else i + stride):
                        exp[h, j, k] = 1
            start = stride - (1 + h % nv) * vs
            for i in range(nb):
                end = i if attention == 'unidirectional' else nb
                for j in range(start, end, stride):
                    for k in range(j, min(j + vs, nb)):
                        exp[h, i, k] = 1
        assert (O.make_layout_py(H, nb, 'fixed', stride, attention, nv, vs) == exp).all()
    assert (O.make_layout_py(2, 4, 'dense', 4, 'unidirectional', 1, 1) == 1).all()


@pytest.mark.skipif(not os.path.isdir(REF_DIR), reason='reference helper not built (oracle/_ref)')
@pytest.mark.parametrize('seed', range(8))
def test_against_compiled_reference(seed):
    sys.path.insert(0, REF_DIR)
    try:
        import torch_blocksparse_cpp_utils as ref
    except ImportError:
        pytest.skip('oracle/_ref present but not importable')
    g = torch.Generator().manual_seed(seed)
    shape = (int(torch.randint(1, 4, (1,), generator=g)), int(torch.randint(1, 20, (1,), generator=g)),
             int(torch.randint(1, 20, (1,), generator=g)))
    lay = random_layout(shape, [0.1, 0.3, 0.5, 0.7, 0.9, 0.95, 0.2, 0.6][seed], seed)
    for sw in (4, 2, 1):
        exp = ref.sdd_segment(lay.to(torch.int32).clone(), sw)
        got = O.sdd_segment(lay.numpy(), sw)
        assert [(p, t.tolist()) for p, t in got] == [(p, t.tolist()) for p, t in exp]
    nb = 4 * int(torch.randint(1, 6, (1,), generator=g))
    for uni in (True, False):
        assert (O.make_layout_cpp(3, nb, 'fixed', 4, uni, 2, 1) == ref.make_layout(3, nb, 'fixed', 4, uni, 2, 1).numpy()).all()


def test_philox_known_answers():
    # Random123's published known-answer vectors for philox4x32-10 (counter, key -> output); they pin the generator
    # behind the dropout mask of the softmax
    from oracle.philox_oracle import philox4x32_10, keep_mask
    kats = [((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
            ((0xffffffff,) * 4, (0xffffffff, 0xffffffff), (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
            ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0), (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1))]
    for ctr, key, want in kats:
        got = philox4x32_10(*[np.array([c], dtype=np.uint64) for c in ctr], *key)
        assert tuple(int(g[0]) for g in got) == want
    # vectorised evaluation = one counter at a time; the mask takes word i % 4 of counter i / 4
    m = keep_mask(1000, 0.25, seed=0x299f31d0a4093822, offset=7)
    w = philox4x32_10(np.array([3], dtype=np.uint64), np.array([0]), 7, 0, 0xa4093822, 0x299f31d0)
    assert [bool(x) for x in m[12:16]] == [((int(v[0]) >> 8) * 2.0 ** -24) >= 0.25 for v in w]
    big = keep_mask(1 << 20, 0.25, seed=12345)
    assert abs(big.mean() - 0.75) < 4 * (0.25 * 0.75 / (1 << 20)) ** 0.5
    assert keep_mask(64, 0.0, seed=1).all()
