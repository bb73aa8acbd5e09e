"""CPU tests of the host side: the C-ABI library loads and exports every declared symbol, the layout
generators match the oracle, the dense oracle's converters round-trip, and argument errors are the reference's."""
import os
import re

import numpy as np
import pytest
import torch

import torch_blocksparse as tb
from torch_blocksparse import _lib
from oracle import dense_oracle as D
from oracle import lut_oracle as O
from helpers import random_layout

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, 'include', 'bsp.h')).read()
    declared = set(re.findall(r'\b(bsp_[a-z0-9_]+)\s*\(', header))
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    lib = _lib.load()
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.bsp_version() >= 1
    assert b'multiple of 16' in lib.bsp_strerror(-7)


def test_no_cpu_fallback():
    lay = torch.ones(1, 2, 2, dtype=torch.int64)
    with pytest.raises(_lib.BlocksparseLibraryError):
        tb.MatMul(lay, 16, 'sdd')(torch.zeros(1, 1, 32, 16), torch.zeros(1, 1, 16, 32))
    with pytest.raises(_lib.BlocksparseLibraryError):
        tb.Softmax(lay, 16)(torch.zeros(1, 4, 16, 16))


def test_constructor_errors():
    lay = torch.ones(1, 2, 2, dtype=torch.int64)
    with pytest.raises(NotImplementedError):
        tb.MatMul(lay, 16, 'ssd')
    with pytest.raises(NotImplementedError):
        tb.SparsityConfig(mode='bigbird')
    with pytest.raises(NotImplementedError):
        tb.SparsityConfig(attention='causal')
    with pytest.raises(ValueError):
        tb.Softmax(lay, 16)(torch.zeros(1, 4, 16, 16, dtype=torch.float16), attn_mask=torch.zeros(32, 32))
    with pytest.raises(ValueError):
        tb.Softmax(lay, 16)(torch.zeros(1, 4, 16, 16, dtype=torch.float16), dropout_p=1.0)
    with pytest.raises(ValueError):
        tb.fixed_layout(2, 16, 'fixed', 4, 'unidirectional', 1, 3)
    with pytest.raises(ValueError):
        tb.fixed_layout(2, 16, 'fixed', 4, 'unidirectional', 8, 1)


def test_layout_generators_match_oracle(golden):
    for c in golden['make_layout_cpp']:
        assert tb.make_layout(*c['args']).tolist() == c['layout']
    # vectors written by the reference's own DeepSpeedSparseSelfAttention._make_layout (vertical stripes wider than one
    # block included): they pin the oracle's restatement and the package's generator alike
    for c in golden['make_layout_py']:
        assert O.make_layout_py(*c['args']).tolist() == c['layout']
        assert tb.fixed_layout(*c['args']).tolist() == c['layout']
    for args in [(2, 8, 'fixed', 4, 'unidirectional', 1, 1), (4, 16, 'fixed', 4, 'bidirectional', 2, 2),
                 (4, 16, 'fixed', 8, 'unidirectional', 4, 2), (3, 32, 'fixed', 8, 'bidirectional', 8, 1),
                 (2, 8, 'dense', 4, 'unidirectional', 1, 1)]:
        assert (tb.fixed_layout(*args).numpy() == O.make_layout_py(*args)).all()
        assert (tb.DeepSpeedSparseSelfAttention._make_layout(*args).numpy() == O.make_layout_py(*args)).all()


def test_config3_layout_statistics():
    lay = tb.sparse_transformer_layout(16, 64, 4, 16, True)
    assert lay.shape == (16, 64, 64) and int(lay[0].sum()) == 256
    assert int(lay[0].sum(1).max()) == 7 and int(lay[0].sum(0).max()) == 49
    assert (lay.triu(1) == 0).all()


def test_bigbird_layout():
    a = tb.bigbird_layout(2, 32, 3, 2, 3, seed=5, causal=True)
    b = tb.bigbird_layout(2, 32, 3, 2, 3, seed=5, causal=True)
    assert (a == b).all() and (a.triu(1) == 0).all() and (a[:, :, 0] == 1).all()
    assert int(a.sum(-1).max()) <= 8
    c = tb.bigbird_layout(1, 32, 3, 2, 3, seed=5, causal=False)
    assert (c[0, :2] == 1).all() and (c[0, :, :2] == 1).all()


def test_dense_oracle_converters_round_trip():
    block = 4
    lay = random_layout((2, 3, 5), 0.5, 3)
    w = torch.randn(2, 2, 3 * block, 5 * block)
    sp = D.dense_to_sparse(w, lay, block)
    # brute force, the reference's loops (tests/utils.py:5-13)
    nz = lay.nonzero()
    for z in range(2):
        for p, (h, i, j) in enumerate(nz.tolist()):
            assert torch.equal(sp[z, p], w[z, h, i * block:(i + 1) * block, j * block:(j + 1) * block])
    dn = D.sparse_to_dense(sp, lay, block)
    assert torch.equal(dn, D.mask_dense(w, lay, block))
    assert torch.equal(D.dense_to_sparse(dn, lay, block), sp)


def test_dense_oracle_softmax_properties():
    block = 4
    lay = random_layout((2, 4, 4), 0.6, 9, at_least_one_per_row=True)
    x = torch.randn(2, int(lay.sum()), block, block)
    dy = torch.randn_like(x)
    y, dx = D.softmax(x, lay, block, scale=0.7, dy=dy)
    rows = D.sparse_to_dense(y, lay, block).sum(-1)
    assert torch.allclose(rows, torch.ones_like(rows), atol=1e-6)
    # the gradient of a softmax row sums to zero
    assert D.sparse_to_dense(dx, lay, block).sum(-1).abs().max() < 1e-5


def test_operand_shapes_are_checked_against_the_layout_before_any_launch():
    # The kernels take every address from the tables, so a wrong extent must be a Python error, never a launch.  The
    # checks run before the library is touched: CPU tensors and a stand-in table are enough to reach them.
    from torch_blocksparse.matmul import _sparse_matmul, _check_dense, _check_sparse
    from torch_blocksparse.softmax import _sparse_softmax

    class Table:
        nnz = 5
    fn, spd, block = _sparse_matmul.fn, (2, 3, 4), 16      # layout [2 heads, 3 block-rows, 4 block-cols]
    ok_sparse = torch.zeros(2, 5, 16, 16)
    t = [None]
    # dsd: a sparse [M=48, K=64], b dense [Z, 2, 64, N]
    for bad_b in (torch.zeros(2, 3, 64, 32), torch.zeros(2, 2, 48, 32), torch.zeros(2, 64, 32)):
        with pytest.raises(ValueError):
            fn['dsd'](ok_sparse, bad_b, False, False, False, spd, block, Table(), 1, 7, None, False, t)
    with pytest.raises(ValueError):                        # read transposed, the reduction runs over the 48 rows
        fn['dsd'](ok_sparse, torch.zeros(2, 2, 64, 32), True, False, False, spd, block, Table(), 1, 7, None, False, t)
    for bad_a in (torch.zeros(2, 4, 16, 16), torch.zeros(2, 5, 16, 32), torch.zeros(3, 5, 16, 16), torch.zeros(5, 16)):
        with pytest.raises(ValueError):
            fn['dsd'](bad_a, torch.zeros(2, 2, 64, 32), False, False, False, spd, block, Table(), 1, 7, None, False, t)
    # dds: a dense [Z, 2, M, K=48], b sparse [48, 64]
    with pytest.raises(ValueError):
        fn['dds'](torch.zeros(2, 2, 32, 64), ok_sparse, False, False, False, spd, block, Table(), 1, 7, None, False, t)
    with pytest.raises(ValueError):
        fn['dds'](torch.zeros(2, 1, 32, 48), ok_sparse, False, False, False, spd, block, Table(), 1, 7, None, False, t)
    # sdd: op(a) [48, K], op(b) [K, 64]
    with pytest.raises(ValueError):
        fn['sdd'](torch.zeros(1, 2, 32, 16), torch.zeros(1, 2, 16, 64), False, False, False, spd, block, [], None, [], [], False, t)
    with pytest.raises(ValueError):
        fn['sdd'](torch.zeros(1, 2, 48, 16), torch.zeros(1, 2, 16, 48), False, False, False, spd, block, [], None, [], [], False, t)
    with pytest.raises(ValueError):
        fn['sdd'](torch.zeros(1, 3, 48, 16), torch.zeros(1, 3, 16, 64), False, False, False, spd, block, [], None, [], [], False, t)
    _check_dense('a', torch.zeros(1, 2, 16, 48), 2, 48, None, True)      # the accepted forms raise nothing
    _check_sparse('b', torch.zeros(5, 16, 16), 5, 16, 3)
    # softmax: x [Z, nnz, block, block], key_padding_mask [Z or 1, >= 64], attn_mask >= [48, 64], rpe broadcastable
    x = torch.zeros(2, 5, 16, 16, dtype=torch.float16)
    chk = _sparse_softmax._check_shapes
    chk(x, torch.zeros(2, 48, 64), torch.zeros(1, 64), torch.zeros(48, 64), spd, block, 5)
    for kw in (dict(x=torch.zeros(2, 4, 16, 16)), dict(x=torch.zeros(2, 5, 16, 8)), dict(kpm=torch.zeros(2, 48)),
               dict(kpm=torch.zeros(3, 64)), dict(attn=torch.zeros(32, 64)), dict(attn=torch.zeros(48, 63)),
               dict(rpe=torch.zeros(2, 2, 48, 32)), dict(rpe=torch.zeros(3, 2, 48, 64)), dict(rpe=torch.zeros(2, 3, 48, 64))):
        with pytest.raises(ValueError):
            chk(kw.get('x', x), kw.get('rpe'), kw.get('kpm'), kw.get('attn'), spd, block, 5)


def test_workspace_size_of_split_chains():
    lib = _lib.load()
    assert lib.bsp_xsd_workspace_bytes(0, 64, 8) == 0
    # 3 split chains x 2 tiles x 2 batches = 12 slots of 8 fp32 tiles of 64 x 64
    assert lib.bsp_xsd_workspace_bytes(3, 128, 2) == 12 * 8 * 64 * 64 * 4


def test_private_gradient_detection():
    # the softmax backward may overwrite its incoming gradient only if nobody else holds it: the detector (reference
    # count of the tensor as the autograd engine hands it over, calibrated with a probe graph) on the CPU
    from torch_blocksparse.softmax import _gradient_is_private, _private_use_count
    assert _private_use_count() >= 1
    seen = {}

    class Spy(torch.autograd.Function):
        @staticmethod
        def forward(ctx, t, tag):
            ctx.tag = tag
            return t * 1.0

        @staticmethod
        def backward(ctx, g):
            seen[ctx.tag] = _gradient_is_private(g)
            return g * 1.0, None
    x = torch.ones(4, requires_grad=True)
    w = torch.ones(4, requires_grad=True)
    (Spy.apply(x, 'fresh') * 2.0).sum().backward()                 # gradient made by the multiplication's backward
    g = torch.ones(4)
    Spy.apply(x, 'user').backward(g)                               # the user's own tensor
    (Spy.apply(x, 'shared') + w).backward(torch.ones(4))           # one tensor handed to two branches by the addition
    big = torch.ones(2, 4)
    Spy.apply(x, 'view').backward(big[0])                          # a view of a larger tensor
    g2 = torch.ones(4)
    Spy.apply(x, 'detached').backward(g2.detach())                 # another tensor object over the user's storage: no base,
    Spy.apply(x, 'data').backward(g2.data)                         # few owners of the object, but the memory is shared
    assert seen == {'fresh': True, 'user': False, 'shared': False, 'view': False, 'detached': False, 'data': False}


def test_sdd_long_reduction_branch_raises_on_a_failed_launch(monkeypatch):
    # the block-32 long-reduction sdd goes to the library with the plan alone; a negative status must raise instead of
    # returning the uninitialised output (library mocked: no GPU needed)
    from torch_blocksparse import matmul as M

    class FakeLib:
        def bsp_sdd_matmul(self, *args):
            return -5

        def bsp_strerror(self, code):
            return b'HIP runtime error'
    monkeypatch.setattr(_lib, 'load', lambda: FakeLib())
    monkeypatch.setattr(_lib, 'ptr', lambda t: 0)
    monkeypatch.setattr(_lib, 'stream_ptr', lambda d: 0)
    monkeypatch.setattr(M, '_Timer', lambda bench, device: type('T', (), {'done': lambda self: None})())
    luts = M.SddTables()
    luts.nnz, luts.spdims = 4, (1, 2, 2)
    plan = M.GroupPlan(torch.zeros(8, dtype=torch.int32), 1, 2)
    luts.gplan, luts.gplan_long = plan, plan
    luts.build = lambda: ([], [], [])
    luts.build_long = lambda: plan
    a = torch.zeros(1, 1, 64, 256, dtype=torch.float16)
    b = torch.zeros(1, 1, 256, 64, dtype=torch.float16)
    with pytest.raises(_lib.BlocksparseLibraryError, match='bsp_sdd_matmul'):
        M._sparse_matmul._sdd_matmul(a, b, False, False, False, (1, 2, 2), 32, luts, 1, None, None, False, [None])
    # the sibling branch (plan alone, short reduction) raises the same way
    luts.build_long = None
    a = torch.zeros(1, 1, 64, 64, dtype=torch.float16)
    b = torch.zeros(1, 1, 64, 64, dtype=torch.float16)
    with pytest.raises(_lib.BlocksparseLibraryError, match='bsp_sdd_matmul'):
        M._sparse_matmul._sdd_matmul(a, b, False, False, False, (1, 2, 2), 32, luts, 1, None, None, False, [None])


def test_replace_mha_takes_the_reference_form_with_one_info_argument():
    # replace_mha(model, info) of the reference (attention.py:267-281): info carries layout and block
    import types
    import torch_blocksparse as tb
    block, heads, E, L = 16, 2, 32, 64
    layout = torch.ones(heads, L // block, L // block, dtype=torch.int64)
    for info in (types.SimpleNamespace(layout=layout, block=block), dict(layout=layout, block=block), (layout, block)):
        model = torch.nn.TransformerEncoderLayer(E, heads, dim_feedforward=64, dropout=0.0)
        before = {k: v.clone() for k, v in model.self_attn.state_dict().items()}
        tb.replace_mha(model, info)
        assert isinstance(model.self_attn, tb.MultiheadAttention) and model.self_attn.block == block
        assert torch.equal(model.self_attn.layout, layout)
        for k, v in model.self_attn.state_dict().items():
            assert torch.equal(v, before[k])
    model = torch.nn.TransformerEncoderLayer(E, heads, dim_feedforward=64, dropout=0.0)
    tb.replace_mha(model, layout, block)
    assert isinstance(model.self_attn, tb.MultiheadAttention)
    with pytest.raises(TypeError):
        tb.replace_mha(model, layout)


def test_sdd_in_parts_argument_checks_and_workspace_size():
    # host-side checks of bsp_sdd_matmul_splitk (nothing is launched: every call below is refused before it touches the GPU)
    import ctypes
    lib = _lib.load()
    assert lib.bsp_sdd_splitk_workspace_bytes(1, 102, 1) == 0
    assert lib.bsp_sdd_splitk_workspace_bytes(2, 10, 4) == 2 * 10 * 4 * 128 * 128 * 4
    buf = (ctypes.c_char * 4096)()
    base = (ctypes.addressof(buf) + 255) // 256 * 256
    ptr = ctypes.c_void_p(base)

    def call(dtype=_lib.F16, a=ptr, K=1024, block=128, parts=4, ws=ptr, ws_bytes=1 << 40, lda=1024, flags=0):
        return lib.bsp_sdd_matmul_splitk(dtype, a, ptr, ptr, 1, 0, 1, K, 0, 0, lda, 0, 0, 1024, 0, block, ptr, None, 5, parts, ws, ws_bytes, flags, None)
    assert call(a=None) == -1 and call(parts=0) == -1 and call(parts=65) == -1 and call(lda=1021) == -1       # BSP_ERR_ARG
    assert call(block=64) == _lib.ERR_UNSUPPORTED and call(dtype=_lib.F32) == _lib.ERR_UNSUPPORTED
    assert call(K=1000) == _lib.ERR_K_MULTIPLE and call(K=1040) == _lib.ERR_UNSUPPORTED                         # 16 | K, 32 | K
    assert call(flags=_lib.FLAG_GENERAL_ONLY) == _lib.ERR_UNSUPPORTED and call(flags=_lib.FLAG_NO_WIDE) == _lib.ERR_UNSUPPORTED
    assert call(ws=None) == -1 and call(ws_bytes=1024) == _lib.ERR_CAPACITY
