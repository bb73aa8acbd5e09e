"""GPU: the attention modules (sdd -> softmax -> dsd) against dense attention."""
import pytest
import torch

import torch_blocksparse as tb
from oracle import dense_oracle as D
from helpers import assert_close

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def test_multihead_attention_matches_dense_module():
    # the reference's test (tests/test_attention.py:13-49): all-ones layout must reproduce nn.MultiheadAttention
    block, bsz, heads, L, E = 16, 2, 2, 128, 128
    layout = torch.ones(heads, L // block, L // block).long()
    torch.manual_seed(0)
    sparse_mha = tb.MultiheadAttention(E, heads, layout, block).to(DEV)
    torch.manual_seed(0)
    dense_mha = torch.nn.MultiheadAttention(E, heads).to(DEV)
    q = torch.rand(L, bsz, E, device=DEV)
    mul_mask = torch.randint(0, 2, (bsz, L), dtype=torch.bool, device=DEV)
    mul_mask[:, 0] = False
    add_mask = mul_mask.float()
    add_mask[add_mask == 1.] = float('-inf')
    sparse_mha, dense_mha, qh, add_mask = sparse_mha.half(), dense_mha.half(), q.half(), add_mask.half()
    s, _ = sparse_mha(qh, qh, qh, key_padding_mask=add_mask, need_weights=False)
    d, _ = dense_mha(qh, qh, qh, key_padding_mask=mul_mask, need_weights=False)
    assert_close(s, d, torch.float16, 'mha')


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16, torch.float32])
def test_sparse_self_attention_forward_backward(dtype):
    torch.manual_seed(2)
    cfg = tb.SparsityConfig(mode='fixed', block=16, stride=64, attention='unidirectional', numverts=2, vertsize=1)
    mod = tb.SparseSelfAttention(cfg)
    B, H, L, dh = 2, 4, 256, 64
    q, k, v, do = [torch.randn(B, H, L, dh).to(dtype) for _ in range(4)]
    kpm = torch.zeros(B, L)
    kpm[0, 200:] = float('-inf')
    lay = tb.fixed_layout(H, L // 16, 'fixed', 4, 'unidirectional', 2, 1)
    ro, rq, rk, rv = D.attention(q, k, v, lay, 16, dh ** -0.5, key_padding_mask=kpm, do=do)
    qg, kg, vg = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    o = mod(qg, kg, vg, key_padding_mask=kpm.to(DEV))
    o.backward(do.to(DEV))
    assert_close(o, ro, dtype, 'attention out')
    assert_close(qg.grad, rq, dtype, 'dq')
    assert_close(kg.grad, rk, dtype, 'dk')
    assert_close(vg.grad, rv, dtype, 'dv')


def test_key_given_transposed():
    torch.manual_seed(4)
    mod = tb.DeepSpeedSparseSelfAttention(tb.SparsityConfig(block=32, stride=64))
    q, k, v = [torch.randn(1, 2, 128, 32, dtype=torch.float16, device=DEV) for _ in range(3)]
    a = mod(q, k, v)
    b = mod(q, k.transpose(2, 3), v)
    assert torch.equal(a, b)


def test_benchmark_chain_block64_seq4096_small_batch():
    # config 3 at batch 1 and 2 heads: fixed layout (local 4 blocks, global every 16), key padding, scale 1/8
    torch.manual_seed(6)
    B, H, L, dh, block = 1, 2, 4096, 64, 64
    lay = tb.sparse_transformer_layout(H, L // block, 4, 16, True)
    q, k, v, do = [torch.randn(B, H, L, dh).half() for _ in range(4)]
    kpm = torch.zeros(B, L)
    kpm[0, 3500:] = float('-inf')
    ro, rq, rk, rv = D.attention(q, k, v, lay, block, 0.125, key_padding_mask=kpm, do=do)
    sdd = tb.MatMul(lay, block, 'sdd', trans_a=False, trans_b=True)
    dsd = tb.MatMul(lay, block, 'dsd')
    sm = tb.Softmax(lay, block)
    qg, kg, vg = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    o = dsd(sm(sdd(qg, kg), scale=0.125, key_padding_mask=kpm.half().to(DEV)), vg)
    o.backward(do.to(DEV))
    assert_close(o, ro, torch.float16, 'out')
    assert_close(qg.grad, rq, torch.float16, 'dq')
    assert_close(kg.grad, rk, torch.float16, 'dk')
    assert_close(vg.grad, rv, torch.float16, 'dv')


def test_specialised_and_general_kernels_agree(monkeypatch):
    # block 64 / fp16 / head_dim 64 takes specialised kernels; the general ones must give the same numbers
    torch.manual_seed(9)
    B, H, L, dh, block = 2, 2, 1024, 64, 64
    lay = tb.sparse_transformer_layout(H, L // block, 4, 8, True)
    sdd = tb.MatMul(lay, block, 'sdd', trans_a=False, trans_b=True)
    dsd = tb.MatMul(lay, block, 'dsd')
    sm = tb.Softmax(lay, block)
    q, k, v, do = [torch.randn(B, H, L, dh, device=DEV, dtype=torch.float16) for _ in range(4)]

    def run():
        qg, kg, vg = [t.clone().requires_grad_(True) for t in (q, k, v)]
        o = dsd(sm(sdd(qg, kg), scale=0.125), vg)
        o.backward(do)
        return o, qg.grad, kg.grad, vg.grad
    grouped = run()                                   # row-group kernels (default for block 64)
    monkeypatch.setenv('BSP_NO_GROUPS', '1')
    fast = run()                                      # per-block / per-segment specialised kernels
    monkeypatch.setenv('BSP_GENERIC_ONLY', '1')
    general = run()                                   # general LDS-tiled kernels
    for a, b, c, name in zip(grouped, fast, general, ('out', 'dq', 'dk', 'dv')):
        assert_close(a, c.float(), torch.float16, name + ' grouped vs general')
        assert_close(b, c.float(), torch.float16, name + ' specialised vs general')


def test_full_size_properties():
    # config 3 at full size (batch 8, 16 heads): no dense oracle fits in seconds, so check what must hold at any
    # size: every softmax row sums to 1, the chain is linear in v, and a shuffled batch gives shuffled outputs
    torch.manual_seed(8)
    B, H, L, dh, block = 8, 16, 4096, 64, 64
    lay = tb.sparse_transformer_layout(H, L // block, 4, 16, True)
    sdd = tb.MatMul(lay, block, 'sdd', trans_a=False, trans_b=True)
    dsd = tb.MatMul(lay, block, 'dsd')
    sm = tb.Softmax(lay, block)
    q, k, v = [torch.randn(B, H, L, dh, device=DEV, dtype=torch.float16) for _ in range(3)]
    p = sm(sdd(q, k), scale=0.125)
    ones = torch.ones(B, H, L, 64, device=DEV, dtype=torch.float16)
    rows = dsd(p, ones)                       # P @ 1 = row sums
    assert (rows.float() - 1).abs().max() < 5e-3
    o1 = dsd(p, v)
    o2 = dsd(p, 2 * v)
    assert torch.allclose(o2.float(), 2 * o1.float(), atol=1e-3, rtol=1e-3)
    perm = torch.randperm(B, device=DEV)
    p2 = sm(sdd(q[perm].contiguous(), k[perm].contiguous()), scale=0.125)
    assert torch.equal(dsd(p2, v[perm].contiguous()), o1[perm])
