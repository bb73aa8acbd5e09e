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


def test_long_context_bigbird_chain_reduced():
    # config 4 at reduced size: BigBird-style layout (window 3 + 2 global + 3 random blocks, causal), block 64, fp16,
    # additive relative-position embedding given per block pair and expanded to [B, H, L, L] with stride-0 views,
    # causal attention mask in 'mul' mode; forward + backward against the dense oracle
    torch.manual_seed(12)
    B, H, L, dh, block = 2, 3, 1024, 64, 64
    nb = L // block
    lay = tb.bigbird_layout(H, nb, 3, 2, 3, seed=3, causal=True)
    q, k, v, do = [torch.randn(B, H, L, dh).half() for _ in range(4)]
    rpe_blocks = (0.1 * torch.randn(nb)).half()                     # one value per block distance
    dist = (torch.arange(nb)[:, None] - torch.arange(nb)[None, :]).abs()
    rpe_bb = rpe_blocks[dist]                                       # [nb, nb]
    rpe = rpe_bb.repeat_interleave(block, 0).repeat_interleave(block, 1)[None, None].expand(B, H, L, L)   # strides 0, 0
    causal = torch.tril(torch.ones(L, L)).half()
    ro, rq, rk, rv = D.attention(q, k, v, lay, block, 0.125, rpe=rpe, attn_mask=causal, attn_mask_mode='mul', do=do)
    sdd = tb.MatMul(lay, block, 'sdd', trans_a=False, trans_b=True)
    dsd = tb.MatMul(lay, block, 'dsd')
    sm = tb.Softmax(lay, block)
    qg, kg, vg = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    rpe_dev = rpe_bb.to(DEV).repeat_interleave(block, 0).repeat_interleave(block, 1)[None, None].expand(B, H, L, L)
    assert rpe_dev.stride(0) == 0 and rpe_dev.stride(1) == 0
    p = sm(sdd(qg, kg), scale=0.125, rpe=rpe_dev, attn_mask=causal.to(DEV), attn_mask_mode='mul')
    o = dsd(p, vg)
    o.backward(do.to(DEV))
    assert_close(o, ro, torch.float16, 'out')
    assert_close(qg.grad, rq, torch.float16, 'dq')
    assert_close(kg.grad, rk, torch.float16, 'dk')
    assert_close(vg.grad, rv, torch.float16, 'dv')


def test_head_dim_128_and_non_contiguous_inputs():
    # head_dim 128 (two 64-wide tiles, sdd reduction of 128) and q/k/v given as strided views of a packed projection
    torch.manual_seed(13)
    B, H, L, dh, block = 2, 2, 512, 128, 64
    lay = tb.sparse_transformer_layout(H, L // block, 2, 4, True)
    qkv = torch.randn(B, L, 3, H, dh).half()
    q, k, v = [qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3)]          # [B, H, L, dh], not contiguous
    do = torch.randn(B, H, L, dh).half()
    ro, rq, rk, rv = D.attention(q, k, v, lay, block, dh ** -0.5, do=do)
    mod = tb.SparseSelfAttention(tb.SparsityConfig(mode='fixed', block=64, stride=128, attention='unidirectional'))
    lay2 = tb.fixed_layout(H, L // block, 'fixed', 2, 'unidirectional', 1, 1)
    ro2, rq2, rk2, rv2 = D.attention(q, k, v, lay2, block, dh ** -0.5, do=do)
    qkv_dev = qkv.to(DEV).requires_grad_(True)
    qd, kd, vd = [qkv_dev[:, :, i].permute(0, 2, 1, 3) for i in range(3)]
    o = mod(qd, kd, vd)
    o.backward(do.to(DEV))
    assert_close(o, ro2, torch.float16, 'out')
    g = qkv_dev.grad
    assert_close(g[:, :, 0].permute(0, 2, 1, 3), rq2, torch.float16, 'dq')
    assert_close(g[:, :, 1].permute(0, 2, 1, 3), rk2, torch.float16, 'dk')
    assert_close(g[:, :, 2].permute(0, 2, 1, 3), rv2, torch.float16, 'dv')


def test_bench_flag_and_second_stream():
    torch.manual_seed(14)
    lay = tb.sparse_transformer_layout(2, 8, 2, 4, True)
    op = tb.MatMul(lay, 64, 'sdd', trans_b=True, bench=True)
    a, b = [torch.randn(1, 2, 512, 64, device=DEV, dtype=torch.float16) for _ in range(2)]
    c = op(a, b)
    assert op.time_c is not None and op.time_c > 0
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        c2 = tb.MatMul(lay, 64, 'sdd', trans_b=True)(a, b)
    s.synchronize()
    assert torch.equal(c, c2)


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
    from torch_blocksparse import _lib, matmul
    monkeypatch.setattr(matmul, 'KERNEL_FLAGS', _lib.FLAG_NO_GROUPS)
    fast = run()                                      # per-block / per-segment specialised kernels
    monkeypatch.setattr(matmul, 'KERNEL_FLAGS', _lib.FLAG_NO_GROUPS | _lib.FLAG_GENERAL_ONLY)
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


@pytest.mark.parametrize('batch_first', [False, True])
def test_replace_mha_in_a_transformer_encoder_layer(batch_first):
    # replace_mha on a small nn.TransformerEncoderLayer (all-ones layout: the replaced model must reproduce the original),
    # in training mode without dropout so that the layer calls the attention module's forward; with a 0/1 key padding
    # mask ('mul' mode: 0 = padded) and an additive causal mask, forward and backward.  Both models run in fp32 (two
    # fp16 pipelines would differ from each other by their own rounding, amplified by the layer norms); the bound is
    # 1e-4 of the largest reference value, the two models share nothing but the weights.
    import copy
    torch.manual_seed(21)
    E, heads, L, B, block = 128, 2, 128, 3, 32
    dense = torch.nn.TransformerEncoderLayer(E, heads, dim_feedforward=256, dropout=0.0, batch_first=batch_first).to(DEV)
    sparse = copy.deepcopy(dense)
    tb.replace_mha(sparse, torch.ones(heads, L // block, L // block, dtype=torch.int64), block)
    assert isinstance(sparse.self_attn, tb.MultiheadAttention) and sparse.self_attn.batch_first == batch_first
    x = torch.randn((B, L, E) if batch_first else (L, B, E), device=DEV)
    causal = torch.full((L, L), float('-inf'), device=DEV).triu(1)
    pad = torch.zeros(B, L, dtype=torch.bool, device=DEV)
    pad[1, 100:] = True                                   # nn.MultiheadAttention: True = ignore this key
    keep = (~pad).float()                                 # 'mul' mode of the sparse softmax: 0 = ignore
    xd, xs = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    yd = dense(xd, src_mask=causal, src_key_padding_mask=pad)
    ys = sparse(xs, src_mask=causal, src_key_padding_mask=keep)
    g = torch.randn_like(yd)
    yd.backward(g)
    ys.backward(g)
    for name, got, ref in (('output', ys, yd), ('input gradient', xs.grad, xd.grad),
                           ('in_proj gradient', sparse.self_attn.in_proj_weight.grad, dense.self_attn.in_proj_weight.grad),
                           ('out_proj gradient', sparse.self_attn.out_proj.weight.grad, dense.self_attn.out_proj.weight.grad)):
        err = float((got.detach() - ref.detach()).abs().max())
        assert err <= 1e-4 * float(ref.detach().abs().max()), 'encoder layer %s: max err %g' % (name, err)


def test_separate_projection_weights_and_no_bias():
    # multi_head_attention_forward with use_separate_proj_weight (q / k / v weights given one by one) and without
    # projection biases, against torch's own functional form on an all-ones layout
    import torch.nn.functional as F
    torch.manual_seed(22)
    E, heads, L, B, block = 64, 2, 64, 2, 16
    lay = torch.ones(heads, L // block, L // block, dtype=torch.int64)
    x = torch.randn(L, B, E, device=DEV, dtype=torch.float16)
    wq, wk, wv, wo = [(0.1 * torch.randn(E, E, device=DEV)).half() for _ in range(4)]
    ops = (tb.MatMul(lay, block, 'sdd', trans_b=True), tb.MatMul(lay, block, 'dsd'), tb.Softmax(lay, block))
    from torch_blocksparse.attention import multi_head_attention_forward
    got, _ = multi_head_attention_forward(x, x, x, E, heads, None, None, None, None, False, 0.0, wo, None, *ops,
                                          use_separate_proj_weight=True, q_proj_weight=wq, k_proj_weight=wk, v_proj_weight=wv)
    ref, _ = F.multi_head_attention_forward(x, x, x, E, heads, None, None, None, None, False, 0.0, wo, None,
                                            use_separate_proj_weight=True, q_proj_weight=wq, k_proj_weight=wk, v_proj_weight=wv,
                                            need_weights=False)
    assert_close(got, ref.float(), torch.float16, 'separate projection weights')


@pytest.mark.parametrize('bias_kv,zero_attn', [(True, False), (False, True), (True, True)])
def test_extra_key_positions_against_torch(bias_kv, zero_attn):
    # add_bias_kv / add_zero_attn append one key position each, visible to every query.  Against nn.MultiheadAttention
    # itself in fp32 with the same weights: the block layout (banded, with a global first column) is handed to torch as
    # an additive mask, which torch pads with zeros for the appended positions; with a key padding mask, forward and
    # backward.  The sparse module keeps the positions in one more block-column whose padding it hides itself.
    import copy
    torch.manual_seed(41)
    E, heads, L, B, block = 64, 2, 128, 3, 16
    nb = L // block
    lay = torch.zeros(heads, nb, nb, dtype=torch.int64)
    for i in range(nb):
        lay[:, i, max(0, i - 1):i + 1] = 1
    lay[:, :, 0] = 1
    lay[1, 2, 5] = 1
    dense = torch.nn.MultiheadAttention(E, heads, add_bias_kv=bias_kv, add_zero_attn=zero_attn).to(DEV)
    sparse = tb.MultiheadAttention(E, heads, lay, block, add_bias_kv=bias_kv, add_zero_attn=zero_attn,
                                   key_padding_mask_mode='mul', attn_mask_mode='add').to(DEV)
    sparse.load_state_dict(dense.state_dict())
    x = torch.randn(L, B, E, device=DEV)
    pad = torch.zeros(B, L, dtype=torch.bool, device=DEV)
    pad[2, 90:] = True
    outside = (lay == 0).repeat_interleave(block, 1).repeat_interleave(block, 2)          # [heads, L, L]
    layout_mask = torch.zeros(heads, L, L).masked_fill(outside, float('-inf')).to(DEV)
    xd, xs = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    yd, _ = dense(xd, xd, xd, key_padding_mask=pad, attn_mask=layout_mask.repeat(B, 1, 1), need_weights=False)
    ys, _ = sparse(xs, xs, xs, key_padding_mask=(~pad).float())
    g = torch.randn_like(yd)
    yd.backward(g)
    ys.backward(g)
    pairs = [('output', ys, yd), ('input gradient', xs.grad, xd.grad), ('in_proj gradient', sparse.in_proj_weight.grad, dense.in_proj_weight.grad)]
    if bias_kv:
        pairs += [('bias_k gradient', sparse.bias_k.grad, dense.bias_k.grad), ('bias_v gradient', sparse.bias_v.grad, dense.bias_v.grad)]
    for name, got, ref in pairs:
        err = float((got.detach() - ref.detach()).abs().max())
        assert err <= 1e-4 * float(ref.detach().abs().max()), 'extra key positions, %s: max err %g' % (name, err)


def test_multihead_attention_with_dropout():
    # dropout on the attention weights: active in training mode only, scaled so that the expectation is unchanged
    torch.manual_seed(31)
    E, heads, L, B, block = 64, 2, 128, 4, 32
    lay = torch.ones(heads, L // block, L // block, dtype=torch.int64)
    mha = tb.MultiheadAttention(E, heads, lay, block, dropout=0.5).to(DEV).half()
    x = torch.randn(L, B, E, device=DEV, dtype=torch.float16)
    mha.eval()
    ref, _ = mha(x, x, x)
    assert torch.equal(ref, mha(x, x, x)[0])
    mha.train()
    torch.manual_seed(1)
    a, _ = mha(x, x, x)
    torch.manual_seed(1)
    b, _ = mha(x, x, x)
    c, _ = mha(x, x, x)
    assert torch.equal(a, b) and not torch.equal(a, c) and not torch.equal(a, ref)
    # the mean over many masks approaches the result without dropout
    acc = torch.zeros_like(ref, dtype=torch.float32)
    n = 200
    for _ in range(n):
        acc += mha(x, x, x)[0].float()
    err = (acc / n - ref.float()).abs().mean() / ref.float().abs().mean()
    assert err < 0.15, err
    a.sum().backward()
    assert torch.isfinite(mha.in_proj_weight.grad).all()
