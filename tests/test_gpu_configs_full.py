"""GPU: the benchmark configurations at their full sizes, against the fp32 dense-masked oracle.

The GPU computes the whole problem once; the oracle, which cannot hold a whole configuration, is evaluated on a few
(batch, head) slices chosen to include the first and last batch and head.  Every launch is independent across batch
and heads, so a slice of the full result must equal the oracle on the slice of the inputs.
"""
import pytest
import torch

import torch_blocksparse as tb
from oracle import dense_oracle as D
from helpers import assert_close, guard_allocations, random_layout, run_matmul_case as run_case

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def head_blocks(lay, h):
    """Storage range [lo, hi) of the blocks of head h."""
    per_head = lay.reshape(lay.shape[0], -1).sum(1)
    lo = int(per_head[:h].sum())
    return lo, lo + int(per_head[h])


def test_config1_readme_sdd_then_softmax_fp32():
    # README shape: sdd with trans_a, fp32, Z=4, H=2, M=256, N=512, K=384, block 16, operands uniform in [0, 1), layout
    # Bernoulli(0.5) of shape [H, M/16, N/16]; then Softmax(layout, 16) on the sparse result.  1e-5 relative at every
    # stage: (1) the product against the oracle (sums of positive terms: pure relative bound); (2) the softmax kernel
    # against the oracle's softmax of the very logits the GPU produced (pure relative bound); (3) the chain against the
    # oracle's chain.  For (3) the bound has to follow the arithmetic: a softmax turns an ABSOLUTE perturbation d of its
    # logits into a RELATIVE one of its result, |dy/y| <= 2 max|d|, and stage (1) leaves d <= 1e-5 |c| with c ~ K/4 = 96
    # here, so the chain is held to 1e-5 (1 + 2 scale max|c|) relative, with max|c| taken per row of the oracle's logits.
    torch.manual_seed(0)
    Z, H, M, N, K, block = 4, 2, 256, 512, 384, 16
    lay = torch.randint(0, 2, (H, M // block, N // block))
    for h in range(H):
        for r in range(M // block):
            if lay[h, r].sum() == 0:
                lay[h, r, 0] = 1
    a = torch.rand(Z, H, K, M)
    b = torch.rand(Z, H, K, N)
    scale = 1.0                                              # Softmax's default, as in the README
    rc = D.matmul(a, b, 'sdd', True, False, lay, block)
    ry = D.softmax(rc, lay, block, scale=scale)
    sdd = tb.MatMul(lay, block, 'sdd', trans_a=True, trans_b=False)
    sm = tb.Softmax(lay, block)
    with guard_allocations('config 1'):
        c = sdd(a.to(DEV), b.to(DEV))
        c_gpu = c.clone()
        y = sm(c, scale=scale)
    assert y.data_ptr() == c.data_ptr()                      # in place, as the reference
    assert_close(c_gpu, rc, torch.float32, 'config 1 sdd', no_cancellation=True)
    assert_close(y, D.softmax(c_gpu, lay, block, scale=scale), torch.float32, 'config 1 softmax of the GPU logits', no_cancellation=True)
    row_max = D.sparse_to_dense(rc, lay, block).abs().amax(-1, keepdim=True)                  # [Z, H, M, 1]
    row_max = D.dense_to_sparse(row_max.expand(-1, -1, -1, N), lay, block)
    bound = 1e-5 * (1 + 2 * scale * row_max) * ry
    err = (y.cpu() - ry).abs()
    assert bool((err <= bound).all()), 'config 1 chain: max err / bound = %g' % float((err / bound.clamp(min=1e-45)).max())
    # rows of the result sum to one
    sums = D.sparse_to_dense(y.cpu(), lay, block).sum(-1)
    assert float((sums - 1).abs().max()) < 1e-5


def test_config3_sparse_transformer_attention_full_size_with_mask_and_backward():
    # The benchmark configuration itself: batch 8, 16 heads, seq 4096, head_dim 64, block 64, fp16, fixed Sparse-Transformer
    # layout (local window of 4 blocks + one global block per 16, causal), scale 1/8, additive key-padding mask with the
    # last 0-25 % of the keys of every sequence padded (random per sequence), forward and backward.  With batch 8 the
    # launches put one batch on each XCD (z = workgroup index mod 8), the scheduling the benchmark figure relies on.
    # Dense oracle on three (batch, head) slices including the first and the last.
    B, H, L, dh, block = 8, 16, 4096, 64, 64
    lay = tb.sparse_transformer_layout(H, L // block, 4, 16, True)
    g = torch.Generator().manual_seed(33)
    q, k, v, do = [torch.randn(B, H, L, dh, generator=g).half() for _ in range(4)]
    kpm = torch.zeros(B, L)
    padded = torch.randint(0, L // 4 + 1, (B,), generator=g)
    for z in range(B):
        if padded[z] > 0:
            kpm[z, L - int(padded[z]):] = float('-inf')
    sdd = tb.MatMul(lay, block, 'sdd', trans_a=False, trans_b=True)
    dsd = tb.MatMul(lay, block, 'dsd')
    sm = tb.Softmax(lay, block)
    kpm_dev, do_dev = kpm.half().to(DEV), do.to(DEV)

    def chain():
        qg, kg, vg = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
        o = dsd(sm(sdd(qg, kg), scale=0.125, key_padding_mask=kpm_dev), vg)
        o.backward(do_dev)
        torch.cuda.synchronize()
        return [t.detach().cpu() for t in (o, qg.grad, kg.grad, vg.grad)]
    got = chain()                                 # as the benchmark runs it (the softmax gradient computed in place)
    with guard_allocations('config 3'):           # and with every output, gradient and workspace inside guard bands
        guarded = chain()
    for x, y in zip(got, guarded):
        assert torch.equal(x, y)
    for z, h in ((0, 0), (B - 1, H - 1), (int(padded.argmax()), 6)):
        sl = (slice(z, z + 1), slice(h, h + 1))
        ref = D.attention(q[sl], k[sl], v[sl], lay[h:h + 1], block, 0.125, key_padding_mask=kpm[z:z + 1], do=do[sl])
        for name, x, r in zip(('out', 'dq', 'dk', 'dv'), got, ref):
            assert not torch.isnan(r).any()
            assert_close(x[sl], r, torch.float16, 'config 3 z=%d h=%d %s' % (z, h, name))


def test_config2_dsd_dds_all_transpositions_full_size():
    # fp16, Z=8, H=16, M=N=K=2048, block 32, a quarter of the blocks kept (at least one per row); values N(0,1)/K^(1/4)
    # in both operands so that the products are N(0,1)-sized; forward and both gradients
    Z, H, S, block = 8, 16, 2048, 32
    lay = random_layout((H, S // block, S // block), 0.25, 2, at_least_one_per_row=True)
    nnz = int(lay.sum())
    g = torch.Generator().manual_seed(22)
    scale = S ** -0.25
    sp = (torch.randn(Z, nnz, block, block, generator=g) * scale).half()
    dn = (torch.randn(Z, H, S, S, generator=g) * scale).half()
    dc = torch.randn(Z, H, S, S, generator=g).half()
    sp_d, dn_d, dc_d = sp.to(DEV), dn.to(DEV), dc.to(DEV)
    slices = [(0, 0), (Z - 1, H - 1), (3, 7)]
    for mode in ('dsd', 'dds'):
        for ta in (False, True):
            for tb_ in (False, True):
                op = tb.MatMul(lay, block, mode, trans_a=ta, trans_b=tb_)
                a_d = (sp_d if mode == 'dsd' else dn_d).clone().requires_grad_(True)
                b_d = (dn_d if mode == 'dsd' else sp_d).clone().requires_grad_(True)
                c = op(a_d, b_d)
                c.backward(dc_d)
                for z, h in slices:
                    lo, hi = head_blocks(lay, h)
                    sps, dns, dcs = sp[z:z + 1, lo:hi], dn[z:z + 1, h:h + 1], dc[z:z + 1, h:h + 1]
                    a, b = (sps, dns) if mode == 'dsd' else (dns, sps)
                    rc, rda, rdb = D.matmul(a, b, mode, ta, tb_, lay[h:h + 1], block, dc=dcs)
                    tag = 'config 2 %s ta=%d tb=%d z=%d h=%d ' % (mode, ta, tb_, z, h)
                    assert_close(c[z:z + 1, h:h + 1], rc, torch.float16, tag + 'c')
                    ga, gb = a_d.grad, b_d.grad
                    if mode == 'dsd':
                        assert_close(ga[z:z + 1, lo:hi], rda, torch.float16, tag + 'da')
                        assert_close(gb[z:z + 1, h:h + 1], rdb, torch.float16, tag + 'db')
                    else:
                        assert_close(ga[z:z + 1, h:h + 1], rda, torch.float16, tag + 'da')
                        assert_close(gb[z:z + 1, lo:hi], rdb, torch.float16, tag + 'db')
                del a_d, b_d, c


def test_config4_long_context_bigbird_full_size():
    # batch 2, 12 heads, seq 16384, head_dim 64, block 64: 3 sliding-window + 2 global + 3 random blocks per row, causal
    # (about 3 % of the blocks; the two global columns of every head are 256 blocks long: chains, cut into parts).
    # Softmax with an additive relative-position embedding (one value per block distance, expanded to [B, H, L, L] by
    # stride-0 views) and a causal attention mask in 'mul' mode; forward and backward.
    B, H, L, dh, block = 2, 12, 16384, 64, 64
    nb = L // block
    lay = tb.bigbird_layout(H, nb, 3, 2, 3, seed=0, causal=True)
    assert int(lay[:, :, 0].sum()) == H * nb              # the global columns are full
    g = torch.Generator().manual_seed(44)
    q, k, v, do = [torch.randn(B, H, L, dh, generator=g).half() for _ in range(4)]
    rpe_blocks = (0.1 * torch.randn(nb, generator=g)).half()
    dist = (torch.arange(nb)[:, None] - torch.arange(nb)[None, :]).abs()
    rpe_bb = rpe_blocks[dist]
    sdd = tb.MatMul(lay, block, 'sdd', trans_a=False, trans_b=True)
    dsd = tb.MatMul(lay, block, 'dsd')
    sm = tb.Softmax(lay, block)
    qg, kg, vg = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    rpe_dev = rpe_bb.to(DEV).repeat_interleave(block, 0).repeat_interleave(block, 1)[None, None].expand(B, H, L, L)
    causal_dev = torch.tril(torch.ones(L, L, dtype=torch.float16, device=DEV))
    p = sm(sdd(qg, kg), scale=0.125, rpe=rpe_dev, attn_mask=causal_dev, attn_mask_mode='mul')
    o = dsd(p, vg)
    o.backward(do.to(DEV))
    torch.cuda.synchronize()
    got = [t.detach().cpu() for t in (o, qg.grad, kg.grad, vg.grad)]
    del rpe_dev, causal_dev, p, o
    rpe = rpe_bb.float().repeat_interleave(block, 0).repeat_interleave(block, 1)[None, None]
    causal = torch.tril(torch.ones(L, L))
    for z, h in ((0, 0), (B - 1, H - 1), (1, 5)):
        sl = (slice(z, z + 1), slice(h, h + 1))
        ref = D.attention(q[sl], k[sl], v[sl], lay[h:h + 1], block, 0.125, rpe=rpe, attn_mask=causal, attn_mask_mode='mul',
                          do=do[sl])
        for name, x, r in zip(('out', 'dq', 'dk', 'dv'), got, ref):
            assert_close(x[sl], r, torch.float16, 'config 4 z=%d h=%d %s' % (z, h, name))


def test_config5_sparse_linear_layer_full_size():
    # dds with trans_b, fp16: activations [1, 1, 8192 tokens, 4096], weight 4096 x 4096 in blocks of 128, a tenth of them
    # kept, values N(0, 0.02); backward: dsd... the dX product and the sdd product for dW restricted to the layout
    M, K, N, block = 8192, 4096, 4096, 128
    lay = random_layout((1, N // block, K // block), 0.1, 5)        # W stored [N, K]: y = x . W^T
    nnz = int(lay.sum())
    g = torch.Generator().manual_seed(55)
    x = torch.randn(1, 1, M, K, generator=g).half()
    w = (0.02 * torch.randn(1, nnz, block, block, generator=g)).half()
    dy = torch.randn(1, 1, M, N, generator=g).half()
    ry, rdx, rdw = D.matmul(x, w, 'dds', False, True, lay, block, dc=dy)
    op = tb.MatMul(lay, block, 'dds', trans_a=False, trans_b=True)
    xg, wg = x.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    y = op(xg, wg)
    y.backward(dy.to(DEV))
    assert_close(y, ry, torch.float16, 'config 5 y')
    assert_close(xg.grad, rdx, torch.float16, 'config 5 dx')
    assert_close(wg.grad, rdw, torch.float16, 'config 5 dw')


@pytest.mark.parametrize('dtype', [torch.float16, torch.bfloat16])
def test_block64_chains_of_hundreds_of_blocks_split_over_workgroups(dtype):
    # Lines of 264 and 600 blocks of 64: chains cut into 5 and 8 parts, each part a workgroup of its own that leaves an
    # fp32 partial tile in the operator's workspace; a second pass adds them up in part order.  Tall layouts give the chains
    # to the transposed product (block-columns are the lines), their transposes to the plain one; free dimension of one
    # and of two 64-wide tiles; Z = 3; every product runs twice.
    from torch_blocksparse.matmul import GroupPlan
    for n, others in ((264, 7), (600, 3)):
        tall = random_layout((2, n, 1 + others), 0.15, n)
        tall[:, :, 1] = 1
        tall[1, :, 0] = 1                                 # head 1: two chains
        plan = GroupPlan.build(tall, False, DEV, thin_min=GroupPlan.thin_min(tall, False, 64), split_len=GroupPlan.SPLIT_LEN)
        assert plan.n_split == 3
        wide = tall.transpose(1, 2).contiguous()
        for free in (64, 128):
            for rep in range(2):
                run_case('dsd', True, False, 64, dtype, Z=3, H=2, M=(1 + others) * 64, K=n * 64, N=free, layout=tall, seed=n + free,
                         dist='randn', scale=0.1)
                run_case('dsd', False, False, 64, dtype, Z=3, H=2, M=(1 + others) * 64, K=n * 64, N=free, layout=wide, seed=n + free + 1,
                         dist='randn', scale=0.1)
        run_case('dds', False, False, 64, dtype, Z=2, H=2, M=64, K=n * 64, N=(1 + others) * 64, layout=tall, seed=n + 2, dist='randn',
                 scale=0.1)
        # one operator called again and again: its workspace is reused, also by a launch with fewer tiles after one with
        # more; the parts are added in a fixed order, so repeated launches agree bit for bit
        op = tb.MatMul(tall, 64, 'dsd', trans_a=True)
        g = torch.Generator().manual_seed(n)
        a = (0.1 * torch.randn(3, int(tall.sum()), 64, 64, generator=g)).to(dtype).to(DEV)
        b = torch.randn(3, 2, n * 64, 128, generator=g).to(dtype).to(DEV)
        c1, c2 = op(a, b), op(a, b)
        c3 = op(a[:2], b[:2, :, :, :64].contiguous())
        c4 = op(a, b)
        assert torch.equal(c1, c2) and torch.equal(c1, c4) and torch.equal(c3, c1[:2, :, :, :64])
