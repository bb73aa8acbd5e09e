"""GPU: the benchmark configurations at their full sizes, against the fp32 dense-masked oracle.

The GPU computes the whole problem once; the oracle, which cannot hold a whole configuration, is evaluated on a few
(batch, head) slices chosen to include the first and last batch and head.  Every launch is independent across batch
and heads, so a slice of the full result must equal the oracle on the slice of the inputs.
"""
import pytest
import torch

import torch_blocksparse as tb
from oracle import dense_oracle as D
from helpers import assert_close, random_layout, run_matmul_case as run_case

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def head_blocks(lay, h):
    """Storage range [lo, hi) of the blocks of head h."""
    per_head = lay.reshape(lay.shape[0], -1).sum(1)
    lo = int(per_head[:h].sum())
    return lo, lo + int(per_head[h])


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
