"""GPU: the launch path under HIP graph capture (torch.cuda.graph).

Nothing on the launch path allocates inside the library, synchronises or clears memory with a memset: after a warm-up
step (which builds the tables and the lazily built plans) the whole forward + backward chain can be captured once and
replayed.  Every replay is checked against the eager result for the same inputs, with eager work between the replays.
"""
import pytest
import torch

import torch_blocksparse as tb

pytestmark = pytest.mark.gpu
DEV = 'cuda'


@pytest.mark.parametrize('block,dtype', [(64, torch.float16), (32, torch.bfloat16), (16, torch.float32)])
def test_attention_chain_captured_and_replayed(block, dtype):
    torch.manual_seed(5)
    B, H, L, dh = 2, 3, 512, 64
    lay = tb.sparse_transformer_layout(H, L // block, 128 // block, 256 // block, True)
    sdd = tb.MatMul(lay, block, 'sdd', trans_a=False, trans_b=True)
    dsd = tb.MatMul(lay, block, 'dsd')
    sm = tb.Softmax(lay, block)
    q, k, v, do = [torch.randn(B, H, L, dh, device=DEV, dtype=dtype) for _ in range(4)]
    kpm = torch.zeros(B, L, device=DEV, dtype=dtype)
    kpm[1, L - 100:] = float('-inf')

    def chain(q, k, v, do):
        qg, kg, vg = [t.detach().clone().requires_grad_(True) for t in (q, k, v)]
        o = dsd(sm(sdd(qg, kg), scale=0.125, key_padding_mask=kpm), vg)
        dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do)
        return o.detach(), dq, dk, dv

    # warm-up on a side stream, as graph capture asks for: builds every table and plan the launches need
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            chain(q, k, v, do)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    static_in = [t.clone() for t in (q, k, v, do)]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = chain(*static_in)
    for rep in range(4):
        fresh = [torch.randn_like(t) for t in static_in]          # eager work between the replays
        eager = chain(*fresh)
        torch.cuda.synchronize()
        for s, f in zip(static_in, fresh):
            s.copy_(f)
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(('out', 'dq', 'dk', 'dv'), static_out, eager):
            assert torch.equal(a, b), 'replay %d differs from the eager run: %s (block %d)' % (rep, name, block)


@pytest.mark.parametrize('masked', [False, True])
def test_fused_attention_chain_captured_and_replayed(masked):
    # the call the attention modules make: one fused launch per direction plus the two transposed products
    from torch_blocksparse import attention_core as ac
    torch.manual_seed(6)
    B, H, L, dh = 2, 3, 1024, 64
    lay = tb.sparse_transformer_layout(H, L // 64, 4, 8, True)
    sdd = tb.MatMul(lay, 64, 'sdd', trans_a=False, trans_b=True)
    dsd = tb.MatMul(lay, 64, 'dsd')
    sm = tb.Softmax(lay, 64)
    q, k, v, do = [torch.randn(B, H, L, dh, device=DEV, dtype=torch.float16) for _ in range(4)]
    kpm = torch.zeros(B, L, device=DEV, dtype=torch.float16)
    kpm[1, L - 100:] = float('-inf')
    kw = dict(scale=0.125, key_padding_mask=kpm)
    if masked:
        kw.update(attn_mask=torch.tril(torch.ones(L, L, device=DEV, dtype=torch.float16)), attn_mask_mode='mul',
                  rpe=(0.2 * torch.randn(L, L, device=DEV)).half())
    old = ac.FUSED
    ac.FUSED = True
    try:
        def chain(q, k, v, do):
            qg, kg, vg = [t.detach().clone().requires_grad_(True) for t in (q, k, v)]
            n0 = ac.fused_calls
            o = ac.attention_chain(sdd, sm, dsd, qg, kg, vg, **kw)
            assert ac.fused_calls == n0 + 1
            dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), do)
            return o.detach(), dq, dk, dv

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                chain(q, k, v, do)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        static_in = [t.clone() for t in (q, k, v, do)]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_out = chain(*static_in)
        for rep in range(4):
            fresh = [torch.randn_like(t) for t in static_in]
            eager = chain(*fresh)
            torch.cuda.synchronize()
            for s_, f in zip(static_in, fresh):
                s_.copy_(f)
            graph.replay()
            torch.cuda.synchronize()
            for name, a, b in zip(('out', 'dq', 'dk', 'dv'), static_out, eager):
                assert torch.equal(a, b), 'replay %d differs from the eager run: %s' % (rep, name)
    finally:
        ac.FUSED = old


def test_split_chains_captured_then_a_larger_eager_call_between_replays():
    # A layout with a line of more than 128 blocks: the chain is cut into parts whose fp32 partial tiles live in the
    # plan's workspace, and a captured launch carries that buffer's address.  An eager call with a larger batch between
    # the replays makes the plan take a larger workspace; the one the graph uses must stay alive and untouched by
    # other tensors, so every replay still equals the eager result.
    torch.manual_seed(11)
    n, block, dtype = 300, 64, torch.float16
    lay = torch.zeros(2, n, 4, dtype=torch.int64)
    lay[:, :, 1] = 1
    lay[0, ::7, 0] = 1
    lay[1, ::5, 3] = 1
    op = tb.MatMul(lay, block, 'dsd', trans_a=True)
    nnz = int(lay.sum())
    a = (0.1 * torch.randn(2, nnz, block, block, device=DEV)).to(dtype)
    b = torch.randn(2, 2, n * block, 64, device=DEV, dtype=dtype)
    a_big = (0.1 * torch.randn(5, nnz, block, block, device=DEV)).to(dtype)
    b_big = torch.randn(5, 2, n * block, 128, device=DEV, dtype=dtype)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            op(a, b)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    plan = op.make_lut(dtype, a.device)[0].gplan
    assert plan.n_split == 2
    small_ws = plan._ws
    sa, sb = a.clone(), b.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = op(sa, sb)
    assert plan._ws is small_ws                         # the capture allocated nothing new for the chains
    for rep in range(3):
        big = op(a_big, b_big)                          # larger batch and free dimension: the workspace grows
        assert plan._ws is not small_ws and any(w is small_ws for w in plan._ws_retired)
        filler = [torch.full((small_ws.numel() // 4,), float(rep), device=DEV) for _ in range(4)]   # would land in a freed buffer
        fa, fb = torch.randn_like(sa) * 0.1, torch.randn_like(sb)
        eager = op(fa, fb)
        torch.cuda.synchronize()
        sa.copy_(fa)
        sb.copy_(fb)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), 'replay %d differs from the eager run' % rep
        assert all(bool((f == float(rep)).all()) for f in filler)
        del big, filler


def test_sparse_linear_layer_captured_and_replayed():
    # A block-128 sparse linear layer, forward and backward: the wide dds kernels and the weight gradient as an sdd
    # in parts (fp32 partial blocks in a workspace of the operator, allocated by the warm-up step).  Replays must equal
    # the eager run bit for bit, with eager work and a larger eager call in between.
    torch.manual_seed(21)
    block, tokens, feat = 128, 1024, 512
    lay = (torch.rand(1, feat // block, feat // block) < 0.5).long()
    lay[0, 0, 0] = 1
    lin = tb.Linear(feat, feat, block, lay).to(DEV).half()
    x = torch.randn(tokens, feat, device=DEV, dtype=torch.float16)
    dy = torch.randn(tokens, feat, device=DEV, dtype=torch.float16)

    def step(x, dy):
        xg = x.detach().clone().requires_grad_(True)
        y = lin(xg)
        dx, dw = torch.autograd.grad(y, (xg, lin.weight), dy)
        return y.detach(), dx, dw

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step(x, dy)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    sx, sdy = x.clone(), dy.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = step(sx, sdy)
    big_x = torch.randn(4 * tokens, feat, device=DEV, dtype=torch.float16)
    for rep in range(3):
        step(big_x, torch.randn_like(big_x))                 # a longer reduction: more parts, a larger workspace
        fx, fdy = torch.randn_like(sx), torch.randn_like(sdy)
        eager = step(fx, fdy)
        torch.cuda.synchronize()
        sx.copy_(fx)
        sdy.copy_(fdy)
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(('y', 'dx', 'dw'), out, eager):
            assert torch.equal(a, b), 'replay %d differs from the eager run: %s' % (rep, name)
