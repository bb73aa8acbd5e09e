"""Shared test helpers: tolerances (stated here, used everywhere) and layout factories."""
import torch


# what the comparisons of a test session reached, per (dtype, quantity, form of the bound); printed at the session's end
# (tests/conftest.py)
ACHIEVED = {}


def assert_close(got, ref, dtype, what='', no_cancellation=False):
    """Tolerances of the parity bar, against the fp32 dense-masked oracle:
         fp32          : |got - ref| <= 1e-5 * |ref| + 1e-5 * max|ref|   (1e-5 relative; the second term keeps
                         elements that cancel to ~0 from being judged against their own rounding noise)
                         no_cancellation (every term of every sum has the same sign: operands drawn from [0, 1), or
                         a softmax's output): the pure relative form |got - ref| <= 1e-5 * |ref|
         fp16 / bf16   : |got - ref| <= 1e-2 * |ref| + 1e-2  (bf16: 2e-2 relative, it has 3 fewer mantissa bits)
    """
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    assert got.shape == ref.shape, '%s shape %s vs %s' % (what, tuple(got.shape), tuple(ref.shape))
    if dtype == torch.float32:
        tol = 1e-5 * ref.abs() + (0.0 if no_cancellation else 1e-5 * ref.abs().max())
    elif dtype == torch.float16:
        tol = 1e-2 * ref.abs() + 1e-2
    else:
        tol = 2e-2 * ref.abs() + 2e-2
    err = (got - ref).abs()
    bad = err > tol
    nan_mismatch = torch.isnan(got) != torch.isnan(ref)
    bad = (bad & ~torch.isnan(ref)) | nan_mismatch
    if bad.any():
        i = torch.nonzero(bad)[0].tolist()
        raise AssertionError('%s: %d of %d elements out of tolerance; first at %s got %r ref %r; max err %g'
                             % (what, int(bad.sum()), bad.numel(), i, got[tuple(i)].item(), ref[tuple(i)].item(),
                                err[~torch.isnan(err)].max().item()))
    # what the comparison actually reached: without cancellation the largest relative error, otherwise the largest
    # share of the tolerance that any element used
    ok = torch.isfinite(ref) & torch.isfinite(got)
    pure = no_cancellation and dtype == torch.float32      # (the 16-bit bounds keep their absolute term)
    key = (str(dtype).replace('torch.', ''), what.split()[0] if what else '', 'pure' if pure else 'mixed')
    if pure:
        ok &= ref != 0
        val = float((err[ok] / ref.abs()[ok]).max()) if ok.any() else 0.0
    else:
        val = float((err[ok] / tol[ok]).max()) if ok.any() else 0.0
    ACHIEVED[key] = max(ACHIEVED.get(key, 0.0), val)


def random_layout(shape, density, seed, at_least_one_per_row=False):
    g = torch.Generator().manual_seed(seed)
    lay = (torch.rand(shape, generator=g) < density).long()
    H, R, C = shape
    for h in range(H):
        if lay[h].sum() == 0:
            lay[h, 0, 0] = 1
    if at_least_one_per_row:
        for h in range(H):
            for r in range(R):
                if lay[h, r].sum() == 0:
                    lay[h, r, r % C] = 1
    return lay


DEV = 'cuda'


def operand_shapes(mode, trans_a, trans_b, M, N, K):
    a = (K, M) if trans_a else (M, K)
    b = (N, K) if trans_b else (K, N)
    sp = {'sdd': (M, N), 'dsd': a, 'dds': b}[mode]
    return a, b, sp


def run_matmul_case(mode, trans_a, trans_b, block, dtype, Z=3, H=2, M=256, N=512, K=384, density=0.5, seed=1, layout=None,
             dist='rand', scale=1.0, backward=True):
    """Same protocol as the reference's run_test_mm (tests/test_matmul.py:44-76): y, dx, dw, through MatMul on the GPU,
    against the fp32 dense-masked oracle."""
    import torch_blocksparse as tb
    from oracle import dense_oracle as D
    torch.manual_seed(seed)
    ashape, bshape, sp = operand_shapes(mode, trans_a, trans_b, M, N, K)
    lay = layout if layout is not None else random_layout((H, sp[0] // block, sp[1] // block), density, seed)
    gen = torch.rand if dist == 'rand' else torch.randn
    a = (gen((Z, H) + ashape) * scale).to(dtype)
    b = (gen((Z, H) + bshape) * scale).to(dtype)
    dc = gen((Z, H, M, N)).to(dtype)
    if mode == 'dsd':
        a = D.dense_to_sparse(a, lay, block)
    if mode == 'dds':
        b = D.dense_to_sparse(b, lay, block)
    if mode == 'sdd':
        dc = D.dense_to_sparse(dc, lay, block)
    rc, rda, rdb = D.matmul(a, b, mode, trans_a, trans_b, lay, block, dc=dc)
    op = tb.MatMul(lay, block, mode, trans_a=trans_a, trans_b=trans_b)
    ag = a.to(DEV).requires_grad_(True)
    bg = b.to(DEV).requires_grad_(True)
    c = op(ag, bg)
    tag = '%s ta=%d tb=%d block=%d %s' % (mode, trans_a, trans_b, block, dtype)
    same_sign = dist == 'rand' and scale > 0          # operands and the incoming gradient all lie in [0, 1): nothing cancels
    assert_close(c, rc, dtype, tag + ' c', no_cancellation=same_sign)
    if not backward:
        return
    c.backward(dc.to(DEV))
    assert_close(ag.grad, rda, dtype, tag + ' da', no_cancellation=same_sign)
    assert_close(bg.grad, rdb, dtype, tag + ' db', no_cancellation=same_sign)
