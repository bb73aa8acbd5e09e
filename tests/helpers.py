"""Shared test helpers: tolerances (stated here, used everywhere) and layout factories."""
import torch

_TORCH_EMPTY = torch.empty          # the real one (guard_allocations replaces torch.empty while it is active)


# what the comparisons of a test session reached, per (dtype, quantity, form of the bound); printed at the session's end
# (tests/conftest.py)
ACHIEVED = {}


def assert_close(got, ref, dtype, what='', no_cancellation=False, mag=None):
    """Tolerances of the parity bar, against the fp32 dense-masked oracle:
         fp32          : 1e-5 relative to the size of what was summed:
                           mag given (the oracle evaluated on the absolute values of the operands, i.e. sum_k |a_k b_k|
                             for a product): |got - ref| <= 1e-5 * mag, element by element.  Where nothing cancels
                             mag = |ref| and this is the plain relative bound; where terms cancel, an element is judged
                             against the terms it was summed from and not against its own, arbitrarily small, value.
                           no_cancellation (every term of every sum has the same sign: operands drawn from [0, 1), or
                             a softmax's output): |got - ref| <= 1e-5 * |ref|
                           neither (compositions of several operators, the dense utility ops): |got - ref| <=
                             1e-5 * |ref| + 1e-5 * max|ref|
         fp16 / bf16   : |got - ref| <= 1e-2 * |ref| + 1e-2  (bf16: 2e-2 relative, it has 3 fewer mantissa bits)
    """
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    assert got.shape == ref.shape, '%s shape %s vs %s' % (what, tuple(got.shape), tuple(ref.shape))
    if dtype == torch.float32 and mag is not None:
        mag = mag.detach().float().cpu()
        assert mag.shape == ref.shape and bool(((mag >= ref.abs() * (1 - 1e-5)) | ~torch.isfinite(ref)).all()), what + ': magnitude bound below |ref|'
        tol = 1e-5 * mag
    elif dtype == torch.float32:
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
    pure = no_cancellation and mag is None and dtype == torch.float32      # (the 16-bit bounds keep their absolute term)
    form = 'pure' if pure else ('terms' if (mag is not None and dtype == torch.float32) else 'mixed')
    key = (str(dtype).replace('torch.', ''), what.split()[0] if what else '', form)
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
    # the sums of the absolute values of the terms of every output element: the oracle on |a|, |b|, |dc|
    mc, mda, mdb = D.matmul(a.abs(), b.abs(), mode, trans_a, trans_b, lay, block, dc=dc.abs()) if dtype == torch.float32 else (None,) * 3
    op = tb.MatMul(lay, block, mode, trans_a=trans_a, trans_b=trans_b)
    ag = a.to(DEV).requires_grad_(True)
    bg = b.to(DEV).requires_grad_(True)
    tag = '%s ta=%d tb=%d block=%d %s' % (mode, trans_a, trans_b, block, dtype)
    # outputs, gradients and workspaces live inside sentinel-filled buffers: nothing may be written around them
    with guard_allocations(tag):
        c = op(ag, bg)
        if backward:
            c.backward(dc.to(DEV))
    same_sign = dist == 'rand' and scale > 0          # operands and the incoming gradient all lie in [0, 1): nothing cancels
    assert_close(c, rc, dtype, tag + ' c', no_cancellation=same_sign, mag=None if same_sign else mc)
    if not backward:
        return
    assert_close(ag.grad, rda, dtype, tag + ' da', no_cancellation=same_sign, mag=None if same_sign else mda)
    assert_close(bg.grad, rdb, dtype, tag + ' db', no_cancellation=same_sign, mag=None if same_sign else mdb)


def softmax_dx_magnitude(y, dy, layout, block, scale):
    """Sum of the absolute values of the terms of the softmax gradient dx = y * (dy - sum_row(y * dy)) * scale, per
    element: y * (|dy| + sum_row(y * |dy|)) * |scale|, from the oracle's y (sparse format in, sparse format out)."""
    from oracle import dense_oracle as D
    y = y.detach().float().cpu()
    t = y * dy.detach().float().cpu().abs()
    rows = D.sparse_to_dense(t, layout, block).sum(-1, keepdim=True)                      # [Z, H, M, 1]
    rows = D.dense_to_sparse(rows.expand(-1, -1, -1, layout.shape[2] * block), layout, block)
    return (t + y * rows) * abs(scale)


class Guarded:
    """A tensor embedded in a larger allocation filled with a sentinel, the role of the reference's `mempad`
    (tests/utils.py:36-40, used at tests/test_matmul.py:56-57): `t` is the interior view handed to the operator,
    `check()` asserts that the kernels wrote nothing outside it.  The interior starts 256-byte aligned, as a fresh
    allocation would; the guard bands are `pad` elements each (at least 64 KiB)."""

    def __init__(self, shape, dtype, device=DEV, pad=None, fill=None, value=None):
        n = 1
        for d in shape:
            n *= d
        item = _TORCH_EMPTY((), dtype=dtype).element_size()
        pad = pad or max(65536 // item, 1)
        pad = (pad + 255) // 256 * 256
        self.sentinel = -1536.0 if dtype.is_floating_point else 0x5A      # exact in fp16, bf16 and fp32
        self.buf = torch.full((n + 2 * pad,), self.sentinel, dtype=dtype, device=device)
        self.pad, self.n = pad, n
        # an alias of the interior that autograd does not see as a view (an in-place operator may then take it as it
        # takes any fresh tensor)
        self.t = _TORCH_EMPTY(0, dtype=dtype, device=device).set_(self.buf.untyped_storage(), pad, tuple(shape))
        if value is not None:
            self.t.copy_(value)
        elif fill is not None:
            self.t.fill_(fill)

    def check(self, what=''):
        torch.cuda.synchronize()
        lo, hi = self.buf[:self.pad], self.buf[self.pad + self.n:]
        bad = int((lo != self.sentinel).sum()) + int((hi != self.sentinel).sum())
        assert bad == 0, '%s: %d guard elements around the tensor were overwritten' % (what, bad)



class guard_allocations:
    """Context manager: every `torch.empty` / `torch.empty_like` on the GPU made inside it (the operators' outputs,
    gradients and the split chains' workspace are all allocated that way by the Python layer) becomes the interior of a
    sentinel-filled buffer (`Guarded`), and on exit every guard band is checked.  A kernel that writes outside a tensor
    it was given -- which the caching allocator would hide inside a slab -- fails the test that ran it."""

    def __init__(self, what=''):
        self.what, self.made = what, []

    def _guarded(self, shape, dtype, device):
        g = Guarded(tuple(int(d) for d in shape), dtype, device)
        self.made.append(g)
        return g.t

    def __enter__(self):
        self._empty, self._empty_like = torch.empty, torch.empty_like
        outer = self

        def empty(*size, **kw):
            dev = kw.get('device')
            if dev is None or torch.device(dev).type != 'cuda' or any(k not in ('dtype', 'device') for k in kw):
                return outer._empty(*size, **kw)
            shape = size[0] if len(size) == 1 and isinstance(size[0], (tuple, list, torch.Size)) else size
            return outer._guarded(shape, kw.get('dtype') or torch.get_default_dtype(), dev)

        def empty_like(t, **kw):
            if not t.is_cuda or kw or not t.is_contiguous():
                return outer._empty_like(t, **kw)
            return outer._guarded(t.shape, t.dtype, t.device)
        torch.empty, torch.empty_like = empty, empty_like
        return self

    def __exit__(self, exc_type, exc, tb):
        torch.empty, torch.empty_like = self._empty, self._empty_like
        if exc_type is None:
            for g in self.made:
                g.check(self.what)
        self.made = []
        return False
