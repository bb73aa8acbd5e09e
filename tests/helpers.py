"""Shared test helpers: tolerances (stated here, used everywhere) and layout factories."""
import torch


def assert_close(got, ref, dtype, what=''):
    """Tolerances of the parity bar, against the fp32 dense-masked oracle:
         fp32          : |got - ref| <= 1e-5 * |ref| + 1e-5 * max|ref|   (1e-5 relative; the second term keeps
                         elements that cancel to ~0 from being judged against their own rounding noise)
         fp16 / bf16   : |got - ref| <= 1e-2 * |ref| + 1e-2  (bf16: 2e-2 relative, it has 3 fewer mantissa bits)
    """
    got = got.detach().float().cpu()
    ref = ref.detach().float().cpu()
    assert got.shape == ref.shape, '%s shape %s vs %s' % (what, tuple(got.shape), tuple(ref.shape))
    if dtype == torch.float32:
        tol = 1e-5 * ref.abs() + 1e-5 * ref.abs().max()
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
