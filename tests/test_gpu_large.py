"""GPU: tensors of more than 2^31 elements (the sparse score tensor of a long batch): every offset must be 64-bit.

No oracle fits this size; each launch is independent across the batch, so the last batches of the large run must equal,
bit for bit, the same batches run on their own (the kernels and their tables do not depend on the batch size).
"""
import pytest
import torch

import torch_blocksparse as tb

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def test_attention_chain_with_a_score_tensor_beyond_2_to_the_31_elements():
    H, L, dh, block = 16, 4096, 64, 64
    lay = tb.sparse_transformer_layout(H, L // block, 4, 16, True)
    nnz = int(lay.sum())
    Z = (1 << 31) // (nnz * block * block) + 2                    # 130 batches: 2.18e9 elements, 4.4 GB in fp16
    assert Z * nnz * block * block > (1 << 31)
    sdd = tb.MatMul(lay, block, 'sdd', trans_a=False, trans_b=True)
    dsd = tb.MatMul(lay, block, 'dsd')
    sm = tb.Softmax(lay, block)
    g = torch.Generator(device=DEV).manual_seed(7)
    q, k, v, do = [torch.randn(Z, H, L, dh, device=DEV, dtype=torch.float16, generator=g) for _ in range(4)]
    kpm = torch.zeros(Z, L, device=DEV, dtype=torch.float16)
    kpm[Z - 1, L - 500:] = float('-inf')

    def run(lo, large=False):
        qg, kg, vg = [t[lo:].clone().requires_grad_(True) for t in (q, k, v)]
        w = sdd(qg, kg)
        assert not large or w.numel() > (1 << 31)
        o = dsd(sm(w, scale=0.125, key_padding_mask=kpm[lo:].contiguous()), vg)
        o.backward(do[lo:].contiguous())
        return o.detach(), qg.grad, kg.grad, vg.grad
    big = run(0, large=True)
    tail = [t[Z - 2:].clone() for t in big]
    first = [t[:1].clone() for t in big]
    del big
    torch.cuda.empty_cache()
    small = run(Z - 2)
    for name, a, b in zip(('out', 'dq', 'dk', 'dv'), tail, small):
        assert torch.equal(a, b), 'batches %d.. of the large run differ from the same batches alone: %s' % (Z - 2, name)
    q, k, v, do, kpm = q[:1].clone(), k[:1].clone(), v[:1].clone(), do[:1].clone(), kpm[:1].clone()
    Z = 1
    head = run(0)
    for name, a, b in zip(('out', 'dq', 'dk', 'dv'), first, head):
        assert torch.equal(a, b), 'batch 0 of the large run differs from the same batch alone: %s' % name
