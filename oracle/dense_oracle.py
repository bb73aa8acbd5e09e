"""TEST INFRASTRUCTURE ONLY: fp32 dense-masked oracle for block-sparse matmul and softmax.

This is the reference's own test oracle restated with vectorised converters: densify the sparse operand,
run the dense PyTorch routine in fp32 on the CPU, mask / re-sparsify (tests/test_matmul.py:10-27,
tests/test_softmax.py:21-34, tests/utils.py:5-25 of the reference).  Only tests, the smoke check and the
benchmark's CPU-baseline leg may import it; the shipped package never does.

Pinned by: round trips of the two converters against brute-force loops on small shapes, and the fact
that everything else is a PyTorch library routine (torch.matmul, torch.softmax, autograd).
"""
import torch


def layout_index(layout):
    """(h, i, j) of every nonzero block in storage order = layout.nonzero() order (tests/utils.py:8-9)."""
    nz = layout.nonzero(as_tuple=False)
    return nz[:, 0], nz[:, 1], nz[:, 2]


def dense_to_sparse(w, layout, block):
    """[Z,H,R*block,C*block] -> [Z,nnz,block,block]  (tests/utils.py:5-13, without the Python loops)."""
    Z, H, M, N = w.shape
    R, C = layout.shape[1], layout.shape[2]
    assert M == R * block and N == C * block and H == layout.shape[0]
    h, i, j = layout_index(layout)
    blocks = w.reshape(Z, H, R, block, C, block).permute(0, 1, 2, 4, 3, 5)  # Z,H,R,C,b,b
    return blocks[:, h, i, j].contiguous()


def sparse_to_dense(w, layout, block, fill=0.0):
    """[Z,nnz,block,block] -> [Z,H,R*block,C*block] with `fill` outside the layout."""
    Z = w.shape[0]
    H, R, C = layout.shape
    h, i, j = layout_index(layout)
    out = torch.full((Z, H, R, C, block, block), fill, dtype=w.dtype, device=w.device)
    out[:, h, i, j] = w
    return out.permute(0, 1, 2, 4, 3, 5).reshape(Z, H, R * block, C * block)


def mask_dense(w, layout, block, fill=0.0):
    """Keep a dense [Z,H,M,N] inside the layout, `fill` elsewhere (tests/utils.py:16-25)."""
    m = layout.to(torch.bool).repeat_interleave(block, 1).repeat_interleave(block, 2)[None]
    return torch.where(m, w, torch.full_like(w, fill))


def matmul(a, b, mode, trans_a, trans_b, layout, block, dc=None):
    """fp32 oracle of MatMul(layout, block, mode, trans_a, trans_b)(a, b)  (tests/test_matmul.py:10-27).

    a, b are given in the op's own formats (sparse operands as [Z,nnz,block,block]); returns c in the op's
    output format and, when dc is given (op output format), also (da, db) in the operands' formats.
    """
    layout = layout.cpu()
    a32 = a.detach().cpu().to(torch.float32)
    b32 = b.detach().cpu().to(torch.float32)
    if mode == 'dsd':
        a32 = sparse_to_dense(a32 if a32.dim() == 4 else a32[None], layout, block)
    if mode == 'dds':
        b32 = sparse_to_dense(b32 if b32.dim() == 4 else b32[None], layout, block)
    while a32.dim() < 4:
        a32 = a32[None]
    while b32.dim() < 4:
        b32 = b32[None]
    a32.requires_grad_(True)
    b32.requires_grad_(True)
    aa = a32.transpose(2, 3) if trans_a else a32
    bb = b32.transpose(2, 3) if trans_b else b32
    y = torch.matmul(aa, bb)
    if mode == 'sdd':
        y = mask_dense(y, layout, block)
    if dc is None:
        with torch.no_grad():
            return dense_to_sparse(y, layout, block) if mode == 'sdd' else y.detach()
    dc32 = dc.detach().cpu().to(torch.float32)
    if mode == 'sdd':
        dc32 = sparse_to_dense(dc32, layout, block)
    y.backward(dc32)
    da, db = a32.grad, b32.grad
    with torch.no_grad():
        c = dense_to_sparse(y, layout, block) if mode == 'sdd' else y.detach()
        if mode == 'dsd':
            da = dense_to_sparse(da, layout, block)
        if mode == 'dds':
            db = dense_to_sparse(db, layout, block)
    return c, da, db


def softmax(x, layout, block, scale=1.0, rpe=None, key_padding_mask=None, attn_mask=None,
            key_padding_mask_mode='add', attn_mask_mode='add', dy=None):
    """fp32 oracle of Softmax(layout, block)(x, scale, rpe, key_padding_mask, attn_mask, modes).

    Semantics (reference softmax.py:74-137): per row over the row's nonzero blocks,
    softmax(x*scale + rpe + kpm + attn), masks in 'mul' mode mean (m == 0) -> -inf else 0.
    x: [Z,nnz,block,block]; rpe: broadcastable [Z,H,L,L]; key_padding_mask: [Z,L]; attn_mask: [L,L].
    Returns y (sparse format) and, when dy is given, dx = dL/dx (sparse format).
    """
    layout = layout.cpu()
    x32 = x.detach().cpu().to(torch.float32).clone().requires_grad_(True)
    xd = sparse_to_dense(x32, layout, block, fill=float('-inf'))
    Z, H, M, N = xd.shape
    s = xd * scale
    if rpe is not None:
        s = s + rpe.detach().cpu().to(torch.float32).expand(Z, H, M, N)
    if key_padding_mask is not None:
        k = key_padding_mask.detach().cpu().to(torch.float32)
        if key_padding_mask_mode == 'mul':
            k = torch.where(k == 0, torch.full_like(k, float('-inf')), torch.zeros_like(k))
        s = s + k[:, None, None, :]
    if attn_mask is not None:
        m = attn_mask.detach().cpu().to(torch.float32)
        if attn_mask_mode == 'mul':
            m = torch.where(m == 0, torch.full_like(m, float('-inf')), torch.zeros_like(m))
        s = s + m[None, None, :, :]
    y = torch.softmax(s, -1)
    ys = dense_to_sparse(y, layout, block)
    if dy is None:
        return ys.detach()
    ys.backward(dy.detach().cpu().to(torch.float32))
    return ys.detach(), x32.grad


def attention(q, k, v, layout, block, scale, rpe=None, key_padding_mask=None, attn_mask=None,
              key_padding_mask_mode='add', attn_mask_mode='mul', do=None):
    """fp32 dense oracle of the chain sdd(q,k^T) -> softmax -> dsd(p,v) (deepspeedsparseselfattention.py:159-165)."""
    q32 = q.detach().cpu().float().requires_grad_(True)
    k32 = k.detach().cpu().float().requires_grad_(True)
    v32 = v.detach().cpu().float().requires_grad_(True)
    s = torch.matmul(q32, k32.transpose(2, 3))
    s = mask_dense(s, layout.cpu(), block, fill=float('-inf')) * scale
    Z, H, M, N = s.shape
    if rpe is not None:
        s = s + rpe.detach().cpu().float().expand(Z, H, M, N)
    if key_padding_mask is not None:
        kp = key_padding_mask.detach().cpu().float()
        if key_padding_mask_mode == 'mul':
            kp = torch.where(kp == 0, torch.full_like(kp, float('-inf')), torch.zeros_like(kp))
        s = s + kp[:, None, None, :]
    if attn_mask is not None:
        m = attn_mask.detach().cpu().float()
        if attn_mask_mode == 'mul':
            m = torch.where(m == 0, torch.full_like(m, float('-inf')), torch.zeros_like(m))
        s = s + m[None, None]
    p = torch.softmax(s, -1)
    o = torch.matmul(p, v32)
    if do is None:
        return o.detach()
    o.backward(do.detach().cpu().float())
    return o.detach(), q32.grad, k32.grad, v32.grad
