"""Block-sparsity layout generators ([heads, blocks, blocks], 0/1).

`make_layout` follows the reference's C++ helper (csrc/utils.cpp:123-148, exported there as
torch_blocksparse.attention.make_layout); `fixed_layout` follows the Python generator of
DeepSpeedSparseSelfAttention (deepspeedsparseselfattention.py:31-65).  The two agree except for
vertsize > 1, where the C++ one only marks the first column of every vertical stripe.
`bigbird_layout` (sliding window + global + seeded random blocks) and `sparse_transformer_layout` have no
counterpart in the reference.

Every generator takes `device=None`.  Without it the result is the reference's: an int64 tensor on the CPU.  On a GPU
device the layout is built there by the library (csrc/layout.hip; int32, same 0/1 values) and never exists on the
host; MatMul, Softmax and the table builders accept it as it is.
"""
import torch

from . import _lib


def _on_gpu(device):
    return device is not None and torch.device(device).type == 'cuda'


def _device_layout(fn_name, num_heads, num_blocks, device, *args):
    dev = torch.device(device)
    out = torch.empty((num_heads, num_blocks, num_blocks), dtype=torch.int32, device=dev)
    rc = getattr(_lib.load(), fn_name)(_lib.ptr(out), num_heads, num_blocks, *args, _lib.stream_ptr(dev))
    _lib.check(rc, fn_name)
    return out


def _local_windows(num_blocks, block_stride, unidirectional):
    i = torch.arange(num_blocks)
    same = (i[:, None] // block_stride) == (i[None, :] // block_stride)
    if unidirectional:
        same = same & (i[None, :] <= i[:, None])
    return same


def _check_window(num_blocks, block_stride):
    if block_stride <= 0 or num_blocks % block_stride != 0:
        raise ValueError('number of blocks (%d) must be a multiple of the stride in blocks (%d)' % (num_blocks, block_stride))


def make_layout(num_heads, num_blocks, mode, block_stride, unidirectional, numverts, vertsize, device=None):
    """Same arguments and result as the reference's torch_blocksparse_cpp_utils.make_layout."""
    if mode != 'dense':
        _check_window(num_blocks, block_stride)
    if _on_gpu(device):
        return _device_layout('bsp_layout_fixed', num_heads, num_blocks, device, int(mode == 'dense'), int(block_stride),
                              int(bool(unidirectional)), int(numverts), int(vertsize), 0)
    if mode == 'dense':
        return torch.ones((num_heads, num_blocks, num_blocks), dtype=torch.int64)
    layout = torch.zeros((num_heads, num_blocks, num_blocks), dtype=torch.int64)
    local = _local_windows(num_blocks, block_stride, unidirectional)
    rows = torch.arange(num_blocks)
    for h in range(num_heads):
        layout[h][local] = 1
        start = block_stride - (1 + h % numverts) * vertsize          # utils.cpp:139
        for j in range(start, num_blocks, block_stride):
            # utils.cpp:143 advances k by num_blocks, so only k = j (and j + num_blocks, ... < j + vertsize) is set
            for k in range(j, j + vertsize, num_blocks):
                if 0 <= k < num_blocks:
                    sel = rows > j if unidirectional else rows >= 0   # j < end, end = i (utils.cpp:141-142)
                    layout[h, sel, k] = 1
    return layout


def fixed_layout(num_heads, num_blocks, mode, block_stride, attention, numverts, vertsize, device=None):
    """Same arguments and result as DeepSpeedSparseSelfAttention._make_layout of the reference."""
    if (block_stride / vertsize) != (block_stride // vertsize):
        raise ValueError('Number of blocks in a stride window %d must be dividable by vertical block size %d'
                         % (block_stride, vertsize))
    if numverts > (block_stride / vertsize):
        raise ValueError('Number of layout versions %d cannot be larger than blocks in a stride window divided by '
                         'vertical block size %d / %d = %g' % (numverts, block_stride, vertsize, block_stride / vertsize))
    if mode == 'fixed':
        _check_window(num_blocks, block_stride)
    if _on_gpu(device) and mode in ('dense', 'fixed'):
        return _device_layout('bsp_layout_fixed', num_heads, num_blocks, device, int(mode == 'dense'), int(block_stride),
                              int(attention == 'unidirectional'), int(numverts), int(vertsize), 1)
    if mode == 'dense':
        return torch.ones((num_heads, num_blocks, num_blocks), dtype=torch.int64)
    layout = torch.zeros((num_heads, num_blocks, num_blocks), dtype=torch.int64)
    if mode != 'fixed':
        return layout
    uni = attention == 'unidirectional'
    local = _local_windows(num_blocks, block_stride, uni)
    rows = torch.arange(num_blocks)
    for h in range(num_heads):
        layout[h][local] = 1                                          # _set_s1_layout
        start = block_stride - (1 + h % numverts) * vertsize          # _set_s2_layout
        for j in range(start, num_blocks, block_stride):
            sel = rows > j if uni else rows >= 0
            layout[h, sel, j:min(j + vertsize, num_blocks)] = 1
    return layout


def bigbird_layout(num_heads, num_blocks, window=3, num_global=2, num_random=3, seed=0, causal=False, device=None):
    """Sliding window of `window` blocks + `num_global` global block columns (and rows, unless causal) at the start
    + `num_random` random blocks per row from a seeded generator; intersected with the causal mask if asked.  The
    random columns are drawn on the host (a [heads, blocks, num_random] table); on a GPU device only that table is
    uploaded and the layout is assembled there."""
    g = torch.Generator().manual_seed(seed)
    i = torch.arange(num_blocks)
    picks = []
    for h in range(num_heads):
        rnd = torch.rand((num_blocks, num_blocks), generator=g)
        if causal:
            rnd = rnd.masked_fill(i[None, :] > i[:, None], 2.0)
        picks.append(rnd.argsort(dim=1)[:, :num_random])
    if _on_gpu(device):
        cols = torch.stack(picks).to(device=device, dtype=torch.int32).contiguous()
        return _device_layout('bsp_layout_bigbird', num_heads, num_blocks, device, int(window), int(num_global), int(bool(causal)),
                              _lib.ptr(cols), int(num_random))
    half = window // 2
    band = (i[:, None] - i[None, :]).abs() <= half
    if causal:
        band = (i[:, None] - i[None, :] >= 0) & (i[:, None] - i[None, :] < window)
    layout = torch.zeros((num_heads, num_blocks, num_blocks), dtype=torch.int64)
    for h in range(num_heads):
        lay = band.clone()
        lay[:, :num_global] = True
        if not causal:
            lay[:num_global, :] = True
        pick = torch.zeros_like(lay)
        pick.scatter_(1, picks[h], True)
        if causal:
            pick &= i[None, :] <= i[:, None]
        lay |= pick
        if causal:
            lay &= i[None, :] <= i[:, None]
        layout[h] = lay.long()
    return layout


def sparse_transformer_layout(num_heads, num_blocks, local_blocks=4, global_stride=16, causal=True, device=None):
    """Sparse-Transformer "fixed" pattern with separate sizes for the two parts: dense local windows of
    `local_blocks` blocks, plus the last block column of every `global_stride` blocks as a global column
    (seen by the rows after it when causal, by every row otherwise)."""
    if _on_gpu(device):
        return _device_layout('bsp_layout_sparse_transformer', num_heads, num_blocks, device, int(local_blocks), int(global_stride),
                              int(bool(causal)))
    i = torch.arange(num_blocks)
    lay = _local_windows(num_blocks, local_blocks, causal)
    glob = (i[None, :] % global_stride) == (global_stride - 1)
    if causal:
        glob = glob & (i[:, None] > i[None, :])
    lay = (lay | glob).long()
    return lay[None].repeat(num_heads, 1, 1).contiguous()
