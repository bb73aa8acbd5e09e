"""The chain scores -> softmax -> context of the attention modules, in one launch per direction where that is possible.

The reference's modules call three operators, sparse_dot_sdd_nt(q, k), sparse_softmax(...), sparse_dot_dsd_nn(p, v)
(deepspeedsparseselfattention.py:152-157; attention.py:190-202).  `attention_chain` takes the same three operator
objects and the same arguments and returns the same context tensor; when the operators are this package's, built on
one layout with blocks of 16, 32 or 64, and the tensors are fp16 / bf16 with a head dimension of 64 or 128, it runs the fused
kernels (bsp_attention_fwd / bsp_attention_bwd) instead: the scores stay in registers between the three steps.
In every other case, and with FUSED = False, it calls the three operators one after the other.
"""
import ctypes
import os

import torch

from . import _lib
from .matmul import MatMul
from .softmax import Softmax, _sparse_softmax

FUSED = os.environ.get('BSP_FUSED_ATTENTION', '1') != '0'
MAX_ROW_BLOCKS = 8          # BSP_ATTENTION_MAX_ROW_BLOCKS: longer rows are streamed (the library decides)
fused_calls = 0             # forward calls that took the fused kernels; tests read it
# dk and dv from the column kernel (bsp_attention_bwd_kv), which computes the softmax gradient again instead of reading it;
# False: the row kernel stores the gradient and the two products are ordinary dsd operators
FUSED_KV = os.environ.get('BSP_FUSED_ATTENTION_KV', '1') != '0'




class _GatheredTiles:
    """64 x 64 tiles over a layout of small blocks (S = 64 / block a side).  A *line* of tiles is S consecutive block-rows;
    a tile takes the line's S block-rows and S block-columns gathered from anywhere in the line: the columns in which
    any of the line's block-rows holds a block, in ascending order, S per tile.  (Tiles cut from a fixed grid would be
    mostly holes wherever the layout has single block-columns, like the global columns of the 'fixed' layouts: a
    kernel that works on whole tiles then does S times the work.)
    sizes / starts: tiles per line and the line's first tile, lines in (head, line) order; cols [tiles, S]: the
    block-columns of a tile (slots past the end of a line repeat the tile's first column); ids [tiles, S, S]: the id of
    the block at (block-row i of the line, gathered column g), -1 where the layout has none or the slot is padding."""

    def __init__(self, lay, ids, S):
        H, R, C = lay.shape
        L = R // S
        pres = lay.reshape(H, L, S, C).any(2)
        n = pres.sum(-1).flatten()
        self.sizes = (n + S - 1) // S
        self.starts = torch.cumsum(self.sizes, 0) - self.sizes
        self.n_tiles = int(self.sizes.sum())
        h, t, c = pres.nonzero().unbind(1)
        line = h * L + t
        rank = torch.arange(c.numel()) - (torch.cumsum(n, 0) - n)[line]
        tile, slot = self.starts[line] + rank // S, rank % S
        cols = torch.full((self.n_tiles, S), -1, dtype=torch.int64)
        cols[tile, slot] = c
        self.cols = torch.where(cols < 0, cols[:, :1], cols)
        self.ids = torch.full((self.n_tiles, S, S), -1, dtype=ids.dtype)
        for i in range(S):
            self.ids[tile, i, slot] = ids[h, t * S + i, c]
        self.lines, self.heads = L, H

    def entries(self, transposed_ids=False):
        """per tile 8 + S * S ints: (tile, 0, line, head, then the tile's block-columns, the last repeated up to four, then
        the ids of its blocks, [block-row of the line][gathered block-column], or the other way round)"""
        t = torch.arange(self.n_tiles)
        line = torch.repeat_interleave(torch.arange(self.heads * self.lines), self.sizes)
        cols = self.cols if self.cols.size(1) == 4 else torch.cat((self.cols, self.cols[:, -1:].expand(-1, 4 - self.cols.size(1))), 1)
        ids = self.ids.transpose(1, 2) if transposed_ids else self.ids
        return torch.cat((torch.stack((t, torch.zeros_like(t), line % self.lines, line // self.lines), 1), cols,
                          ids.reshape(self.n_tiles, -1).to(torch.int64)), 1)


KV_PART_BLOCKS = 16         # columns of more blocks than this (and than twice the average column) are computed in parts of about this size


class _ColumnTable:
    """The tables of the column kernel: the layout read along columns, cut into work items.
    items: per item twelve ints (entries, offset of its entries, head, column, slot of its partial sums or -1, 0, 0, 0, then
    the column's block-columns, the last repeated up to four), then the entries, a column's by row.  Blocks of 64: a
    column is a block-column, an entry (id, row, column, head); the ids are the positions in the row-major order of the
    nonzero blocks, as everywhere.  Smaller blocks: a column is S block-columns (the long ones of a head together, the others
    with their neighbours), its entries the tiles
    of _GatheredTiles over the transposed layout (S block-rows gathered per tile): 8 + S * S ints, the last S * S the ids
    of the tile's blocks, [gathered block-row][block-column of the group].  A column of more than `part`
    entries is cut into parts of near-equal size, each with a slot; split: per such column eight ints (head, column,
    first slot, parts, then its block-columns)."""

    def __init__(self, layout, device, part=None, S=1, ids=None):
        lay = (layout != 0).cpu()
        H, R, C = lay.shape
        if S == 1:
            h, r, c = lay.nonzero().unbind(1)
            col = h * C + c
            order = torch.argsort(col * R + r)
            sizes = torch.bincount(col, minlength=H * C)
            starts = torch.cumsum(sizes, 0) - sizes
            entries = torch.stack((order, r[order], c[order], h[order]), 1)
            groups = torch.arange(H * C).reshape(H * C, 1) % C
        else:
            # a column of tiles: S block-columns whose blocks lie in the same block-rows as far as possible, so that the
            # block-rows gathered into a tile hold blocks in most of them: first the long block-columns of the head (more
            # than four times the median: the global columns of a layout), longest first, then the others as they lie
            # (neighbours share their rows in banded layouts)
            layT, idsT = lay.transpose(1, 2), ids.transpose(1, 2)
            length = layT.sum(-1)                                                         # [H, C]
            is_long = length > 4 * length.float().median(dim=1, keepdim=True).values.clamp(min=1)
            key = torch.where(is_long, -length.double() - 2.0 * R, torch.arange(C, dtype=torch.float64)[None].expand_as(length))
            order = torch.argsort(key, dim=1, stable=True)                                # [H, C]
            pick = order[:, :, None].expand(-1, -1, R)
            g = _GatheredTiles(torch.gather(layT, 1, pick), torch.gather(idsT, 1, pick), S)
            C = C // S
            # an entry carries the ids of its tile's blocks, [gathered block-row][block-column of the group]
            sizes, starts, entries = g.sizes, g.starts, g.entries(transposed_ids=True)
            groups = order.reshape(H * C, S)
        groups = torch.cat((groups, groups[:, -1:].expand(-1, 4 - groups.size(1))), 1) if groups.size(1) < 4 else groups
        if part is None:
            # only columns that stand out are cut (every part costs a slot written and read): those of more than twice the
            # average length
            part = max(KV_PART_BLOCKS, -(-2 * int(sizes.sum()) // max(1, H * C)))
        parts = torch.clamp((sizes + part - 1) // part, min=1)
        first_item = torch.cumsum(parts, 0) - parts
        item_col = torch.repeat_interleave(torch.arange(H * C), parts)
        n_items = int(item_col.numel())
        k = torch.arange(n_items) - first_item[item_col]
        base, rem = sizes[item_col] // parts[item_col], sizes[item_col] % parts[item_col]
        count = base + (k < rem).long()
        begin = starts[item_col] + k * base + torch.minimum(k, rem)
        is_part = parts[item_col] > 1
        slot = torch.where(is_part, torch.cumsum(is_part.long(), 0) - 1, torch.full_like(count, -1))
        zero = torch.zeros_like(count)
        header = torch.cat((torch.stack((count, 12 * n_items + entries.size(1) * begin, item_col // C, item_col % C, slot, zero, zero, zero), 1),
                            groups[item_col]), 1).reshape(-1)
        self.items = torch.cat((header, entries.reshape(-1))).to(torch.int32).to(device)
        self.n_items = n_items
        self.columns = C
        self.n_slots = int(is_part.sum())
        long_cols = (parts > 1).nonzero().flatten()
        self.n_split = int(long_cols.numel())
        self.split = None
        if self.n_split:
            self.split = torch.cat((torch.stack((long_cols // C, long_cols % C, slot[first_item[long_cols]], parts[long_cols]), 1),
                                    groups[long_cols]), 1).reshape(-1).to(torch.int32).to(device)


def _vec_ok(t):
    """16-byte vector accesses: unit inner stride, every other stride a multiple of 8 elements, aligned base."""
    return t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in t.stride()[:-1])


def _vec(t):
    return t if _vec_ok(t) else t.contiguous()


class AttentionCore:
    """What the fused kernels need beside the tensors: the softmax table of the layout (for blocks of 16 or 32: the table
    of its 64 x 64 tiles with gathered block-columns and the ids of each tile's blocks), the tables of the column
    kernel, and the two products that are ordinary operators in the backward pass when the column kernel is not used
    (dv = p^T . do and dk = ds^T . q)."""

    def __init__(self, layout, block, softmax=None):
        self.layout = layout
        self.block = block
        self.spdims = tuple(layout.shape)
        self.softmax = softmax if softmax is not None else Softmax(layout, block)
        self.dsd_tn = MatMul(layout, block, 'dsd', trans_a=True, trans_b=False)
        self.nnz = None
        self._tables = dict()

    def blocks(self):
        if self.nnz is None:
            self.nnz = int((self.layout != 0).sum())
        return self.nnz

    def tables(self, device):
        """(table, longest row, None, rows of the table's layout, present blocks per present tile as a share,
        tables of the column kernel) on `device`, or None when the layout does not divide into 64 x 64 tiles."""
        key = str(device)
        if key not in self._tables:
            S = 64 // self.block
            H, R, C = self.spdims
            if S == 1:
                lut, maxlut = self.softmax.make_lut(device)
                self._tables[key] = (lut, maxlut, None, R, 1., _ColumnTable(self.layout, device))
            elif R % S or C % S:
                self._tables[key] = None
            else:
                # tiles of 64 x 64 with gathered block-columns (rows: forward and the row kernel of the backward pass) and with
                # gathered block-rows (the column kernel): each view has its own tiles; p lives in the small blocks either way
                lay = (self.layout != 0).cpu()
                ids = torch.full(lay.shape, -1, dtype=torch.int32)
                ids[lay] = torch.arange(int(lay.sum()), dtype=torch.int32)
                g = _GatheredTiles(lay, ids, S)
                header = torch.stack((g.sizes, 2 * g.sizes.numel() + (8 + S * S) * g.starts), 1).reshape(-1)
                lut = torch.cat((header, g.entries().reshape(-1))).to(torch.int32).to(device)
                maxlut = int(g.sizes.max()) if g.n_tiles else 0
                ct = _ColumnTable(self.layout, device, S=S, ids=ids)
                self._tables[key] = (lut, maxlut, None, R // S, self.blocks() / max(1, g.n_tiles * S * S), ct)
        return self._tables[key]

    def usable(self, q, k, v, dropout_p=0.):
        """Can this call take the fused kernels?  (Shapes that do not fit the layout are left to the operators, which
        raise the reference's errors.)"""
        if not FUSED or self.block not in (16, 32, 64) or dropout_p:
            return False
        if not (q.is_cuda and q.dtype in (torch.float16, torch.bfloat16) and k.dtype == q.dtype and v.dtype == q.dtype):
            return False
        if q.dim() != 4 or k.dim() != 4 or v.dim() != 4 or q.size(3) not in (64, 128):
            return False
        H, R, C = self.spdims
        Z, D, b = q.size(0), q.size(3), self.block
        if tuple(q.shape) != (Z, H, R * b, D) or tuple(k.shape) != (Z, H, C * b, D) or tuple(v.shape) != (Z, H, C * b, D):
            return False
        t = self.tables(q.device)
        if t is None or t[1] <= 0:
            return False
        return t[1] * 64 < 32768                           # the softmax operator's bound on a row (softmax.py:225-227)

    def __call__(self, q, k, v, scale=1., rpe=None, key_padding_mask=None, attn_mask=None,
                 key_padding_mask_mode='add', attn_mask_mode='add'):
        for name, m in (('relative position embedding', rpe), ('Attention mask', attn_mask), ('Key padding mask', key_padding_mask)):
            if m is not None and m.dtype != q.dtype:      # softmax.py:348-353
                raise ValueError('%s must be %s' % (name, q.dtype))
        lut, maxlut, _, rows = self.tables(q.device)[:4]
        # p is kept for the backward pass; a forward pass that no backward pass can follow does not store it
        keep_p = torch.is_grad_enabled() and (q.requires_grad or k.requires_grad or v.requires_grad)
        return _attention_core.apply(q, k, v, float(scale), rpe, key_padding_mask, attn_mask, key_padding_mask_mode,
                                     attn_mask_mode, self, lut, maxlut, keep_p, rows)


class _attention_core(torch.autograd.Function):

    @staticmethod
    def forward(ctx, q, k, v, scale, rpe, key_padding_mask, attn_mask, kp_mask_mode, attn_mask_mode, core, lut, maxlut, keep_p, rows):
        global fused_calls
        H, R, C = core.spdims
        Z, D, block = q.size(0), q.size(3), core.block
        nnz = core.blocks()
        # the masks against the layout, exactly as the softmax operator checks them (it takes every address from the table)
        if rpe is not None or key_padding_mask is not None or attn_mask is not None:
            _sparse_softmax._check_shapes(torch.empty((Z, nnz, block, block), device='meta'), rpe, key_padding_mask, attn_mask, core.spdims, block, nnz)
        q, k, v = _vec(q), _vec(k), _vec(v)
        null = ctypes.c_void_p(0)
        rpe_args = (null, 0, 0, 0)
        if rpe is not None:                                # element (z, h, r, c), softmax.py:50-55, 265
            while rpe.dim() < 4:
                rpe = rpe.unsqueeze(0)
            rpe = _sparse_softmax._strided16(rpe.expand(Z, H, rpe.size(2), rpe.size(3)), 'rpe')
            rpe_args = (_lib.ptr(rpe), rpe.stride(0), rpe.stride(1), rpe.stride(2))
        kpm_args = (null, 0)
        if key_padding_mask is not None:                   # element (z, c), softmax.py:60-62, 274
            key_padding_mask = _sparse_softmax._strided16(key_padding_mask, 'key_padding_mask')
            kpm_args = (_lib.ptr(key_padding_mask), key_padding_mask.stride(0) if key_padding_mask.size(0) > 1 else 0)
        attn_args = (null, 0)
        if attn_mask is not None:                          # element (r, c), softmax.py:67-70, 283
            attn_mask = _sparse_softmax._strided16(attn_mask, 'attn_mask')
            attn_args = (_lib.ptr(attn_mask), attn_mask.stride(0))
        p = torch.empty((Z, nnz, block, block), dtype=q.dtype, device=q.device) if keep_p else None
        o = torch.empty((Z, H, R * block, D), dtype=q.dtype, device=q.device)
        rc = _lib.load().bsp_attention_fwd(
            _lib.DTYPES[q.dtype], _lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.ptr(p), _lib.ptr(o), Z, H, rows, D,
            q.stride(0), q.stride(1), q.stride(2), k.stride(0), k.stride(1), k.stride(2), v.stride(0), v.stride(1), v.stride(2),
            o.stride(0), o.stride(1), o.stride(2), p.stride(0) if keep_p else 0, block, scale, _lib.ptr(lut), maxlut,
            rpe_args[0], rpe_args[1], rpe_args[2], rpe_args[3], kpm_args[0], kpm_args[1], int(kp_mask_mode == 'mul'),
            attn_args[0], attn_args[1], int(attn_mask_mode == 'mul'), _lib.stream_ptr(q.device))
        _lib.check(rc, 'bsp_attention_fwd')
        fused_calls += 1
        ctx.save_for_backward(q, k, v, p, o, lut)
        ctx.core, ctx.scale, ctx.maxlut, ctx.rows = core, scale, maxlut, rows
        ctx.columns = core.tables(q.device)[5]
        return o

    @staticmethod
    def rows_kernel(ctx, do, ds, delta):
        """dq; with it the softmax gradient ds (if a tensor is given) and / or the rows' sums delta = sum_d do . o"""
        q, k, v, p, o, lut = ctx.saved_tensors
        core = ctx.core
        Z, H, D = q.size(0), q.size(1), q.size(3)
        dq = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        rc = _lib.load().bsp_attention_bwd(
            _lib.DTYPES[q.dtype], _lib.ptr(do), _lib.ptr(v), _lib.ptr(k), _lib.ptr(p), _lib.ptr(o), _lib.ptr(ds), _lib.ptr(dq), Z, H, ctx.rows, D,
            do.stride(0), do.stride(1), do.stride(2), v.stride(0), v.stride(1), v.stride(2), k.stride(0), k.stride(1), k.stride(2),
            o.stride(0), o.stride(1), o.stride(2), dq.stride(0), dq.stride(1), dq.stride(2), p.stride(0), ds.stride(0) if ds is not None else 0,
            core.block, ctx.scale, _lib.ptr(lut), ctx.maxlut, _lib.ptr(delta), delta.stride(1) if delta is not None else 0,
            _lib.stream_ptr(q.device))
        _lib.check(rc, 'bsp_attention_bwd')
        return dq

    @staticmethod
    def columns_kernel(ctx, do, delta):
        """dk and dv, the softmax gradient computed again from p and delta"""
        q, k, v, p, o, lut = ctx.saved_tensors
        Z, H, D = q.size(0), q.size(1), q.size(3)
        ct = ctx.columns
        dk = torch.empty(k.shape, dtype=k.dtype, device=k.device)
        dv = torch.empty(v.shape, dtype=v.dtype, device=v.device)
        partial = torch.empty((Z, ct.n_slots, 2, 64, D), dtype=torch.float32, device=q.device) if ct.n_slots else None
        rc = _lib.load().bsp_attention_bwd_kv(
            _lib.DTYPES[q.dtype], _lib.ptr(do), _lib.ptr(q), _lib.ptr(v), _lib.ptr(p), _lib.ptr(delta), _lib.ptr(dk), _lib.ptr(dv), Z, H, ct.columns, D,
            do.stride(0), do.stride(1), do.stride(2), q.stride(0), q.stride(1), q.stride(2), v.stride(0), v.stride(1), v.stride(2),
            dk.stride(0), dk.stride(1), dk.stride(2), dv.stride(0), dv.stride(1), dv.stride(2), p.stride(0), delta.stride(1),
            ctx.core.block, ctx.scale, _lib.ptr(ct.items), ct.n_items, _lib.ptr(partial), ct.n_slots, _lib.ptr(ct.split), ct.n_split,
            _lib.stream_ptr(q.device))
        _lib.check(rc, 'bsp_attention_bwd_kv')
        return dk, dv

    @staticmethod
    def backward(ctx, do):
        q, k, v, p, o, lut = ctx.saved_tensors
        core = ctx.core
        do = _vec(do)
        need_q, need_k, need_v = ctx.needs_input_grad[:3]
        dq = dk = dv = None
        if need_k and FUSED_KV:
            # two launches: rows (dq, delta), then columns (dk and dv)
            delta = torch.empty((q.size(0), q.size(1), ctx.rows * 64), dtype=torch.float32, device=q.device)
            dq = _attention_core.rows_kernel(ctx, do, None, delta)
            dk, dv = _attention_core.columns_kernel(ctx, do, delta)
        else:
            if need_v:
                dv = core.dsd_tn(p, do)                    # p^T . do, as the dsd operator's backward does (matmul.py:598-601)
            if need_k:
                ds = torch.empty_like(p)
                dq = _attention_core.rows_kernel(ctx, do, ds, None)
                dk = core.dsd_tn(ds, q)                    # ds^T . q (matmul.py:598-601 of the sdd operator)
            elif need_q:
                dq = _attention_core.rows_kernel(ctx, do, None, None)
        return (dq if need_q else None, dk, dv if need_v else None) + (None,) * 11


def _core_for(sdd_nt, softmax, dsd_nn):
    """The fused core that stands for this triple of operators, or None when they are not such a triple."""
    if not (isinstance(sdd_nt, MatMul) and isinstance(dsd_nn, MatMul) and isinstance(softmax, Softmax)):
        return None
    core = getattr(softmax, '_attention_core', None)
    if core is not None and core[0] is sdd_nt and core[1] is dsd_nn:
        return core[2]
    ok = (sdd_nt.mode == 'sdd' and not sdd_nt.trans_a and sdd_nt.trans_b and dsd_nn.mode == 'dsd' and not dsd_nn.trans_a
          and not dsd_nn.trans_b and sdd_nt.block == softmax.block == dsd_nn.block and softmax.block in (16, 32, 64))
    if ok:
        for other in (sdd_nt.layout, dsd_nn.layout):
            ok = ok and (other is softmax.layout or (other.shape == softmax.layout.shape and bool((other == softmax.layout).all())))
    made = AttentionCore(softmax.layout, softmax.block, softmax) if ok else None
    softmax._attention_core = (sdd_nt, dsd_nn, made)
    return made


def attention_chain(sdd_nt, softmax, dsd_nn, q, k, v, scale=1., rpe=None, key_padding_mask=None, attn_mask=None,
                    key_padding_mask_mode='add', attn_mask_mode='add', dropout_p=0.):
    """dsd_nn(softmax(sdd_nt(q, k), ...), v): fused when the operators and tensors allow it, else the three calls."""
    core = _core_for(sdd_nt, softmax, dsd_nn)
    if core is not None and core.usable(q, k, v, dropout_p):
        return core(q, k, v, scale, rpe, key_padding_mask, attn_mask, key_padding_mask_mode, attn_mask_mode)
    w = sdd_nt(q, k)
    kwargs = dict(dropout_p=dropout_p) if dropout_p else {}
    w = softmax(w, scale=scale, rpe=rpe, key_padding_mask=key_padding_mask, attn_mask=attn_mask,
                key_padding_mask_mode=key_padding_mask_mode, attn_mask_mode=attn_mask_mode, **kwargs)
    return dsd_nn(w, v)
