"""Block-sparse matrix multiplication (sdd / dsd / dds) on MI355X.

Drop-in for the reference's torch_blocksparse/matmul.py: same `MatMul(layout, block, mode, trans_a, trans_b,
bench)` object, same sparse storage ([Z, nnz, block, block], blocks in layout.nonzero() order), same
look-up tables (built on the GPU, bit-identical to matmul.py:221-297 and :372-458), same autograd wiring
(matmul.py:558-606).  The kernels are HIP/MFMA kernels reached through the C ABI in include/bsp.h.
"""
import ctypes
import math

import torch

from . import _lib


# Flags handed to every matmul launch (bsp_launch_flags of the C ABI).  0 in normal use; the tests that compare the kernel
# families with each other set _lib.FLAG_GENERAL_ONLY / _lib.FLAG_NO_GROUPS here.
KERNEL_FLAGS = 0


def _vec(dtype):
    return 4 if dtype == torch.float32 else 8


class _LayoutOnDevice:
    """The int32 copy of a layout on the device, its number of blocks and the builders' workspace: made once per
    `MatMul.make_lut` and shared by the tables it builds."""

    def __init__(self, layout, device):
        self.device = torch.device(device)
        self.lay = _lib.layout_to_device(layout, self.device)
        self.ws, self.ws_bytes = _lib.workspace(self.lay, self.device)
        self.nnz = int((layout != 0).sum())
        self._coarse = None

    @staticmethod
    def of(layout, device, ctx):
        return ctx if ctx is not None else _LayoutOnDevice(layout, device)

    def coarse(self, S):
        """The layout coarsened to tiles of S x S blocks (a tile is present if any of its blocks is), as a context of its
        own, and per present tile the ids of its S * S blocks (-1 where absent), tiles in nonzero() order.  Made once
        and shared by the plans over tiles of all three products."""
        if self._coarse is None:
            H, R, C = self.lay.shape
            lay = self.lay != 0
            tiles5 = lay.reshape(H, R // S, S, C // S, S)
            present = tiles5.any(4).any(2)
            cctx = _LayoutOnDevice.__new__(_LayoutOnDevice)
            cctx.device, cctx.lay = self.device, present.to(torch.int32).contiguous()
            cctx.ws, cctx.ws_bytes = _lib.workspace(cctx.lay, self.device)
            cctx.nnz = int(present.sum())
            cctx._coarse = None
            fine = torch.where(lay, torch.cumsum(lay.reshape(-1), 0, dtype=torch.int32).reshape(lay.shape) - 1, -1).to(torch.int32)
            ids = fine.reshape(H, R // S, S, C // S, S).permute(0, 1, 3, 2, 4)[present].reshape(-1, S * S)
            self._coarse = (cctx, ids)
        return self._coarse


def _prep(x):
    """Operands are read with 16-byte vector loads along a unit inner stride."""
    v = _vec(x.dtype)
    ok = x.stride(-1) == 1 and x.data_ptr() % 16 == 0 and all(s % v == 0 for s in x.stride()[:-1])
    return x if ok else x.contiguous()


class _Timer:
    """Event timing of one launch when bench=True (milliseconds); the reference stores the JIT's own timing."""

    def __init__(self, bench, device):
        self.bench = bench
        if bench:
            self.start = torch.cuda.Event(enable_timing=True)
            self.stop = torch.cuda.Event(enable_timing=True)
            self.start.record(torch.cuda.current_stream(device))
        self.device = device

    def done(self):
        if not self.bench:
            return None
        self.stop.record(torch.cuda.current_stream(self.device))
        self.stop.synchronize()
        return self.start.elapsed_time(self.stop)


class GroupPlan:
    """Work list of the row-group kernels (see bsp_group_plan_build): device table, number of header rows, lines per
    head, number of split chains (their fp32 partial tiles live in `workspace`)."""

    def __init__(self, table, n_groups, lines, n_split=0):
        self.table, self.n_groups, self.lines, self.n_split = table, n_groups, lines, n_split
        self.coarse = False
        self.rowpair = False
        self._max_entries = None
        self._ws = None
        self._ws_retired = []

    @staticmethod
    def thin_min(layout, by_rows, block=64, nnz=None):
        """Lines at least this long become chains: well above the average line, so that dense-ish layouts (whose
        groups share every dense tile four times) keep their groups and only outliers such as global columns split.
        The kernels for blocks 16 and 32 give a chain less than the block-64 kernel does (measured on the attention
        mask: chains of 98 blocks of 32 cost 3 us, chains of 196 blocks of 16 save 15), so only very long lines split."""
        H, R, C = layout.shape
        mean = float((layout != 0).sum() if nnz is None else nnz) / max(1, H * (R if by_rows else C))
        return max(16 if block >= 64 else 128, int(2 * mean + 0.5))

    # A chain with more entries than this is cut into parts that run as workgroups of their own (block-64 kernels).
    SPLIT_LEN = 128

    @staticmethod
    def order_buckets(layout, by_rows, block):
        """Coarse (8 steps) rather than exact longest-first order of the groups when the dense rows one head reads are
        few (at most 8192): the short groups then run head by head and find those rows in L2.  Measured on the
        attention mask at seq 4096: transposed products 81 -> 77 and 92 -> 87 us at block 32, no change at block 64;
        at seq 16384 (BigBird layout) the coarse order is 2 % slower, so long sequences keep the exact order."""
        H, R, C = layout.shape
        return 8 if (C if by_rows else R) * block <= 8192 else 0

    @staticmethod
    def build(layout, by_rows, device, thin_min=None, order_buckets=0, split_len=0, ctx=None):
        """thin_min: lines at least this long become chains; None = GroupPlan.thin_min(...), 0 = no chains.
        order_buckets: see GroupPlan.order_buckets; 0 = exact longest-first order.  split_len: chains longer than this
        are cut into parts (0 = never; only the block-64 dsd/dds kernels know how to add the parts up)."""
        lib = _lib.load()
        ctx = _LayoutOnDevice.of(layout, device, ctx)
        dev, lay = ctx.device, ctx.lay
        H, R, C = lay.shape
        cap = lib.bsp_group_plan_cap(H, R, C, ctx.nnz, int(bool(by_rows)))
        table = torch.empty((cap,), dtype=torch.int32, device=dev)
        n_groups, n_split, n = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int64(0)
        thin = GroupPlan.thin_min(layout, by_rows) if thin_min is None else int(thin_min)
        rc = lib.bsp_group_plan_build(_lib.ptr(lay), H, R, C, int(bool(by_rows)), thin, int(split_len), int(order_buckets),
                                      _lib.ptr(table), cap, _lib.ptr(ctx.ws), ctx.ws_bytes, ctypes.byref(n_groups),
                                      ctypes.byref(n_split), ctypes.byref(n), _lib.stream_ptr(dev))
        _lib.check(rc, 'bsp_group_plan_build')
        return GroupPlan(table[:n.value], n_groups.value, R if by_rows else C, n_split.value)

    @staticmethod
    def build_coarse(layout, block, by_rows, device, for_sdd=False, ctx=None):
        """Plan of a block-16 layout over 64 x 64 tiles: the groups, chains and order of `build` on the layout coarsened
        to 64 (a tile is present if any of its S x S blocks is, S = 64 / block), with entries that carry the ids of the
        small blocks: (position, 4 tile ids, 4 x S*S block ids, -1 where absent).  The launchers are told by a
        negative line count.  for_sdd: the plan bsp_sdd_matmul takes: no chains, and the longer half of the groups before
        the shorter half, head by head in each (measured on the attention mask: the sdd and the softmax that reads
        its result 2-3 us faster each than with the exact longest-first order).  None if the layout does not divide
        into tiles."""
        S = 64 // block
        H, R, C = layout.shape
        if R % S or C % S:
            return None
        ctx = _LayoutOnDevice.of(layout, device, ctx)
        cctx, tiles = ctx.coarse(S)
        coarse = cctx.lay
        plan = GroupPlan.build(coarse, by_rows, ctx.device, thin_min=0 if for_sdd else GroupPlan.thin_min(coarse, by_rows, 64, nnz=cctx.nnz),
                               order_buckets=2 if for_sdd else GroupPlan.order_buckets(coarse, by_rows, 64),
                               split_len=0 if for_sdd else GroupPlan.SPLIT_LEN, ctx=cctx)
        ng, G = plan.n_groups, 4
        table = plan.table
        header, entries = table[:4 * ng], table[4 * ng:].view(-1, G + 1)
        ids = entries[:, 1:].to(torch.int64)                                    # [entries, G] tile ids or -1
        sub = torch.where((ids >= 0).unsqueeze(2), tiles[ids.clamp(min=0)], -1)
        wide = torch.cat([entries, sub.reshape(entries.shape[0], G * S * S)], 1)
        out = GroupPlan(torch.cat([header, wide.reshape(-1)]).contiguous(), ng, plan.lines, plan.n_split)
        out.coarse = True
        return out

    @staticmethod
    def build_rowpair(layout, device, ctx=None):
        """Plan of a block-16 layout for the long-reduction sdd kernel: every two consecutive block-rows form a member of 32
        rows (present at a block-column if either has a block there), four members a group (128 rows of A), no chains,
        groups head by head.  Entries: (position, 4 member ids, then the ids of the two blocks of each member, -1 where
        absent).  None if the layout has an odd number of block-rows."""
        H, R, C = layout.shape
        if R % 2:
            return None
        ctx = _LayoutOnDevice.of(layout, device, ctx)
        lay = ctx.lay != 0
        pairs = lay.reshape(H, R // 2, 2, C)
        present = pairs.any(2)
        pctx = _LayoutOnDevice.__new__(_LayoutOnDevice)
        pctx.device, pctx.lay = ctx.device, present.to(torch.int32).contiguous()
        pctx.ws, pctx.ws_bytes = _lib.workspace(pctx.lay, ctx.device)
        pctx.nnz = int(present.sum())
        pctx._coarse = None
        fine = torch.where(lay, torch.cumsum(lay.reshape(-1), 0, dtype=torch.int32).reshape(lay.shape) - 1, -1).to(torch.int32)
        ids2 = fine.reshape(H, R // 2, 2, C).permute(0, 1, 3, 2)[present].reshape(-1, 2)        # per present pair, in nonzero() order
        plan = GroupPlan.build(pctx.lay, True, ctx.device, thin_min=0, order_buckets=1, ctx=pctx)
        ng, G = plan.n_groups, 4
        header, entries = plan.table[:4 * ng], plan.table[4 * ng:].view(-1, G + 1)
        ids = entries[:, 1:].to(torch.int64)
        sub = torch.where((ids >= 0).unsqueeze(2), ids2[ids.clamp(min=0)], -1)
        wide = torch.cat([entries, sub.reshape(entries.shape[0], 2 * G)], 1)
        out = GroupPlan(torch.cat([header, wide.reshape(-1)]).contiguous(), ng, plan.lines, 0)
        out.rowpair = True
        return out

    def max_entries(self):
        """The largest number of entries of any group of the plan (read back from the device once and kept)."""
        if self._max_entries is None:
            self._max_entries = int(self.table[:4 * self.n_groups].view(-1, 4)[:, 1].max()) if self.n_groups else 0
        return self._max_entries

    def workspace(self, free_dim, Z):
        """(pointer, bytes) of the scratch buffer the split chains of this plan need for a launch with this free dimension
        and batch (fp32 partial tiles; kept for the next call, contents never matter); (NULL, 0) for a plan without
        split chains.  One buffer per plan: launches of one operator are assumed to be ordered on one stream.
        A launch that needs more than the buffer holds gets a larger one, and the smaller one stays allocated for the
        life of the plan: a captured HIP graph replays launches that carry its address."""
        if self.n_split == 0:
            return ctypes.c_void_p(0), 0
        need = _lib.load().bsp_xsd_workspace_bytes(self.n_split, int(free_dim), int(Z))
        if self._ws is None or self._ws.numel() < need:
            if self._ws is not None:
                self._ws_retired.append(self._ws)
            self._ws = torch.empty(need, dtype=torch.uint8, device=self.table.device)
        return _lib.ptr(self._ws), self._ws.numel()

    @staticmethod
    def args(plan):
        if plan is None:
            return ctypes.c_void_p(0), 0, 0
        return _lib.ptr(plan.table), plan.n_groups, (-plan.lines if plan.coarse else plan.lines)

    @staticmethod
    def xsd_args(plan, free_dim, Z):
        """The plan, its split chains and their workspace, as bsp_dsd_matmul / bsp_dds_matmul take them."""
        if plan is None:
            return ctypes.c_void_p(0), 0, 0, 0, ctypes.c_void_p(0), 0
        ws, ws_bytes = plan.workspace(free_dim, Z)
        return GroupPlan.args(plan) + (plan.n_split, ws, ws_bytes)


def _check_dense(name, x, heads, rows, cols, trans):
    """A dense operand against the layout: [Z, heads, rows, cols] as stored when not read transposed, [Z, heads, cols,
    rows] otherwise; None = the free dimension, any size.  The kernels take every address from the tables (head,
    block-row, block id), so a wrong extent would be an out-of-bounds access on the device, not an error."""
    if x.dim() != 4:
        raise ValueError('matmul operand %s must have 4 dimensions [batch, heads, rows, cols], got %s' % (name, tuple(x.shape)))
    if x.size(1) != heads:
        raise ValueError('matmul operand %s has %d heads, the layout has %d' % (name, x.size(1), heads))
    r, c = (x.size(3), x.size(2)) if trans else (x.size(2), x.size(3))
    if rows is not None and r != rows:
        raise ValueError('matmul operand %s: op(%s) has %d rows, the layout needs %d' % (name, name, r, rows))
    if cols is not None and c != cols:
        raise ValueError('matmul operand %s: op(%s) has %d columns, the layout needs %d' % (name, name, c, cols))


def _check_sparse(name, x, nnz, block, Z):
    """A sparse operand: [nnz, block, block] (shared by the batch) or [Z or 1, nnz, block, block]."""
    if x.dim() not in (3, 4):
        raise ValueError('sparse matmul operand %s must be [nnz, block, block] or [batch, nnz, block, block], got %s' % (name, tuple(x.shape)))
    if tuple(x.shape[-2:]) != (block, block):
        raise ValueError('sparse matmul operand %s has blocks of %s, expected (%d, %d)' % (name, tuple(x.shape[-2:]), block, block))
    if nnz is not None and x.size(-3) != nnz:
        raise ValueError('sparse matmul operand %s has %d blocks, the layout has %d' % (name, x.size(-3), nnz))
    if x.dim() == 4 and x.size(0) not in (1, Z):
        raise ValueError('sparse matmul operand %s has batch %d, the dense operand has %d' % (name, x.size(0), Z))


class SddTables(list):
    """The per-pack sdd tables, in the reference's order; `nnz` is the number of blocks of the output, `gplan` the
    optional row-group plan of the layout.  Built by `MatMul.make_lut` the list starts empty and `build` fills it when a
    product first needs the tables: the greedy packing behind them is the one sequential step of the builders
    (milliseconds at block 16), and the kernels that work from the plan alone never read them."""
    nnz = 0
    gplan = None
    spdims = None
    build = None          # callable -> (tables, widths, packs), or None when the list is complete
    gplan_long = None     # block 32: the plan of the long-reduction kernel (head by head), built by build_long on demand
    build_long = None
    widths = None
    packs = None

    def materialize(self):
        if self.build is not None:
            tables, self.widths, self.packs = self.build()
            self.extend(tables)
            self.build = None
        return self.widths, self.packs


class _sparse_matmul(torch.autograd.Function):

    ##########################
    # SPARSE = DENSE x DENSE #
    ##########################
    @staticmethod
    def make_sdd_lut(layout, block, dtype, device, ctx=None, lazy=False):
        """-> (luts, None, widths, packs) as the reference (matmul.py:281-297); built on `device`.

        start_width is 64 // block in the reference, which is 0 for block 128 and leaves the table empty
        (matmul.py:283, csrc/utils.cpp:117); max(1, .) gives block 128 the single-block table it needs.
        Each table tensor carries `.valid` (None, or a uint8 tensor marking the rows that really are blocks).
        lazy: return (luts, None, None, None) with the tables not built yet; `luts.materialize()` builds them (the
        row-group plan, which the specialised kernels work from, is always built here).
        """
        lib = _lib.load()
        ctx = _LayoutOnDevice.of(layout, device, ctx)
        dev, lay, nnz = ctx.device, ctx.lay, ctx.nnz
        H, R, C = lay.shape

        def build_tables():
            start_width = max(1, 64 // block)
            cap = nnz + nnz // 8 + 64
            n_levels = ctypes.c_int(0)
            packs = (ctypes.c_int * 8)()
            rows = (ctypes.c_int64 * 8)()
            total = ctypes.c_int64(0)
            all_valid = ctypes.c_int(1)
            for attempt in range(2):
                lut = torch.empty((cap, 4), dtype=torch.int32, device=dev)
                valid = torch.empty((cap,), dtype=torch.uint8, device=dev)
                rc = lib.bsp_sdd_lut_build(_lib.ptr(lay), H, R, C, start_width, _lib.ptr(lut), _lib.ptr(valid), cap, _lib.ptr(ctx.ws),
                                           ctx.ws_bytes, ctypes.byref(n_levels), packs, rows, ctypes.byref(total),
                                           ctypes.byref(all_valid), _lib.stream_ptr(dev))
                if rc == _lib.ERR_CAPACITY and attempt == 0:
                    cap = int(total.value)
                    continue
                _lib.check(rc, 'bsp_sdd_lut_build')
                break
            tables, widths, out_packs = [], [], []
            done = 0
            for k in range(n_levels.value):
                p, r = int(packs[k]), int(rows[k])
                t = lut[done:done + r].reshape(-1)
                t.valid = None if all_valid.value else valid[done:done + r]
                tables.append(t)
                widths.append(r // (p * p))
                out_packs.append(p)
                done += r
            return tables, widths, out_packs

        luts = SddTables()
        luts.nnz = nnz
        luts.spdims = tuple(layout.shape)
        luts.build = build_tables
        if block in (16, 32, 64):
            luts.gplan = GroupPlan.build_coarse(layout, block, True, dev, for_sdd=True, ctx=ctx) if block == 16 else None
            if luts.gplan is None:
                luts.gplan = GroupPlan.build(layout, True, dev, thin_min=0, ctx=ctx)
        # blocks of 32 with a long reduction take a kernel of their own, whose plan runs head by head (the workgroups on
        # an XCD at one time then read the same rows of B; the attention-shape kernels prefer the longest group first:
        # measured 0.64 against 0.67 ms per attention step); built when such a product first comes
        luts.gplan_long = None
        if block == 32:
            luts.build_long = lambda: GroupPlan.build(layout, True, dev, thin_min=0, order_buckets=1, ctx=ctx)
        elif block == 16 and R % 2 == 0:
            # blocks of 16: the same kernel on pairs of block-rows (a plan and a flag of its own)
            luts.build_long = lambda: GroupPlan.build_rowpair(layout, dev, ctx=ctx)
        if lazy and luts.gplan is not None:
            return luts, None, None, None
        widths, packs = luts.materialize()
        return luts, None, widths, packs

    @staticmethod
    def _sdd_matmul(a, b, trans_a, trans_b, trans_c, spdims, block, luts, num_locks, widths, packs, bench, time):
        if trans_c:                                   # matmul.py:303-305
            a, b = b, a
            trans_a, trans_b = not trans_b, not trans_a
        a, b = _prep(a), _prep(b)
        AS0 = a.size(0)
        AS3 = a.size(2 if trans_a else 3)
        if AS3 % 16 != 0:
            raise ValueError('Reduction size for SDD must be a multiple of 16')
        if b.size(0) != AS0 or b.size(1) != a.size(1) or b.size(3 if trans_b else 2) != AS3:
            raise ValueError('incompatible operand shapes for sdd: %s and %s' % (tuple(a.shape), tuple(b.shape)))
        _check_dense('a', a, spdims[0], block * spdims[1], None, trans_a)
        _check_dense('b', b, spdims[0], None, block * spdims[2], trans_b)
        lib = _lib.load()
        lazy = isinstance(luts, SddTables)
        total_width = luts.nnz if lazy else sum(w * p * p for w, p in zip(widths, packs))
        c = torch.empty((AS0, total_width, block, block), dtype=a.dtype, device=a.device)
        timer = _Timer(bench, a.device)
        operands = (_lib.DTYPES[a.dtype], _lib.ptr(a), _lib.ptr(b), _lib.ptr(c), int(trans_a), int(trans_b),
                    AS0, AS3, a.stride(0), a.stride(1), a.stride(2), b.stride(0), b.stride(1), b.stride(2), c.stride(0), block)
        # The group plan describes the whole layout.  If the tables are not built yet it goes first on its own: a kernel
        # that works from the plan writes every block (status OK_WHOLE_LAYOUT) and the tables are never needed; otherwise
        # nothing was launched (NEEDS_TABLE), the tables are built and the plan goes with the first pack level.
        gplan = GroupPlan.args(getattr(luts, 'gplan', None))
        rc = _lib.NEEDS_TABLE
        long_k = (lazy and block in (16, 32) and AS3 >= 256 and AS3 % 32 == 0 and a.dtype != torch.float32
                  and getattr(luts, 'build_long', None) is not None)
        if long_k:
            # the kernel for long reductions works from its own plan, whether the tables exist or not
            if luts.gplan_long is None:
                luts.gplan_long = luts.build_long()
            lp = GroupPlan.args(luts.gplan_long)
            flags = KERNEL_FLAGS | (_lib.FLAG_PLAN_ROWPAIR if luts.gplan_long.rowpair else 0)
            # (the largest group of the plan sizes the grid: workgroups for block-columns that no group reaches are not launched)
            rc = lib.bsp_sdd_matmul(*operands, 0, ctypes.c_void_p(0), ctypes.c_void_p(0), min(spdims[2], luts.gplan_long.max_entries()),
                                    lp[0], lp[1], lp[2], flags, _lib.stream_ptr(a.device))
            if rc not in (_lib.OK_WHOLE_LAYOUT, _lib.NEEDS_TABLE):
                _lib.check(rc, 'bsp_sdd_matmul')
        elif lazy and luts.gplan is not None and luts.build is not None:
            rc = lib.bsp_sdd_matmul(*operands, 0, ctypes.c_void_p(0), ctypes.c_void_p(0), spdims[2], gplan[0], gplan[1], gplan[2],
                                    KERNEL_FLAGS, _lib.stream_ptr(a.device))
            if rc not in (_lib.OK_WHOLE_LAYOUT, _lib.NEEDS_TABLE):
                _lib.check(rc, 'bsp_sdd_matmul')
        if rc == _lib.NEEDS_TABLE:
            if lazy:
                widths, packs = luts.materialize()
            if _sparse_matmul._sdd_splitk(lib, operands, a, AS0, AS3, block, luts, widths, packs):
                time[0] = timer.done()
                return c
            for lut, width, pack in zip(luts, widths, packs):
                rc = lib.bsp_sdd_matmul(*operands, pack, _lib.ptr(lut), _lib.ptr(getattr(lut, 'valid', None)), width,
                                        gplan[0], gplan[1], gplan[2], KERNEL_FLAGS, _lib.stream_ptr(a.device))
                if rc == _lib.OK_WHOLE_LAYOUT:
                    break
                _lib.check(rc, 'bsp_sdd_matmul')
                gplan = GroupPlan.args(None)
        time[0] = timer.done()
        return c

    # Blocks of 128, few of them and a long reduction (the weight gradient of a sparse linear layer): the reduction is cut
    # into parts that run side by side, as many as fill the chip once (three workgroups of this kernel fit a CU: 768),
    # each part at least 256 long.  Measured on 110 blocks over a reduction of 8192: 1 part 0.092 ms (the general
    # kernel), 2 parts 0.102, 4 parts 0.069, 6 parts 0.063, 8 parts (more workgroups than fit at once) 0.081.
    SPLITK_TARGET_WORKGROUPS = 768

    @staticmethod
    def _sdd_splitk(lib, operands, a, Z, K, block, luts, widths, packs):
        if block != 128 or a.dtype == torch.float32 or K % 32 or K < 512 or len(luts) != 1 or packs[0] != 1 or (KERNEL_FLAGS & 5):
            return False
        n = widths[0]
        if n <= 0 or n * Z >= _sparse_matmul.SPLITK_TARGET_WORKGROUPS:
            return False
        parts = max(1, min(_sparse_matmul.SPLITK_TARGET_WORKGROUPS // (n * Z), K // 256, 16))
        need = lib.bsp_sdd_splitk_workspace_bytes(Z, n, parts)
        ws = getattr(luts, '_splitk_ws', None)
        if need and (ws is None or ws.numel() < need):
            if ws is not None:
                luts._splitk_retired = getattr(luts, '_splitk_retired', []) + [ws]      # a captured graph may still use it
            ws = luts._splitk_ws = torch.empty(need, dtype=torch.uint8, device=a.device)
        lut = luts[0]
        rc = lib.bsp_sdd_matmul_splitk(*operands, _lib.ptr(lut), _lib.ptr(getattr(lut, 'valid', None)), n, parts,
                                       _lib.ptr(ws) if need else ctypes.c_void_p(0), ws.numel() if need else 0, KERNEL_FLAGS,
                                       _lib.stream_ptr(a.device))
        if rc == _lib.ERR_UNSUPPORTED:
            return False
        _lib.check(rc, 'bsp_sdd_matmul_splitk')
        return True

    ##########################
    # DENSE = DENSE x SPARSE #
    ##########################
    @staticmethod
    def make_dxx_lut(layout, block, step, trans, device, transform=lambda idx: idx, ctx=None):
        """-> (lut, num_locks, width, None) as the reference (matmul.py:372-458); built on `device`.

        The table tensor carries `.plan`: per block, in table order, (position in the dense operand's reduction
        dimension, storage index) -- the absolute values the table's increments are differences of -- and
        `.planbuf`, the buffer the launchers take: the order in which they dispatch the segments, then `.plan`.
        """
        lib = _lib.load()
        ctx = _LayoutOnDevice.of(layout, device, ctx)
        dev, lay, nnz = ctx.device, ctx.lay, ctx.nnz
        H, R, C = lay.shape
        cap = lib.bsp_dxx_lut_cap(H, R, C, nnz, block, step, int(bool(trans)))
        lut = torch.empty((cap,), dtype=torch.int32, device=dev)
        planbuf = torch.empty((lib.bsp_dxx_plan_cap(H, R, C, max(nnz, 1), int(bool(trans))),), dtype=torch.int32, device=dev)
        n = ctypes.c_int64(0)
        width = ctypes.c_int(0)
        num_locks = ctypes.c_int(0)
        rc = lib.bsp_dxx_lut_build(_lib.ptr(lay), H, R, C, block, step, int(bool(trans)), _lib.ptr(lut), cap, _lib.ptr(planbuf),
                                   _lib.ptr(ctx.ws), ctx.ws_bytes, ctypes.byref(n), ctypes.byref(width), ctypes.byref(num_locks),
                                   _lib.stream_ptr(dev))
        if rc == _lib.ERR_EMPTY_HEAD:
            raise RuntimeError('block-sparse layout has a head without any nonzero block')
        _lib.check(rc, 'bsp_dxx_lut_build')
        lut = lut[:n.value]
        first = lib.bsp_dxx_plan_pairs_offset(width.value)
        lut.planbuf = planbuf
        lut.plan = planbuf[first:first + 2 * nnz].view(nnz, 2)
        lut.nnz = nnz
        lut.spdims = tuple(layout.shape)
        lut.gplan = GroupPlan.build_coarse(layout, block, trans, dev, ctx=ctx) if block == 16 else None
        if lut.gplan is None and block in (16, 32, 64):
            lut.gplan = GroupPlan.build(layout, trans, dev, thin_min=GroupPlan.thin_min(layout, trans, block, nnz=nnz),
                                        order_buckets=GroupPlan.order_buckets(layout, trans, block),
                                        split_len=GroupPlan.SPLIT_LEN if block == 64 else 0, ctx=ctx)
        # blocks of 32 with a wide free dimension take a kernel of their own (dense tiles shared by the four lines of a
        # group): its plan has no chains and runs head by head; built when such a product first comes
        lut.gplan_wide = None
        if block == 32:
            lut.build_wide = lambda: GroupPlan.build(layout, trans, dev, thin_min=0, order_buckets=1, ctx=ctx)
        return lut, num_locks.value, width.value, None

    @staticmethod
    def _plan_for(lut, block, free_dim, dtype, dense_k_contiguous):
        """The group plan that goes with a dsd / dds launch: the wide-free-dimension plan for blocks of 32 (16-bit types,
        256 dense rows or more, dense operand with the reduction contiguous: the products the wide kernel takes), else
        the table's ordinary plan."""
        if (block == 32 and free_dim >= 256 and dtype != torch.float32 and dense_k_contiguous
                and getattr(lut, 'build_wide', None) is not None):
            if lut.gplan_wide is None:
                lut.gplan_wide = lut.build_wide()
            return lut.gplan_wide
        return getattr(lut, 'gplan', None)

    @staticmethod
    def _pad_free_dim(x, dim, v):
        pad = (-x.size(dim)) % v
        if pad == 0:
            return x
        shape = list(x.shape)
        shape[dim] = pad
        return torch.cat((x, x.new_zeros(shape)), dim=dim)

    @staticmethod
    def _dds_matmul(a, b, trans_a, trans_b, trans_c, spdims, block, lut, num_locks, width, packs, bench, time):
        v = _vec(a.dtype)
        _check_sparse('b', b, getattr(lut, 'nnz', None), block, a.size(0))
        _check_dense('a', a, spdims[0], None, block * spdims[2 if trans_b else 1], trans_a)
        AS2 = a.size(3 if trans_a else 2)                     # free dimension M (matmul.py:467)
        a = _prep(_sparse_matmul._pad_free_dim(a, 3 if trans_a else 2, v))
        M = a.size(3 if trans_a else 2)
        b = b if b.is_contiguous() else b.contiguous()
        BS2 = block * spdims[1 if trans_b else 2]             # matmul.py:471
        CS2, CS3 = (BS2, M) if trans_c else (M, BS2)
        c = torch.empty((a.size(0), a.size(1), CS2, CS3), dtype=a.dtype, device=a.device)
        b_sz = b.stride(0) if (b.dim() == 4 and b.size(0) > 1) else 0   # a 3-D (or batch-1) sparse operand is shared by the batch
        timer = _Timer(bench, a.device)
        rc = _lib.load().bsp_dds_matmul(_lib.DTYPES[a.dtype], _lib.ptr(a), _lib.ptr(b), _lib.ptr(c), int(trans_a), int(trans_b),
                                        int(trans_c), a.size(0), M, a.stride(0), a.stride(1), a.stride(2), b_sz, c.stride(0),
                                        c.stride(1), c.stride(2), block, _lib.ptr(lut), _lib.ptr(lut.planbuf), width,
                                        *GroupPlan.xsd_args(_sparse_matmul._plan_for(lut, block, M, a.dtype, not trans_a), M, a.size(0)), KERNEL_FLAGS,
                                        _lib.stream_ptr(a.device))
        _lib.check(rc, 'bsp_dds_matmul')
        time[0] = timer.done()
        if M != AS2:
            c = c[:, :, :, :AS2] if trans_c else c[:, :, :AS2, :]
        return c

    @staticmethod
    def _dsd_matmul(a, b, trans_a, trans_b, trans_c, spdims, block, lut, num_locks, width, packs, bench, time):
        v = _vec(b.dtype)
        _check_sparse('a', a, getattr(lut, 'nnz', None), block, b.size(0))
        _check_dense('b', b, spdims[0], block * spdims[1 if trans_a else 2], None, trans_b)
        BS3 = b.size(2 if trans_b else 3)                     # free dimension N (matmul.py:518)
        b = _prep(_sparse_matmul._pad_free_dim(b, 2 if trans_b else 3, v))
        N = b.size(2 if trans_b else 3)
        a = a if a.is_contiguous() else a.contiguous()
        AS1 = block * spdims[2 if trans_a else 1]             # matmul.py:513
        CS2, CS3 = (N, AS1) if trans_c else (AS1, N)
        c = torch.empty((b.size(0), b.size(1), CS2, CS3), dtype=b.dtype, device=b.device)
        a_sz = a.stride(0) if (a.dim() == 4 and a.size(0) > 1) else 0
        timer = _Timer(bench, b.device)
        rc = _lib.load().bsp_dsd_matmul(_lib.DTYPES[b.dtype], _lib.ptr(a), _lib.ptr(b), _lib.ptr(c), int(trans_a), int(trans_b),
                                        int(trans_c), b.size(0), N, a_sz, b.stride(0), b.stride(1), b.stride(2), c.stride(0),
                                        c.stride(1), c.stride(2), block, _lib.ptr(lut), _lib.ptr(lut.planbuf), width,
                                        *GroupPlan.xsd_args(_sparse_matmul._plan_for(lut, block, N, b.dtype, bool(trans_b)), N, b.size(0)), KERNEL_FLAGS,
                                        _lib.stream_ptr(b.device))
        _lib.check(rc, 'bsp_dsd_matmul')
        time[0] = timer.done()
        if N != BS3:
            c = c[:, :, :BS3, :] if trans_c else c[:, :, :, :BS3]
        return c

    fn = {'sdd': _sdd_matmul.__get__(object),
          'dsd': _dsd_matmul.__get__(object),
          'dds': _dds_matmul.__get__(object)}

    @staticmethod
    def forward(ctx, a, b, trans_a, trans_b, trans_c, mode, spdims, block,
                c_lut, c_num_locks, c_width, c_packs, c_bench, c_time,
                da_lut, da_num_locks, da_width, da_packs, da_bench, da_time,
                db_lut, db_num_locks, db_width, db_packs, db_bench, db_time):
        _lib.require_gpu_tensor(a, 'matmul operand a')
        _lib.require_gpu_tensor(b, 'matmul operand b')
        if a.dtype != b.dtype or a.dtype not in _lib.DTYPES:
            raise ValueError('matmul operands must both be float16, bfloat16 or float32 (got %s, %s)' % (a.dtype, b.dtype))
        c = _sparse_matmul.fn[mode](a, b, trans_a, trans_b, trans_c, spdims, block,
                                    c_lut, c_num_locks, c_width, c_packs, c_bench, c_time)
        ctx.save_for_backward(a, b)
        ctx.da = (da_lut, da_num_locks, da_width, da_packs, da_bench, da_time)
        ctx.db = (db_lut, db_num_locks, db_width, db_packs, db_bench, db_time)
        ctx.mode, ctx.spdims, ctx.block = mode, spdims, block
        ctx.trans_a, ctx.trans_b = trans_a, trans_b
        return c

    @staticmethod
    def backward(ctx, dc):
        a, b = ctx.saved_tensors
        mode = ctx.mode
        da = db = None
        # db before da: in an attention chain da of the dsd product (an sdd launch) is what the softmax backward
        # reads next, and da of the sdd product is what the caller's next op reads; measured 1 % faster per step.
        if ctx.needs_input_grad[1]:                        # matmul.py:598-601
            mode_db = mode[2] + mode[1] + mode[0]
            db = _sparse_matmul.fn[mode_db](a, dc, not ctx.trans_a, False, ctx.trans_b, ctx.spdims, ctx.block, *ctx.db)
            if db.shape != b.shape:
                db = db.reshape(b.shape) if db.numel() == b.numel() else db.sum(0).reshape(b.shape)
        if ctx.needs_input_grad[0]:                           # matmul.py:593-596
            mode_da = mode[1] + mode[0] + mode[2]
            da = _sparse_matmul.fn[mode_da](dc, b, False, not ctx.trans_b, ctx.trans_a, ctx.spdims, ctx.block, *ctx.da)
            if da.shape != a.shape:
                da = da.reshape(a.shape) if da.numel() == a.numel() else da.sum(0).reshape(a.shape)
        return (da, db) + (None,) * 24


class MatMul:
    """C = op(A) @ op(B) with one block-sparse participant.

    mode 'sdd': C sparse, A and B dense; 'dsd': A sparse; 'dds': B sparse.  `layout` ([H, R, C], 0/1, on the CPU)
    always describes the sparse tensor as stored.
    """

    def make_lut(self, dtype, device):
        key = (dtype, device)
        if key in self.lut_cache:
            return self.lut_cache[key]
        layout, block = self.layout, self.block
        step = 8 if dtype == torch.float32 else 16             # matmul.py:617
        ctx = _LayoutOnDevice(layout, device)                  # one upload of the layout and one workspace for all tables
        sdd = lambda: _sparse_matmul.make_sdd_lut(layout, block, dtype, device, ctx=ctx, lazy=True)
        dxx = lambda trans: _sparse_matmul.make_dxx_lut(layout, block, step, trans, device, ctx=ctx)
        if self.mode == 'sdd':                                 # matmul.py:618-637
            c, da, db = sdd(), dxx(True), dxx(False)
        elif self.mode == 'dsd':
            c, da, db = dxx(not self.trans_a), sdd(), dxx(self.trans_a)
        else:
            c, da, db = dxx(self.trans_b), dxx(not self.trans_b), sdd()
        self.lut_cache[key] = c + da + db
        return self.lut_cache[key]

    def __init__(self, layout, block, mode, trans_a=False, trans_b=False, bench=False):
        if mode not in ['sdd', 'dsd', 'dds']:
            raise NotImplementedError('Supported modes are: sdd, dsd, dds')
        if block not in (16, 32, 64, 128):
            raise ValueError('block must be 16, 32, 64 or 128')
        self.lut_cache = dict()
        self.trans_a = trans_a
        self.trans_b = trans_b
        self.mode = mode
        self.spdims = layout.shape
        self.block = block
        self.layout = layout
        self.bench = bench
        self.time_c = None
        self.time_da = None
        self.time_db = None

    @staticmethod
    def _pad_shape(x, is_sparse):
        max_dim = 3 if is_sparse else 4                        # matmul.py:663-668
        for _ in range(max_dim - x.dim()):
            x = x.unsqueeze(0)
        return x

    def __call__(self, a, b):
        _lib.require_gpu_tensor(a, 'matmul operand a')
        luts = self.make_lut(a.dtype, a.device)
        time_c, time_da, time_db = [None], [None], [None]
        a = MatMul._pad_shape(a, self.mode == 'dsd')
        b = MatMul._pad_shape(b, self.mode == 'dds')
        c = _sparse_matmul.apply(a, b, self.trans_a, self.trans_b, False, self.mode, self.spdims, self.block,
                                 luts[0], luts[1], luts[2], luts[3], self.bench, time_c,
                                 luts[4], luts[5], luts[6], luts[7], self.bench, time_da,
                                 luts[8], luts[9], luts[10], luts[11], self.bench, time_db)
        self.time_c, self.time_da, self.time_db = time_c[0], time_da[0], time_db[0]
        return c


class Linear(torch.nn.Module):
    """y = x @ W with a block-sparse W of shape [in_features, out_features] (blocks [nnz, block, block]).

    The reference's constructor passes its arguments to MatMul in the wrong order (matmul.py:702) and cannot be
    instantiated; this one builds the dds product it meant.
    """

    def __init__(self, in_features, out_features, block, layout, bench=False):
        super(Linear, self).__init__()
        if layout.dim() == 2:
            layout = layout[None]
        if layout.shape[0] != 1 or layout.shape[1] * block != in_features or layout.shape[2] * block != out_features:
            raise ValueError('layout must be [1, in_features/block, out_features/block]')
        self.in_features = in_features
        self.out_features = out_features
        self.block = block
        self.weight = torch.nn.Parameter(torch.empty(int(layout.sum()), block, block))
        self.reset_parameters()
        self.matmul = MatMul(layout, block, 'dds', False, False, bench)

    def reset_parameters(self):
        torch.nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))

    def forward(self, input):
        shape = input.shape
        x = input.reshape(1, 1, -1, shape[-1])
        tokens = x.size(2)
        pad = (-tokens) % 16     # the weight gradient is an sdd product reducing over the tokens (multiple of 16)
        if pad:
            x = torch.cat((x, x.new_zeros(1, 1, pad, shape[-1])), dim=2)
        y = self.matmul(x, self.weight)[:, :, :tokens]
        return y.reshape(shape[:-1] + (self.out_features,))
