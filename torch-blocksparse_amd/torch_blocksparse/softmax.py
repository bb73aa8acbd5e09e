"""Block-sparse softmax (forward + backward) on MI355X.

Drop-in for the reference's torch_blocksparse/softmax.py: `Softmax(layout, block, bench)` and
`softmax(x, scale, rpe, key_padding_mask, attn_mask, key_padding_mask_mode, attn_mask_mode)`, in place on x,
same look-up table (softmax.py:201-221, built on the GPU), same autograd behaviour (softmax.py:253-326).
"""
import ctypes

import torch

from . import _lib
from .matmul import _Timer


_PRIVATE_USE_COUNT = None


def _private_use_count():
    """How many owners the autograd engine itself gives a gradient that nobody else holds, as seen from inside a custom
    backward: measured once with a two-element CPU graph rather than assumed."""
    global _PRIVATE_USE_COUNT
    if _PRIVATE_USE_COUNT is None:
        seen = []

        class Probe(torch.autograd.Function):
            @staticmethod
            def forward(ctx, t):
                return t * 1.0

            @staticmethod
            def backward(ctx, g):
                seen.append(g._use_count() if hasattr(g, '_use_count') else 0)
                return g * 1.0
        t = torch.ones(2, requires_grad=True)
        with torch.enable_grad():
            (Probe.apply(t) * 3.0).sum().backward()        # the gradient is a fresh tensor made by the multiplication's backward
        _PRIVATE_USE_COUNT = seen[0] if seen else 0
    return _PRIVATE_USE_COUNT


def _storage_owners(g):
    """How many tensors share g's storage (g itself counts), or a large number when that cannot be told."""
    try:
        return int(torch._C._storage_Use_Count(g.untyped_storage()._cdata))
    except Exception:
        return 1 << 30


_PRIVATE_STORAGE_COUNT = None


def _gradient_is_private(g):
    """True when no one but the autograd engine holds g (then overwriting it cannot be observed): neither the tensor
    object (its own reference count), nor a view of it, nor its storage through another tensor object such as
    `g.detach()` or `g.data`, which share the memory but have no base."""
    global _PRIVATE_STORAGE_COUNT
    base = _private_use_count()
    if not (base > 0 and hasattr(g, '_use_count') and g._use_count() <= base and g._base is None):
        return False
    if _PRIVATE_STORAGE_COUNT is None:
        _PRIVATE_STORAGE_COUNT = _storage_owners(torch.ones(2))      # what a tensor nobody shares reads
    return _storage_owners(g) <= _PRIVATE_STORAGE_COUNT


class _sparse_softmax(torch.autograd.Function):
    in_place_backwards = 0          # backward calls that overwrote their (private) incoming gradient; tests read it

    @staticmethod
    def make_lut(layout, block, device):
        """-> (lut int32 on device, maxlut) as the reference (softmax.py:201-221)."""
        lib = _lib.load()
        dev = torch.device(device)
        lay = _lib.layout_to_device(layout, dev)
        H, R, C = lay.shape
        ws, ws_bytes = _lib.workspace(lay, dev)
        cap = 2 * H * R + 4 * int((layout != 0).sum())
        lut = torch.empty((max(cap, 1),), dtype=torch.int32, device=dev)
        n = ctypes.c_int64(0)
        maxlut = ctypes.c_int(0)
        rc = lib.bsp_softmax_lut_build(_lib.ptr(lay), H, R, C, _lib.ptr(lut), cap, _lib.ptr(ws), ws_bytes, ctypes.byref(n),
                                       ctypes.byref(maxlut), _lib.stream_ptr(dev))
        _lib.check(rc, 'bsp_softmax_lut_build')
        return lut[:n.value], int(maxlut.value)

    @staticmethod
    def _check_rows(maxlut, block):
        if maxlut * block >= 32768:                        # softmax.py:225-227
            raise NotImplementedError('Reductions larger than 32768 elements are not yet implemented')

    @staticmethod
    def _check_shapes(x, rpe, key_padding_mask, attn_mask, spdims, block, nnz):
        """Operand extents against the layout.  The kernels take every address from the table (block id, block-row,
        block-column, head), so a tensor that is too small would be read or written out of bounds on the device."""
        H, R, C = spdims
        if x.dim() != 4 or x.size(1) != nnz or tuple(x.shape[2:]) != (block, block):
            raise ValueError('softmax input must be [batch, %d, %d, %d] for this layout, got %s' % (nnz, block, block, tuple(x.shape)))
        Z = x.size(0)
        if key_padding_mask is not None:
            if key_padding_mask.dim() != 2 or key_padding_mask.size(0) not in (1, Z) or key_padding_mask.size(1) < C * block:
                raise ValueError('key_padding_mask must be [%d or 1, >= %d], got %s' % (Z, C * block, tuple(key_padding_mask.shape)))
        if attn_mask is not None:
            if attn_mask.dim() != 2 or attn_mask.size(0) < R * block or attn_mask.size(1) < C * block:
                raise ValueError('attn_mask must be at least [%d, %d], got %s' % (R * block, C * block, tuple(attn_mask.shape)))
        if rpe is not None:
            shape = (1,) * (4 - rpe.dim()) + tuple(rpe.shape)
            if len(shape) != 4 or shape[0] not in (1, Z) or shape[1] not in (1, H) or shape[2] < R * block or shape[3] < C * block:
                raise ValueError('rpe must broadcast to [%d, %d, >= %d, >= %d], got %s' % (Z, H, R * block, C * block, tuple(rpe.shape)))

    @staticmethod
    def _strided16(t, what):
        """Masks are read with vector loads: unit inner stride, 16-byte aligned rows."""
        v = 4 if t.dtype == torch.float32 else 8
        if t.stride(-1) != 1 and t.size(-1) != 1:
            t = t.contiguous()
        if t.data_ptr() % 16 != 0 or any(s % v for s in t.stride()[:-1]):
            t = t.contiguous()
            if t.data_ptr() % 16 != 0:
                t = t.clone()
        return t

    @staticmethod
    def forward(ctx, x, scale, rpe, key_padding_mask, attn_mask, kp_mask_mode, attn_mask_mode,
                spdims, block, lut, maxlut, bench, time, dropout=None):
        _lib.require_gpu_tensor(x, 'softmax input')
        if x.dtype not in _lib.DTYPES:
            raise ValueError('softmax input must be float16, bfloat16 or float32')
        if not x.is_contiguous():
            raise ValueError('softmax works in place on a contiguous [Z, nnz, block, block] tensor')
        _sparse_softmax._check_rows(maxlut, block)
        _sparse_softmax._check_shapes(x, rpe, key_padding_mask, attn_mask, spdims, block, (lut.numel() - 2 * spdims[0] * spdims[1]) // 4)
        null = ctypes.c_void_p(0)
        rpe_args = (null, 0, 0, 0)
        if rpe is not None:                                # element (z, h, r, c), softmax.py:50-55, 265
            while rpe.dim() < 4:
                rpe = rpe.unsqueeze(0)
            rpe = _sparse_softmax._strided16(rpe.expand(x.size(0), spdims[0], rpe.size(2), rpe.size(3)), 'rpe')
            rpe_args = (_lib.ptr(rpe), rpe.stride(0), rpe.stride(1), rpe.stride(2))
        kpm_args = (null, 0)
        if key_padding_mask is not None:                   # element (z, c), softmax.py:60-62, 274
            key_padding_mask = _sparse_softmax._strided16(key_padding_mask, 'key_padding_mask')
            kpm_args = (_lib.ptr(key_padding_mask), key_padding_mask.stride(0) if key_padding_mask.size(0) > 1 else 0)
        attn_args = (null, 0)
        if attn_mask is not None:                          # element (r, c), softmax.py:67-70, 283
            attn_mask = _sparse_softmax._strided16(attn_mask, 'attn_mask')
            attn_args = (_lib.ptr(attn_mask), attn_mask.stride(0))
        timer = _Timer(bench, x.device)
        common = (rpe_args[0], rpe_args[1], rpe_args[2], rpe_args[3],
                  kpm_args[0], kpm_args[1], int(kp_mask_mode == 'mul'),
                  attn_args[0], attn_args[1], int(attn_mask_mode == 'mul'),
                  x.size(0), spdims[0], spdims[1], block, x.stride(0))
        ctx.dropout = dropout
        if dropout is None:
            rc = _lib.load().bsp_softmax_fwd(_lib.DTYPES[x.dtype], _lib.ptr(x), float(scale), _lib.ptr(lut), maxlut, *common,
                                             _lib.stream_ptr(x.device))
            _lib.check(rc, 'bsp_softmax_fwd')
            out = x
            ctx.mark_dirty(x)
        else:
            # x keeps the softmax itself (the backward pass needs it), the dropped copy is a tensor of its own; the mask is
            # a function of (seed, offset, element), re-created in the backward pass
            p, seed, offset = dropout
            out = torch.empty_like(x)
            rc = _lib.load().bsp_softmax_dropout_fwd(_lib.DTYPES[x.dtype], _lib.ptr(x), _lib.ptr(out), float(scale), _lib.ptr(lut), maxlut,
                                                     *common, out.stride(0), float(p), int(seed), int(offset), _lib.stream_ptr(x.device))
            _lib.check(rc, 'bsp_softmax_dropout_fwd')
            ctx.mark_dirty(x)      # x now holds the softmax: autograd must know, as on the path without dropout
        time[0] = timer.done()
        ctx.save_for_backward(x, lut)
        ctx.spdims, ctx.block, ctx.maxlut, ctx.scale = spdims, block, maxlut, scale
        return out if dropout is None else (out, x)

    @staticmethod
    def backward(ctx, dx, dy_plain=None):
        """dx: gradient of the (dropped) result; dy_plain: with dropout, the gradient of the second output, the softmax
        itself that x was overwritten with (None unless the caller went on using x).
        The kernel computes the gradient in place, as the reference does on every incoming gradient (softmax.py:316-325).
        Here that happens only when the incoming tensor is private to this call: a gradient that something else still
        holds (the tensor the user handed to backward(), a gradient that an addition passes to two branches) is copied
        first, so nobody else sees it change."""
        x, lut = ctx.saved_tensors
        if dx is None:             # with dropout: only the softmax left in x was used
            dx = torch.zeros_like(x)
        if dx.shape != x.shape:
            raise ValueError('softmax gradient has shape %s, the output has %s' % (tuple(dx.shape), tuple(x.shape)))
        private = _gradient_is_private(dx)
        dx = dx.contiguous()
        if dx.data_ptr() % 16 != 0 or not private:
            dx = torch.empty_like(dx).copy_(dx)
        _sparse_softmax.in_place_backwards += int(private)
        args = (_lib.DTYPES[x.dtype], _lib.ptr(x), _lib.ptr(dx), float(ctx.scale), _lib.ptr(lut), ctx.maxlut, x.size(0),
                ctx.spdims[0], ctx.spdims[1], ctx.block, x.stride(0), dx.stride(0))
        if ctx.dropout is None:
            rc = _lib.load().bsp_softmax_bwd(*args, _lib.stream_ptr(x.device))
        else:
            p, seed, offset = ctx.dropout
            rc = _lib.load().bsp_softmax_dropout_bwd(*args, float(p), int(seed), int(offset), _lib.stream_ptr(x.device))
        _lib.check(rc, 'bsp_softmax_bwd')
        if dy_plain is not None:
            extra = torch.empty_like(x).copy_(dy_plain)
            rc = _lib.load().bsp_softmax_bwd(*(args[:2] + (_lib.ptr(extra),) + args[3:-1] + (extra.stride(0),)), _lib.stream_ptr(x.device))
            _lib.check(rc, 'bsp_softmax_bwd')
            dx = dx + extra
        return (dx,) + (None,) * 13


class Softmax:
    """softmax over each row of a block-sparse matrix, restricted to the row's nonzero blocks."""

    sparse_softmax = _sparse_softmax.apply

    def make_lut(self, device):
        key = (device,)
        if key not in self.lut_cache:
            self.lut_cache[key] = _sparse_softmax.make_lut(self.layout, self.block, device)
        return self.lut_cache[key]

    def __init__(self, layout, block, bench=False):
        if block not in (16, 32, 64, 128):
            raise ValueError('block must be 16, 32, 64 or 128')
        self.spdims = layout.shape
        self.layout = layout
        self.block = block
        self.bench = bench
        self.lut_cache = dict()
        self.time_y = None

    def __call__(self, x, scale=1., rpe=None, key_padding_mask=None, attn_mask=None,
                 key_padding_mask_mode='add', attn_mask_mode='add', dropout_p=0., dropout_seed=None, dropout_offset=0):
        """The reference's arguments (softmax.py:345-361), plus dropout on the result (not in the reference): with
        dropout_p > 0 the result is softmax(...) * mask / (1 - p) in a new tensor (x itself still receives the softmax).
        The mask is a counter-based function of (dropout_seed, dropout_offset, element); the seed is drawn from
        torch's default generator when not given, so torch.manual_seed makes a run repeatable."""
        time_y = [None]
        if rpe is not None and rpe.dtype != x.dtype:
            raise ValueError('relative position embedding must be %s' % x.dtype)
        if attn_mask is not None and attn_mask.dtype != x.dtype:
            raise ValueError('Attention mask must be %s' % x.dtype)
        if key_padding_mask is not None and key_padding_mask.dtype != x.dtype:
            raise ValueError('Key padding mask must be %s' % x.dtype)
        if not 0. <= dropout_p < 1.:
            raise ValueError('dropout probability must be in [0, 1), got %r' % (dropout_p,))
        _lib.require_gpu_tensor(x, 'softmax input')
        lut, maxlut = self.make_lut(x.device)
        dropout = None
        if dropout_p > 0.:
            seed = int(torch.randint(0, 2 ** 62, (1,)).item()) if dropout_seed is None else int(dropout_seed)
            dropout = (float(dropout_p), seed, int(dropout_offset))
        x = Softmax.sparse_softmax(x, scale, rpe, key_padding_mask, attn_mask, key_padding_mask_mode, attn_mask_mode,
                                   self.spdims, self.block, lut, maxlut, self.bench, time_y, dropout)
        self.time_y = time_y[0]
        return x if dropout is None else x[0]
