"""Benchmark of the hot path on one MI355X: fp16 block-64 sparse self-attention, forward + backward.

Workload (the configuration the headline metric is quoted on): batch 8, 16 heads, sequence 4096, head_dim 64,
block 64, fixed Sparse-Transformer layout (local window of 4 blocks + one global block column per 16 blocks,
causal), softmax scale 1/8 and an additive key-padding mask hiding the last 0-25% of the keys of each sequence.
One step = sdd(q, k^T) -> softmax -> dsd(p, v), then the backward pass (softmax backward and four matmuls).

Prints one JSON line.  `value` is the effective matmul throughput of the whole step: the FLOPs of the six
block-sparse products over their nonzero blocks (2*Z*64*nnz*64^2 each, the reference's formula,
tests/test_matmul.py:82-84) divided by the wall time of the full step, softmax included.  `kernels` lists every
launch of the step with its own HIP-event time, effective TFLOP/s or GB/s and roofline fractions; `roofline`
repeats the entry of the launch that takes the largest share of the step.  `cpu_baseline` is the same chain
computed by the fp32 dense-masked oracle on the host cores, on a slice of the batch.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, 'torch-blocksparse_amd')):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_PEAK_TFLOPS = 2500.0   # dense fp16 MFMA

# HBM bytes per launch at batch 8, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch), each scaled by what
# the same counter reads for the calibration copy of known size (profiles/attention_seq4096_fp16_blk64.txt).  None = not
# measured for this build of the kernel.
TRAFFIC_BYTES = {
    'sdd_fwd  q.k^T': 143501257 + 268435475, 'sdd_bwd  do.v^T': 143501257 + 268435475,
    'dsd_fwd  p.v': 362576945 + 67108868, 'dsd_bwd  ds.k': 362576945 + 67108868,
    'dsd_bwd  p^T.do': 403227301 + 67108864, 'dds_bwd  (q^T.ds)^T': 403227301 + 67108864,
    'softmax_fwd': 269842570 + 268435456, 'softmax_bwd': 538083047 + 268435456,
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=200)
    ap.add_argument('--warmup', type=int, default=30)
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--batch', type=int, default=8)
    ap.add_argument('--block', type=int, default=64, choices=[16, 32, 64],
                    help='config 3 only: express the same attention mask in smaller blocks (64 = the headline workload)')
    ap.add_argument('--config', type=int, default=3, choices=[1, 2, 3, 4, 5],
                    help='3 = the headline workload (default); 1, 2, 4, 5 = the other configurations, matmul/softmax launches timed one by one')
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit('bench.py measures one GPU: the path shards over batch and heads without communication, '
                 'and no multi-GPU run is part of this build (got --gpus %d)' % args.gpus)
    if args.config != 3:
        return other_config(args)

    import torch
    import torch_blocksparse as tb
    from torch_blocksparse.matmul import _sparse_matmul
    dev = torch.device('cuda:0')
    torch.manual_seed(0)
    B, H, L, dh, block = args.batch, 16, 4096, 64, args.block
    dtype = torch.float16
    scale = 0.125
    lay = tb.sparse_transformer_layout(H, L // 64, 4, 16, True)
    if block != 64:   # the same mask, every 64-block split into (64 / block)^2 blocks: same flops, same bytes
        lay = lay.repeat_interleave(64 // block, 1).repeat_interleave(64 // block, 2)
    nnz = int(lay.sum())
    q, k, v, do = [torch.randn(B, H, L, dh, dtype=dtype, device=dev) for _ in range(4)]
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    g = torch.Generator().manual_seed(1)
    kpm = torch.zeros(B, L, dtype=dtype)
    for z in range(B):
        pad = int(torch.randint(0, L // 4 + 1, (1,), generator=g))
        if pad:
            kpm[z, L - pad:] = float('-inf')
    kpm = kpm.to(dev)
    sdd = tb.MatMul(lay, block, 'sdd', trans_a=False, trans_b=True)
    dsd = tb.MatMul(lay, block, 'dsd')
    sm = tb.Softmax(lay, block)

    def step():
        q.grad = k.grad = v.grad = None
        w = sdd(q, k)
        p = sm(w, scale=scale, key_padding_mask=kpm)
        o = dsd(p, v)
        o.backward(do)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    flops_mm = 2.0 * B * dh * nnz * block * block          # per product (K = N = M = head_dim in all six)
    es = 2
    x_bytes = B * nnz * block * block * es
    dense_bytes = B * H * L * dh * es
    mm_bytes = x_bytes + 2 * dense_bytes                    # one sparse tensor + two dense tensors, each touched once

    # Per-launch timing with HIP events on the launch stream, the eight launches of a step issued back to back in
    # step order (so each kernel sees the cache state its predecessor leaves), K steps, one synchronisation at the end.
    luts = {m: m.make_lut(dtype, dev) for m in (sdd, dsd)}
    sm_lut, sm_maxlut = sm.make_lut(dev)
    t = [None]
    fn = _sparse_matmul.fn
    sl, dl = luts[sdd], luts[dsd]
    spd = lay.shape
    st = {}

    def k_sdd_fwd():
        st['w'] = fn['sdd'](q, k, False, True, False, spd, block, sl[0], sl[1], sl[2], sl[3], False, t)

    def k_softmax_fwd():
        st['p'] = tb.Softmax.sparse_softmax(st['w'], scale, None, kpm, None, 'add', 'add', spd, block, sm_lut, sm_maxlut, False, t)

    def k_dsd_fwd():
        st['o'] = fn['dsd'](st['p'], v, False, False, False, spd, block, dl[0], dl[1], dl[2], dl[3], False, t)

    def k_sdd_bwd():     # dp = do . v^T restricted to the layout
        st['dp'] = fn['sdd'](do, v, False, True, False, spd, block, dl[4], dl[5], dl[6], dl[7], False, t)

    def k_dsd_bwd_t():   # dv = p^T . do
        st['dv'] = fn['dsd'](st['p'], do, True, False, False, spd, block, dl[8], dl[9], dl[10], dl[11], False, t)

    def k_softmax_bwd():
        _bwd_softmax(tb, st['p'], st['dp'], scale, sm_lut, sm_maxlut, spd, block)

    def k_dsd_bwd():     # dq = ds . k
        st['dq'] = fn['dsd'](st['dp'], k, False, False, False, spd, block, sl[4], sl[5], sl[6], sl[7], False, t)

    def k_dds_bwd():     # dk = (q^T . ds)^T
        st['dk'] = fn['dds'](q, st['dp'], True, False, True, spd, block, sl[8], sl[9], sl[10], sl[11], False, t)

    def k_copy():        # plain copy of |x| bytes: the known-size kernel the traffic counters are calibrated on
        st['copy'] = st['dp'].clone()

    launches = [
        ('sdd_fwd  q.k^T', k_sdd_fwd, flops_mm, mm_bytes),
        ('softmax_fwd', k_softmax_fwd, 0.0, 2 * x_bytes + kpm.numel() * es),
        ('dsd_fwd  p.v', k_dsd_fwd, flops_mm, mm_bytes),
        ('dsd_bwd  p^T.do', k_dsd_bwd_t, flops_mm, mm_bytes),
        ('sdd_bwd  do.v^T', k_sdd_bwd, flops_mm, mm_bytes),
        ('softmax_bwd', k_softmax_bwd, 0.0, 3 * x_bytes),
        ('dds_bwd  (q^T.ds)^T', k_dds_bwd, flops_mm, mm_bytes),
        ('dsd_bwd  ds.k', k_dsd_bwd, flops_mm, mm_bytes),
        ('calibration_copy', k_copy, 0.0, 2 * x_bytes),
    ]
    reps = max(args.steps, 10)
    events = {name: [] for name, _, _, _ in launches}
    with torch.no_grad():
        for it in range(3 + reps):
            for name, f, _, _ in launches:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                f()
                e1.record()
                if it >= 3:
                    events[name].append((e0, e1))
    torch.cuda.synchronize()
    kernels = {}
    for name, _, flops, nbytes in launches:
        ms = sum(a.elapsed_time(b) for a, b in events[name]) / len(events[name])
        ent = {'ms': round(ms, 4), 'GB/s': round(nbytes / ms * 1e-6, 1), 'hbm_frac': round(nbytes / ms * 1e-6 / HBM_PEAK_GBS, 4),
               'bytes': nbytes, 'traffic': TRAFFIC_BYTES.get(name) if (B == 8 and block == 64) else None}
        if flops:
            ent['TFLOP/s'] = round(flops / ms * 1e-9, 2)
            ent['mfma_frac'] = round(flops / ms * 1e-9 / MFMA_PEAK_TFLOPS, 4)
        kernels[name] = ent
    calib = kernels.pop('calibration_copy')
    dom = max(kernels, key=lambda n: kernels[n]['ms'])
    roofline = {'kernel': dom, 'bound': 'hbm', 'achieved': kernels[dom]['GB/s'], 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
                'frac': kernels[dom]['hbm_frac'], 'traffic': kernels[dom]['traffic']}

    out = {
        'metric': 'effective TFLOP/s (nonzero blocks) sdd/dsd/dds + softmax GB/s, fp16 blk%d' % block,
        'value': round(6 * flops_mm / ms_per_step * 1e-9, 3), 'unit': 'TFLOP/s',
        'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': round(ms_per_step, 4),
        'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f16', 'data': 'synthetic',
        'config': {'workload': 'sparse self-attention fwd+bwd: batch %d, 16 heads, seq 4096, head_dim 64, block %d, fixed '
                               'layout (local 4 blocks + 1 global per 16 at block 64, causal), scale 1/8, additive key-padding mask' % (B, block),
                   'nnz_blocks': nnz, 'sum_of_kernel_ms': round(sum(e['ms'] for e in kernels.values()), 4)},
        'matmul_TFLOP/s_kernel_time_only': round(6 * flops_mm / sum(e['ms'] for n, e in kernels.items() if 'softmax' not in n) * 1e-9, 2),
        'softmax_GB/s': {'fwd': kernels['softmax_fwd']['GB/s'], 'bwd': kernels['softmax_bwd']['GB/s']},
        'roofline': roofline, 'kernels': kernels, 'calibration_copy': calib,
    }
    if not args.no_cpu_baseline:
        out['cpu_baseline'] = cpu_baseline(lay, block, dh, scale, L)
    print(json.dumps(out))


def other_config(args):
    """The configurations the headline metric is not quoted on: every launch timed on its own (HIP events, mean of
    `--steps` back-to-back launches), effective throughput over the nonzero blocks.  One JSON line, not the headline."""
    import torch
    import torch_blocksparse as tb
    dev = torch.device('cuda:0')
    out = []

    def timeit(f):
        for _ in range(max(args.warmup, 1)):
            f()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            f()
        e1.record()
        e1.synchronize()
        return e0.elapsed_time(e1) / args.steps

    def bernoulli(shape, density, seed, one_per_row=False):
        g = torch.Generator().manual_seed(seed)
        lay = (torch.rand(shape, generator=g) < density).long()
        if one_per_row:
            for h in range(shape[0]):
                for r in range(shape[1]):
                    if lay[h, r].sum() == 0:
                        lay[h, r, int(torch.randint(0, shape[2], (1,), generator=g))] = 1
        return lay

    def mm(name, mode, ta, tb_, block, dtype, Z, H, M, N, K, lay, scale=1.0):
        nnz = int(lay.sum())
        a = torch.randn((Z, H) + ((K, M) if ta else (M, K)), device=dev, dtype=dtype) * scale
        b = torch.randn((Z, H) + ((N, K) if tb_ else (K, N)), device=dev, dtype=dtype) * scale
        if mode == 'dsd':
            a = torch.randn(Z, nnz, block, block, device=dev, dtype=dtype)
        if mode == 'dds':
            b = torch.randn(Z, nnz, block, block, device=dev, dtype=dtype)
        op = tb.MatMul(lay, block, mode, trans_a=ta, trans_b=tb_)
        with torch.no_grad():
            ms = timeit(lambda: op(a, b))
        D = {'sdd': K, 'dsd': N, 'dds': M}[mode]
        fl = 2.0 * Z * D * nnz * block * block
        peak = 157.3 if dtype == torch.float32 else MFMA_PEAK_TFLOPS
        out.append({'launch': name, 'ms': round(ms, 4), 'TFLOP/s': round(fl / ms * 1e-9, 2), 'mfma_frac': round(fl / ms * 1e-9 / peak, 4)})

    if args.config == 1:
        torch.manual_seed(0)
        lay = torch.randint(0, 2, (2, 16, 32))
        mm('sdd trans_a fp32 blk16 Z4 H2 256x512x384', 'sdd', True, False, 16, torch.float32, 4, 2, 256, 512, 384, lay)
        x = torch.rand(4, int(lay.sum()), 16, 16, device=dev)
        sm = tb.Softmax(lay, 16)
        with torch.no_grad():
            ms = timeit(lambda: sm(x))
        out.append({'launch': 'softmax fwd fp32 blk16', 'ms': round(ms, 4), 'GB/s': round(2 * x.numel() * 4 / ms * 1e-6, 1)})
        workload = 'README shape: sdd trans_a fp32 block 16 + softmax'
    elif args.config == 2:
        lay = bernoulli((16, 64, 64), 0.25, 2, one_per_row=True)
        for ta in (False, True):
            for tb_ in (False, True):
                mm('dsd trans_a=%d trans_b=%d' % (ta, tb_), 'dsd', ta, tb_, 32, torch.float16, 8, 16, 2048, 2048, 2048, lay, 2048 ** -0.25)
                mm('dds trans_a=%d trans_b=%d' % (ta, tb_), 'dds', ta, tb_, 32, torch.float16, 8, 16, 2048, 2048, 2048, lay, 2048 ** -0.25)
        mm('sdd (gradient of the sparse operand)', 'sdd', False, True, 32, torch.float16, 8, 16, 2048, 2048, 2048, lay)
        workload = 'fp16 block 32, Z 8, H 16, M=N=K=2048, Bernoulli(0.25) layout'
    elif args.config == 5:
        lay = bernoulli((1, 32, 32), 0.1, 5)
        mm('dds trans_b (y = x.W^T)', 'dds', False, True, 128, torch.float16, 1, 1, 8192, 4096, 4096, lay, 0.1)
        mm('dds (dx = dy.W)', 'dds', False, False, 128, torch.float16, 1, 1, 8192, 4096, 4096, lay, 0.1)
        mm('sdd trans_a (dW = dy^T.x on the layout)', 'sdd', True, False, 128, torch.float16, 1, 1, 4096, 4096, 8192, lay, 0.1)
        workload = 'block-sparse linear layer: 8192 tokens, 4096x4096 weight, block 128, 10 % density, fp16'
    else:
        lay = tb.bigbird_layout(12, 256, 3, 2, 3, seed=0, causal=True)
        B, H, L, dh, block = 2, 12, 16384, 64, 64
        nnz = int(lay.sum())
        q, k, v = [torch.randn(B, H, L, dh, device=dev, dtype=torch.float16) for _ in range(3)]
        sdd = tb.MatMul(lay, block, 'sdd', trans_b=True)
        dsd = tb.MatMul(lay, block, 'dsd')
        sm = tb.Softmax(lay, block)
        nb = L // block
        idx = torch.arange(nb)
        rpe_bb = (0.1 * torch.randn(nb)).half()[(idx[:, None] - idx[None, :]).abs()].to(dev)
        rpe = rpe_bb.repeat_interleave(block, 0).repeat_interleave(block, 1)[None, None].expand(B, H, L, L)
        causal = torch.tril(torch.ones(L, L, dtype=torch.float16, device=dev))
        fl = 2.0 * B * dh * nnz * block * block
        xb = B * nnz * block * block * 2
        do = torch.randn_like(q)
        from torch_blocksparse.matmul import _sparse_matmul
        fn, spd, t = _sparse_matmul.fn, lay.shape, [None]
        sl, dl = sdd.make_lut(torch.float16, dev), dsd.make_lut(torch.float16, dev)   # (c, da, db) tables of each op
        sm_lut, sm_maxlut = sm.make_lut(dev)
        with torch.no_grad():
            w = sdd(q, k)
            dw = torch.randn_like(w)
            for name, f, flops, nbytes in (
                    ('sdd q.k^T', lambda: sdd(q, k), fl, xb + 2 * B * H * L * dh * 2),
                    ('softmax fwd, scale only', lambda: sm(w, scale=0.125), 0, 2 * xb),
                    ('softmax fwd, rpe + causal mask', lambda: sm(w, scale=0.125, rpe=rpe, attn_mask=causal, attn_mask_mode='mul'), 0, 2 * xb),   # x only: both masks are shared by batch and heads
                    ('dsd p.v', lambda: dsd(w, v), fl, xb + 2 * B * H * L * dh * 2),
                    # backward, in the order autograd runs it (the products of MatMul.backward are MatMul modes of their own)
                    ('dsd p^T.do', lambda: fn['dsd'](w, do, True, False, False, spd, block, dl[8], dl[9], dl[10], dl[11], False, t), fl, xb + 2 * B * H * L * dh * 2),
                    ('sdd do.v^T', lambda: fn['sdd'](do, v, False, True, False, spd, block, dl[4], dl[5], dl[6], dl[7], False, t), fl, xb + 2 * B * H * L * dh * 2),
                    ('softmax bwd', lambda: _bwd_softmax(tb, w, dw, 0.125, sm_lut, sm_maxlut, spd, block), 0, 3 * xb),
                    ('dds (q^T.ds)^T', lambda: fn['dds'](q, dw, True, False, True, spd, block, sl[8], sl[9], sl[10], sl[11], False, t), fl, xb + 2 * B * H * L * dh * 2),
                    ('dsd ds.k', lambda: fn['dsd'](dw, k, False, False, False, spd, block, sl[4], sl[5], sl[6], sl[7], False, t), fl, xb + 2 * B * H * L * dh * 2)):
                ms = timeit(f)
                ent = {'launch': name, 'ms': round(ms, 4), 'GB/s': round(nbytes / ms * 1e-6, 1), 'hbm_frac': round(nbytes / ms * 1e-6 / HBM_PEAK_GBS, 4)}
                if flops:
                    ent['TFLOP/s'] = round(flops / ms * 1e-9, 2)
                out.append(ent)
        workload = 'BigBird layout (3 window + 2 global + 3 random blocks, causal), batch 2, 12 heads, seq 16384, head_dim 64, block 64, fp16, forward and backward launches'
    print(json.dumps({'metric': 'per-launch effective throughput (nonzero blocks), not the headline metric', 'n_gpus': 1,
                      'steps': args.steps, 'warmup': args.warmup, 'data': 'synthetic', 'config': {'workload': workload, 'config': args.config},
                      'launches': out}))


def _bwd_softmax(tb, y, dy, scale, lut, maxlut, spdims, block):
    import ctypes
    from torch_blocksparse import _lib
    rc = _lib.load().bsp_softmax_bwd(_lib.DTYPES[y.dtype], _lib.ptr(y), _lib.ptr(dy), float(scale), _lib.ptr(lut), maxlut,
                                     y.size(0), spdims[0], spdims[1], block, y.stride(0), dy.stride(0), _lib.stream_ptr(y.device))
    _lib.check(rc, 'bsp_softmax_bwd')


def cpu_baseline(lay, block, dh, scale, L):
    """The reference's CPU path = its test oracle: dense fp32 matmuls + layout mask + dense softmax, forward and
    backward (oracle/dense_oracle.py).  Timed on the same workload, one sequence at a time (the dense score tensors
    of one sequence are ~1 GB each), repeating the sequence-sized pass for about 12 s."""
    import torch
    from oracle import dense_oracle as D
    torch.manual_seed(0)
    H = lay.shape[0]
    kpm = torch.zeros(1, L)
    kpm[0, L - L // 8:] = float('-inf')
    q, k, v, do = [torch.randn(1, H, L, dh) for _ in range(4)]
    D.attention(q[:, :1], k[:, :1], v[:, :1], lay[:1], block, scale, key_padding_mask=kpm, do=do[:, :1])   # warm-up
    done, t0 = 0, time.perf_counter()
    while done < 24 and time.perf_counter() - t0 < 12.0:
        D.attention(q, k, v, lay, block, scale, key_padding_mask=kpm, do=do)
        done += 1
    dt = time.perf_counter() - t0
    flops = 6 * 2.0 * done * dh * int(lay.sum()) * block * block
    return {'value': round(flops / dt * 1e-12, 5), 'unit': 'TFLOP/s', 'cores': torch.get_num_threads(), 'kind': 'port',
            'sample': 'same chain fwd+bwd, %d sequence-sized passes (1 sequence = 16 heads x seq 4096; the workload has 8), fp32 dense matmul + mask + softmax, '
                      '%.1f s; throughput counts only the nonzero-block FLOPs, like the GPU figure' % (done, dt)}


if __name__ == '__main__':
    main()
