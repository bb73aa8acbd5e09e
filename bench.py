"""Benchmark of the hot path on one MI355X: fp16 block-64 sparse self-attention, forward + backward.

Workload (the configuration the headline metric is quoted on): batch 8, 16 heads, sequence 4096, head_dim 64,
block 64, fixed Sparse-Transformer layout (local window of 4 blocks + one global block column per 16 blocks,
causal), softmax scale 1/8 and an additive key-padding mask hiding the last 0-25% of the keys of each sequence.
One step = sdd(q, k^T) -> softmax -> dsd(p, v), then the backward pass (softmax backward and four matmuls).

Prints one JSON line.  `value` is the effective matmul throughput of the whole step: the FLOPs of the six
block-sparse products over their nonzero blocks (2*Z*64*nnz*64^2 each, the reference's formula,
tests/test_matmul.py:82-84) divided by the wall time of the full step, softmax included.  `kernels` lists every
launch of the step with its own HIP-event time, effective TFLOP/s or GB/s and roofline fractions; `roofline` is the
kernel that takes the largest share of the step (all its launches together).  `other_configs` holds the per-launch
figures of the other benchmark configurations (block-32 dsd/dds round trip, long-context BigBird attention,
block-128 sparse linear layer).  `cpu_baseline` is the same chain computed by the fp32 dense-masked oracle on the host
cores, on a slice of the batch.

Other modes:  --config N        one of the other configurations alone (one JSON line, not the headline)
              --calibrate       what this box streams: read / write / copy / in-place / 1r:2w probes at 4 GiB and at the
                                step's 268 MB footprint, and the step's launches with the caches flushed before each
              --record-traffic  turn two rocprofv3 --pmc runs of this script (FETCH_SIZE, WRITE_SIZE) into the file that
                                `traffic` in the JSON line is read from
"""
import argparse
import ctypes
import glob
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.join(ROOT, 'torch-blocksparse_amd')
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_PEAK_TFLOPS = 2500.0   # dense fp16 MFMA
FP32_PEAK_TFLOPS = 157.3    # fp32 matrix

TRAFFIC_FILE = os.path.join(ROOT, 'profiles', 'traffic_attention_seq4096_fp16_blk64.json')

SETTLE_STEPS = 30         # untimed steps in front of the warm-up steps (see main)

# kernel behind each launch of the step, for the per-kernel totals (the headline block size; kernel_of() for the others)
KERNEL_OF = {
    'sdd_fwd  q.k^T': 'k_sdd64_rg', 'sdd_bwd  do.v^T': 'k_sdd64_rg',
    'dsd_fwd  p.v': 'k_xsd64_rg<sparse operand as stored>', 'dsd_bwd  ds.k': 'k_xsd64_rg<sparse operand as stored>',
    'dsd_bwd  p^T.do': 'k_xsd64_rg<sparse operand transposed>', 'dds_bwd  (q^T.ds)^T': 'k_xsd64_rg<sparse operand transposed>',
    'softmax_fwd': 'k_softmax_fwd', 'softmax_bwd': 'k_softmax_bwd',
}


def kernel_of(block):
    """--block 32 runs the one-member-per-wavefront kernels, --block 16 the block-64 kernels on gathered 4 x 4 tiles."""
    if block == 64:
        return KERNEL_OF
    def ren(k):
        if block == 32:
            return k.replace('k_sdd64_rg', 'k_sdd_rg_small').replace('k_xsd64_rg', 'k_xsd_rg_small')
        if '64_rg' not in k:
            return k
        return k.replace('>', ', tiles of 4 x 4 blocks>') if '<' in k else k + '<tiles of 4 x 4 blocks>'
    return {name: ren(k) for name, k in KERNEL_OF.items()}


def kernel_sources_sha():
    """Hash of the HIP sources the library is built from: ties recorded counter readings to a build of the kernels."""
    h = hashlib.sha256()
    for f in sorted(glob.glob(os.path.join(PKG, 'csrc', '*'))):
        if f.endswith(('.hip', '.h')) and not f.endswith('probe.hip'):
            h.update(os.path.basename(f).encode())
            h.update(open(f, 'rb').read())
    return h.hexdigest()


def recorded_traffic():
    """HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (profiles/), or {} when the kernels' sources have
    changed since the counters were read (the figure would describe other kernels)."""
    try:
        rec = json.load(open(TRAFFIC_FILE))
    except (OSError, ValueError):
        return {}
    return rec.get('bytes_per_launch', {}) if rec.get('kernel_sources_sha256') == kernel_sources_sha() else {}


def recorded_kernel_traffic(kernel):
    """HBM bytes per launch of one kernel from the same record (None when absent or stale)."""
    try:
        rec = json.load(open(TRAFFIC_FILE))
    except (OSError, ValueError):
        return None
    return rec.get('bytes_per_kernel_launch', {}).get(kernel) if rec.get('kernel_sources_sha256') == kernel_sources_sha() else None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=200)
    ap.add_argument('--warmup', type=int, default=30)
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--no-other-configs', action='store_true', help='headline only: skip configurations 2, 4 and 5')
    ap.add_argument('--batch', type=int, default=8)
    ap.add_argument('--block', type=int, default=64, choices=[16, 32, 64],
                    help='config 3 only: express the same attention mask in smaller blocks (64 = the headline workload)')
    ap.add_argument('--config', default='3', choices=['1', '2', '3', '4', '5', 'ref'],
                    help='3 = the headline workload (default); 1, 2, 4, 5 = the other configurations, matmul/softmax launches timed one by one; '
                         'ref = the shapes of the reference\'s own benchmark functions (tests/test_matmul.py:105-122, tests/test_softmax.py:92-128)')
    ap.add_argument('--dtype', default='f16', choices=['f16', 'bf16'], help='config 3 only: the 16-bit type of the workload (the headline is quoted on f16)')
    ap.add_argument('--calibrate', action='store_true')
    ap.add_argument('--kernel-flags', type=int, default=0,
                    help='--config runs only: the flags argument of the matmul launchers (include/bsp.h: 1 general kernels only, '
                         '2 no group plans, 4 no direct-to-LDS kernels), to time one kernel family against another')
    ap.add_argument('--record-traffic', nargs=2, metavar=('FETCH_DIR', 'WRITE_DIR'))
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit('bench.py measures one GPU: the path shards over batch and heads without communication, '
                 'and no multi-GPU run is part of this build (got --gpus %d)' % args.gpus)
    if args.record_traffic:
        return record_traffic(*args.record_traffic)
    if args.calibrate:
        return calibrate(args)
    if args.config != 'ref':
        args.config = int(args.config)
    if args.kernel_flags and args.config == 3:
        sys.exit('--kernel-flags is for --config 1|2|4|5 runs: the headline figure is always taken with the default kernels')
    if args.config != 3:
        from torch_blocksparse import matmul as _mm
        _mm.KERNEL_FLAGS = args.kernel_flags
        if args.config == 'ref':
            res = reference_bench_shapes(min(args.steps, 50), max(1, min(args.warmup, 5)))
        else:
            res = other_config(args.config, min(args.steps, 50), max(1, min(args.warmup, 5)))
        print(json.dumps({'metric': 'per-launch effective throughput (nonzero blocks), not the headline metric', 'n_gpus': 1,
                          'steps': args.steps, 'warmup': args.warmup, 'data': 'synthetic',
                          'config': {'workload': res['workload'], 'config': args.config, 'kernel_flags': args.kernel_flags},
                          'launches': res['launches'], **({'ms_per_step': res['ms_per_step']} if 'ms_per_step' in res else {})}))
        return

    import torch
    import torch_blocksparse as tb
    w = Attention(args.batch, args.block, args.dtype)
    step = w.step
    # The literal reading of the command line first: W warm-up steps and K timed steps on a GPU that has done nothing
    # else in this process (tables built, no settle steps, no per-launch pass before).  Reported as
    # `ms_per_step_first_window`; `ms_per_step` further down is the steady state.
    import gc
    gc.collect()
    gc.disable()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_first_window = (time.perf_counter() - t0) * 1e3 / args.steps
    # Per-launch timing with HIP events on the launch stream, the eight launches of a step issued back to back in
    # step order (so each kernel sees the cache state its predecessor leaves), K steps, one synchronisation at the end.
    launches = w.launches() + [('calibration_copy', w.k_copy, 0.0, 2 * w.x_bytes)]
    # No garbage collection inside the measured regions: a full collection stops the host for tens of milliseconds, the
    # launch queue runs dry, and the idle time lands between the two events of whichever launch comes next.
    import gc
    gc.collect()
    gc.disable()
    reps = max(args.steps, 50)                    # at least ~40 ms of work: past the power-management transient that follows an idle GPU
    events = {name: [] for name, _, _, _ in launches}
    with torch.no_grad():
        for it in range(10 + reps):                  # the first ten passes are not recorded
            for name, f, _, _ in launches:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                f()
                e1.record()
                if it >= 10:
                    events[name].append((e0, e1))
    torch.cuda.synchronize()
    # The step itself: W untimed steps, then exactly K steps between two synchronisations.  (The per-launch pass above
    # runs first so that clocks, caches and the allocator are in their steady state whatever W is.)
    # After any change of the launch pattern (an idle GPU, or the per-launch pass above) the step time needs about 25
    # steps to settle (0.63 -> 0.59 ms here, the GPU's power management): SETTLE_STEPS more untimed steps in front of the
    # W warm-up steps, so that the K timed steps measure the steady state whatever W is.  Reported as config.settle_steps.
    for _ in range(SETTLE_STEPS):
        step()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    gc.enable()

    traffic = recorded_traffic() if (args.batch == 8 and args.block == 64 and args.dtype == 'f16') else {}
    kernels = {}
    stalls = 0
    for name, _, flops, nbytes in launches:
        # mean over the passes; a sample more than three times the median is not a launch duration but a launch that the
        # GPU had to wait for (the host was held up: the events bracket the wait too) and is left out, and counted
        samples = sorted(a.elapsed_time(b) for a, b in events[name])
        kept = [t for t in samples if t <= 3.0 * samples[len(samples) // 2]]
        stalls += len(samples) - len(kept)
        ms = sum(kept) / len(kept)
        ent = {'ms': round(ms, 4), 'GB/s': round(nbytes / ms * 1e-6, 1), 'hbm_frac': round(nbytes / ms * 1e-6 / HBM_PEAK_GBS, 4),
               'bytes': nbytes, 'traffic': traffic.get(name)}
        if flops:
            ent['TFLOP/s'] = round(flops / ms * 1e-9, 2)
            ent['mfma_frac'] = round(flops / ms * 1e-9 / MFMA_PEAK_TFLOPS, 4)
        kernels[name] = ent
    calib = kernels.pop('calibration_copy')
    # the dominant kernel = the one with the largest total time per step over all its launches
    per_kernel = {}
    for name, ent in kernels.items():
        k = per_kernel.setdefault(kernel_of(args.block)[name], {'launches_per_step': 0, 'ms_per_step': 0.0, 'bytes': 0, 'traffic': 0, 'have_traffic': True})
        k['launches_per_step'] += 1
        k['ms_per_step'] += ent['ms']
        k['bytes'] += ent['bytes']
        k['have_traffic'] = k['have_traffic'] and ent['traffic'] is not None
        k['traffic'] += ent['traffic'] or 0
    dom = max(per_kernel, key=lambda n: per_kernel[n]['ms_per_step'])
    d = per_kernel[dom]
    n_l = d['launches_per_step']
    avg_ms = d['ms_per_step'] / n_l
    achieved = d['bytes'] / n_l / avg_ms * 1e-6
    roofline = {'kernel': dom, 'launches_per_step': n_l, 'avg_launch_ms': round(avg_ms, 4), 'bound': 'hbm',
                'achieved': round(achieved, 1), 'peak': HBM_PEAK_GBS, 'unit': 'GB/s', 'frac': round(achieved / HBM_PEAK_GBS, 4),
                'traffic': (d['traffic'] // n_l) if d['have_traffic'] else None,
                'share_of_step': round(d['ms_per_step'] / sum(k['ms_per_step'] for k in per_kernel.values()), 4)}

    block, B = args.block, args.batch
    out = {
        'metric': 'effective TFLOP/s (nonzero blocks) sdd/dsd/dds + softmax GB/s, %s blk%d' % ({'f16': 'fp16', 'bf16': 'bf16'}[args.dtype], block),
        'value': round(6 * w.flops_mm / ms_per_step * 1e-9, 3), 'unit': 'TFLOP/s',
        'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': round(ms_per_step, 4),
        'ms_per_step_first_window': round(ms_first_window, 4),
        'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None, 'dtype': args.dtype, 'data': 'synthetic',
        'config': {'workload': 'sparse self-attention fwd+bwd: batch %d, 16 heads, seq 4096, head_dim 64, block %d, fixed '
                               'layout (local 4 blocks + 1 global per 16 at block 64, causal), scale 1/8, additive key-padding mask' % (B, block),
                   'nnz_blocks': w.nnz, 'sum_of_kernel_ms': round(sum(e['ms'] for e in kernels.values()), 4),
                   'per_launch_samples_left_out_as_host_stalls': stalls, 'settle_steps': SETTLE_STEPS},
        'matmul_TFLOP/s_kernel_time_only': round(6 * w.flops_mm / sum(e['ms'] for n, e in kernels.items() if 'softmax' not in n) * 1e-9, 2),
        'softmax_GB/s': {'fwd': kernels['softmax_fwd']['GB/s'], 'bwd': kernels['softmax_bwd']['GB/s']},
        'roofline': roofline, 'kernels': kernels, 'calibration_copy': calib,
        'traffic_source': os.path.relpath(TRAFFIC_FILE, ROOT) if traffic else None,
    }
    if True:
        # not the headline: the same workload through the call the attention modules make, which takes the fused kernels
        ms_fused = fused_chain_step(w, args.steps, args.warmup)
        if ms_fused is not None:
            def timeit(f, reps=max(20, min(args.steps, 100))):
                for _ in range(5):
                    f()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(reps):
                    f()
                e1.record()
                e1.synchronize()
                return e0.elapsed_time(e1) / reps
            out['fused_attention_chain'] = {
                'what': 'attention_chain(sdd, softmax, dsd, q, k, v): bsp_attention_fwd, then in the backward pass bsp_attention_bwd (dq) '
                        'and bsp_attention_bwd_kv (dk, dv; the softmax gradient is computed twice and never stored); same workload, '
                        'flop count of the six products of the three-operator chain',
                'ms_per_step': round(ms_fused, 4), 'TFLOP/s': round(6 * w.flops_mm / ms_fused * 1e-9, 3),
                'vs_three_operators': round(ms_per_step / ms_fused, 3),
                'launches': fused_chain_launches(w.lay, w.q.detach(), w.k.detach(), w.v.detach(), w.do, w.scale, timeit,
                                                 [('additive key-padding mask', dict(key_padding_mask=w.kpm))], block)}
            if traffic:
                for ent in out['fused_attention_chain']['launches']:
                    ent['roofline']['traffic'] = recorded_kernel_traffic(ent['roofline']['kernel'])
    lay, dh, scale = w.lay, w.dh, w.scale
    del w
    torch.cuda.empty_cache()
    if not args.no_other_configs:
        out['other_configs'] = {str(c): other_config(c, 20, 3) for c in (2, 4, 5)}
        out['other_configs']['module default'] = module_default_config(20, 5)
    if not args.no_cpu_baseline:
        out['cpu_baseline'] = cpu_baseline(lay, block, dh, scale, 4096)
    print(json.dumps(out))


class Attention:
    """The headline workload: operands, operators, the autograd step and its eight launches one by one."""

    def __init__(self, B=8, block=64, dtype='f16'):
        import torch
        import torch_blocksparse as tb
        from torch_blocksparse.matmul import _sparse_matmul
        self.tb, self.torch = tb, torch
        dev = torch.device('cuda:0')
        torch.manual_seed(0)
        H, L, dh = 16, 4096, 64
        dtype = {'f16': torch.float16, 'bf16': torch.bfloat16}[dtype]
        self.scale, self.dh, self.block = 0.125, dh, block
        lay = tb.sparse_transformer_layout(H, L // 64, 4, 16, True)
        if block != 64:   # the same mask, every 64-block split into (64 / block)^2 blocks: same flops, same bytes
            lay = lay.repeat_interleave(64 // block, 1).repeat_interleave(64 // block, 2)
        self.lay, self.nnz = lay, int(lay.sum())
        self.q, self.k, self.v, self.do = [torch.randn(B, H, L, dh, dtype=dtype, device=dev) for _ in range(4)]
        for t in (self.q, self.k, self.v):
            t.requires_grad_(True)
        g = torch.Generator().manual_seed(1)
        kpm = torch.zeros(B, L, dtype=dtype)
        for z in range(B):
            pad = int(torch.randint(0, L // 4 + 1, (1,), generator=g))
            if pad:
                kpm[z, L - pad:] = float('-inf')
        self.kpm = kpm.to(dev)
        self.sdd = tb.MatMul(lay, block, 'sdd', trans_a=False, trans_b=True)
        self.dsd = tb.MatMul(lay, block, 'dsd')
        self.sm = tb.Softmax(lay, block)
        es = 2
        self.flops_mm = 2.0 * B * dh * self.nnz * block * block     # per product (K = N = M = head_dim in all six)
        self.x_bytes = B * self.nnz * block * block * es
        self.dense_bytes = B * H * L * dh * es
        self.mm_bytes = self.x_bytes + 2 * self.dense_bytes          # one sparse tensor + two dense tensors, each touched once
        self.kpm_bytes = self.kpm.numel() * es
        self.sl, self.dl = self.sdd.make_lut(dtype, dev), self.dsd.make_lut(dtype, dev)
        self.sm_lut, self.sm_maxlut = self.sm.make_lut(dev)
        self.fn, self.spd, self.t, self.st = _sparse_matmul.fn, lay.shape, [None], {}

    def step(self):
        q, k, v = self.q, self.k, self.v
        q.grad = k.grad = v.grad = None
        w = self.sdd(q, k)
        p = self.sm(w, scale=self.scale, key_padding_mask=self.kpm)
        o = self.dsd(p, v)
        o.backward(self.do)

    # the launches of a step, callable one by one (no autograd)
    def k_sdd_fwd(self):
        sl = self.sl
        self.st['w'] = self.fn['sdd'](self.q, self.k, False, True, False, self.spd, self.block, sl[0], sl[1], sl[2], sl[3], False, self.t)

    def k_softmax_fwd(self):
        self.st['p'] = self.tb.Softmax.sparse_softmax(self.st['w'], self.scale, None, self.kpm, None, 'add', 'add', self.spd, self.block,
                                                      self.sm_lut, self.sm_maxlut, False, self.t)

    def k_dsd_fwd(self):
        dl = self.dl
        self.st['o'] = self.fn['dsd'](self.st['p'], self.v, False, False, False, self.spd, self.block, dl[0], dl[1], dl[2], dl[3], False, self.t)

    def k_sdd_bwd(self):     # dp = do . v^T restricted to the layout
        dl = self.dl
        self.st['dp'] = self.fn['sdd'](self.do, self.v, False, True, False, self.spd, self.block, dl[4], dl[5], dl[6], dl[7], False, self.t)

    def k_dsd_bwd_t(self):   # dv = p^T . do
        dl = self.dl
        self.st['dv'] = self.fn['dsd'](self.st['p'], self.do, True, False, False, self.spd, self.block, dl[8], dl[9], dl[10], dl[11], False, self.t)

    def k_softmax_bwd(self):
        _bwd_softmax(self.tb, self.st['p'], self.st['dp'], self.scale, self.sm_lut, self.sm_maxlut, self.spd, self.block)

    def k_dsd_bwd(self):     # dq = ds . k
        sl = self.sl
        self.st['dq'] = self.fn['dsd'](self.st['dp'], self.k, False, False, False, self.spd, self.block, sl[4], sl[5], sl[6], sl[7], False, self.t)

    def k_dds_bwd(self):     # dk = (q^T . ds)^T
        sl = self.sl
        self.st['dk'] = self.fn['dds'](self.q, self.st['dp'], True, False, True, self.spd, self.block, sl[8], sl[9], sl[10], sl[11], False, self.t)

    def k_copy(self):        # plain copy of |x| bytes: the known-size kernel the traffic counters are calibrated on
        self.st['copy'] = self.st['dp'].clone()

    def launches(self):
        """(name, callable, flops, algorithmic bytes) in step order."""
        f, b, x = self.flops_mm, self.mm_bytes, self.x_bytes
        return [('sdd_fwd  q.k^T', self.k_sdd_fwd, f, b), ('softmax_fwd', self.k_softmax_fwd, 0.0, 2 * x + self.kpm_bytes),
                ('dsd_fwd  p.v', self.k_dsd_fwd, f, b), ('dsd_bwd  p^T.do', self.k_dsd_bwd_t, f, b),
                ('sdd_bwd  do.v^T', self.k_sdd_bwd, f, b), ('softmax_bwd', self.k_softmax_bwd, 0.0, 3 * x),
                ('dds_bwd  (q^T.ds)^T', self.k_dds_bwd, f, b), ('dsd_bwd  ds.k', self.k_dsd_bwd, f, b)]


def launch_roofline(kernel, flops, nbytes, ms, peak_tflops=MFMA_PEAK_TFLOPS):
    """The roofline object of one launch.  A product is bound by min(matrix peak, arithmetic intensity x HBM peak) with the
    intensity taken from the algorithmic bytes (every tensor touched once); a softmax by the HBM peak.  `frac` is the
    achieved rate over that binding roof; products also carry their fraction of the raw matrix peak."""
    if not flops:
        gbs = nbytes / ms * 1e-6
        return {'kernel': kernel, 'bound': 'hbm', 'achieved': round(gbs, 1), 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
                'frac': round(gbs / HBM_PEAK_GBS, 4), 'traffic': None}
    tf = flops / ms * 1e-9
    hbm_roof = flops / nbytes * HBM_PEAK_GBS * 1e-3            # TFLOP/s at 8 TB/s for this flop : byte ratio
    roof = min(peak_tflops, hbm_roof)
    return {'kernel': kernel, 'bound': 'mfma' if peak_tflops <= hbm_roof else 'hbm', 'achieved': round(tf, 2), 'peak': round(roof, 1),
            'unit': 'TFLOP/s', 'frac': round(tf / roof, 4), 'frac_of_matrix_peak': round(tf / peak_tflops, 4),
            'flop_per_byte': round(flops / nbytes, 1), 'traffic': None}


def xsd_kernel_name(block, dtype_bits, free_dim, sp_trans, dn_kc):
    """Which kernel the library's dispatch gives a dsd/dds launch (csrc/capi.hip xsd_dispatch, in its order)."""
    if dtype_bits == 16 and free_dim >= 256:
        if block == 32 and dn_kc:
            return 'k_xsd_rg_dl'
        if block in (64, 128) and not (sp_trans and dn_kc):
            return 'k_xsd_dl<%d>' % block
    if dtype_bits == 16 and not dn_kc and free_dim % 64 == 0:
        if block == 64:
            return 'k_xsd64_rg<sparse operand %s>' % ('transposed' if sp_trans else 'as stored')
        if block == 16:
            return 'k_xsd64_rg<tiles of 4 x 4 blocks>'
        if block == 32 and free_dim <= 128:
            return 'k_xsd_rg_small'
    return 'k_xsd (general)'


def fused_chain_launches(lay, q, k, v, do, scale, timeit, variants, block=64):
    """The fused attention kernels (bsp_attention_fwd / bsp_attention_bwd: what the attention modules launch instead of
    sdd -> softmax -> dsd when block, dtype and head dimension allow), each timed on its own through the C ABI.
    variants: [(label, softmax keyword arguments)] for the forward kernel.  Algorithmic bytes: forward q, k, v, o and
    the sparse p once each; backward rows do, o, v, k, dq and the sparse p once each, backward columns do, q, v, dk, dv and p (masks: what the layout touches
    is counted by the caller's softmax figures, not here)."""
    import torch
    from torch_blocksparse import attention_core as ac
    core = ac.AttentionCore(lay, block)
    B, H, L, dh = q.shape
    nnz = core.blocks()
    dense = q.numel() * q.element_size()
    xb = B * nnz * block * block * q.element_size()
    out = []
    state = {}
    for label, kw in variants:
        def fwd():
            with torch.no_grad():
                state['o'] = ac._attention_core.forward(state.setdefault('ctx', _Ctx()), q, k, v, float(scale), kw.get('rpe'), kw.get('key_padding_mask'),
                                                        kw.get('attn_mask'), kw.get('key_padding_mask_mode', 'add'), kw.get('attn_mask_mode', 'add'),
                                                        core, *_fwd_tables(core, q.device))
        ms = timeit(fwd)
        nbytes = 4 * dense + xb
        out.append({'launch': 'fused forward: q.k^T, softmax, p.v (%s)' % label, 'ms': round(ms, 4), 'GB/s': round(nbytes / ms * 1e-6, 1),
                    'hbm_frac': round(nbytes / ms * 1e-6 / HBM_PEAK_GBS, 4), 'roofline': launch_roofline('k_attn64_fwd', 0, nbytes, ms)})
    ctx = state['ctx']
    delta = torch.empty((B, H, ctx.rows * 64), dtype=torch.float32, device=q.device)

    def rows():
        with torch.no_grad():
            ac._attention_core.rows_kernel(ctx, do, None, delta)
    ms = timeit(rows)
    nbytes = 5 * dense + xb
    out.append({'launch': 'fused backward, rows: do.v^T, softmax gradient, ds.k -> dq', 'ms': round(ms, 4), 'GB/s': round(nbytes / ms * 1e-6, 1),
                'hbm_frac': round(nbytes / ms * 1e-6 / HBM_PEAK_GBS, 4), 'roofline': launch_roofline('k_attn64_bwd', 0, nbytes, ms)})

    def columns():
        with torch.no_grad():
            ac._attention_core.columns_kernel(ctx, do, delta)
    ms = timeit(columns)
    ct = ctx.columns
    nbytes = 5 * dense + xb + 2 * B * ct.n_slots * 2 * 64 * dh * 4      # (the partial sums of the long columns' parts: written, read)
    out.append({'launch': 'fused backward, columns: softmax gradient again, p^T.do -> dv, ds^T.q -> dk (%d of %d columns in parts)' % (ct.n_split, H * ct.columns),
                'ms': round(ms, 4), 'GB/s': round(nbytes / ms * 1e-6, 1),
                'hbm_frac': round(nbytes / ms * 1e-6 / HBM_PEAK_GBS, 4), 'roofline': launch_roofline('k_attn64_bwd_kv', 0, nbytes, ms)})
    return out


def _fwd_tables(core, device, keep_p=True):
    """the table arguments of _attention_core.forward: (table, longest row, keep p for a backward pass, rows)"""
    lut, maxlut, _, rows = core.tables(device)[:4]
    return lut, maxlut, keep_p, rows


class _Ctx:
    """Stand-in for the autograd context when the fused kernels are called outside autograd (timing only)."""
    needs_input_grad = (True, True, True)

    def save_for_backward(self, *t):
        self.saved_tensors = t


def fused_chain_step(w, steps, warmup):
    """The headline workload through attention_chain (the call the attention modules make): forward and backward with the
    fused kernels, timed like the headline step."""
    import torch
    from torch_blocksparse import attention_core as ac

    def step():
        w.q.grad = w.k.grad = w.v.grad = None
        o = ac.attention_chain(w.sdd, w.sm, w.dsd, w.q, w.k, w.v, scale=w.scale, key_padding_mask=w.kpm)
        o.backward(w.do)
    before = ac.fused_calls
    for _ in range(SETTLE_STEPS + warmup):
        step()
    torch.cuda.synchronize()
    if ac.fused_calls == before:
        return None
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def module_default_config(steps, warmup):
    """The sparse self-attention module as its defaults configure it (deepspeedsparseselfattention.py:13: 'fixed' layout,
    block 16, stride 64, unidirectional), same batch, heads, sequence and head dimension as the headline: forward +
    backward through autograd, the three operators (FUSED off) against the fused chain the module calls."""
    import torch
    import torch_blocksparse as tb
    from torch_blocksparse import attention_core as ac
    dev = torch.device('cuda:0')
    torch.manual_seed(0)
    B, H, L, dh = 8, 16, 4096, 64
    mod = tb.SparseSelfAttention(tb.SparsityConfig())
    q, k, v = [torch.randn(B, H, L, dh, device=dev, dtype=torch.float16, requires_grad=True) for _ in range(3)]
    do = torch.randn(B, H, L, dh, device=dev, dtype=torch.float16)

    def step():
        q.grad = k.grad = v.grad = None
        mod(q, k, v).backward(do)
    res = {}
    old = ac.FUSED
    try:
        for name, fused in (('three operators', False), ('fused chain', True)):
            ac.FUSED = fused
            for _ in range(warmup):
                step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                step()
            torch.cuda.synchronize()
            res[name] = round((time.perf_counter() - t0) * 1e3 / steps, 4)
    finally:
        ac.FUSED = old
    sdd, dsd, sm = mod.get_ops(H, L, dev)
    nnz = int((sm.layout != 0).sum())
    t = ac._core_for(sdd, sm, dsd).tables(dev)
    torch.cuda.empty_cache()
    return {'workload': "SparseSelfAttention(SparsityConfig()): 'fixed' layout, block 16, stride 64, unidirectional; batch 8, 16 heads, seq 4096, head_dim 64, fp16, "
                        'forward + backward', 'blocks_per_head': nnz // H, 'ms_per_step': res,
            'tiles': {'longest_line': t[1], 'blocks_present_per_tile': round(t[4], 3)}}


def other_config(config, steps, warmup):
    """The configurations the headline metric is not quoted on: every launch timed on its own (HIP events, mean of
    `steps` back-to-back launches), effective throughput over the nonzero blocks, as a fraction of the fp16 MFMA peak
    (the MFMA-bound configurations 2 and 5; fp32 peak for configuration 1) or of the HBM peak (configuration 4).
    Returns {'workload': ..., 'launches': [...]}."""
    import torch
    import torch_blocksparse as tb
    dev = torch.device('cuda:0')
    out = []

    def timeit(f):
        import gc
        # warm-up by time, not by count: after a change of the launch pattern the GPU needs about 20 ms of the new work
        # before its launch times settle (see SETTLE_STEPS), whether that is 15 launches or 400
        for _ in range(max(warmup, 1)):
            f()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        f()
        torch.cuda.synchronize()
        one = max(time.perf_counter() - t0, 2e-5)
        for _ in range(min(2000, int(0.025 / one) + 1)):
            f()
        gc.collect()
        gc.disable()                                   # (a collection pause would leave the GPU waiting inside the timed loop)
        try:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(steps):
                f()
            e1.record()
            e1.synchronize()
        finally:
            gc.enable()
        return e0.elapsed_time(e1) / steps

    def bernoulli(shape, density, seed, one_per_row=False):
        g = torch.Generator().manual_seed(seed)
        lay = (torch.rand(shape, generator=g) < density).long()
        if one_per_row:
            for h in range(shape[0]):
                for r in range(shape[1]):
                    if lay[h, r].sum() == 0:
                        lay[h, r, int(torch.randint(0, shape[2], (1,), generator=g))] = 1
        return lay

    def mm(name, mode, ta, tb_, block, dtype, Z, H, M, N, K, lay, scale=1.0, sp_scale=1.0):
        # operands N(0, scale) (dense) and N(0, sp_scale) (sparse): the matrix pipes' clock under load depends on the data
        nnz = int(lay.sum())
        a = torch.randn((Z, H) + ((K, M) if ta else (M, K)), device=dev, dtype=dtype) * scale
        b = torch.randn((Z, H) + ((N, K) if tb_ else (K, N)), device=dev, dtype=dtype) * scale
        if mode == 'dsd':
            a = torch.randn(Z, nnz, block, block, device=dev, dtype=dtype) * sp_scale
        if mode == 'dds':
            b = torch.randn(Z, nnz, block, block, device=dev, dtype=dtype) * sp_scale
        op = tb.MatMul(lay, block, mode, trans_a=ta, trans_b=tb_)
        with torch.no_grad():
            ms = timeit(lambda: op(a, b))
        D = {'sdd': K, 'dsd': N, 'dds': M}[mode]
        fl = 2.0 * Z * D * nnz * block * block
        es = a.element_size()
        nbytes = es * (Z * nnz * block * block + Z * H * (M * K if mode != 'dsd' else K * N) + Z * H * (M * N if mode != 'sdd' else K * N))
        peak = FP32_PEAK_TFLOPS if dtype == torch.float32 else MFMA_PEAK_TFLOPS
        bits = 32 if dtype == torch.float32 else 16
        if mode == 'sdd':
            kernel = ('k_sdd_rg_dl' if (block in (16, 32) and K >= 256 and K % 32 == 0 and bits == 16) else
                      'k_sdd128_splitk + k_sdd_splitk_sum' if (block == 128 and bits == 16 and K >= 512 and K % 32 == 0 and nnz * Z < 768) else
                      'k_sdd64_rg' if (block in (16, 64) and bits == 16 and K in (64, 128) and not ta and tb_) else
                      'k_sdd_rg_small' if (block == 32 and bits == 16 and K == 64 and not ta and tb_) else 'k_sdd (general)')
        elif mode == 'dsd':      # kernel rows = rows of op(A); dense operand reduction-contiguous when B is read transposed
            kernel = xsd_kernel_name(block, bits, N, ta, tb_)
        else:                    # dds = dsd on the transposed problem
            kernel = xsd_kernel_name(block, bits, M, not tb_, not ta)
        out.append({'launch': name, 'ms': round(ms, 4), 'TFLOP/s': round(fl / ms * 1e-9, 2), 'mfma_frac': round(fl / ms * 1e-9 / peak, 4),
                    'GB/s': round(nbytes / ms * 1e-6, 1), 'hbm_frac': round(nbytes / ms * 1e-6 / HBM_PEAK_GBS, 4),
                    'roofline': launch_roofline(kernel, fl, nbytes, ms, peak)})

    if config == 1:
        torch.manual_seed(0)
        lay = torch.randint(0, 2, (2, 16, 32))
        mm('sdd trans_a fp32 blk16 Z4 H2 256x512x384', 'sdd', True, False, 16, torch.float32, 4, 2, 256, 512, 384, lay)
        x = torch.rand(4, int(lay.sum()), 16, 16, device=dev)
        sm = tb.Softmax(lay, 16)
        with torch.no_grad():
            ms = timeit(lambda: sm(x))
        out.append({'launch': 'softmax fwd fp32 blk16', 'ms': round(ms, 4), 'GB/s': round(2 * x.numel() * 4 / ms * 1e-6, 1),
                    'roofline': launch_roofline('k_softmax_fwd', 0, 2 * x.numel() * 4, ms)})
        workload = 'README shape: sdd trans_a fp32 block 16 + softmax'
    elif config == 2:
        lay = bernoulli((16, 64, 64), 0.25, 2, one_per_row=True)
        for ta in (False, True):
            for tb_ in (False, True):
                mm('dsd trans_a=%d trans_b=%d' % (ta, tb_), 'dsd', ta, tb_, 32, torch.float16, 8, 16, 2048, 2048, 2048, lay, 2048 ** -0.5)
                mm('dds trans_a=%d trans_b=%d' % (ta, tb_), 'dds', ta, tb_, 32, torch.float16, 8, 16, 2048, 2048, 2048, lay, 2048 ** -0.5)
        mm('sdd (gradient of the sparse operand)', 'sdd', False, True, 32, torch.float16, 8, 16, 2048, 2048, 2048, lay, 2048 ** -0.5)
        workload = 'fp16 block 32, Z 8, H 16, M=N=K=2048, Bernoulli(0.25) layout, dense operands N(0,1)/sqrt(K), sparse N(0,1); bound: MFMA'
    elif config == 5:
        lay = bernoulli((1, 32, 32), 0.1, 5)
        mm('dds trans_b (y = x.W^T)', 'dds', False, True, 128, torch.float16, 1, 1, 8192, 4096, 4096, lay, 1.0, 0.02)
        mm('dds (dx = dy.W)', 'dds', False, False, 128, torch.float16, 1, 1, 8192, 4096, 4096, lay, 1.0, 0.02)
        mm('sdd trans_a (dW = dy^T.x on the layout)', 'sdd', True, False, 128, torch.float16, 1, 1, 4096, 4096, 8192, lay, 1.0)
        workload = 'block-sparse linear layer: 8192 tokens, 4096x4096 weight N(0, 0.02), block 128, 10 % density, activations and gradients N(0,1), fp16; bound: MFMA'
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
        # both masks are shared by batch and heads (the rpe through stride-0 views): the bytes of each that the layout
        # touches are the block positions present in any head
        touched = int(lay.sum(0).ne(0).sum()) * block * block * 2
        do = torch.randn_like(q)
        from torch_blocksparse.matmul import _sparse_matmul
        fn, spd, t = _sparse_matmul.fn, lay.shape, [None]
        sl, dl = sdd.make_lut(torch.float16, dev), dsd.make_lut(torch.float16, dev)   # (c, da, db) tables of each op
        sm_lut, sm_maxlut = sm.make_lut(dev)
        mmb = xb + 2 * B * H * L * dh * 2
        with torch.no_grad():
            w = sdd(q, k)
            dw = torch.randn_like(w)
            for name, f, flops, nbytes in (
                    ('sdd q.k^T', lambda: sdd(q, k), fl, mmb),
                    ('softmax fwd, scale only', lambda: sm(w, scale=0.125), 0, 2 * xb),
                    ('softmax fwd, rpe + causal mask', lambda: sm(w, scale=0.125, rpe=rpe, attn_mask=causal, attn_mask_mode='mul'), 0, 2 * xb + 2 * touched),
                    ('dsd p.v', lambda: dsd(w, v), fl, mmb),
                    # backward, in the order autograd runs it (the products of MatMul.backward are MatMul modes of their own)
                    ('dsd p^T.do', lambda: fn['dsd'](w, do, True, False, False, spd, block, dl[8], dl[9], dl[10], dl[11], False, t), fl, mmb),
                    ('sdd do.v^T', lambda: fn['sdd'](do, v, False, True, False, spd, block, dl[4], dl[5], dl[6], dl[7], False, t), fl, mmb),
                    ('softmax bwd', lambda: _bwd_softmax(tb, w, dw, 0.125, sm_lut, sm_maxlut, spd, block), 0, 3 * xb),
                    ('dds (q^T.ds)^T', lambda: fn['dds'](q, dw, True, False, True, spd, block, sl[8], sl[9], sl[10], sl[11], False, t), fl, mmb),
                    ('dsd ds.k', lambda: fn['dsd'](dw, k, False, False, False, spd, block, sl[4], sl[5], sl[6], sl[7], False, t), fl, mmb)):
                ms = timeit(f)
                ent = {'launch': name, 'ms': round(ms, 4), 'GB/s': round(nbytes / ms * 1e-6, 1), 'hbm_frac': round(nbytes / ms * 1e-6 / HBM_PEAK_GBS, 4)}
                if flops:
                    ent['TFLOP/s'] = round(flops / ms * 1e-9, 2)
                kernel = ('k_softmax_fwd' if 'softmax fwd' in name else 'k_softmax_bwd' if 'softmax bwd' in name else 'k_sdd64_rg' if name.startswith('sdd')
                          else 'k_xsd64_rg<sparse operand %s>' % ('transposed' if '^T.' in name else 'as stored'))
                ent['roofline'] = launch_roofline(kernel, flops, nbytes, ms)
                out.append(ent)
        out.extend(fused_chain_launches(lay, q, k, v, do, 0.125, timeit,
                                        [('scale only', {}), ('rpe + causal mask', dict(rpe=rpe, attn_mask=causal, attn_mask_mode='mul'))]))
        # the whole step, forward + backward through autograd: the three operators against attention_chain (what the modules call)
        from torch_blocksparse import attention_core as ac
        qg, kg, vg = [t.detach().requires_grad_(True) for t in (q, k, v)]
        steps_ms = {}
        for label, kw in (('scale only', {}), ('rpe + causal mask', dict(rpe=rpe, attn_mask=causal, attn_mask_mode='mul'))):
            for fused in (False, True):
                def step():
                    qg.grad = kg.grad = vg.grad = None
                    ac.attention_chain(sdd, sm, dsd, qg, kg, vg, scale=0.125, **kw).backward(do)
                old_fused, ac.FUSED = ac.FUSED, fused
                try:
                    steps_ms.setdefault(label, {})['fused chain' if fused else 'three operators'] = round(timeit(step), 4)
                finally:
                    ac.FUSED = old_fused
        workload = ('BigBird layout (3 window + 2 global + 3 random blocks, causal), batch 2, 12 heads, seq 16384, head_dim 64, block 64, fp16, '
                    'forward and backward launches; bound: HBM (softmax bytes: 2|x| + the mask and rpe bytes the layout touches)')
        torch.cuda.empty_cache()
        return {'workload': workload, 'launches': out, 'ms_per_step': steps_ms}
    torch.cuda.empty_cache()
    return {'workload': workload, 'launches': out}


def reference_bench_shapes(steps, warmup):
    """The shapes the reference's own benchmark functions run (they are all it ever names; it publishes no numbers):
      * tests/test_matmul.py:105-122  sdd, batch 1, 12 heads, hidden 512, block 16, 'fixed' layout of stride 64 with 4
        vertical blocks, bidirectional, seq 4096, fp16, operands uniform in [0, 1); reported as the reference does:
        2 * Z * K * nnz * block^2 flops over the time of the forward call
      * tests/test_softmax.py:92-128  block 16, Z 2, H 4, density 0.4: 256 rows x (256 .. 3072) columns and (32 .. 480)
        rows x 512 columns; block 64, Z 1, H 1, 'fixed' layout of stride 64 with 4 vertical blocks, unidirectional and
        bidirectional, seq 1024 .. 8192; forward and backward; bytes counted as the reference counts them:
        forward 2|x| + |attn_mask| + |kp_mask|, backward 3|x|  (tests/test_softmax.py:76-77)
    Every launch timed on its own with HIP events, `steps` back-to-back launches after a warm-up."""
    import gc
    import torch
    import torch_blocksparse as tb
    dev = torch.device('cuda:0')
    torch.manual_seed(1)

    def timeit(f):
        for _ in range(max(warmup, 3)):
            f()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        f()
        torch.cuda.synchronize()
        one = max(time.perf_counter() - t0, 2e-5)
        for _ in range(min(2000, int(0.025 / one) + 1)):
            f()
        gc.collect()
        gc.disable()
        try:
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(steps):
                f()
            e1.record()
            e1.synchronize()
        finally:
            gc.enable()
        return e0.elapsed_time(e1) / steps

    out = []
    # matmul: bench_op of tests/test_matmul.py
    batch, heads, hidden, block, stride, L = 1, 12, 512, 16, 64, 4096
    lay = tb.make_layout(heads, L // block, 'fixed', stride // block, False, 4, 1)
    nnz = int(lay.sum())
    x = torch.rand(batch, heads, L, hidden, device=dev, dtype=torch.float16)
    w = torch.rand(batch, heads, hidden, L, device=dev, dtype=torch.float16)
    op = tb.MatMul(lay, block, 'sdd', trans_a=False, trans_b=False)
    with torch.no_grad():
        ms = timeit(lambda: op(x, w))
    fl = 2.0 * batch * hidden * nnz * block * block
    nbytes = 2 * (batch * nnz * block * block + 2 * batch * heads * L * hidden)
    out.append({'launch': 'sdd  batch 1, 12 heads, seq 4096, hidden 512, block 16, fixed layout (stride 64, 4 vertical), fp16', 'nnz_blocks': nnz,
                'ms': round(ms, 4), 'TFLOP/s': round(fl / ms * 1e-9, 2), 'roofline': launch_roofline('k_sdd_rg_dl<block 16>', fl, nbytes, ms)})

    # softmax: bench_op of tests/test_softmax.py
    def softmax_case(label, Z, lay, block):
        n = int(lay.sum())
        N = lay.shape[2] * block
        xs = torch.rand(Z, n, block, block, device=dev, dtype=torch.float16)
        dx = torch.rand_like(xs)
        sm = tb.Softmax(lay, block)
        lut, maxlut = sm.make_lut(dev)
        with torch.no_grad():
            sm(xs, 0.4)                                     # leaves a softmax in xs: what the backward pass reads
            ms_y = timeit(lambda: sm(xs, 0.4))
            ms_dx = timeit(lambda: _bwd_softmax(tb, xs, dx, 0.4, lut, maxlut, lay.shape, block))
        xb = xs.numel() * 2
        gb_y, gb_dx = 2 * xb + N * N * 2 + Z * N * 2, 3 * xb      # as the reference counts (masks included although it passes none)
        out.append({'launch': 'softmax ' + label, 'nnz_blocks': n, 'fwd_ms': round(ms_y, 4), 'bwd_ms': round(ms_dx, 4),
                    'fwd_GB/s': round(gb_y / ms_y * 1e-6, 1), 'bwd_GB/s': round(gb_dx / ms_dx * 1e-6, 1),
                    'fwd_GB/s_x_only': round(2 * xb / ms_y * 1e-6, 1),
                    'roofline': launch_roofline('k_softmax_fwd', 0, 2 * xb, ms_y)})

    def bernoulli(shape, density, seed):
        g = torch.Generator().manual_seed(seed)
        lay = (torch.rand(shape, generator=g) < density).long()
        for h in range(shape[0]):
            for r in range(shape[1]):
                if lay[h, r].sum() == 0:
                    lay[h, r, 0] = 1
        return lay
    for N in (256, 1024, 2048, 3072):                       # "# Columns" sweep (the reference runs every multiple of 256)
        softmax_case('block 16, Z 2, H 4, 256 rows x %d columns, density 0.4' % N, 2, bernoulli((4, 16, N // 16), 0.4, N), 16)
    for M in (32, 256, 480):                                # "# Rows" sweep
        softmax_case('block 16, Z 2, H 4, %d rows x 512 columns, density 0.4' % M, 2, bernoulli((4, M // 16, 32), 0.4, M), 16)
    for uni, tag in ((True, 'Sparse GPT2 (unidirectional)'), (False, 'Sparse BERT (bidirectional)')):
        for ctx_len in (1024, 2048, 4096, 8192):
            lay = tb.make_layout(1, ctx_len // 64, 'fixed', 1, uni, 4, 1)
            softmax_case('%s, block 64, Z 1, H 1, seq %d' % (tag, ctx_len), 1, lay, 64)
    torch.cuda.empty_cache()
    return {'workload': "the reference's own benchmark shapes: tests/test_matmul.py:105-122 (sdd, block 16) and tests/test_softmax.py:92-128 "
                        "(softmax sweeps); the reference publishes no numbers for them", 'launches': out}


def _bwd_softmax(tb, y, dy, scale, lut, maxlut, spdims, block):
    from torch_blocksparse import _lib
    rc = _lib.load().bsp_softmax_bwd(_lib.DTYPES[y.dtype], _lib.ptr(y), _lib.ptr(dy), float(scale), _lib.ptr(lut), maxlut,
                                     y.size(0), spdims[0], spdims[1], block, y.stride(0), dy.stride(0), _lib.stream_ptr(y.device))
    _lib.check(rc, 'bsp_softmax_bwd')


def calibrate(args):
    """What this box streams, and the step's kernels with cold caches.  Probes (libbsp_probe.so): 16-byte accesses in
    address order over a 4 GiB footprint (far beyond the 256 MB memory-side cache) and over the 268 MB footprint of the
    step's sparse tensor (which fits it).  Then every launch of the headline step timed alone, once as in the step
    (its predecessor's output still cached) and once after a 1 GiB write that flushes L2 and the memory-side cache."""
    import torch
    from torch_blocksparse import _lib
    probe_path = os.path.join(PKG, 'lib', 'libbsp_probe.so')
    if not os.path.exists(probe_path):
        sys.exit('%s not found: build it with `python torch-blocksparse_amd/build.py`' % probe_path)
    probe = ctypes.CDLL(probe_path)
    probe.bsp_probe_stream.restype = ctypes.c_int
    probe.bsp_probe_stream.argtypes = [ctypes.c_int] + [ctypes.c_void_p] * 3 + [ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
    dev = torch.device('cuda:0')
    stream = _lib.stream_ptr(dev)
    reps = 20

    def timed(f, before=None):
        total = 0.0
        for it in range(reps + 2):
            if before:
                before()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            f()
            e1.record()
            e1.synchronize()
            if it >= 2:
                total += e0.elapsed_time(e1)
        return total / reps

    res = {'probes': []}
    moved = {0: 1, 1: 1, 2: 2, 3: 2, 4: 3}
    names = {0: 'read only', 1: 'write only', 2: 'copy (1 read : 1 write)', 3: 'in place (read + write back)', 4: '1 read : 2 writes'}
    for nbytes, label in ((4 << 30, '4 GiB per buffer'), (268435456, '268 MB per buffer')):
        bufs = [torch.empty(nbytes, dtype=torch.uint8, device=dev) for _ in range(3)]
        for b in bufs:
            b.zero_()
        for mode in range(5):
            for groups in (256 * 8, 256 * 32):
                ms = timed(lambda: probe.bsp_probe_stream(mode, _lib.ptr(bufs[0]), _lib.ptr(bufs[1]), _lib.ptr(bufs[2]), nbytes, groups, stream))
                res['probes'].append({'probe': names[mode], 'footprint': label, 'workgroups': groups, 'ms': round(ms, 4),
                                      'GB/s': round(moved[mode] * nbytes / ms * 1e-6, 1)})
        del bufs
        torch.cuda.empty_cache()
    w = Attention(8, 64)
    flush_buf = torch.empty(1 << 30, dtype=torch.uint8, device=dev)

    def flush():           # 1 GiB written: L2 and the memory-side cache end up full of DIRTY lines of another buffer
        probe.bsp_probe_stream(1, _lib.ptr(flush_buf), None, None, flush_buf.numel(), 256 * 16, stream)

    def flush_clean():     # 1 GiB read: the caches end up full of CLEAN lines of another buffer (nothing to write back)
        probe.bsp_probe_stream(0, _lib.ptr(flush_buf), None, None, flush_buf.numel(), 256 * 16, stream)

    launches = w.launches()
    with torch.no_grad():
        for _ in range(3):
            for _, f, _, _ in launches:
                f()
        res['launches'] = []
        for i, (name, f, flops, nbytes) in enumerate(launches):
            prev = launches[i - 1][1]
            warm = timed(f, before=prev)        # the cache state of the step: the predecessor has just run
            cold = timed(f, before=flush)
            flush()
            torch.cuda.synchronize()
            cold_clean = timed(f, before=flush_clean)
            res['launches'].append({'launch': name, 'bytes': nbytes, 'ms_after_predecessor': round(warm, 4),
                                    'GB/s_after_predecessor': round(nbytes / warm * 1e-6, 1), 'ms_cold': round(cold, 4),
                                    'GB/s_cold': round(nbytes / cold * 1e-6, 1), 'ms_cold_clean': round(cold_clean, 4),
                                    'GB/s_cold_clean': round(nbytes / cold_clean * 1e-6, 1)})
    print(json.dumps({'metric': 'streaming calibration, not the headline metric', 'n_gpus': 1, 'data': 'synthetic', **res}))


def record_traffic(fetch_dir, write_dir):
    """Reads the counter CSVs of two runs
         rocprofv3 --pmc FETCH_SIZE --output-format csv -d FETCH_DIR -o f -- python3 bench.py --steps 3 --warmup 1 --no-cpu-baseline --no-other-configs
         rocprofv3 --pmc WRITE_SIZE --output-format csv -d WRITE_DIR -o w -- python3 bench.py --steps 3 --warmup 1 --no-cpu-baseline --no-other-configs
    and writes the HBM bytes per launch of each of the step's kernels to profiles/, scaled by what the same counter reads
    for the run's calibration copy of 268 435 456 bytes, together with the hash of the kernel sources they belong to."""
    import csv
    import collections

    def read(d, counter):
        per = collections.defaultdict(list)
        for f in glob.glob(os.path.join(d, '**', '*counter_collection.csv'), recursive=True):
            for r in csv.DictReader(open(f)):
                if r['Counter_Name'] == counter:
                    per[r['Kernel_Name']].append(float(r['Counter_Value']))
        return per

    fetch, write = read(fetch_dir, 'FETCH_SIZE'), read(write_dir, 'WRITE_SIZE')

    def copy_scale(per):
        vals = [v for k, vs in per.items() if 'copyBuffer' in k for v in vs if v > 100000]    # the 268 MB copies only
        return 268435456.0 / (sum(vals) / len(vals))
    fs, ws = copy_scale(fetch), copy_scale(write)

    split = {}

    def kernel_bytes(name, sub, *more):
        def pick(per):
            vals = [v for k, vs in per.items() if sub in k and all(m in k for m in more) for v in vs]
            return sum(vals) / len(vals)
        split[name] = {'FETCH_SIZE_KiB': round(pick(fetch)), 'WRITE_SIZE_KiB': round(pick(write)),
                       'read_bytes': int(pick(fetch) * fs), 'written_bytes': int(pick(write) * ws)}
        return split[name]['read_bytes'] + split[name]['written_bytes']
    per_kernel = {name: kernel_bytes(name, *subs) for name, subs in (
        ('k_sdd64_rg', ('k_sdd64_rg',)), ('k_xsd64_rg<sparse operand as stored>', ('k_xsd64_rg', 'Lb0E')),
        ('k_xsd64_rg<sparse operand transposed>', ('k_xsd64_rg', 'Lb1E')), ('k_softmax_fwd', ('k_softmax_fwd',)),
        ('k_softmax_bwd', ('k_softmax_bwd',)))}
    for name in ('k_attn64_fwd', 'k_attn64_bwd', 'k_attn64_bwd_kv'):   # the fused chain of the attention modules, run after the headline step
        for sub in (name + 'I', name + '<'):               # (the template's name as mangled or as written: k_attn64_bwd is not k_attn64_bwd_kv)
            if any(sub in k for k in fetch) and any(sub in k for k in write):
                per_kernel[name] = kernel_bytes(name, sub)
    rec = {'kernel_sources_sha256': kernel_sources_sha(), 'bytes_per_counted_KiB': {'FETCH_SIZE': round(fs, 1), 'WRITE_SIZE': round(ws, 1)},
           'bytes_per_kernel_launch': per_kernel, 'counters_per_kernel_launch': split,
           'bytes_per_launch': {name: per_kernel[k] for name, k in KERNEL_OF.items()},
           'note': 'averages over the launches of each kernel in a 3-step run; launches of one kernel share a figure'}
    with open(TRAFFIC_FILE, 'w') as f:
        json.dump(rec, f, indent=1)
    print(json.dumps(rec))


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
