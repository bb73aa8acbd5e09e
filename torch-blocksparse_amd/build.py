"""Compiles the HIP sources in csrc/ into torch-blocksparse_amd/lib/libbsp_hip.so for gfx950.

hipcc cross-compiles without a GPU.  Run as a script or call build().  The translation units are compiled
in parallel and linked into one shared library with a plain C ABI (include/bsp.h).
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
LIBDIR = os.path.join(HERE, 'lib')
OBJDIR = os.path.join(HERE, 'build')
LIBNAME = 'libbsp_hip.so'
PROBE_LIBNAME = 'libbsp_probe.so'
SOURCES = ['lut.hip', 'layout.hip', 'softmax.hip', 'softmax_row.hip', 'attention_core.hip', 'attention_long.hip', 'attention_kv.hip', 'matmul_f16.hip', 'matmul_bf16.hip', 'matmul_f32.hip', 'matmul_fast64.hip', 'matmul_dl.hip', 'elementwise.hip', 'capi.hip']
FLAGS = ['--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC', '-fno-gpu-rdc', '-Wall', '-Wno-unused-function',
         # packed-fp32 instruction selection is switched off on purpose
         '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops']


def lib_path():
    return os.path.join(LIBDIR, LIBNAME)


# Kernels that count their own outstanding vector-memory operations (s_waitcnt vmcnt(n) in front of the barriers of an
# LDS ring of direct global -> LDS loads).  A register spill adds scratch loads and stores to that count and the waits
# would then let a tile be read before it has landed: the build refuses such a kernel.
COUNTED_WAITS = {'attention_core.hip': 'k_attn64', 'attention_long.hip': 'k_attn64', 'attention_kv.hip': 'k_attn64', 'matmul_dl.hip': 'k_'}


def _spilled_kernels(remarks, prefix):
    bad, name = [], None
    for line in remarks.splitlines():
        if 'Function Name:' in line:
            name = line.split('Function Name:')[1].split()[0]
        elif 'ScratchSize [bytes/lane]:' in line and name and prefix in name:
            if int(line.split('ScratchSize [bytes/lane]:')[1].split()[0]) > 0:
                bad.append(name)
    return bad


def _compile(src):
    obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + '.o')
    check = COUNTED_WAITS.get(src)
    cmd = ['hipcc'] + FLAGS + (['-Rpass-analysis=kernel-resource-usage'] if check else []) + ['-c', os.path.join(CSRC, src), '-o', obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = '\n'.join(l for l in r.stderr.splitlines() if 'packed-fp32-ops' not in l)
    if r.returncode != 0:
        raise RuntimeError('hipcc failed on %s:\n%s' % (src, err))
    if check:
        bad = _spilled_kernels(err, check)
        if bad:
            raise RuntimeError('%s: kernels with counted waits use scratch memory (register spills):\n  %s' % (src, '\n  '.join(bad)))
        err = '\n'.join(l for l in err.splitlines() if any(w in l for w in ('warning', 'error', 'note:')))   # (not the remarks and their source lines)
    return obj, err


def build(verbose=False, jobs=None, sources=None):
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    jobs = jobs or min(len(SOURCES), os.cpu_count() or 4, 16)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(_compile, sources or SOURCES))
    if verbose:
        for _, err in results:
            if err.strip():
                print(err)
    objs = [os.path.join(OBJDIR, os.path.splitext(s)[0] + '.o') for s in SOURCES]
    subprocess.check_call(['hipcc', '--offload-arch=gfx950', '-shared', '-fPIC', '-o', lib_path()] + objs)
    if sources is None:
        build_probe()
    return lib_path()


def build_probe():
    """The streaming probes of `bench.py --calibrate`: a separate small library, not part of the operator ABI."""
    out = os.path.join(LIBDIR, PROBE_LIBNAME)
    r = subprocess.run(['hipcc'] + FLAGS + ['-shared', os.path.join(CSRC, 'probe.hip'), '-o', out], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError('hipcc failed on probe.hip:\n%s' % r.stderr)
    return out


if __name__ == '__main__':
    print(build(verbose=True, sources=sys.argv[1:] or None))
