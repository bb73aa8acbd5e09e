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


def _compile(src):
    obj = os.path.join(OBJDIR, os.path.splitext(src)[0] + '.o')
    cmd = ['hipcc'] + FLAGS + ['-c', os.path.join(CSRC, src), '-o', obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = '\n'.join(l for l in r.stderr.splitlines() if 'packed-fp32-ops' not in l)
    if r.returncode != 0:
        raise RuntimeError('hipcc failed on %s:\n%s' % (src, err))
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
