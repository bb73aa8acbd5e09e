"""Writes the golden look-up-table vectors under tests/golden/ (run once, in the build container).

Two sources, both only available where the reference checkout is mounted:
  * oracle/_ref : the reference's csrc/utils.cpp compiled as is (oracle/Makefile) -> sdd_segment, make_layout
  * the reference's Python `_sparse_matmul.load_balance` / `make_dxx_lut` (matmul.py:221-267, 372-458) and
    `DeepSpeedSparseSelfAttention._make_layout` (deepspeedsparseselfattention.py:31-65), imported from the
    checkout.  No other reference function is run: every other table has a closed form.
The vectors are plain JSON (inputs + expected outputs); the reference itself is not stored anywhere.

usage: python tests/golden/make_golden.py [/root/reference]
"""
import importlib.util
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REF = sys.argv[1] if len(sys.argv) > 1 else '/root/reference'


def layouts():
    """Named int64 layouts covering the cases the builders branch on."""
    g = torch.Generator().manual_seed(1234)
    out = {}
    out['kat_2x2_lower'] = torch.tensor([[[1, 0], [1, 1]]])
    out['kat_2x2_full'] = torch.tensor([[[1, 1], [1, 1]]])
    out['single_block'] = torch.tensor([[[1]]])
    out['one_row'] = torch.tensor([[[1, 0, 1, 1, 0, 1, 1, 1]]])
    out['one_col'] = torch.tensor([[[1], [0], [1], [1], [1], [1]]])
    for name, shape, p in [('rand_h2_4x6_p50', (2, 4, 6), 0.5), ('rand_h3_8x8_p30', (3, 8, 8), 0.3),
                           ('rand_h2_16x32_p50', (2, 16, 32), 0.5), ('rand_h4_12x7_p70', (4, 12, 7), 0.7),
                           ('rand_h2_16x16_p10', (2, 16, 16), 0.1), ('rand_h1_24x24_p90', (1, 24, 24), 0.9)]:
        lay = (torch.rand(shape, generator=g) < p).long()
        for h in range(shape[0]):          # the reference cannot handle an all-zero head
            if lay[h].sum() == 0:
                lay[h, 0, 0] = 1
        out[name] = lay
    # empty rows and columns next to full ones
    lay = torch.zeros(2, 6, 6, dtype=torch.long)
    lay[0, 0, :] = 1
    lay[0, 3, 2] = 1
    lay[1, :, 4] = 1
    lay[1, 5, 0] = 1
    out['empty_lines'] = lay
    out['dense_h2_4x4'] = torch.ones(2, 4, 4, dtype=torch.long)
    # Sparse-Transformer "fixed" layouts in both directions (what the attention modules feed in)
    sys.path.insert(0, os.path.join(ROOT, 'oracle', '_ref'))
    import torch_blocksparse_cpp_utils as ref_cpp
    out['fixed_uni_h2_16_s4'] = ref_cpp.make_layout(2, 16, 'fixed', 4, True, 1, 1)
    out['fixed_bi_h4_16_s4_nv4'] = ref_cpp.make_layout(4, 16, 'fixed', 4, False, 4, 1)
    out['fixed_uni_h2_32_s8_nv2'] = ref_cpp.make_layout(2, 32, 'fixed', 8, True, 2, 1)
    return out, ref_cpp


def load_reference_matmul(ref_cpp):
    sys.modules['torch_blocksparse_cpp_utils'] = ref_cpp
    spec = importlib.util.spec_from_file_location('_ref_matmul', os.path.join(REF, 'torch_blocksparse', 'matmul.py'))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod._sparse_matmul


def load_reference_make_layout(ref_cpp):
    """DeepSpeedSparseSelfAttention._make_layout of the reference, through the reference's own package."""
    sys.modules['torch_blocksparse_cpp_utils'] = ref_cpp
    sys.path.insert(0, REF)
    import torch_blocksparse                                  # the reference checkout (this script never adds the repository's package)
    assert os.path.dirname(torch_blocksparse.__file__).startswith(REF)
    from torch_blocksparse.deepspeedsparseselfattention import DeepSpeedSparseSelfAttention
    return DeepSpeedSparseSelfAttention._make_layout


def main():
    lays, ref_cpp = layouts()
    sm = load_reference_matmul(ref_cpp)
    gold = {'layouts': {k: v.tolist() for k, v in lays.items()}, 'sdd_segment': [], 'dxx_lut': [], 'load_balance': [],
            'make_layout_cpp': []}   # 'make_layout_py' is added below
    for name, lay in lays.items():
        for start_width in (4, 2, 1):
            seg = ref_cpp.sdd_segment(lay.to(torch.int32).clone(), start_width)
            gold['sdd_segment'].append({'layout': name, 'start_width': start_width,
                                        'tables': [[int(p), t.reshape(-1).tolist()] for p, t in seg]})
        combos = ((16, 16), (16, 8), (32, 16), (32, 8), (64, 16), (64, 8), (128, 16))
        if int(lay.sum()) > 100:           # keep the file small: large layouts get three combinations
            combos = ((16, 16), (32, 8), (64, 16))
        for block, step in combos:
            for trans in (False, True):
                lut, num_locks, width, _ = sm.make_dxx_lut(lay.clone(), block, step, trans, 'cpu')
                gold['dxx_lut'].append({'layout': name, 'block': block, 'step': step, 'trans': trans,
                                        'num_locks': int(num_locks), 'width': int(width), 'lut': lut.tolist()})
    g = torch.Generator().manual_seed(7)
    size_cases = [[1, 2], [3, 3, 3], [0, 5, 0, 2], [4, 4, 1], [17, 3, 9, 0, 16, 1], [64, 1, 1, 1, 2, 7, 8, 33], [1], [2, 0, 0]]
    size_cases += [torch.randint(0, hi, (n,), generator=g).tolist() for hi, n in ((4, 9), (6, 12), (40, 16), (100, 5))]
    for sizes in size_cases:
        if max(sizes) == 0:
            continue
        seg, col, lock, mx, off = sm.load_balance(torch.tensor(sizes, dtype=torch.int64), 16)
        gold['load_balance'].append({'sizes': sizes, 'segments': seg.tolist(), 'column': col.tolist(), 'lockid': lock.tolist(),
                                     'maxid': mx.tolist(), 'offsets': off.tolist()})
    for args in [(2, 8, 'fixed', 4, True, 1, 1), (3, 16, 'fixed', 4, False, 2, 1), (4, 16, 'fixed', 8, True, 4, 2),
                 (2, 16, 'fixed', 4, False, 2, 2), (1, 4, 'dense', 4, True, 1, 1), (4, 64, 'fixed', 16, True, 1, 1)]:
        gold['make_layout_cpp'].append({'args': list(args), 'layout': ref_cpp.make_layout(*args).tolist()})
    make_layout_py = load_reference_make_layout(ref_cpp)
    gold['make_layout_py'] = []
    for args in [(2, 8, 'fixed', 4, 'unidirectional', 1, 1), (4, 16, 'fixed', 4, 'bidirectional', 2, 2),
                 (4, 16, 'fixed', 8, 'unidirectional', 4, 2), (3, 32, 'fixed', 8, 'bidirectional', 8, 1),
                 (3, 24, 'fixed', 6, 'unidirectional', 2, 3), (5, 16, 'fixed', 8, 'unidirectional', 2, 4),
                 (2, 12, 'fixed', 4, 'bidirectional', 1, 4), (2, 8, 'dense', 4, 'unidirectional', 1, 1)]:
        gold['make_layout_py'].append({'args': list(args), 'layout': make_layout_py(*args).tolist()})
    path = os.path.join(HERE, 'lut_golden.json')
    with open(path, 'w') as f:
        json.dump(gold, f, separators=(',', ':'))
    print('wrote', path, os.path.getsize(path), 'bytes')


if __name__ == '__main__':
    main()
