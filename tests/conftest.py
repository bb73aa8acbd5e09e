import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, 'torch-blocksparse_amd')):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs a real MI355X (run with -m gpu on the GPU box)')


def pytest_terminal_summary(terminalreporter):
    """What each comparison against the oracle actually reached (tests/helpers.py): the largest relative error where the
    bound is purely relative, the largest used share of the tolerance where it has an absolute term."""
    try:
        from helpers import ACHIEVED
    except ImportError:
        return
    if not ACHIEVED:
        return
    bound = {'float32': 1e-5, 'float16': 1e-2, 'bfloat16': 2e-2}
    terminalreporter.write_sep('-', 'parity against the oracle: what the comparisons reached')
    for (dtype, what, form), val in sorted(ACHIEVED.items()):
        if form == 'pure':
            terminalreporter.write_line('%-9s %-12s max relative error %.3g (bound %g, no absolute term)' % (dtype, what, val, bound[dtype]))
        elif form == 'terms':
            terminalreporter.write_line('%-9s %-12s %.0f %% of the tolerance used at most (bound %g of the summed |terms|, no absolute term)'
                                        % (dtype, what, 100 * val, bound[dtype]))
        else:
            terminalreporter.write_line('%-9s %-12s %.0f %% of the tolerance used at most' % (dtype, what, 100 * val))


@pytest.fixture(scope='session')
def golden():
    import json
    import numpy as np
    with open(os.path.join(ROOT, 'tests', 'golden', 'lut_golden.json')) as f:
        g = json.load(f)
    g['layouts'] = {k: np.array(v, dtype=np.int64) for k, v in g['layouts'].items()}
    return g
