import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, 'torch-blocksparse_amd')):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs a real MI355X (run with -m gpu on the GPU box)')


@pytest.fixture(scope='session')
def golden():
    import json
    import numpy as np
    with open(os.path.join(ROOT, 'tests', 'golden', 'lut_golden.json')) as f:
        g = json.load(f)
    g['layouts'] = {k: np.array(v, dtype=np.int64) for k, v in g['layouts'].items()}
    return g
