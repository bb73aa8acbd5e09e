"""GPU: a seeded random sweep over the matmul dispatch space (mode, transpositions, block, dtype, batch, heads, layout
shape and density, free dimension / reduction length on both sides of every kernel-selection threshold), each case
checked like the directed ones: result and both gradients against the fp32 dense-masked oracle."""
import random

import pytest
import torch

from helpers import random_layout, run_matmul_case

pytestmark = pytest.mark.gpu

FREE = [8, 24, 64, 72, 128, 256, 264, 320, 520]        # multiples of 8 around the 64 / 128 / 256 thresholds
REDUCTION = [16, 48, 64, 128, 256, 272, 288, 512]       # multiples of 16 around the 64 / 128 / 256 thresholds


def cases(n, seed):
    rng = random.Random(seed)
    out = []
    for i in range(n):
        block = rng.choice([16, 32, 32, 64, 64, 128])
        dtype = rng.choice([torch.float16, torch.float16, torch.bfloat16, torch.float32])
        mode = rng.choice(['sdd', 'dsd', 'dds'])
        ta, tb_ = rng.random() < 0.5, rng.random() < 0.5
        Z, H = rng.choice([1, 2, 3]), rng.choice([1, 2, 3])
        R, C = rng.randint(1, 6 if block <= 64 else 3), rng.randint(1, 6 if block <= 64 else 3)
        if mode == 'sdd':
            M, N, K = R * block, C * block, rng.choice(REDUCTION)
        elif mode == 'dsd':
            M, K, N = R * block, C * block, rng.choice(FREE)
            if ta:
                M, K = C * block, R * block
        else:
            K, N, M = R * block, C * block, rng.choice(FREE)
            if tb_:
                K, N = C * block, R * block
        out.append((i, mode, ta, tb_, block, dtype, Z, H, M, N, K, (R, C), rng.choice([0.25, 0.5, 0.8, 1.0])))
    return out


@pytest.mark.parametrize('case', cases(72, 20240607), ids=lambda c: '%d-%s-%d%d-b%d-%s' % (c[0], c[1], c[2], c[3], c[4], str(c[5])[6:]))
def test_random_case(case):
    i, mode, ta, tb_, block, dtype, Z, H, M, N, K, (R, C), density = case
    lay = random_layout((H, R, C), density, 1000 + i)
    # the gradient of the sparse operand of dsd / dds is an sdd product over the free dimension, which the reference's rule
    # (matmul.py:313-314, kept here) wants to be a multiple of 16: other free dimensions are checked forward only
    free = {'sdd': 16, 'dsd': N, 'dds': M}[mode]
    run_matmul_case(mode, ta, tb_, block, dtype, Z=Z, H=H, M=M, N=N, K=K, layout=lay, seed=i, dist='randn', scale=0.5,
                    backward=free % 16 == 0)


def softmax_cases(n, seed):
    rng = random.Random(seed)
    out = []
    for i in range(n):
        block = rng.choice([16, 16, 32, 64, 64, 128])
        dtype = rng.choice([torch.float16, torch.float16, torch.bfloat16, torch.float32])
        # row lengths on both sides of every register bucket (1, 2, 4, 6, 7, 8, 16, 32 blocks) and of the streaming variant
        C = rng.choice([1, 2, 3, 5, 6, 7, 8, 9, 15, 17, 31, 33, 40])
        if block == 128:
            C = min(C, 9)
        out.append((i, rng.choice([1, 2, 3, 4]), rng.choice([1, 2, 3]), rng.randint(1, 4), C, block, dtype, rng.choice([0.3, 0.6, 1.0]),
                    rng.random() < 0.4, rng.choice([None, None, 'add', 'mul']), rng.choice([None, None, 'add', 'mul'])))
    return out


@pytest.mark.parametrize('case', softmax_cases(48, 20240608), ids=lambda c: '%d-b%d-%s-c%d' % (c[0], c[5], str(c[6])[6:], c[4]))
def test_random_softmax_case(case):
    from test_gpu_softmax import run_case
    i, Z, H, R, C, block, dtype, density, rpe, kpm, attn = case
    run_case(Z, H, R, C, block, dtype, density, 3000 + i, scale=0.3, rpe=rpe, kpm=kpm, attn=attn)
