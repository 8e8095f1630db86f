import math
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs an MI355X (ROCm device); run with -m gpu on the GPU box')


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason='no ROCm device in this process')
    for item in items:
        if 'gpu' in item.keywords:
            item.add_marker(skip)


SEED = 322  # the reference's tests seed with 322; inputs here are drawn on the CPU so they are portable


def cpu_gen(seed=SEED):
    return torch.Generator('cpu').manual_seed(seed)


def rand_cl3d(gen, n, c, h, w, d, mean=0.0, std=1.0):
    """fp16 (N,C,H,W,D) channels_last_3d tensor ~ N(mean, std^2), drawn in fp32 on the CPU."""
    x = torch.randn(n, c, h, w, d, generator=gen) * std + mean
    return x.half().to(memory_format=torch.channels_last_3d)


def rand_dw_weight(gen, c):
    """torch-layout depthwise weight (C,1,3,3,3) ~ N(0, 1/27) and its [3,3,3,C] kernel layout
    (the permutation of tests/ops/test_conv.py:23 of the reference)."""
    w = (torch.randn(c, 1, 3, 3, 3, generator=gen) / math.sqrt(27)).half()
    return w, w[:, 0].permute(1, 2, 3, 0).contiguous()


def from_bits(arr):
    """uint16 numpy array in logical order -> fp16 tensor (contiguous, logical shape)."""
    return torch.from_numpy(arr.view(np.int16).copy()).view(torch.float16)


@pytest.fixture(scope='session')
def golden():
    return np.load(os.path.join(ROOT, 'tests', 'golden', 'hotpath_small.npz'))


@pytest.fixture(scope='session')
def golden_config1():
    return np.load(os.path.join(ROOT, 'tests', 'golden', 'config1_dwconv.npz'))
