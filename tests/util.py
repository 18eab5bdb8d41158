"""Shared helpers for the test-suite: package loader, synthetic inputs of the benchmark configs."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as graft  # noqa: E402


def mesh():
    return graft.load_package()


def codec_input(T, h=4096):
    """Boundary hidden state of the codec config: N(0,1) with 0.1% of channels (fixed indices) scaled x50."""
    rng = np.random.Generator(np.random.PCG64(1234 + T))
    x = rng.standard_normal((T, h)).astype(np.float32)
    n_out = int(np.ceil(h * 0.001))
    ch = np.random.Generator(np.random.PCG64(1234)).choice(h, size=n_out, replace=False)
    x[:, ch] *= 50
    return x


def bits_equal_nan_aware(a, b):
    """f32 arrays equal bit-for-bit, except that any NaN matches any NaN."""
    a = np.ascontiguousarray(a, np.float32).reshape(-1)
    b = np.ascontiguousarray(b, np.float32).reshape(-1)
    na, nb = np.isnan(a), np.isnan(b)
    return np.array_equal(na, nb) and np.array_equal(a[~na].view(np.uint32), b[~nb].view(np.uint32))
