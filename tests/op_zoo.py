"""Closed forms (numpy) for extra_kernels.int_ops / float_ops: used to pin the lane oracle on the CPU and to check the
GPU backend bit for bit."""
import numpy as np


def int_inputs(n, seed=0):
    rng = np.random.default_rng(seed)
    x = rng.integers(-2**31, 2**31, n).astype(np.int32)
    y = rng.integers(-2**31, 2**31, n).astype(np.int32)
    y[y == 0] = 7
    x[:4] = [-7, 7, -2**31, 2**31 - 1]
    y[:4] = [2, -2, 3, -1]
    return x, y


def int_expected(x, y):
    ux, uy = x.astype(np.uint32), y.astype(np.uint32)
    sh = y & 31
    x64, y64 = x.astype(np.int64), y.astype(np.int64)
    q = (np.abs(x64) // np.abs(y64)) * np.where((x64 < 0) == (y64 < 0), 1, -1)   # division truncates towards zero
    r = x64 - q * y64
    return np.stack([
        q.astype(np.int32), r.astype(np.int32), (ux // uy).view(np.int32), (ux % uy).view(np.int32),
        (x64 << sh).astype(np.uint64).astype(np.uint32).view(np.int32), x >> sh, (ux >> sh.astype(np.uint32)).view(np.int32),
        ((ux.astype(np.uint64) * uy.astype(np.uint64)) >> np.uint64(32)).astype(np.uint32).view(np.int32),
        np.abs(x64).astype(np.uint32).view(np.int32), np.where(ux < uy, x, y), (x ^ y) | (x & ~y), np.maximum(ux, uy).view(np.int32)])


def float_inputs(n, seed=1):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal(n) * 100).astype(np.float32)
    y = (rng.standard_normal(n) * 3).astype(np.float32)
    y[y == 0] = 1
    return x, y


def float_expected(x, y, lo, hi):
    ax = np.abs(x)
    return np.stack([
        np.fmin(np.fmax(x, np.float32(lo)), np.float32(hi)), np.sqrt(ax), x / y, np.trunc(x).astype(np.int32).astype(np.float32),
        np.trunc(ax).astype(np.uint32).astype(np.float32), x.view(np.int32).astype(np.float32), np.floor(x) + np.ceil(y),
        (x.astype(np.float64) * y.astype(np.float64) + x.astype(np.float64)).astype(np.float32)])
