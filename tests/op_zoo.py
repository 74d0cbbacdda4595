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


def philox_uniform(seed, offsets):
    """Philox-4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3") keyed by a 64-bit seed, counter =
    (offset, 0, 0, 0), first output word mapped to [0, 1): what tl.rand(seed, offset) is defined to return."""
    A, B = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
    KA, KB = 0x9E3779B9, 0xBB67AE85
    M = np.uint64(0xFFFFFFFF)
    c0 = offsets.astype(np.uint32).astype(np.uint64)
    c1 = np.zeros_like(c0)
    c2 = np.zeros_like(c0)
    c3 = np.zeros_like(c0)
    k0, k1 = int(seed) & 0xFFFFFFFF, (int(seed) >> 32) & 0xFFFFFFFF
    for _ in range(10):
        p0, p2 = A * c0, B * c2                       # 64-bit products of 32-bit values
        c0, c1, c2, c3 = ((p2 >> np.uint64(32)) ^ c1 ^ np.uint64(k0)) & M, p2 & M, ((p0 >> np.uint64(32)) ^ c3 ^ np.uint64(k1)) & M, p0 & M
        k0, k1 = (k0 + KA) & 0xFFFFFFFF, (k1 + KB) & 0xFFFFFFFF
    x = c0.astype(np.uint32).view(np.int32)
    x = np.where(x < 0, -x - 1, x)
    return x.astype(np.float32) * np.float32(4.6566127342e-10)
