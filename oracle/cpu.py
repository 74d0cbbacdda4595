"""TEST INFRASTRUCTURE - ctypes wrapper over oracle/cpu_path.c (see its header).

Functions take and return torch CPU tensors and mirror the launch of the Triton
kernels in triton-shared_amd/examples/kernels.py (same arguments, same grids).
"""
import ctypes
import os
import subprocess

import torch

_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_DIR, "liboracle_cpu.so")
_lib = None


def build():
    res = subprocess.run(["make", "-C", _DIR, "-B", "liboracle_cpu.so"], capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("building the oracle failed:\n" + res.stdout + res.stderr)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = ctypes.CDLL(LIB_PATH)
        L.oracle_f16_to_f32.restype = ctypes.c_float
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f32_to_f16.restype = ctypes.c_uint16
        L.oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.oracle_valid_extent.restype = ctypes.c_int64
        L.oracle_valid_extent.argtypes = [ctypes.c_int64] * 3
        i32, p, f32 = ctypes.c_int32, ctypes.c_void_p, ctypes.c_float
        L.ref_vec_add.argtypes = [p, p, p, i32, i32, i32]
        L.ref_row_softmax.argtypes = [p, p, i32, i32, i32, i32, i32]
        L.ref_layer_norm_fwd.argtypes = [p, p, p, p, p, p, i32, i32, f32, i32, i32, i32]
        L.ref_matmul_tiles.argtypes = [p, p, p] + [i32] * 16
        L.ref_w8a16_matmul.argtypes = [p, p, p, p] + [i32] * 15
        for f in (L.ref_vec_add, L.ref_row_softmax, L.ref_layer_norm_fwd, L.ref_matmul_tiles, L.ref_w8a16_matmul):
            f.restype = None
        _lib = L
    return _lib


def _cpu(t):
    assert t.device.type == "cpu", "the oracle works on host tensors"
    return t


def cdiv(a, b):
    return (a + b - 1) // b


def vec_add(x, y, BLOCK=1024):
    x, y = _cpu(x).contiguous(), _cpu(y).contiguous()
    n = x.numel()
    z = torch.empty_like(x)
    lib().ref_vec_add(x.data_ptr(), y.data_ptr(), z.data_ptr(), n, BLOCK, cdiv(n, BLOCK))
    return z


def row_softmax(x, BLOCK=None, rows=None):
    x = _cpu(x)
    assert x.stride(1) == 1
    n_rows, n_cols = x.shape
    if BLOCK is None:
        BLOCK = 1 << (n_cols - 1).bit_length()
    rows = n_rows if rows is None else rows
    out = torch.empty((n_rows, n_cols), dtype=x.dtype)
    lib().ref_row_softmax(out.data_ptr(), x.data_ptr(), x.stride(0), out.stride(0), n_cols, BLOCK, rows)
    return out


def layer_norm_fwd(x, w, b, eps, BLOCK=1024, rows=None):
    x, w, b = _cpu(x), _cpu(w).contiguous(), _cpu(b).contiguous()
    assert x.stride(1) == 1 and x.dtype in (torch.float16, torch.bfloat16)
    M, N = x.shape
    rows = M if rows is None else rows
    y = torch.empty_like(x)
    mean = torch.empty(M, dtype=torch.float32)
    rstd = torch.empty(M, dtype=torch.float32)
    lib().ref_layer_norm_fwd(x.data_ptr(), y.data_ptr(), w.data_ptr(), b.data_ptr(), mean.data_ptr(), rstd.data_ptr(),
                             x.stride(0), N, eps, BLOCK, rows, int(x.dtype == torch.bfloat16))
    return y, mean, rstd


def matmul_tiles(a, b, BM=128, BN=128, BK=64, GROUP_M=8, pids=None, out=None):
    a, b = _cpu(a), _cpu(b)
    assert a.dtype == b.dtype and a.dtype in (torch.float16, torch.bfloat16)
    M, K = a.shape
    _, N = b.shape
    c = torch.zeros((M, N), dtype=a.dtype) if out is None else out
    grid = cdiv(M, BM) * cdiv(N, BN)
    lo, hi = (0, grid) if pids is None else pids
    lib().ref_matmul_tiles(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, a.stride(0), a.stride(1), b.stride(0),
                           b.stride(1), c.stride(0), c.stride(1), BM, BN, BK, GROUP_M, lo, hi,
                           int(a.dtype == torch.bfloat16))
    return c


def w8a16_matmul(a, w, s, BM=16, BN=128, BK=128, ys=None, out=None):
    a, w, s = _cpu(a), _cpu(w), _cpu(s).contiguous()
    assert a.dtype == torch.float16 and w.dtype == torch.int8 and s.dtype == torch.float16
    M, K = a.shape
    _, N = w.shape
    c = torch.zeros((M, N), dtype=torch.float16) if out is None else out
    gy = cdiv(N, BN)
    lo, hi = (0, gy) if ys is None else ys
    lib().ref_w8a16_matmul(a.data_ptr(), w.data_ptr(), s.data_ptr(), c.data_ptr(), M, N, K, a.stride(0), a.stride(1),
                           w.stride(0), w.stride(1), c.stride(0), c.stride(1), BM, BN, BK, cdiv(M, BM), lo, hi)
    return c
