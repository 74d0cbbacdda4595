"""Kernels for the language features that the reference runs from Triton's own core test file
(python/examples/conftest.py:52-92 names the functions it enables).  That file is not part of the
reference tree, so these are written from the language definition: one small kernel per feature,
with closed-form expectations in core_cases.py."""
import triton
import triton.language as tl


@triton.jit
def umulhi_pairs(x_ptr, y_ptr, out_ptr, BLOCK: tl.constexpr):
    o = tl.arange(0, BLOCK)
    tl.store(out_ptr + o, tl.umulhi(tl.load(x_ptr + o), tl.load(y_ptr + o)))


@triton.jit
def sum_of_loop_indices(out_ptr, lo, hi, STEP: tl.constexpr):
    # the induction variable takes the (64-bit) type of the bounds
    acc = 0
    acc = acc.to(tl.int64)
    for i in range(lo, hi, STEP):
        acc += i
    tl.store(out_ptr, acc)


@triton.jit
def _scaled(x, k):
    return x * k


@triton.jit(noinline=True)
def _plus_one(x):
    return x + 1


@triton.jit(noinline=True)
def _plus_two(x):
    return x + 2


@triton.jit(noinline=True)
def _store_sum(x, y, dst_ptr):
    tl.store(dst_ptr, x + y)


@triton.jit(noinline=True)
def _store_sum_of_calls(x, y, dst_ptr):
    _store_sum(_plus_one(x), _plus_two(y), dst_ptr)


@triton.jit(noinline=True)
def _store_by_sign(x, y, dst_ptr):
    if x >= 1:
        x = _plus_one(x)
    else:
        x = _plus_two(x)
    tl.store(dst_ptr, x + y)


@triton.jit(noinline=True)
def _square_tile_plus(x, y, tile_ptr):
    o = tl.arange(0, 16)[:, None] * 16 + tl.arange(0, 16)[None, :]
    z = tl.load(tile_ptr + o)
    tl.store(tile_ptr + o, tl.dot(z, z) + x + y)


@triton.jit(noinline=True)
def _sum_and_difference(x, y):
    return x + y, x - y


@triton.jit
def calls_helpers(x_ptr, y_ptr, dst_ptr, KIND: tl.constexpr):
    # scalars loaded by the caller, work done in functions kept out of line (KIND 0: an inlined helper for comparison)
    x = tl.load(x_ptr)
    y = tl.load(y_ptr)
    if KIND == 0:
        tl.store(dst_ptr, _scaled(x, 2.0) + y)
    elif KIND == 1:
        _store_sum(x, y, dst_ptr)
    elif KIND == 2:
        _store_sum_of_calls(x, y, dst_ptr)
    elif KIND == 3:
        _store_by_sign(x, y, dst_ptr)
    elif KIND == 4:
        _square_tile_plus(x, y, dst_ptr)
    else:
        s, d = _sum_and_difference(x, y)
        tl.store(dst_ptr, s)
        tl.store(dst_ptr + 1, d)


@triton.jit
def index_with_new_axes(x_ptr, z2_ptr, z3_ptr, N: tl.constexpr, A: tl.constexpr, C: tl.constexpr):
    i = tl.arange(0, N)
    x = tl.load(x_ptr + i)
    z2 = x[:, None] * 100 + x[None, :]
    tl.store(z2_ptr + i[:, None] * N + i[None, :], z2)
    a = tl.arange(0, A)
    c = tl.arange(0, C)
    z3 = x[None, :, None] + (a * 1000)[:, None, None] + (c * 100000)[None, None, :]
    tl.store(z3_ptr + a[:, None, None] * (N * C) + i[None, :, None] * C + c[None, None, :], z3)


@triton.jit
def fill_constants(i8_ptr, i16_ptr, i32_ptr, i64_ptr, u8_ptr, f16_ptr, bf16_ptr, f32_ptr, f64_ptr, BLOCK: tl.constexpr):
    o = tl.arange(0, BLOCK)
    tl.store(i8_ptr + o, tl.full((BLOCK,), -7, tl.int8))
    tl.store(i16_ptr + o, tl.full((BLOCK,), -300, tl.int16))
    tl.store(i32_ptr + o, tl.full((BLOCK,), 1 << 20, tl.int32))
    tl.store(i64_ptr + o, tl.full((BLOCK,), -(1 << 40), tl.int64))
    tl.store(u8_ptr + o, tl.full((BLOCK,), 200, tl.uint8))
    tl.store(f16_ptr + o, tl.full((BLOCK,), 0.333251953125, tl.float16))
    tl.store(bf16_ptr + o, tl.full((BLOCK,), -2.5, tl.bfloat16))
    tl.store(f32_ptr + o, tl.full((BLOCK,), 3.1415927410125732, tl.float32))
    tl.store(f64_ptr + o, tl.full((BLOCK,), 2.718281828459045, tl.float64))


@triton.jit
def double_precision_ops(x_ptr, y_ptr, s_ptr, out_ptr, sum_ptr, k, n, BLOCK: tl.constexpr):
    o = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = o < n
    x = tl.load(x_ptr + o, mask=m, other=1.0)
    y = tl.load(y_ptr + o, mask=m, other=1.0)
    s = tl.load(s_ptr + o, mask=m, other=0.0)                       # fp32
    tl.store(out_ptr + 0 * n + o, x + y * k, mask=m)
    tl.store(out_ptr + 1 * n + o, x / y, mask=m)
    tl.store(out_ptr + 2 * n + o, tl.sqrt(tl.abs(x)), mask=m)
    tl.store(out_ptr + 3 * n + o, tl.maximum(x, y), mask=m)
    tl.store(out_ptr + 4 * n + o, s.to(tl.float64) * x, mask=m)
    tl.store(out_ptr + 5 * n + o, tl.where(x > y, x, -y), mask=m)
    tl.store(out_ptr + 6 * n + o, (x * 1000.0).to(tl.int32).to(tl.float64), mask=m)
    tl.store(sum_ptr + tl.program_id(0), tl.sum(tl.where(m, x, 0.0), axis=0))


@triton.jit
def does_nothing(x_ptr, SIZE: tl.constexpr):
    pass


@triton.jit
def return_inside_if(flag_ptr, out_ptr, MODE: tl.constexpr):
    f = tl.load(flag_ptr)
    if MODE == 0:
        if f > 0:
            tl.store(out_ptr, 1)
            return
        tl.store(out_ptr, 2)
    else:
        if f > 0:
            tl.store(out_ptr, 1)
            return
        else:
            if f < -5:
                tl.store(out_ptr, 3)
                return
        tl.store(out_ptr + 1, 4)


@triton.jit
def min_max_nan_rules(x_ptr, y_ptr, out_ptr, BLOCK: tl.constexpr):
    o = tl.arange(0, BLOCK)
    x = tl.load(x_ptr + o)
    y = tl.load(y_ptr + o)
    tl.store(out_ptr + o, tl.minimum(x, y))
    tl.store(out_ptr + BLOCK + o, tl.maximum(x, y))
    tl.store(out_ptr + 2 * BLOCK + o, tl.minimum(x, y, propagate_nan=tl.PropagateNan.ALL))
    tl.store(out_ptr + 3 * BLOCK + o, tl.maximum(x, y, propagate_nan=tl.PropagateNan.ALL))
    tl.store(out_ptr + 4 * BLOCK + o, tl.clamp(x, -1.0, 1.0))
    tl.store(out_ptr + 5 * BLOCK + o, tl.clamp(x, -1.0, 1.0, propagate_nan=tl.PropagateNan.ALL))


@triton.jit
def clamp_between_blocks(x_ptr, lo_ptr, hi_ptr, out_ptr, n, BLOCK: tl.constexpr):
    o = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = o < n
    x = tl.load(x_ptr + o, mask=m)
    lo = tl.load(lo_ptr + o, mask=m)
    hi = tl.load(hi_ptr + o, mask=m)
    tl.store(out_ptr + o, tl.clamp(x, lo, hi), mask=m)


@triton.jit
def permute_3d(src_ptr, dst_ptr, A: tl.constexpr, B: tl.constexpr, C: tl.constexpr):
    a = tl.arange(0, A)
    b = tl.arange(0, B)
    c = tl.arange(0, C)
    x = tl.load(src_ptr + a[:, None, None] * (B * C) + b[None, :, None] * C + c[None, None, :])
    y = tl.permute(x, (2, 0, 1))                                     # [C, A, B]
    tl.store(dst_ptr + c[:, None, None] * (A * B) + a[None, :, None] * B + b[None, None, :], y)


@triton.jit
def permute_4d_block_ptr(src_ptr, dst_ptr, S0: tl.constexpr, S1: tl.constexpr, S2: tl.constexpr, S3: tl.constexpr):
    # dims (0, 1, 2, 3) -> (3, 1, 0, 2)
    src = tl.make_block_ptr(src_ptr, (S0, S1, S2, S3), (S1 * S2 * S3, S2 * S3, S3, 1), (0, 0, 0, 0), (S0, S1, S2, S3), (3, 2, 1, 0))
    dst = tl.make_block_ptr(dst_ptr, (S3, S1, S0, S2), (S1 * S0 * S2, S0 * S2, S2, 1), (0, 0, 0, 0), (S3, S1, S0, S2), (3, 2, 1, 0))
    tl.store(dst, tl.load(src).permute((3, 1, 0, 2)))


@triton.jit
def broadcast_pair(x_ptr, y_ptr, out_ptr, M: tl.constexpr, N: tl.constexpr):
    i = tl.arange(0, M)
    j = tl.arange(0, N)
    x = tl.load(x_ptr + i)[:, None]                                   # [M, 1]
    y = tl.load(y_ptr + i[:, None] * N + j[None, :])                  # [M, N]
    xb, yb = tl.broadcast(x, y)
    z = tl.broadcast_to(tl.load(x_ptr + j)[None, :], (M, N))
    tl.store(out_ptr + i[:, None] * N + j[None, :], xb * 2 + yb + z * 3)


@triton.jit
def dot_of_constants(out_ptr, B: tl.constexpr):
    a = tl.full((B, B), 0.5, tl.float32)
    b = tl.full((B, B), 3.0, tl.float32)
    i = tl.arange(0, B)
    tl.store(out_ptr + i[:, None] * B + i[None, :], tl.dot(a, b))


@triton.jit
def product_by_broadcast_and_sum(a_ptr, b_ptr, c_ptr, M: tl.constexpr, N: tl.constexpr, K: tl.constexpr):
    i = tl.arange(0, M)
    j = tl.arange(0, N)
    k = tl.arange(0, K)
    a = tl.load(a_ptr + i[:, None] * K + k[None, :])
    b = tl.load(b_ptr + k[:, None] * N + j[None, :])
    a3 = tl.broadcast_to(a[:, :, None], (M, K, N))
    b3 = tl.broadcast_to(b[None, :, :], (M, K, N))
    tl.store(c_ptr + i[:, None] * N + j[None, :], tl.sum(a3 * b3, axis=1))


@triton.jit
def scalar_load_under_mask(src_ptr, dst_ptr, index, n, OTHER: tl.constexpr):
    v = tl.load(src_ptr + index, mask=index < n, other=OTHER)
    tl.store(dst_ptr, v)


@triton.jit
def fused_multiply_add(x_ptr, y_ptr, z_ptr, out_ptr, BLOCK: tl.constexpr):
    o = tl.arange(0, BLOCK)
    tl.store(out_ptr + o, tl.fma(tl.load(x_ptr + o), tl.load(y_ptr + o), tl.load(z_ptr + o)))


@triton.jit
def copy_from_const(src_ptr: tl.const, dst_ptr, n, BLOCK: tl.constexpr):
    o = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    tl.store(dst_ptr + o, tl.load(src_ptr + o, mask=o < n), mask=o < n)


@triton.jit
def arange_from(out_ptr, START: tl.constexpr, BLOCK: tl.constexpr):
    tl.store(out_ptr + tl.arange(0, BLOCK), tl.arange(START, START + BLOCK))


@triton.jit
def widen_halves(src_ptr, dst_ptr, BLOCK: tl.constexpr):
    o = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    tl.store(dst_ptr + o, tl.load(src_ptr + o).to(tl.float32))


@triton.jit
def absolute_values(xi_ptr, xf_ptr, xh_ptr, oi_ptr, of_ptr, oh_ptr, BLOCK: tl.constexpr):
    o = tl.arange(0, BLOCK)
    tl.store(oi_ptr + o, tl.abs(tl.load(xi_ptr + o)))
    tl.store(of_ptr + o, tl.abs(tl.load(xf_ptr + o)))
    tl.store(oh_ptr + o, tl.abs(tl.load(xh_ptr + o)))


@triton.jit
def hinted_copy(src_ptr, dst_ptr, n, BLOCK: tl.constexpr):
    o = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    o = tl.max_contiguous(tl.multiple_of(o, 8), 8)
    v = tl.load(src_ptr + o, mask=o < n, cache_modifier=".cg", eviction_policy="evict_first")
    tl.store(dst_ptr + o, v + 1, mask=o < n, cache_modifier=".wt", eviction_policy="evict_last")


@triton.jit
def volatile_copy(src_ptr, dst_ptr, BLOCK: tl.constexpr):
    o = tl.arange(0, BLOCK)
    tl.store(dst_ptr + o, tl.load(src_ptr + o, volatile=True, cache_modifier=".ca"), cache_modifier=".cs")


@triton.jit
def unary_ops(xi_ptr, xf_ptr, oi_ptr, of_ptr, BLOCK: tl.constexpr):
    o = tl.arange(0, BLOCK)
    xi = tl.load(xi_ptr + o)
    xf = tl.load(xf_ptr + o)
    tl.store(oi_ptr + o, -xi)
    tl.store(oi_ptr + BLOCK + o, ~xi)
    tl.store(oi_ptr + 2 * BLOCK + o, (xi == 0).to(tl.int32))
    tl.store(of_ptr + o, -xf)


@triton.jit
def floor_division(x_ptr, y_ptr, q_ptr, r_ptr, BLOCK: tl.constexpr):
    o = tl.arange(0, BLOCK)
    x = tl.load(x_ptr + o)
    y = tl.load(y_ptr + o)
    tl.store(q_ptr + o, x // y)
    tl.store(r_ptr + o, x % y)


@triton.jit
def scale_by_argument(x_ptr, out_ptr, k, BLOCK: tl.constexpr):
    # k == 1 is specialised to a constant by the front end; a value past 32 bits arrives as i64
    o = tl.arange(0, BLOCK)
    tl.store(out_ptr + o, tl.load(x_ptr + o).to(tl.int64) * k)


@triton.jit
def unary_math(x_ptr, out_ptr, BLOCK: tl.constexpr):
    o = tl.arange(0, BLOCK)
    x = tl.load(x_ptr + o)
    tl.store(out_ptr + 0 * BLOCK + o, tl.exp(x))
    tl.store(out_ptr + 1 * BLOCK + o, tl.log(tl.abs(x) + 1.0))
    tl.store(out_ptr + 2 * BLOCK + o, tl.cos(x))
    tl.store(out_ptr + 3 * BLOCK + o, tl.sin(x))
    tl.store(out_ptr + 4 * BLOCK + o, tl.sqrt(tl.abs(x)))
    tl.store(out_ptr + 5 * BLOCK + o, tl.rsqrt(tl.abs(x) + 0.5))
    tl.store(out_ptr + 6 * BLOCK + o, tl.erf(x))
    tl.store(out_ptr + 7 * BLOCK + o, tl.floor(x))
    tl.store(out_ptr + 8 * BLOCK + o, tl.ceil(x))
    tl.store(out_ptr + 9 * BLOCK + o, tl.exp2(x))
    tl.store(out_ptr + 10 * BLOCK + o, tl.log2(tl.abs(x) + 1.0))
    tl.store(out_ptr + 11 * BLOCK + o, tl.sigmoid(x))


@triton.jit
def dot_in_half_precision(a_ptr, b_ptr, c_ptr, M: tl.constexpr, N: tl.constexpr, K: tl.constexpr, ACC_IN: tl.constexpr):
    i = tl.arange(0, M)
    j = tl.arange(0, N)
    k = tl.arange(0, K)
    a = tl.load(a_ptr + i[:, None] * K + k[None, :])
    b = tl.load(b_ptr + k[:, None] * N + j[None, :])
    if ACC_IN:
        c = tl.load(c_ptr + i[:, None] * N + j[None, :])
        c = tl.dot(a, b, c)
    else:
        c = tl.dot(a, b)
    tl.store(c_ptr + i[:, None] * N + j[None, :], c)


@triton.jit
def dot_with_epilogue(x_ptr, y_ptr, w_ptr, z_ptr, M: tl.constexpr, N: tl.constexpr, K: tl.constexpr, EPI: tl.constexpr):
    # one tile product, then: 0 nothing, 1 + matrix, 2 + a value per row, 3 + a value per column, 4 row softmax,
    # 5 a second product with w[N, N], 6 the result stored transposed
    i = tl.arange(0, M)
    j = tl.arange(0, N)
    k = tl.arange(0, K)
    x = tl.load(x_ptr + i[:, None] * K + k[None, :])
    y = tl.load(y_ptr + k[:, None] * N + j[None, :])
    z = tl.dot(x, y)
    at = z_ptr + i[:, None] * N + j[None, :]
    if EPI == 1:
        z += tl.load(at)
    if EPI == 2:
        z += tl.load(z_ptr + i * N)[:, None]
    if EPI == 3:
        z += tl.load(z_ptr + j)[None, :]
    if EPI == 4:
        z = z - tl.max(z, 1)[:, None]
        num = tl.exp(z)
        z = num / tl.sum(num, 1)[:, None]
    if EPI == 5:
        w = tl.load(w_ptr + j[:, None] * N + j[None, :])
        z = tl.dot(z.to(w.dtype), w)
    if EPI == 6:
        tl.store(z_ptr + i[:, None] + j[None, :] * M, z)
    else:
        tl.store(at, z)


@triton.jit
def integer_ops_any_width(x_ptr, y_ptr, out_ptr, n, BLOCK: tl.constexpr):
    # the planes of test_bin_op / test_bitwise_op / test_shift_op / comparisons for whatever integer type the pointers have
    o = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = o < n
    x = tl.load(x_ptr + o, mask=m, other=1)
    y = tl.load(y_ptr + o, mask=m, other=1)
    s = (y & 3).to(x.dtype)
    tl.store(out_ptr + 0 * n + o, x + y, mask=m)
    tl.store(out_ptr + 1 * n + o, x - y, mask=m)
    tl.store(out_ptr + 2 * n + o, x * y, mask=m)
    tl.store(out_ptr + 3 * n + o, x // y, mask=m)
    tl.store(out_ptr + 4 * n + o, x % y, mask=m)
    tl.store(out_ptr + 5 * n + o, x & y, mask=m)
    tl.store(out_ptr + 6 * n + o, x | y, mask=m)
    tl.store(out_ptr + 7 * n + o, x ^ y, mask=m)
    tl.store(out_ptr + 8 * n + o, x << s, mask=m)
    tl.store(out_ptr + 9 * n + o, x >> s, mask=m)
    tl.store(out_ptr + 10 * n + o, (x < y).to(x.dtype) + (x <= y).to(x.dtype) * 2 + (x == y).to(x.dtype) * 4, mask=m)
    tl.store(out_ptr + 11 * n + o, tl.maximum(x, y) - tl.minimum(x, y), mask=m)
    tl.store(out_ptr + 12 * n + o, tl.where(x > y, x, y), mask=m)


@triton.jit
def fill_values_that_are_data(x_ptr, alt_ptr, out_ptr, n, fill, BLOCK: tl.constexpr):
    # `other` of a masked load as a kernel argument (test/Conversion/TritonToStructured/masked_ldst_sitofp_other.mlir
    # converts an integer argument for it), then as a block loaded from elsewhere
    o = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    a = tl.load(x_ptr + o, mask=o < n, other=fill.to(tl.float32))
    b = tl.load(x_ptr + o, mask=o < n, other=tl.load(alt_ptr + o))
    tl.store(out_ptr + o, a)
    tl.store(out_ptr + tl.num_programs(0) * BLOCK + o, b)


@triton.jit
def scalar_store_under_mask(dst_ptr, flag, value):
    tl.store(dst_ptr, value, mask=flag > 0)
    tl.store(dst_ptr + 1, value + 1, mask=flag <= 0)


@triton.jit
def copy_with_offsets_first(x_ptr, y_ptr, ORDER: tl.constexpr, SIZE: tl.constexpr):
    # pointer + offsets in either order; SIZE = 1 is a block of one element
    o = tl.arange(0, SIZE)
    if ORDER == 0:
        tl.store(y_ptr + o, tl.load(x_ptr + o))
    else:
        tl.store(o + y_ptr, tl.load(o + x_ptr))


@triton.jit
def dot_accumulating_in_half(a_ptr, b_ptr, c_ptr, M: tl.constexpr, N: tl.constexpr, K: tl.constexpr):
    i = tl.arange(0, M)
    j = tl.arange(0, N)
    k = tl.arange(0, K)
    a = tl.load(a_ptr + i[:, None] * K + k[None, :])
    b = tl.load(b_ptr + k[:, None] * N + j[None, :])
    tl.store(c_ptr + i[:, None] * N + j[None, :], tl.dot(a, b, out_dtype=tl.float16))
