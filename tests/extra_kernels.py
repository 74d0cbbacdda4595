"""Triton kernels used only by the tests (shapes taken from what the reference's
lit tests exercise; the code is ours)."""
import triton
import triton.language as tl


@triton.jit
def masked_copy_2d(src, dst, rows, cols):
    # a 128x256 window at (2, 3) of a buffer whose second index has pitch 1024; the same
    # access test/Conversion/TritonToStructured/masked_ldst_2d.mlir describes
    i = 2 + tl.arange(0, 128)
    j = 3 + tl.arange(0, 256)
    idx = i[:, None] + (j * 1024)[None, :]
    m = (i[:, None] < rows) & (j[None, :] < cols)
    v = tl.load(src + idx, mask=m, other=float("-inf"))
    tl.store(dst + idx, v, mask=m)


@triton.jit
def wraparound_rows(src, dst, M, BLOCK: tl.constexpr):
    # modulo addressing outside a matmul: a structured access with a period, run by the generic tile-program family
    i = (tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)) % M
    tl.store(dst + tl.arange(0, BLOCK), tl.load(src + i))


@triton.jit
def gather_rows(src, idx, dst, BLOCK: tl.constexpr):
    # data-dependent addressing: not a structured access
    k = tl.load(idx + tl.arange(0, BLOCK))
    tl.store(dst + tl.arange(0, BLOCK), tl.load(src + k))


@triton.jit
def fused_mul_add(x_ptr, y_ptr, z_ptr, n, BLOCK: tl.constexpr):
    # two ops in the map: runs on the fused-map interpreter kernel
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = i < n
    a = tl.load(x_ptr + i, mask=m)
    b = tl.load(y_ptr + i, mask=m)
    tl.store(z_ptr + i, a * b + a, mask=m)


@triton.jit
def vec_sub_swapped(x_ptr, y_ptr, z_ptr, n, BLOCK: tl.constexpr):
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = i < n
    a = tl.load(x_ptr + i, mask=m)
    b = tl.load(y_ptr + i, mask=m)
    tl.store(z_ptr + i, b - a, mask=m)


@triton.jit
def block_sum(x_ptr, out_ptr, n, BLOCK: tl.constexpr):
    # a reduction to one value per program: no hand-written family, run by the generic one
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    v = tl.load(x_ptr + i, mask=i < n, other=0.0)
    tl.store(out_ptr + tl.program_id(0), tl.sum(v, axis=0))


@triton.jit
def atomic_accumulate(x_ptr, out_ptr, n, BLOCK: tl.constexpr):
    # read-modify-write memory ops have no structured lowering: refused
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    tl.atomic_add(out_ptr + i, tl.load(x_ptr + i, mask=i < n, other=0.0), mask=i < n)


@triton.jit
def small_dot(a_ptr, b_ptr, c_ptr, B: tl.constexpr):
    # a matrix product that is not shaped like the tiled matmul kernels (no K loop): no family takes it
    i = tl.arange(0, B)
    at = i[:, None] * B + i[None, :]
    tl.store(c_ptr + at, tl.dot(tl.load(a_ptr + at), tl.load(b_ptr + at)))


# ---- small tile programs (the shapes of the reference's functional tests in python/examples; the code is ours)
@triton.jit
def wrap_rows_loop(a_ptr, c_ptr, M, N, s_am, s_an, s_cm, s_cn, BK: tl.constexpr):
    # rows 2..5 of A modulo M, two steps of BK columns (test_modulo.py: stacked wraparound)
    ra = (2 + tl.arange(0, 4)) % M
    pa = a_ptr + (ra[:, None] * s_am + tl.arange(0, 4)[None, :] * s_an)
    pc = c_ptr + s_cm * tl.arange(0, 4)[:, None] + s_cn * tl.arange(0, 4)[None, :]
    for k in range(0, 2):
        tl.store(pc, tl.load(pa))
        pa += BK * s_an
        pc += BK * s_an


@triton.jit
def wrap_cols_row(a_ptr, c_ptr, M, N, s_am, s_an, s_cm, s_cn):
    # row 7, columns 6..9 modulo N (test_modulo.py: 1-D)
    ca = (6 + tl.arange(0, 4)) % N
    tl.store(c_ptr + s_cn * tl.arange(0, 4)[None, :], tl.load(a_ptr + 7 * s_am + ca[None, :] * s_an))


@triton.jit
def wrap_cols_tile(a_ptr, c_ptr, M, N, s_am, s_an, s_cm, s_cn):
    # rows 2..5, columns 6..9 modulo N (test_modulo.py: side by side)
    ra = 2 + tl.arange(0, 4)
    ca = (6 + tl.arange(0, 4)) % N
    pa = a_ptr + (ra[:, None] * s_am + ca[None, :] * s_an)
    pc = c_ptr + s_cm * tl.arange(0, 4)[:, None] + s_cn * tl.arange(0, 4)[None, :]
    tl.store(pc, tl.load(pa))


@triton.jit
def wrap_cols_masked_loop(a_ptr, c_ptr, M, N, s_am, s_an, s_cm, s_cn, BK: tl.constexpr):
    # as above with a row mask (other = -99) and two steps down the rows (test_modulo.py: masked loop)
    ra = 2 + tl.arange(0, BK)
    ca = (6 + tl.arange(0, BK)) % N
    pa = a_ptr + (ra[:, None] * s_am + ca[None, :] * s_an)
    rk = tl.arange(0, BK)
    pc = c_ptr + s_cm * tl.arange(0, BK)[:, None] + s_cn * tl.arange(0, BK)[None, :]
    for k in range(0, 2):
        tl.store(pc, tl.load(pa, mask=rk[:, None] < 2, other=-99))
        pa += BK * s_am
        pc += BK * s_an


@triton.jit
def masked_gather_const(in0, out0):
    # every lane masked off: the store writes `other` (test_mask.py)
    offs = 100 + tl.arange(0, 4)
    tl.store(out0 + tl.arange(0, 4), tl.load(in0 + offs, mask=offs < 4, other=-1))


@triton.jit
def mask_with_scalar(in0, out0, bound, value):
    # a scalar condition in conjunction with a lane mask (test_mask.py)
    offs = tl.arange(0, 8)
    tl.store(out0 + offs, tl.load(in0 + offs, mask=(value < 5) & (offs < bound), other=-1))


@triton.jit
def swap_blocks(x_ptr, y_ptr, BLOCK: tl.constexpr):
    # in-place exchange: both loads must complete before either store (test_swap.py)
    o = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    x = tl.load(x_ptr + o)
    y = tl.load(y_ptr + o)
    tl.store(x_ptr + o, y)
    tl.store(y_ptr + o, x)


@triton.jit
def fill_rows(val, out, s_row, s_col, BC: tl.constexpr):
    # a splatted scalar argument stored as a 2-row tile (test_splat.py)
    x = tl.full((2, BC), val, dtype=tl.float32)
    r = 2 * tl.program_id(0) + tl.arange(0, 2)
    tl.store(out + (r[:, None] * s_row + tl.arange(0, BC)[None, :] * s_col), x)


@triton.jit
def scalar_walk(in0, out0):
    # scalar loads and stores through pointers advanced in a loop (test_addptr.py)
    for i in range(0, 10, 2):
        p = in0 + 1 + i
        q = out0 + 1 + i
        a = tl.load(p)
        b = tl.load(p + 1)
        tl.store(q, a)
        tl.store(q + 1, b)


@triton.jit
def affine_tile_2d(x_ptr, y_ptr, n_rows, n_cols, s0, s1, BR: tl.constexpr, BC: tl.constexpr):
    # y = 2 x + 1 on a 2-D grid of tiles (test_load_2d_tensor_block.py, with ordinary pointers)
    r = tl.program_id(0) * BR + tl.arange(0, BR)
    c = tl.program_id(1) * BC + tl.arange(0, BC)
    m = (r[:, None] < n_rows) & (c[None, :] < n_cols)
    x = tl.load(x_ptr + r[:, None] * s0 + c[None, :] * s1, mask=m, other=0.0)
    tl.store(y_ptr + r[:, None] * s0 + c[None, :] * s1, 2 * x + 1, mask=m)


@triton.jit
def copy_tile_strided(x_ptr, y_ptr, n_rows, n_cols, sx0, sx1, sy0, sy1, BR: tl.constexpr, BC: tl.constexpr):
    # masked 2-D copy between tensors of unrelated strides (a transposing read when sx1 != 1)
    r = tl.program_id(0) * BR + tl.arange(0, BR)
    c = tl.program_id(1) * BC + tl.arange(0, BC)
    m = (r[:, None] < n_rows) & (c[None, :] < n_cols)
    tl.store(y_ptr + r[:, None] * sy0 + c[None, :] * sy1, tl.load(x_ptr + r[:, None] * sx0 + c[None, :] * sx1, mask=m), mask=m)


@triton.jit
def block_ptr_affine(x_ptr, y_ptr, n_rows, n_cols, s0, s1, BR: tl.constexpr, BC: tl.constexpr):
    # y = 2 x + 1 through block pointers, boundary-checked on both dimensions (test_load_2d_tensor_block.py)
    px = tl.make_block_ptr(base=x_ptr, shape=[n_rows, n_cols], strides=[s0, s1],
                           offsets=[tl.program_id(0) * BR, tl.program_id(1) * BC], block_shape=[BR, BC], order=[1, 0])
    py = tl.make_block_ptr(base=y_ptr, shape=[n_rows, n_cols], strides=[s0, s1],
                           offsets=[tl.program_id(0) * BR, tl.program_id(1) * BC], block_shape=[BR, BC], order=[1, 0])
    x = tl.load(px, boundary_check=(0, 1), padding_option="zero")
    tl.store(py, 2 * x + 1, boundary_check=(0, 1))


@triton.jit
def block_ptr_matmul(a_ptr, b_ptr, c_ptr, M, N, K, sam, sbk, scm, BM: tl.constexpr, BN: tl.constexpr, BK: tl.constexpr, PAD: tl.constexpr):
    # C = A @ B with both operands and the result behind block pointers that advance along K (the tutorial's block-pointer
    # product, test/Conversion/TritonToStructured/block_ptr_advance.mlir's shape); PAD picks the padding of the A tiles
    pa = tl.make_block_ptr(base=a_ptr, shape=[M, K], strides=[sam, 1], offsets=[tl.program_id(0) * BM, 0], block_shape=[BM, BK], order=[1, 0])
    pb = tl.make_block_ptr(base=b_ptr, shape=[K, N], strides=[sbk, 1], offsets=[0, tl.program_id(1) * BN], block_shape=[BK, BN], order=[1, 0])
    acc = tl.zeros([BM, BN], dtype=tl.float32)
    for _ in range(0, tl.cdiv(K, BK)):
        a = tl.load(pa, boundary_check=(0, 1), padding_option=PAD)
        b = tl.load(pb, boundary_check=(0, 1), padding_option="zero")
        acc = tl.dot(a, b, acc)
        pa = tl.advance(pa, [0, BK])
        pb = tl.advance(pb, [BK, 0])
    pc = tl.make_block_ptr(base=c_ptr, shape=[M, N], strides=[scm, 1], offsets=[tl.program_id(0) * BM, tl.program_id(1) * BN], block_shape=[BM, BN], order=[1, 0])
    tl.store(pc, acc, boundary_check=(0, 1))


@triton.jit
def block_ptr_row_walk(x_ptr, y_ptr, n_rows, n_cols, s0, BR: tl.constexpr, BC: tl.constexpr):
    # one program per row block walks the columns with tl.advance
    px = tl.make_block_ptr(base=x_ptr, shape=[n_rows, n_cols], strides=[s0, 1], offsets=[tl.program_id(0) * BR, 0],
                           block_shape=[BR, BC], order=[1, 0])
    py = tl.make_block_ptr(base=y_ptr, shape=[n_rows, n_cols], strides=[s0, 1], offsets=[tl.program_id(0) * BR, 0],
                           block_shape=[BR, BC], order=[1, 0])
    for _ in range(0, tl.cdiv(n_cols, BC)):
        tl.store(py, tl.load(px, boundary_check=(0, 1)) * 0.5, boundary_check=(0, 1))
        px = tl.advance(px, [0, BC])
        py = tl.advance(py, [0, BC])


# ---- unstructured (gather / scatter) accesses --------------------------------------------
# The four kernels below compute what python/examples/test_gather_scatter.py's kernels compute
# (same index arithmetic, written our way), so that the literal tensors that test asserts are
# the expected outputs.
@triton.jit
def gather_div10(src, dst):
    lane = tl.arange(0, 64)
    where = lane
    for step in range(0, 2):
        where = where // 10 + (step + 5)
        tl.store(dst + lane + 64 * step, tl.load(src + where))
        where += 64


@triton.jit
def gather_quarter_masked(src, dst):
    lane = tl.arange(0, 64)
    for step in range(0, 2):
        pick = (lane + 64 * step) // 4
        got = tl.load(src + pick, mask=pick < 8 + 16 * step)
        tl.store(dst + lane + 64 * step, got)


@triton.jit
def gather_quarter_masked_other(src, dst):
    lane = tl.arange(0, 64)
    limit = 8
    for step in range(0, 2):
        pick = (lane + 64 * step) // 4
        got = tl.load(src + pick, mask=pick < limit, other=-1)
        tl.store(dst + lane + 64 * step, got)
        limit += 16


@triton.jit
def gather_div12_masked_store(src, dst):
    where = tl.arange(0, 64)
    to = tl.arange(0, 64)
    for step in range(0, 2):
        where = where // 12
        got = tl.load(src + where, mask=where < 64, other=99)
        tl.store(dst + to, got, mask=to < 77)
        where += 64
        to += 64


@triton.jit
def scatter_by_index(src, idx, dst, n, BLOCK: tl.constexpr):
    # dst[idx[i]] = src[i]
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = i < n
    tl.store(dst + tl.load(idx + i, mask=m), tl.load(src + i, mask=m), mask=m)


@triton.jit
def select_rows(src, dst, rows, pitch_rows, pitch_src, pitch_dst, period, R: tl.constexpr, C: tl.constexpr):
    # dst[r, :] = src[rows[r] + r % period, :]  (python/examples/test_index_select.py checks this against
    # torch.index_select)
    r = tl.arange(0, R)
    c = tl.arange(0, C)
    which = tl.load(rows + r * pitch_rows)
    tile = tl.load(src + (which[:, None] + r[:, None] % period) * pitch_src + c[None, :])
    tl.store(dst + r[:, None] * pitch_dst + c[None, :], tile)


@triton.jit
def _move_masked(src, dst, where):
    # dst[where] = src[where] where where < 32, else 0 (the store is not masked); returns the next offsets
    tl.store(dst + where, tl.load(src + where, mask=where < 32))
    return where + 32


@triton.jit
def gather_scatter_nested(src, dst):
    # python/examples/test_gather_scatter.py's nested-loop case: offsets carried through two loop levels
    where = tl.arange(0, 32)
    for i in range(0, 2):
        where = _move_masked(src, dst, where // 3 + i)
        for j in range(0, 2):
            where = _move_masked(src, dst, where // ((i + 1) * (j + 1)) + i)
        where = _move_masked(src, dst, where // 3 + i)


# ---- reductions and scans in the generic family ---------------------------------------------
@triton.jit
def reduce_rows_2d(x_ptr, out_ptr, n_rows, n_cols, pitch, BR: tl.constexpr, BC: tl.constexpr, KIND: tl.constexpr):
    # out[r] = sum / max / min over the columns of row r (one program per BR rows)
    r = tl.program_id(0) * BR + tl.arange(0, BR)
    c = tl.arange(0, BC)
    m = (r[:, None] < n_rows) & (c[None, :] < n_cols)
    if KIND == 0:
        x = tl.load(x_ptr + r[:, None] * pitch + c[None, :], mask=m, other=0.0)
        v = tl.sum(x, axis=1)
    elif KIND == 1:
        x = tl.load(x_ptr + r[:, None] * pitch + c[None, :], mask=m, other=float("-inf"))
        v = tl.max(x, axis=1)
    else:
        x = tl.load(x_ptr + r[:, None] * pitch + c[None, :], mask=m, other=float("inf"))
        v = tl.min(x, axis=1)
    tl.store(out_ptr + r, v, mask=r < n_rows)


@triton.jit
def reduce_cols_2d(x_ptr, out_ptr, n_rows, n_cols, pitch, BR: tl.constexpr, BC: tl.constexpr):
    # out[c] = sum over the rows of column c (one program per BC columns)
    r = tl.arange(0, BR)
    c = tl.program_id(0) * BC + tl.arange(0, BC)
    m = (r[:, None] < n_rows) & (c[None, :] < n_cols)
    x = tl.load(x_ptr + r[:, None] * pitch + c[None, :], mask=m, other=0.0)
    tl.store(out_ptr + c, tl.sum(x, axis=0), mask=c < n_cols)


@triton.jit
def centre_rows(x_ptr, y_ptr, n_cols, pitch, BC: tl.constexpr):
    # y[row, :] = x[row, :] - mean(x[row, :]): a reduction whose result feeds an elementwise op of the block
    row = tl.program_id(0)
    c = tl.arange(0, BC)
    m = c < n_cols
    x = tl.load(x_ptr + row * pitch + c, mask=m, other=0.0)
    mean = tl.sum(x, axis=0) / n_cols
    tl.store(y_ptr + row * pitch + c, x - mean, mask=m)


@triton.jit
def int_reductions(x_ptr, out_ptr, n, BLOCK: tl.constexpr):
    # integer sum, max, min and xor of one block
    i = tl.arange(0, BLOCK)
    x = tl.load(x_ptr + i, mask=i < n, other=0)
    tl.store(out_ptr + 0, tl.sum(x, axis=0))
    tl.store(out_ptr + 1, tl.max(x, axis=0))
    tl.store(out_ptr + 2, tl.min(x, axis=0))
    tl.store(out_ptr + 3, tl.xor_sum(x, axis=0))


@triton.jit
def arg_extremes_rows(x_ptr, max_ptr, min_ptr, n_cols, pitch, BC: tl.constexpr):
    # index of the first maximum and of the first minimum of each row
    row = tl.program_id(0)
    c = tl.arange(0, BC)
    m = c < n_cols
    hi = tl.load(x_ptr + row * pitch + c, mask=m, other=float("-inf"))
    lo = tl.load(x_ptr + row * pitch + c, mask=m, other=float("inf"))
    tl.store(max_ptr + row, tl.argmax(hi, axis=0))
    tl.store(min_ptr + row, tl.argmin(lo, axis=0))


@triton.jit
def running_sum(x_ptr, y_ptr, n, BLOCK: tl.constexpr):
    # inclusive prefix sum of each program's block
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = i < n
    tl.store(y_ptr + i, tl.cumsum(tl.load(x_ptr + i, mask=m, other=0.0), axis=0), mask=m)


@triton.jit
def running_sum_2d(x_ptr, y_ptr, pitch, BR: tl.constexpr, BC: tl.constexpr, AXIS: tl.constexpr):
    r = tl.arange(0, BR)
    c = tl.arange(0, BC)
    at = r[:, None] * pitch + c[None, :]
    tl.store(y_ptr + at, tl.cumsum(tl.load(x_ptr + at), axis=AXIS))


# ---- control flow and data-dependent scalars (semantics of python/examples/test_early_return.py,
# test_scalar_store.py, test_sign_extend.py; the code is ours)
@triton.jit
def stop_on_flag(flags, dst):
    # a program whose flag is -1 writes nothing
    flag = tl.load(flags + tl.program_id(0))
    if flag == -1:
        return
    i = tl.arange(0, 4)
    tl.store(dst + i, i + 1)


@triton.jit
def count_up_scalars(dst, N: tl.constexpr):
    # dst[0 .. N) = 0, 1, 2, ... written one scalar at a time from two nested loops
    at = dst + tl.program_id(0)
    for a in range(0, N // 2):
        v = 2 * a
        for b in range(0, N // 4):
            v += b
            tl.store(at, v)
            at += 1


@triton.jit
def window_at_loaded_offset(start_ptr, src, dst, n):
    # the window's start is read from memory and widened to 64 bits
    first = tl.load(start_ptr).to(tl.int64)
    i = first + tl.arange(0, 4)
    tl.store(dst + tl.arange(0, 4), tl.load(src + i, mask=i < n, other=11))


# ---- more access patterns of the reference's functional tests (python/examples/test_blockptr_complex_offset.py,
# test_gather_scatter_continuous.py, test_load_2d_tensor_col.py, test_mask_loop_iter_arg.py, test_nested_loops.py,
# test_reduce.py, test_tensor_index_iterargs.py, test_unstructured_mask.py, test_einsum_qhmd_hmpd_to_qhmp.py);
# the kernels are ours, written to the same semantics so that those tests' expectations apply
@triton.jit
def block_ptr_shifted_base(src, dst):
    # a 2x2 block pointer whose base is 8 elements into the buffer
    a = tl.make_block_ptr(base=src + 8, shape=(2, 2), strides=(2, 1), offsets=(0, 0), block_shape=(2, 2), order=(1, 0))
    b = tl.make_block_ptr(base=dst, shape=(2, 2), strides=(2, 1), offsets=(0, 0), block_shape=(2, 2), order=(1, 0))
    tl.store(b, tl.load(a, boundary_check=(0,)), boundary_check=(0,))


@triton.jit
def copy_as_3d(src, dst, X: tl.constexpr, Y: tl.constexpr, Z: tl.constexpr, MASK: tl.constexpr):
    # a contiguous [X, Y, Z] buffer addressed as [(X*Y), Z] with the row index split by // and %;
    # MASK 1 masks the load to z < 4 (other = 0), MASK 2 masks the store
    row = tl.arange(0, X * Y)[:, None]
    z = tl.arange(0, Z)[None, :]
    at = (row // Y) * (Y * Z) + (row % Y) * Z + z
    if MASK == 1:
        v = tl.load(src + at, mask=z < 4, other=0)
    else:
        v = tl.load(src + at)
    if MASK == 2:
        tl.store(dst + at, v, mask=z < 4)
    else:
        tl.store(dst + at, v)


@triton.jit
def block_ptr_column(src, dst, n_rows, n_cols, BR: tl.constexpr, PITCH: tl.constexpr):
    # each program copies one whole column through a [BR, 1] block pointer
    col = tl.program_id(0)
    a = tl.make_block_ptr(base=src, shape=[n_rows, n_cols], strides=[PITCH, 1], offsets=[0, col], block_shape=[BR, 1], order=[1, 0])
    b = tl.make_block_ptr(base=dst, shape=[n_rows, n_cols], strides=[PITCH, 1], offsets=[0, col], block_shape=[BR, 1], order=[1, 0])
    tl.store(b, tl.load(a))


@triton.jit
def grid_stride_copy(dst, src, total, BLOCK: tl.constexpr):
    # a grid-stride loop whose offsets are a loop-carried block and whose bound is a 64-bit argument
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    hop = tl.num_programs(0) * BLOCK
    for _ in range(tl.cdiv(total, 4)):
        m = i < total
        tl.store(dst + i, tl.load(src + i, mask=m).to(tl.float32), mask=m)
        i += hop


@triton.jit
def nested_walk(src, dst, pitch_m, pitch_n):
    # 2x2 blocks walked by pointers carried through three loop levels; three loads interleaved with three stores
    r = tl.arange(0, 2)
    a = src + (r[:, None] * pitch_m + r[None, :] * pitch_n)
    c = dst + (r[:, None] * pitch_m + r[None, :] * pitch_n)
    for i in range(0, 2):
        v1 = tl.load(a)
        for j in range(0, 2):
            a += 2 * pitch_n
            v2 = tl.load(a)
            for k in range(0, 2):
                a += 2 * pitch_n
                v3 = tl.load(a)
                tl.store(c, v1)
                c += 2 * pitch_n
                tl.store(c, v2)
                c += 2 * pitch_n
                tl.store(c, v3)
                c += 2 * pitch_n
        a += 2 * pitch_n


@triton.jit
def block_ptr_row_sum(x_ptr, out_ptr, pitch, n, BLOCK: tl.constexpr):
    # one row per program through a rank-1 block pointer with a boundary check, summed
    row = tl.program_id(0)
    p = tl.make_block_ptr(base=x_ptr, shape=[n * tl.num_programs(0)], strides=[1], offsets=[pitch * row], block_shape=[BLOCK], order=[0])
    x = tl.load(p, boundary_check=[0])
    tl.store(out_ptr + row, tl.sum(x, axis=0).to(x.dtype))


@triton.jit
def carried_offsets_masked(src, dst, bound):
    # 4 blocks of 4; the mask on the carried offsets only bites in the last block (other = -11)
    i = tl.arange(0, 4)
    o = tl.arange(0, 4)
    for _ in range(0, 4):
        tl.store(dst + o, tl.load(src + i, mask=i < bound, other=-11))
        i += 4
        o += 4


@triton.jit
def carried_offsets_nested(src, dst):
    i = tl.arange(0, 4)
    o = tl.arange(0, 4)
    for a in range(0, 2):
        i += a * 2
        tl.store(dst + o, tl.load(src + i))
        i += 4
        o += 4
        for b in range(0, 3):
            i += b * 3
            tl.store(dst + o, tl.load(src + i))
            i += 4
            o += 4


@triton.jit
def store_carried_block(dst):
    v = tl.arange(0, 4)
    o = tl.arange(0, 4)
    for _ in range(0, 2):
        tl.store(dst + o, v)
        o += 4
        v += 4


@triton.jit
def masks_from_memory_2d(src, dst, keep_rows, keep_cols, m, n, M: tl.constexpr, N: tl.constexpr):
    # rows are loaded where keep_rows says so (other = -2), columns stored where keep_cols says so
    r = tl.arange(0, M)
    c = tl.arange(0, N)
    kr = tl.load(keep_rows + r, mask=r < m, other=0) != 0
    kc = tl.load(keep_cols + c, mask=c < n, other=0) != 0
    at = r[:, None] * N + c[None, :]
    v = tl.load(src + at, mask=kr[:, None] & (c[None, :] < n), other=-2)
    tl.store(dst + at, v, mask=(r[:, None] < m) & kc[None, :])


@triton.jit
def rows_by_index_masked(src, dst, idx, n_idx, m, n, pitch_m, pitch_n, IM: tl.constexpr, N: tl.constexpr):
    # dst[k, :] = src[idx[k], :] for idx[k] < m (else -2)
    k = tl.arange(0, IM)
    c = tl.arange(0, N)
    which = tl.load(idx + k, mask=k < n_idx, other=0)
    ok = (which < m) & (k < n_idx)
    v = tl.load(src + which[:, None] * pitch_m + c[None, :] * pitch_n, mask=ok[:, None] & (c[None, :] < n), other=-2)
    tl.store(dst + k[:, None] * pitch_m + c[None, :] * pitch_n, v, mask=(k[:, None] < n_idx) & (c[None, :] < n))


@triton.jit
def einsum_qhmd_hmpd(a_ptr, b_ptr, c_ptr, Q, H, M, P, D, a_q, a_h, a_m, a_d, b_h, b_m, b_p, b_d, c_q, c_h, c_m, c_p,
                     BQ: tl.constexpr, BP: tl.constexpr):
    # C[q,h,m,p] = sum_d A[q,h,m,d] * B[h,m,p,d]; (q,h,m) flattened into one block dimension and split again by // and %
    f = tl.program_id(0) * BQ + tl.arange(0, BQ)
    p = tl.program_id(1) * BP + tl.arange(0, BP)
    okf = f < Q * H * M
    okp = p < P
    q = f // (H * M)
    h = (f % (H * M)) // M
    m = (f % (H * M)) % M
    acc = tl.zeros((BQ, BP), dtype=tl.float32)
    for d in range(D):
        av = tl.load(a_ptr + q * a_q + h * a_h + m * a_m + d * a_d, mask=okf, other=0.0)
        bv = tl.load(b_ptr + (h * b_h + m * b_m + d * b_d)[:, None] + p[None, :] * b_p, mask=okf[:, None] & okp[None, :], other=0.0)
        acc += av[:, None] * bv
    tl.store(c_ptr + (q * c_q + h * c_h + m * c_m)[:, None] + p[None, :] * c_p, acc, mask=okf[:, None] & okp[None, :])


@triton.jit
def mm_peeled(a_ptr, b_ptr, c_ptr, M, N, K, s_am, s_ak, s_bk, s_bn, s_cm, s_cn,
              BM: tl.constexpr, BN: tl.constexpr, BK: tl.constexpr):
    # the shape of python/examples/test_mm.py: whole K blocks without masks, then one masked remainder block; operand
    # rows and columns wrap (% M, % N) instead of being masked; 32x32x32 blocks, so the generic family's small products
    tn_count = tl.cdiv(N, BN)
    tm = tl.program_id(0) // tn_count
    tn = tl.program_id(0) % tn_count
    rm = tm * BM + tl.arange(0, BM)
    rn = tn * BN + tl.arange(0, BN)
    am = rm % M
    bn = rn % N
    whole = (tl.cdiv(K, BK) - 1) * BK
    acc = tl.zeros((BM, BN), dtype=tl.float32)
    for k0 in range(0, whole, BK):
        rk = k0 + tl.arange(0, BK)
        a = tl.load(a_ptr + am[:, None] * s_am + rk[None, :] * s_ak)
        b = tl.load(b_ptr + rk[:, None] * s_bk + bn[None, :] * s_bn)
        acc += tl.dot(a, b)
    rk = whole + tl.arange(0, BK)
    a = tl.load(a_ptr + am[:, None] * s_am + rk[None, :] * s_ak, mask=(rk < K)[None, :], other=0.0)
    b = tl.load(b_ptr + rk[:, None] * s_bk + bn[None, :] * s_bn, mask=(rk < K)[:, None], other=0.0)
    acc += tl.dot(a, b)
    tl.store(c_ptr + rm[:, None] * s_cm + rn[None, :] * s_cn, acc.to(c_ptr.dtype.element_ty), mask=(rm < M)[:, None] & (rn < N)[None, :])


# ---- integer, bit and conversion ops (the op classes of test_core's test_bin_op / test_bitwise_op / test_shift_op /
# test_umulhi / test_abs / test_clamp / test_floordiv / test_precise_math, which the reference's conftest whitelists)
@triton.jit
def int_ops(x_ptr, y_ptr, out_ptr, n, BLOCK: tl.constexpr):
    # 12 results per element, stored as 12 planes of n
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = i < n
    x = tl.load(x_ptr + i, mask=m, other=1)
    y = tl.load(y_ptr + i, mask=m, other=1)
    ux = x.to(tl.uint32, bitcast=True)
    uy = y.to(tl.uint32, bitcast=True)
    sh = y & 31
    tl.store(out_ptr + 0 * n + i, x // y, mask=m)                                   # signed division (truncating in the IR)
    tl.store(out_ptr + 1 * n + i, x % y, mask=m)
    tl.store(out_ptr + 2 * n + i, (ux // uy).to(tl.int32, bitcast=True), mask=m)    # unsigned division
    tl.store(out_ptr + 3 * n + i, (ux % uy).to(tl.int32, bitcast=True), mask=m)
    tl.store(out_ptr + 4 * n + i, x << sh, mask=m)
    tl.store(out_ptr + 5 * n + i, x >> sh, mask=m)                                  # arithmetic shift
    tl.store(out_ptr + 6 * n + i, (ux >> sh.to(tl.uint32)).to(tl.int32, bitcast=True), mask=m)   # logical shift
    tl.store(out_ptr + 7 * n + i, tl.umulhi(ux, uy).to(tl.int32, bitcast=True), mask=m)
    tl.store(out_ptr + 8 * n + i, tl.abs(x), mask=m)
    tl.store(out_ptr + 9 * n + i, tl.where(ux < uy, x, y), mask=m)                  # unsigned compare
    tl.store(out_ptr + 10 * n + i, (x ^ y) | (x & ~y), mask=m)
    tl.store(out_ptr + 11 * n + i, tl.maximum(ux, uy).to(tl.int32, bitcast=True), mask=m)


@triton.jit
def float_ops(x_ptr, y_ptr, out_ptr, n, lo, hi, BLOCK: tl.constexpr):
    # 8 results per element, stored as 8 planes of n
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = i < n
    x = tl.load(x_ptr + i, mask=m, other=1.0)
    y = tl.load(y_ptr + i, mask=m, other=1.0)
    tl.store(out_ptr + 0 * n + i, tl.clamp(x, lo, hi), mask=m)
    tl.store(out_ptr + 1 * n + i, tl.sqrt_rn(tl.abs(x)), mask=m)
    tl.store(out_ptr + 2 * n + i, tl.div_rn(x, y), mask=m)
    tl.store(out_ptr + 3 * n + i, x.to(tl.int32).to(tl.float32), mask=m)             # fptosi then sitofp
    tl.store(out_ptr + 4 * n + i, tl.abs(x).to(tl.uint32).to(tl.float32), mask=m)    # fptoui then uitofp
    tl.store(out_ptr + 5 * n + i, x.to(tl.int32, bitcast=True).to(tl.float32), mask=m)   # the bits as an integer
    tl.store(out_ptr + 6 * n + i, tl.floor(x) + tl.ceil(y), mask=m)
    tl.store(out_ptr + 7 * n + i, tl.fma(x, y, x), mask=m)


# ---- shape ops (test_core's whitelisted test_trans_2d / test_transpose and reshapes between ranks 1 and 2)
@triton.jit
def transpose_tile(src, dst, R: tl.constexpr, C: tl.constexpr):
    # dst[C, R] = src[R, C]^T with a bias that depends on the destination column, so a wrong index order shows
    r = tl.arange(0, R)
    c = tl.arange(0, C)
    x = tl.load(src + r[:, None] * C + c[None, :])
    y = tl.trans(x) + r[None, :].to(tl.float32)
    tl.store(dst + c[:, None] * R + r[None, :], y)


@triton.jit
def fold_and_sum(src, dst, R: tl.constexpr, C: tl.constexpr):
    # a flat block of R*C elements viewed as [R, C], summed along the columns, and written back flat after scaling
    i = tl.arange(0, R * C)
    x = tl.load(src + i)
    m = tl.reshape(x, (R, C))
    s = tl.sum(m, axis=1)
    tl.store(dst + tl.arange(0, R), s)
    tl.store(dst + R + i, tl.reshape(m * 2.0, (R * C,)))


# ---- extern elementwise functions (the libdevice symbols test/Conversion/TritonToLinalg/convert_extern_elementwise.mlir lists)
from triton.language.extra.cuda import libdevice as _libdevice  # noqa: E402  (only the symbol names matter: "__nv_powf" ...)


@triton.jit
def extern_math(x_ptr, y_ptr, out_ptr, n, BLOCK: tl.constexpr):
    # 6 planes: pow, atan2, log1p, tanh via sinh / cosh, trunc, asin of a clamped value
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = i < n
    x = tl.load(x_ptr + i, mask=m, other=1.0)
    y = tl.load(y_ptr + i, mask=m, other=1.0)
    tl.store(out_ptr + 0 * n + i, _libdevice.pow(tl.abs(x), y), mask=m)
    tl.store(out_ptr + 1 * n + i, _libdevice.atan2(x, y), mask=m)
    tl.store(out_ptr + 2 * n + i, _libdevice.log1p(tl.abs(x)), mask=m)
    tl.store(out_ptr + 3 * n + i, _libdevice.sinh(y) / _libdevice.cosh(y), mask=m)
    tl.store(out_ptr + 4 * n + i, _libdevice.trunc(x), mask=m)
    tl.store(out_ptr + 5 * n + i, _libdevice.asin(tl.minimum(tl.maximum(y, -1.0), 1.0)), mask=m)
    tl.device_assert(n > 0, "n must be positive")


# ---- kernels in the style of the Triton tutorials, run by the generic family
@triton.jit
def seeded_dropout(x_ptr, out_ptr, n, p, seed, BLOCK: tl.constexpr):
    # tutorial 04: a Philox random number per element (umulhi, xor, shifts), compare, select, scale
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = i < n
    x = tl.load(x_ptr + i, mask=m)
    keep = tl.rand(seed, i) > p
    tl.store(out_ptr + i, tl.where(keep, x / (1 - p), 0.0), mask=m)


@triton.jit
def rms_norm_rows(x_ptr, w_ptr, y_ptr, pitch, n_cols, eps, BLOCK: tl.constexpr):
    # y = x / sqrt(mean(x^2) + eps) * w, one row per program, fp16 in and out, fp32 arithmetic
    row = tl.program_id(0)
    c = tl.arange(0, BLOCK)
    m = c < n_cols
    x = tl.load(x_ptr + row * pitch + c, mask=m, other=0.0).to(tl.float32)
    w = tl.load(w_ptr + c, mask=m, other=0.0).to(tl.float32)
    r = 1.0 / tl.sqrt(tl.sum(x * x, axis=0) / n_cols + eps)
    tl.store(y_ptr + row * pitch + c, (x * r * w).to(tl.float16), mask=m)


@triton.jit
def column_sums_looped(x_ptr, out_ptr, n_rows, n_cols, pitch, BR: tl.constexpr, BC: tl.constexpr):
    # the shape of the tutorial's LayerNorm backward dw/db kernel: a [BR, BC] accumulator carried down the rows, summed at the end
    c = tl.program_id(0) * BC + tl.arange(0, BC)
    acc = tl.zeros((BR, BC), dtype=tl.float32)
    for r0 in range(0, n_rows, BR):
        r = r0 + tl.arange(0, BR)
        m = (r[:, None] < n_rows) & (c[None, :] < n_cols)
        acc += tl.load(x_ptr + r[:, None] * pitch + c[None, :], mask=m, other=0.0)
    tl.store(out_ptr + c, tl.sum(acc, axis=0), mask=c < n_cols)


@triton.jit
def log_sum_exp_rows(x_ptr, out_ptr, pitch, n_cols, BLOCK: tl.constexpr):
    row = tl.program_id(0)
    c = tl.arange(0, BLOCK)
    x = tl.load(x_ptr + row * pitch + c, mask=c < n_cols, other=-float("inf"))
    top = tl.max(x, axis=0)
    tl.store(out_ptr + row, top + tl.log(tl.sum(tl.exp(x - top), axis=0)))


@triton.jit
def join_split_cat(a_ptr, b_ptr, out_ptr, N: tl.constexpr):
    # out[0 : 2N] = interleave(a, b) (join + reshape); out[2N : 4N] = cat(a + 1, b + 1); out[4N : 5N], out[5N : 6N] = the two
    # halves split out of the joined block again, swapped
    i = tl.arange(0, N)
    a = tl.load(a_ptr + i)
    b = tl.load(b_ptr + i)
    tl.store(out_ptr + tl.arange(0, 2 * N), tl.interleave(a, b))
    tl.store(out_ptr + 2 * N + tl.arange(0, 2 * N), tl.cat(a + 1, b + 1, can_reorder=True))
    first, second = tl.split(tl.join(a, b))
    tl.store(out_ptr + 4 * N + i, second)
    tl.store(out_ptr + 5 * N + i, first)


@triton.jit
def branch_with_results(x_ptr, flag_ptr, out_ptr, N: tl.constexpr):
    # an if / else on a value read from memory that produces a block, a float scalar and an integer scalar
    pid = tl.program_id(0)
    i = tl.arange(0, N)
    x = tl.load(x_ptr + i)
    f = tl.load(flag_ptr + pid)
    if f > 0:
        y = x * 2.0
        s = 1.0
        k = f * 3
    else:
        y = x - 1.0
        s = -1.0
        k = 7 - f
    tl.store(out_ptr + pid * N + i, y + s + k.to(tl.float32))


@triton.jit
def softmax_persistent(out_ptr, in_ptr, in_pitch, out_pitch, n_rows, n_cols, BLOCK: tl.constexpr):
    # the current fused-softmax tutorial: each program walks rows pid, pid + num_programs, ...
    first = tl.program_id(0)
    hop = tl.num_programs(0)
    for row in tl.range(first, n_rows, hop):
        c = tl.arange(0, BLOCK)
        m = c < n_cols
        x = tl.load(in_ptr + row * in_pitch + c, mask=m, other=-float("inf"))
        e = tl.exp(x - tl.max(x, axis=0))
        tl.store(out_ptr + row * out_pitch + c, e / tl.sum(e, axis=0), mask=m)


@triton.jit
def matmul_leaky(a_ptr, b_ptr, c_ptr, M, N, K, s_am, s_bk, s_cm, slope, BM: tl.constexpr, BN: tl.constexpr, BK: tl.constexpr,
                 ACT: tl.constexpr = 0, bias_ptr=None):
    # a tiled matmul with elementwise ops fused before the narrowing store (the tutorial's ACTIVATION hook).  ACT 0: leaky
    # relu, 1: x * sigmoid(slope * x) -- functions of the accumulator alone, which the matmul kernels take as an epilogue;
    # 2: a bias per column before the leaky relu, 3: slope * acc + what the output held -- these depend on the element's
    # position, which the epilogue finds through the table of tile owners
    tm = tl.program_id(0)
    tn = tl.program_id(1)
    rm = tm * BM + tl.arange(0, BM)
    rn = tn * BN + tl.arange(0, BN)
    rk = tl.arange(0, BK)
    pa = a_ptr + rm[:, None] * s_am + rk[None, :]
    pb = b_ptr + rk[:, None] * s_bk + rn[None, :]
    acc = tl.zeros((BM, BN), dtype=tl.float32)
    for k in range(0, tl.cdiv(K, BK)):
        left = K - k * BK
        a = tl.load(pa, mask=(rm[:, None] < M) & (rk[None, :] < left), other=0.0)
        b = tl.load(pb, mask=(rk[:, None] < left) & (rn[None, :] < N), other=0.0)
        acc = tl.dot(a, b, acc)
        pa += BK
        pb += BK * s_bk
    if ACT == 1:
        acc = acc * tl.sigmoid(acc * slope)
    elif ACT == 3:
        at = c_ptr + rm[:, None] * s_cm + rn[None, :]
        acc = acc * slope + tl.load(at, mask=(rm[:, None] < M) & (rn[None, :] < N), other=0.0).to(tl.float32)
    else:
        if ACT == 2:
            acc += tl.load(bias_ptr + rn, mask=rn < N, other=0.0)[None, :]
        acc = tl.where(acc >= 0, acc, slope * acc)
    tl.store(c_ptr + rm[:, None] * s_cm + rn[None, :], acc.to(c_ptr.dtype.element_ty), mask=(rm[:, None] < M) & (rn[None, :] < N))


@triton.jit
def masks_from_memory_3d(src, dst, keep_rows, keep_cols, b, m, n, B: tl.constexpr, M: tl.constexpr, N: tl.constexpr):
    # masks_from_memory_2d for every matrix of a batch: the middle index masked by data on the load, the last one on the store
    q = tl.arange(0, B)
    r = tl.arange(0, M)
    c = tl.arange(0, N)
    kr = tl.load(keep_rows + r, mask=r < m, other=0) != 0
    kc = tl.load(keep_cols + c, mask=c < n, other=0) != 0
    at = q[:, None, None] * (m * n) + r[None, :, None] * n + c[None, None, :]
    v = tl.load(src + at, mask=(q[:, None, None] < b) & kr[None, :, None] & (c[None, None, :] < n), other=-2)
    tl.store(dst + at, v, mask=(q[:, None, None] < b) & (r[None, :, None] < m) & kc[None, None, :])


@triton.jit
def columns_by_index_masked(src, dst, idx, n_idx, m, n, pitch_m, pitch_n, M: tl.constexpr, IN: tl.constexpr):
    # dst[:, idx[k]] = src[:, k] for idx[k] < n
    r = tl.arange(0, M)
    k = tl.arange(0, IN)
    which = tl.load(idx + k, mask=k < n_idx, other=0)
    ok = (which < n) & (k < n_idx)
    v = tl.load(src + r[:, None] * pitch_m + k[None, :] * pitch_n, mask=(r[:, None] < m) & (k[None, :] < n_idx), other=-2)
    tl.store(dst + r[:, None] * pitch_m + which[None, :] * pitch_n, v, mask=(r[:, None] < m) & ok[None, :])


@triton.jit
def rows_by_index_masked_3d(src, dst, idx, n_idx, b, m, n, s_b, s_m, s_n, d_b, d_m, d_n, B: tl.constexpr, IM: tl.constexpr, N: tl.constexpr):
    # dst[q, k, :] = src[q, idx[k], :] for idx[k] < m (else -2)
    q = tl.arange(0, B)
    k = tl.arange(0, IM)
    c = tl.arange(0, N)
    which = tl.load(idx + k, mask=k < n_idx, other=0)
    ok = (which < m) & (k < n_idx)
    v = tl.load(src + q[:, None, None] * s_b + which[None, :, None] * s_m + c[None, None, :] * s_n,
                mask=(q[:, None, None] < b) & ok[None, :, None] & (c[None, None, :] < n), other=-2)
    tl.store(dst + q[:, None, None] * d_b + k[None, :, None] * d_m + c[None, None, :] * d_n, v,
             mask=(q[:, None, None] < b) & (k[None, :, None] < n_idx) & (c[None, None, :] < n))


@triton.jit
def columns_by_index_masked_3d(src, dst, idx, n_idx, b, m, n, s_b, s_m, s_n, B: tl.constexpr, M: tl.constexpr, IN: tl.constexpr):
    # dst[q, :, idx[k]] = src[q, :, k] for idx[k] < n
    q = tl.arange(0, B)
    r = tl.arange(0, M)
    k = tl.arange(0, IN)
    which = tl.load(idx + k, mask=k < n_idx, other=0)
    ok = (which < n) & (k < n_idx)
    v = tl.load(src + q[:, None, None] * s_b + r[None, :, None] * s_m + k[None, None, :] * s_n,
                mask=(q[:, None, None] < b) & (r[None, :, None] < m) & (k[None, None, :] < n_idx), other=-2)
    tl.store(dst + q[:, None, None] * s_b + r[None, :, None] * s_m + which[None, None, :] * s_n, v,
             mask=(q[:, None, None] < b) & (r[None, :, None] < m) & ok[None, None, :])


@triton.jit
def masks_above_program_id(src, dst, m, n, s_pid, s_m, s_n, M: tl.constexpr, N: tl.constexpr):
    # rows beyond the program id are loaded (other = -2), columns beyond it stored: comparisons against a value that is
    # not a bound of the block, together with the ordinary bounds
    pid = tl.program_id(0)
    r = tl.arange(0, M)
    c = tl.arange(0, N)
    at = pid * s_pid + r[:, None] * s_m + c[None, :] * s_n
    v = tl.load(src + at, mask=(r[:, None] < m) & (c[None, :] < n) & (r > pid)[:, None], other=-2)
    tl.store(dst + at, v, mask=(r[:, None] < m) & (c[None, :] < n) & (c > pid)[None, :])


# ---- blocks past the register budget, reductions of rank-3 blocks -----------------------------
@triton.jit
def reduce_big_block_2d(x_ptr, out_ptr, R: tl.constexpr, C: tl.constexpr, AXIS: tl.constexpr, KIND: tl.constexpr):
    # one program reduces a whole [R, C] block (test/Conversion/TritonToLinalg/reducesum_512_256_*_axis{0,1}.mlir do this at 512 x 256)
    r = tl.arange(0, R)
    c = tl.arange(0, C)
    x = tl.load(x_ptr + r[:, None] * C + c[None, :])
    if KIND == 0:
        v = tl.sum(x, axis=AXIS)
    else:
        v = tl.max(x, axis=AXIS)
    if AXIS == 0:
        tl.store(out_ptr + c, v)
    else:
        tl.store(out_ptr + r, v)


@triton.jit
def block_total_and_extremes(x_ptr, out_ptr, n, BLOCK: tl.constexpr):
    i = tl.arange(0, BLOCK)
    x = tl.load(x_ptr + i, mask=i < n, other=0)
    tl.store(out_ptr, tl.sum(x, axis=0))
    tl.store(out_ptr + 1, tl.max(x, axis=0))
    tl.store(out_ptr + 2, tl.min(x, axis=0))


@triton.jit
def reduce_3d(x_ptr, out_ptr, A: tl.constexpr, B: tl.constexpr, C: tl.constexpr, AXIS: tl.constexpr, KIND: tl.constexpr):
    # test/Conversion/StructuredToMemref/reducesum_middle_dim.mlir reduces the middle index of a rank-3 block
    a = tl.arange(0, A)
    b = tl.arange(0, B)
    c = tl.arange(0, C)
    x = tl.load(x_ptr + a[:, None, None] * (B * C) + b[None, :, None] * C + c[None, None, :])
    if KIND == 0:
        v = tl.sum(x, axis=AXIS)
    else:
        v = tl.max(x, axis=AXIS)
    if AXIS == 0:
        tl.store(out_ptr + b[:, None] * C + c[None, :], v)
    elif AXIS == 1:
        tl.store(out_ptr + a[:, None] * C + c[None, :], v)
    else:
        tl.store(out_ptr + a[:, None] * B + b[None, :], v)


@triton.jit
def shift_left_in_place(x_ptr, R: tl.constexpr, C: tl.constexpr):
    # every element takes its right neighbour's old value: all loads come before any store, whatever the block's size
    at = tl.arange(0, R)[:, None] * C + tl.arange(0, C)[None, :]
    tl.store(x_ptr + at, tl.load(x_ptr + at + 1))


@triton.jit
def grouped_rows_matmul(a_ptr, b_ptr, c_ptr, rows_ptr, expert_ptr, n_rows, K, N, s_am, s_be, s_bk, s_cm,
                        BM: tl.constexpr, BN: tl.constexpr, BK: tl.constexpr):
    # C[i, :] = A[rows[i], :] @ B[expert of i's block] -- the shape of a mixture-of-experts layer
    # (test/Conversion/TritonToLinalgExperimental/unstructured_ptr_used_in_loop.mlir is such a kernel): a scalar read
    # from memory picks the weight matrix and may end the program early, the rows of A come through loaded indices,
    # and both blocks of pointers are carried along K by the loop
    pid_m = tl.program_id(0)
    pid_n = tl.program_id(1)
    expert = tl.load(expert_ptr + pid_m)
    if expert < 0:
        return
    i = pid_m * BM + tl.arange(0, BM)
    ok = i < n_rows
    which = tl.load(rows_ptr + i, mask=ok, other=0)
    j = pid_n * BN + tl.arange(0, BN)
    k = tl.arange(0, BK)
    a_ptrs = a_ptr + which[:, None] * s_am + k[None, :]
    b_ptrs = b_ptr + expert * s_be + k[:, None] * s_bk + j[None, :]
    acc = tl.zeros((BM, BN), tl.float32)
    for k0 in range(0, K, BK):
        a = tl.load(a_ptrs, mask=ok[:, None] & (k[None, :] < K - k0), other=0.0)
        b = tl.load(b_ptrs, mask=(k[:, None] < K - k0) & (j[None, :] < N), other=0.0)
        acc = tl.dot(a, b, acc)
        a_ptrs += BK
        b_ptrs += BK * s_bk
    tl.store(c_ptr + i[:, None] * s_cm + j[None, :], acc, mask=ok[:, None] & (j[None, :] < N))


@triton.jit
def pointer_picked_by_branch(src, dst, which):
    # both sides of a branch produce a pointer into the same argument (test/Conversion/TritonToStructured/conditional_ptr_as_src.mlir)
    if which == 5:
        p = src + which * 2
    else:
        p = src + which
    i = tl.arange(0, 4)
    tl.store(dst + i, tl.load(p + 6 + i))


@triton.jit
def matmul_grouped_order_plus_bias(a_ptr, b_ptr, c_ptr, bias_ptr, M, N, K, s_am, s_bk, s_cm, BM: tl.constexpr, BN: tl.constexpr, BK: tl.constexpr,
                                   GROUP_M: tl.constexpr):
    # the tutorial's one-dimensional grid (tiles walked in groups of GROUP_M rows) with a bias per row and per column added
    # before the cast: the epilogue has to find the program that owns an element through that tile order
    pid = tl.program_id(0)
    tiles_m = tl.cdiv(M, BM)
    tiles_n = tl.cdiv(N, BN)
    per_group = GROUP_M * tiles_n
    m0 = (pid // per_group) * GROUP_M
    rows_in_group = min(tiles_m - m0, GROUP_M)
    tm = m0 + (pid % rows_in_group)
    tn = (pid % per_group) // rows_in_group
    rm = tm * BM + tl.arange(0, BM)
    rn = tn * BN + tl.arange(0, BN)
    rk = tl.arange(0, BK)
    pa = a_ptr + rm[:, None] * s_am + rk[None, :]
    pb = b_ptr + rk[:, None] * s_bk + rn[None, :]
    acc = tl.zeros((BM, BN), dtype=tl.float32)
    for k in range(0, tl.cdiv(K, BK)):
        left = K - k * BK
        a = tl.load(pa, mask=(rm[:, None] < M) & (rk[None, :] < left), other=0.0)
        b = tl.load(pb, mask=(rk[:, None] < left) & (rn[None, :] < N), other=0.0)
        acc = tl.dot(a, b, acc)
        pa += BK
        pb += BK * s_bk
    acc += tl.load(bias_ptr + rn, mask=rn < N, other=0.0)[None, :] + 16.0 * tl.load(bias_ptr + N + rm, mask=rm < M, other=0.0)[:, None]
    tl.store(c_ptr + rm[:, None] * s_cm + rn[None, :], acc.to(c_ptr.dtype.element_ty), mask=(rm[:, None] < M) & (rn[None, :] < N))


@triton.jit
def pointer_blocks_by_branch(src, idx, dst, flag, pitch, BLOCK: tl.constexpr):
    # a block of pointers chosen by an if / else (one side gathered through loaded row numbers, the other strided) and then
    # by tl.where between two blocks of pointers (TritonToStructured/conditional_ptr_as_src_for_yield_input.mlir's shape)
    offs = tl.arange(0, BLOCK)
    rows = tl.load(idx + offs)
    if flag == 0:
        p = src + rows * pitch + offs
    else:
        p = src + offs * 2
    q = tl.where((offs % 2) == 0, p, src + offs + tl.program_id(0))
    tl.store(dst + tl.program_id(0) * BLOCK + offs, tl.load(q))


@triton.jit
def float_bits_through_pointer_cast(x_ptr, bits_ptr, y_ptr, n, BLOCK: tl.constexpr):
    # the same buffer read as fp32 and, through a pointer cast, as its bit patterns; the sign bit is cleared in the integer
    # view and the result written back through a float buffer seen as integers
    offs = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = offs < n
    xi = x_ptr.to(tl.pointer_type(tl.int32))
    b = tl.load(xi + offs, mask=m, other=0)
    tl.store(bits_ptr + offs, b, mask=m)
    yi = (y_ptr + 0).to(tl.pointer_type(tl.int32))
    tl.store(yi + offs, b & 0x7FFFFFFF, mask=m)


@triton.jit
def double_in_place_then_square(p_ptr, q_ptr, n, BLOCK: tl.constexpr):
    # a load that follows a store to the same buffer inside one program has to see the store: q = (2 p)^2, not p^2
    offs = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = offs < n
    x = tl.load(p_ptr + offs, mask=m)
    tl.store(p_ptr + offs, x + x, mask=m)
    y = tl.load(p_ptr + offs, mask=m)
    tl.store(q_ptr + offs, y * y, mask=m)


@triton.jit
def bump_counter_and_report(acc_ptr, out_ptr, BLOCK: tl.constexpr):
    # a scalar read, then a scalar write of the same address, then the value read goes out as a block: every element of
    # `out` is the old value; and a second read after the write sees the new one
    old = tl.load(acc_ptr)
    tl.store(acc_ptr, old + 1)
    offs = tl.arange(0, BLOCK)
    tl.store(out_ptr + offs, tl.zeros((BLOCK,), tl.int32) + old)
    new = tl.load(acc_ptr)
    tl.store(out_ptr + BLOCK + offs, tl.zeros((BLOCK,), tl.int32) + new)


@triton.jit
def strided_row_softmax(out_ptr, in_ptr, in_pitch, out_pitch, col_stride, n_cols, BLOCK: tl.constexpr):
    # the row softmax over every col_stride-th element of the input row
    r = tl.program_id(0)
    cols = tl.arange(0, BLOCK)
    v = tl.load(in_ptr + r * in_pitch + cols * col_stride, mask=cols < n_cols, other=-float("inf"))
    e = tl.exp(v - tl.max(v, axis=0))
    p = e / tl.sum(e, axis=0)
    tl.store(out_ptr + r * out_pitch + cols, p, mask=cols < n_cols)


@triton.jit
def transpose_tiles(src, dst, R, C, BR: tl.constexpr, BC: tl.constexpr):
    # dst[C, R] = src[R, C]^T in tiles of [BR, BC]: the transposed tile is read coalesced, turned in LDS and written coalesced
    pr = tl.program_id(0)
    pc = tl.program_id(1)
    r = pr * BR + tl.arange(0, BR)
    c = pc * BC + tl.arange(0, BC)
    m = (r[:, None] < R) & (c[None, :] < C)
    x = tl.load(src + r[:, None] * C + c[None, :], mask=m, other=0.0)
    tl.store(dst + c[:, None] * R + r[None, :], tl.trans(x * 2.0), mask=tl.trans(m))


@triton.jit
def attention_fwd(Q, K, V, O, sm_scale, seq, stride_h, stride_s, BM: tl.constexpr, BN: tl.constexpr, D: tl.constexpr):
    # flash-attention forward, one (query block, head) per program, plain pointer arithmetic on fp16 tensors: two tile products
    # per step, an online softmax whose running maximum and sum (vectors of BM) are carried next to the [BM, D] accumulator
    pm = tl.program_id(0)
    ph = tl.program_id(1)
    rm = pm * BM + tl.arange(0, BM)
    rd = tl.arange(0, D)
    q = tl.load(Q + ph * stride_h + rm[:, None] * stride_s + rd[None, :], mask=rm[:, None] < seq, other=0.0)
    m_i = tl.zeros([BM], dtype=tl.float32) - float("inf")
    l_i = tl.zeros([BM], dtype=tl.float32)
    acc = tl.zeros([BM, D], dtype=tl.float32)
    for start in range(0, seq, BN):
        rn = start + tl.arange(0, BN)
        k = tl.load(K + ph * stride_h + rn[:, None] * stride_s + rd[None, :], mask=rn[:, None] < seq, other=0.0)
        v = tl.load(V + ph * stride_h + rn[:, None] * stride_s + rd[None, :], mask=rn[:, None] < seq, other=0.0)
        qk = tl.dot(q, tl.trans(k)) * sm_scale
        qk = tl.where(rn[None, :] < seq, qk, -float("inf"))
        m_new = tl.maximum(m_i, tl.max(qk, axis=1))
        p = tl.exp(qk - m_new[:, None])
        alpha = tl.exp(m_i - m_new)
        l_i = l_i * alpha + tl.sum(p, axis=1)
        acc = acc * alpha[:, None] + tl.dot(p.to(tl.float16), v)
        m_i = m_new
    acc = acc / l_i[:, None]
    tl.store(O + ph * stride_h + rm[:, None] * stride_s + rd[None, :], acc.to(tl.float16), mask=rm[:, None] < seq)


@triton.jit
def narrow_scaled(x_ptr, y_ptr, n, scale, BLOCK: tl.constexpr):
    # y = (x * scale) narrowed to y's element type: one elementwise pass
    o = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    x = tl.load(x_ptr + o, mask=o < n, other=0.0)
    tl.store(y_ptr + o, (x * scale).to(y_ptr.dtype.element_ty), mask=o < n)


@triton.jit
def narrow_scaled_with_row_max(x_ptr, y_ptr, m_ptr, n_cols, scale, BLOCK: tl.constexpr):
    # the same narrowing next to a reduction (a row per program): the generic family
    r = tl.program_id(0)
    c = tl.arange(0, BLOCK)
    x = tl.load(x_ptr + r * n_cols + c, mask=c < n_cols, other=0.0)
    tl.store(m_ptr + r, tl.max(tl.abs(x), axis=0))
    tl.store(y_ptr + r * n_cols + c, (x * scale).to(y_ptr.dtype.element_ty), mask=c < n_cols)


@triton.jit
def stamp_tiles(out_ptr, R, C, BR: tl.constexpr, BC: tl.constexpr):
    # every element gets its program's ids and the grid's extents: rows on program_id(0), columns on program_id(1)
    p0 = tl.program_id(0)
    p1 = tl.program_id(1)
    r = p0 * BR + tl.arange(0, BR)
    c = p1 * BC + tl.arange(0, BC)
    v = p0 * 100 + p1 + 10000 * tl.num_programs(0) + 1000000 * tl.num_programs(1)
    tile = tl.zeros((BR, BC), dtype=tl.int32) + v
    tl.store(out_ptr + r[:, None] * C + c[None, :], tile, mask=(r[:, None] < R) & (c[None, :] < C))


@triton.jit
def softmax_row_in_pieces(x_ptr, y_ptr, cnt_ptr, stride, N, BLOCK: tl.constexpr):
    # a row longer than a block: running maximum and sum carried through the loop as scalars (an online softmax), and a
    # carried integer that counts the positive elements
    row = tl.program_id(0)
    m_i = -float("inf")
    l_i = 0.0
    pos = 0
    for s in range(0, N, BLOCK):
        cols = s + tl.arange(0, BLOCK)
        x = tl.load(x_ptr + row * stride + cols, mask=cols < N, other=-float("inf"))
        m_new = tl.maximum(m_i, tl.max(x, 0))
        l_i = l_i * tl.exp(m_i - m_new) + tl.sum(tl.exp(x - m_new), 0)
        m_i = m_new
        pos += tl.sum((x > 0).to(tl.int32), 0)
    for s in range(0, N, BLOCK):
        cols = s + tl.arange(0, BLOCK)
        x = tl.load(x_ptr + row * stride + cols, mask=cols < N, other=0.0)
        tl.store(y_ptr + row * stride + cols, tl.exp(x - m_i) / l_i, mask=cols < N)
    tl.store(cnt_ptr + row, pos)


@triton.jit
def scale_add_2d(x_ptr, y_ptr, out_ptr, n_cols, stride, alpha, ROWS_ON_X: tl.constexpr, BLOCK: tl.constexpr):
    # out[r, c] = alpha * x[r, c] + y[r, c] + r + c / 1024 on a two-dimensional grid, rows on either axis: the result
    # tells which program wrote an element
    if ROWS_ON_X:
        row = tl.program_id(0)
        cb = tl.program_id(1)
    else:
        row = tl.program_id(1)
        cb = tl.program_id(0)
    cols = cb * BLOCK + tl.arange(0, BLOCK)
    m = cols < n_cols
    x = tl.load(x_ptr + row * stride + cols, mask=m, other=0.0)
    y = tl.load(y_ptr + row * stride + cols, mask=m, other=0.0)
    tl.store(out_ptr + row * stride + cols, alpha * x + y, mask=m)


@triton.jit
def while_halve(x_ptr, y_ptr, n, BLOCK: tl.constexpr):
    # y = x / 2^floor(log2 n): a `while` that carries an integer and a block
    offs = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    acc = tl.load(x_ptr + offs, mask=offs < n, other=0.0)
    k = n
    while k > 1:
        acc = acc * 0.5
        k = k // 2
    tl.store(y_ptr + offs, acc, mask=offs < n)


@triton.jit
def while_sum_until(x_ptr, out_ptr, cnt_ptr, stride, n, limit, BLOCK: tl.constexpr):
    # a row is summed piece by piece until the sum reaches `limit` or the row ends: how often the loop runs depends on
    # the data, and differs from program to program
    row = tl.program_id(0)
    k = 0
    acc = 0.0
    while (k < n) & (acc < limit):
        cols = k + tl.arange(0, BLOCK)
        x = tl.load(x_ptr + row * stride + cols, mask=cols < n, other=0.0)
        acc += tl.sum(x, 0)
        k += BLOCK
    tl.store(out_ptr + row, acc)
    tl.store(cnt_ptr + row, k)


@triton.jit
def while_carried_pointer(x_ptr, out_ptr, stride, n, BLOCK: tl.constexpr):
    # a block of pointers carried by a `while`, stepped along the row
    row = tl.program_id(0)
    offs = tl.arange(0, BLOCK)
    p = x_ptr + row * stride + offs
    k = 0
    acc = tl.zeros((BLOCK,), dtype=tl.float32)
    while k < n:
        acc += tl.load(p, mask=k + offs < n, other=0.0)
        p += BLOCK
        k += BLOCK
    tl.store(out_ptr + row, tl.sum(acc, 0))


@triton.jit
def while_inside_for(x_ptr, out_ptr, n, BLOCK: tl.constexpr):
    # a `while` inside a `for`: out = x * sum over i < n of (i + i // 2 + i // 4 + ...)
    offs = tl.arange(0, BLOCK)
    acc = tl.zeros((BLOCK,), dtype=tl.float32)
    for i in range(0, n):
        k = i
        while k > 0:
            acc += tl.load(x_ptr + offs) * k
            k = k // 2
    tl.store(out_ptr + offs, acc)


@triton.jit
def grid_stamp(out_ptr, BLOCK: tl.constexpr):
    # every program writes a block of integers made from its ids and the grid's extents: what a launch hands to
    # program_id / num_programs on each axis, whatever the extents are
    x = tl.program_id(0)
    y = tl.program_id(1)
    z = tl.program_id(2)
    nx = tl.num_programs(0)
    ny = tl.num_programs(1)
    offs = tl.arange(0, BLOCK)
    lin = (z * ny + y) * nx + x
    vals = x * 1000003 + y * 7 + z * 131 + offs * 3 + tl.num_programs(2)
    tl.store(out_ptr + lin * BLOCK + offs, vals)


@triton.jit
def add_rows_2d(x_ptr, y_ptr, z_ptr, n_cols, BLOCK: tl.constexpr):
    # z = x + y on [rows, n_cols]: column blocks on program_id(0), rows on program_id(1)
    row = tl.program_id(1)
    cols = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    mask = cols < n_cols
    a = tl.load(x_ptr + row * n_cols + cols, mask=mask)
    b = tl.load(y_ptr + row * n_cols + cols, mask=mask)
    tl.store(z_ptr + row * n_cols + cols, a + b, mask=mask)


@triton.jit
def scale_tile_and_row_sums(x_ptr, s_ptr, y_ptr, sums_ptr, n_rows, n_cols, pitch, BR: tl.constexpr, BC: tl.constexpr):
    # y = x * s[None, :] on [BR, BC] tiles (x and y in a 16-bit type, s in fp32), and each tile's row sums of x
    r = tl.program_id(0) * BR + tl.arange(0, BR)
    c = tl.program_id(1) * BC + tl.arange(0, BC)
    m = (r[:, None] < n_rows) & (c[None, :] < n_cols)
    x = tl.load(x_ptr + r[:, None] * pitch + c[None, :], mask=m, other=0.0).to(tl.float32)
    s = tl.load(s_ptr + c, mask=c < n_cols, other=0.0)
    tl.store(y_ptr + r[:, None] * pitch + c[None, :], (x * s[None, :]).to(y_ptr.dtype.element_ty), mask=m)
    tl.store(sums_ptr + tl.program_id(1) * n_rows + r, tl.sum(x, axis=1), mask=r < n_rows)


@triton.jit
def running_mean_of_rows(x_ptr, y_ptr, n_rows, n_cols, pitch, BLOCK: tl.constexpr):
    # y[r, :] = mean(x[0..r, :]) for a block of columns: a carried fp32 accumulator next to 16-bit loads and stores
    c = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = c < n_cols
    acc = tl.zeros((BLOCK,), dtype=tl.float32)
    for r in range(0, n_rows):
        acc += tl.load(x_ptr + r * pitch + c, mask=m, other=0.0).to(tl.float32)
        tl.store(y_ptr + r * pitch + c, (acc / (r + 1)).to(y_ptr.dtype.element_ty), mask=m)


@triton.jit
def widen_and_count(x_ptr, y_ptr, k_ptr, n, BLOCK: tl.constexpr):
    # fp32 copy of a 16-bit block, and an i32 block counting the elements up to each position that are positive
    # (4-byte stores next to 16-bit loads)
    o = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = o < n
    x = tl.load(x_ptr + o, mask=m, other=-1.0).to(tl.float32)
    tl.store(y_ptr + o, x * 2.0, mask=m)
    tl.store(k_ptr + o, tl.where(x > 0, o, -o), mask=m)


@triton.jit
def quantize_rows_int8(x_ptr, q_ptr, s_ptr, n_cols, pitch, BLOCK: tl.constexpr):
    # row-wise symmetric int8 quantisation: q = round-half-away(x / (max|x| / 127)), one row per program
    row = tl.program_id(0)
    c = tl.arange(0, BLOCK)
    m = c < n_cols
    x = tl.load(x_ptr + row * pitch + c, mask=m, other=0.0).to(tl.float32)
    scale = tl.max(tl.abs(x), axis=0) / 127.0
    q = x / scale
    q = tl.where(q >= 0, q + 0.5, q - 0.5).to(tl.int8)
    tl.store(q_ptr + row * pitch + c, q, mask=m)
    tl.store(s_ptr + row, scale)


@triton.jit
def dequantize_rows_int8(q_ptr, s_ptr, y_ptr, n_cols, pitch, BLOCK: tl.constexpr):
    row = tl.program_id(0)
    c = tl.arange(0, BLOCK)
    m = c < n_cols
    q = tl.load(q_ptr + row * pitch + c, mask=m, other=0)
    tl.store(y_ptr + row * pitch + c, (q.to(tl.float32) * tl.load(s_ptr + row)).to(y_ptr.dtype.element_ty), mask=m)


@triton.jit
def scale_rows_on_a_2d_grid(x_ptr, w_ptr, y_ptr, n_rows, n_cols, BLOCK: tl.constexpr):
    # y[b, r, :] = x[b, r, :] * w + (b - r): one row per program, rows on program_id(0), batches on program_id(1); w is the
    # same block for every program
    r = tl.program_id(0)
    b = tl.program_id(1)
    c = tl.arange(0, BLOCK)
    m = c < n_cols
    w = tl.load(w_ptr + c, mask=m, other=0.0).to(tl.float32)
    x = tl.load(x_ptr + (b * n_rows + r) * n_cols + c, mask=m, other=0.0).to(tl.float32)
    tl.store(y_ptr + (b * n_rows + r) * n_cols + c, (x * w + (b - r)).to(y_ptr.dtype.element_ty), mask=m)
