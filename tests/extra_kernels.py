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
    # modulo addressing outside a matmul: lowered to a structured access with a period, refused at the plan stage
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
    # structured, but matches no hand-written kernel family (a reduction to one value per program)
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    v = tl.load(x_ptr + i, mask=i < n, other=0.0)
    tl.store(out_ptr + tl.program_id(0), tl.sum(v, axis=0))
