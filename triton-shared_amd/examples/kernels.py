"""The five Triton kernels of the hot path, written against the unchanged Triton
frontend (`@triton.jit`, `tl.*`).  They are ordinary user code: nothing in them
knows which driver is active.

Provenance of the algorithms (reference, read as text):
  * vector add      - python/examples/test_vec_add.py:8-34
  * row softmax     - python/examples/test_softmax.py:8-29
  * LayerNorm fwd   - python/examples/test_layernorm.py:29-76
  * blocked matmul  - python/examples/test_matmul.py:33-108, with edge masks on
                      M/N instead of the `% M` wraparound and a narrowing epilogue
  * W8A16 matmul    - no counterpart in the reference; weight-only int8 with
                      per-output-channel scales, dequantised inside the K loop
"""
import triton
import triton.language as tl


@triton.jit
def vec_add(x_ptr, y_ptr, z_ptr, n, BLOCK: tl.constexpr):
    first = tl.program_id(0) * BLOCK
    idx = first + tl.arange(0, BLOCK)
    live = idx < n
    a = tl.load(x_ptr + idx, mask=live)
    b = tl.load(y_ptr + idx, mask=live)
    tl.store(z_ptr + idx, a + b, mask=live)


@triton.jit
def row_softmax(out_ptr, in_ptr, in_pitch, out_pitch, n_cols, BLOCK: tl.constexpr):
    r = tl.program_id(0)
    cols = tl.arange(0, BLOCK)
    v = tl.load(in_ptr + r * in_pitch + cols, mask=cols < n_cols, other=-float("inf"))
    e = tl.exp(v - tl.max(v, axis=0))
    p = e / tl.sum(e, axis=0)
    tl.store(out_ptr + r * out_pitch + cols, p, mask=cols < n_cols)


@triton.jit
def layer_norm_fwd(X, Y, W, B, Mean, Rstd, pitch, N, eps, BLOCK: tl.constexpr):
    r = tl.program_id(0)
    X += r * pitch
    Y += r * pitch
    acc = tl.zeros([BLOCK], dtype=tl.float32)
    for base in range(0, N, BLOCK):
        c = base + tl.arange(0, BLOCK)
        acc += tl.load(X + c, mask=c < N, other=0.).to(tl.float32)
    mean = tl.sum(acc, axis=0) / N
    acc2 = tl.zeros([BLOCK], dtype=tl.float32)
    for base in range(0, N, BLOCK):
        c = base + tl.arange(0, BLOCK)
        d = tl.load(X + c, mask=c < N, other=0.).to(tl.float32)
        d = tl.where(c < N, d - mean, 0.)
        acc2 += d * d
    var = tl.sum(acc2, axis=0) / N
    rstd = 1 / tl.sqrt(var + eps)
    tl.store(Mean + r, mean)
    tl.store(Rstd + r, rstd)
    for base in range(0, N, BLOCK):
        c = base + tl.arange(0, BLOCK)
        ok = c < N
        w = tl.load(W + c, mask=ok)
        b = tl.load(B + c, mask=ok)
        d = tl.load(X + c, mask=ok, other=0.).to(tl.float32)
        y = (d - mean) * rstd * w + b
        tl.store(Y + c, y, mask=ok)


@triton.jit
def matmul_tiles(a_ptr, b_ptr, c_ptr, M, N, K,
                 s_am, s_ak, s_bk, s_bn, s_cm, s_cn,
                 BM: tl.constexpr, BN: tl.constexpr, BK: tl.constexpr, GROUP_M: tl.constexpr):
    pid = tl.program_id(0)
    tiles_m = tl.cdiv(M, BM)
    tiles_n = tl.cdiv(N, BN)
    per_group = GROUP_M * tiles_n
    g = pid // per_group
    m0 = g * GROUP_M
    rows_in_group = min(tiles_m - m0, GROUP_M)
    tm = m0 + (pid % rows_in_group)
    tn = (pid % per_group) // rows_in_group

    rm = tm * BM + tl.arange(0, BM)
    rn = tn * BN + tl.arange(0, BN)
    rk = tl.arange(0, BK)
    pa = a_ptr + (rm[:, None] * s_am + rk[None, :] * s_ak)
    pb = b_ptr + (rk[:, None] * s_bk + rn[None, :] * s_bn)

    acc = tl.zeros((BM, BN), dtype=tl.float32)
    for k in range(0, tl.cdiv(K, BK)):
        left = K - k * BK
        a = tl.load(pa, mask=(rm[:, None] < M) & (rk[None, :] < left), other=0.0)
        b = tl.load(pb, mask=(rk[:, None] < left) & (rn[None, :] < N), other=0.0)
        acc += tl.dot(a, b)
        pa += BK * s_ak
        pb += BK * s_bk
    out = acc.to(c_ptr.dtype.element_ty)
    pc = c_ptr + s_cm * rm[:, None] + s_cn * rn[None, :]
    tl.store(pc, out, mask=(rm[:, None] < M) & (rn[None, :] < N))


@triton.jit
def matmul_wrapped(a_ptr, b_ptr, c_ptr, M, N, K,
                   s_am, s_ak, s_bk, s_bn, s_cm, s_cn,
                   BM: tl.constexpr, BN: tl.constexpr, BK: tl.constexpr, GROUP_M: tl.constexpr, ACTIVATION: tl.constexpr = ""):
    """The stock tutorial form of the tiled matmul: rows of A and columns of B beyond the problem are read
    modulo M and N instead of being masked; only K and the output carry masks.  ACTIVATION="leaky_relu" fuses the
    tutorial's activation before the cast (python/examples/test_matmul.py:98-99 in the reference)."""
    pid = tl.program_id(0)
    tiles_m = tl.cdiv(M, BM)
    tiles_n = tl.cdiv(N, BN)
    per_group = GROUP_M * tiles_n
    g = pid // per_group
    m0 = g * GROUP_M
    rows_in_group = min(tiles_m - m0, GROUP_M)
    tm = m0 + (pid % rows_in_group)
    tn = (pid % per_group) // rows_in_group

    ra = (tm * BM + tl.arange(0, BM)) % M
    rb = (tn * BN + tl.arange(0, BN)) % N
    rk = tl.arange(0, BK)
    pa = a_ptr + (ra[:, None] * s_am + rk[None, :] * s_ak)
    pb = b_ptr + (rk[:, None] * s_bk + rb[None, :] * s_bn)

    acc = tl.zeros((BM, BN), dtype=tl.float32)
    for k in range(0, tl.cdiv(K, BK)):
        left = K - k * BK
        a = tl.load(pa, mask=rk[None, :] < left, other=0.0)
        b = tl.load(pb, mask=rk[:, None] < left, other=0.0)
        acc += tl.dot(a, b)
        pa += BK * s_ak
        pb += BK * s_bk
    if ACTIVATION == "leaky_relu":
        acc = tl.where(acc >= 0, acc, 0.01 * acc)
    out = acc.to(c_ptr.dtype.element_ty)
    rm = tm * BM + tl.arange(0, BM)
    rn = tn * BN + tl.arange(0, BN)
    pc = c_ptr + s_cm * rm[:, None] + s_cn * rn[None, :]
    tl.store(pc, out, mask=(rm[:, None] < M) & (rn[None, :] < N))


@triton.jit
def w8a16_matmul(a_ptr, w_ptr, s_ptr, c_ptr, M, N, K,
                 s_am, s_ak, s_wk, s_wn, s_cm, s_cn,
                 BM: tl.constexpr, BN: tl.constexpr, BK: tl.constexpr):
    tm = tl.program_id(0)
    tn = tl.program_id(1)
    rm = tm * BM + tl.arange(0, BM)
    rn = tn * BN + tl.arange(0, BN)
    rk = tl.arange(0, BK)
    pa = a_ptr + (rm[:, None] * s_am + rk[None, :] * s_ak)
    pw = w_ptr + (rk[:, None] * s_wk + rn[None, :] * s_wn)
    scale = tl.load(s_ptr + rn, mask=rn < N, other=0.0)

    acc = tl.zeros((BM, BN), dtype=tl.float32)
    for k in range(0, tl.cdiv(K, BK)):
        left = K - k * BK
        a = tl.load(pa, mask=(rm[:, None] < M) & (rk[None, :] < left), other=0.0)
        q = tl.load(pw, mask=(rk[:, None] < left) & (rn[None, :] < N), other=0)
        w = q.to(tl.float16) * scale[None, :]
        acc += tl.dot(a, w)
        pa += BK * s_ak
        pw += BK * s_wk
    pc = c_ptr + s_cm * rm[:, None] + s_cn * rn[None, :]
    tl.store(pc, acc.to(tl.float16), mask=(rm[:, None] < M) & (rn[None, :] < N))


# ---- fused elementwise maps (one-dimensional blocks; any number of inputs, constants and scalar arguments)
@triton.jit
def gelu_tanh_bias(x_ptr, b_ptr, y_ptr, n, BLOCK: tl.constexpr):
    """y = gelu(x + b), tanh approximation written with exp, on fp32."""
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = i < n
    x = tl.load(x_ptr + i, mask=m, other=0.0) + tl.load(b_ptr + i, mask=m, other=0.0)
    u = 0.7978845608028654 * (x + 0.044715 * x * x * x)
    t = 1.0 - 2.0 / (tl.exp(2.0 * u) + 1.0)
    tl.store(y_ptr + i, 0.5 * x * (1.0 + t), mask=m)


@triton.jit
def clamp_scale_where(x_ptr, y_ptr, out_ptr, n, lo, hi, alpha, BLOCK: tl.constexpr):
    """out = where(x > y, alpha * clamp(x, lo, hi), sqrt(|y|)), fp32 with scalar arguments."""
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = i < n
    x = tl.load(x_ptr + i, mask=m, other=0.0)
    y = tl.load(y_ptr + i, mask=m, other=0.0)
    c = tl.minimum(tl.maximum(x, lo), hi)
    tl.store(out_ptr + i, tl.where(x > y, alpha * c, tl.sqrt(tl.abs(y))), mask=m)


@triton.jit
def silu_mul_f16(g_ptr, u_ptr, out_ptr, n, BLOCK: tl.constexpr):
    """out = silu(g) * u on fp16 tensors, computed in fp32 (the SwiGLU gate)."""
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = i < n
    g = tl.load(g_ptr + i, mask=m, other=0.0).to(tl.float32)
    u = tl.load(u_ptr + i, mask=m, other=0.0).to(tl.float32)
    tl.store(out_ptr + i, (g / (1.0 + tl.exp(-g)) * u).to(tl.float16), mask=m)


# ---- generic family: gathers, reductions along an axis, scans
@triton.jit
def take_rows(src_ptr, rows_ptr, dst_ptr, n_rows, n_cols, pitch_src, pitch_dst, BR: tl.constexpr, BC: tl.constexpr):
    """dst[r, :] = src[rows[r], :]: a gather of whole rows through an index vector (torch.index_select along dim 0)."""
    r = tl.program_id(0) * BR + tl.arange(0, BR)
    c = tl.arange(0, BC)
    which = tl.load(rows_ptr + r, mask=r < n_rows, other=0)
    m = (r[:, None] < n_rows) & (c[None, :] < n_cols)
    tile = tl.load(src_ptr + which[:, None].to(tl.int64) * pitch_src + c[None, :], mask=m, other=0.0)
    tl.store(dst_ptr + r[:, None].to(tl.int64) * pitch_dst + c[None, :], tile, mask=m)


@triton.jit
def row_sums(x_ptr, out_ptr, n_rows, n_cols, pitch, BR: tl.constexpr, BC: tl.constexpr):
    """out[r] = sum of row r, BR rows per program."""
    r = tl.program_id(0) * BR + tl.arange(0, BR)
    c = tl.arange(0, BC)
    m = (r[:, None] < n_rows) & (c[None, :] < n_cols)
    x = tl.load(x_ptr + r[:, None].to(tl.int64) * pitch + c[None, :], mask=m, other=0.0)
    tl.store(out_ptr + r, tl.sum(x, axis=1), mask=r < n_rows)


@triton.jit
def block_cumsum(x_ptr, y_ptr, n, BLOCK: tl.constexpr):
    """Inclusive prefix sum inside each block of BLOCK elements."""
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = i < n
    tl.store(y_ptr + i, tl.cumsum(tl.load(x_ptr + i, mask=m, other=0.0), axis=0), mask=m)


@triton.jit
def matmul_leaky_relu(a_ptr, b_ptr, c_ptr, M, N, K, s_am, s_bk, s_cm, slope, BM: tl.constexpr, BN: tl.constexpr, BK: tl.constexpr):
    """C = leaky_relu(A @ B): a tiled matmul with an activation fused before the narrowing store.  Not the shape the
    hand-written MFMA kernels take: it runs on the generic family (operands staged in LDS, 32x32 MFMA blocks)."""
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
    acc = tl.where(acc >= 0, acc, slope * acc)
    tl.store(c_ptr + rm[:, None] * s_cm + rn[None, :], acc.to(c_ptr.dtype.element_ty), mask=(rm[:, None] < M) & (rn[None, :] < N))


@triton.jit
def expert_rows_matmul(a_ptr, b_ptr, c_ptr, rows_ptr, expert_ptr, n_rows, K, N, s_am, s_be, s_bk, s_cm,
                       BM: tl.constexpr, BN: tl.constexpr, BK: tl.constexpr):
    """C[i, :] = A[rows[i], :] @ B[expert of i's block of BM rows]: the product of a mixture-of-experts layer.  The
    expert id is read from memory (negative: nothing to do for this block), the rows of A come through loaded indices,
    and both blocks of pointers are carried along K.  Runs on the generic family."""
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
    tl.store(c_ptr + i[:, None] * s_cm + j[None, :], acc.to(c_ptr.dtype.element_ty), mask=ok[:, None] & (j[None, :] < N))


# ---- the machine's stream ceilings, measured through this backend: a 1:1 read/write stream and a read-only stream
@triton.jit
def copy_blocks(x_ptr, z_ptr, n, BLOCK: tl.constexpr):
    """z = x: one byte written for every byte read."""
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    m = i < n
    tl.store(z_ptr + i, tl.load(x_ptr + i, mask=m), mask=m)


@triton.jit
def block_sums(x_ptr, out_ptr, n, BLOCK: tl.constexpr):
    """out[p] = sum of block p of x: BLOCK elements read for one written."""
    i = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    tl.store(out_ptr + tl.program_id(0), tl.sum(tl.load(x_ptr + i, mask=i < n, other=0.0), axis=0))


@triton.jit
def batched_matmul(a_ptr, b_ptr, c_ptr, M, N, K, s_ab, s_am, s_bb, s_bk, s_cb, s_cm, BM: tl.constexpr, BN: tl.constexpr, BK: tl.constexpr):
    # C[b] = A[b] @ B[b]: tiles of one product on program_id(0), the product on program_id(1); a batch stride of 0 shares an operand
    pid = tl.program_id(0)
    bid = tl.program_id(1)
    nn = tl.cdiv(N, BN)
    pm = pid // nn
    pn = pid % nn
    rm = pm * BM + tl.arange(0, BM)
    rn = pn * BN + tl.arange(0, BN)
    rk = tl.arange(0, BK)
    pa = a_ptr + bid * s_ab + rm[:, None] * s_am + rk[None, :]
    pb = b_ptr + bid * s_bb + rk[:, None] * s_bk + rn[None, :]
    acc = tl.zeros((BM, BN), dtype=tl.float32)
    for k in range(0, tl.cdiv(K, BK)):
        a = tl.load(pa, mask=(rm[:, None] < M) & (rk[None, :] < K - k * BK), other=0.0)
        b = tl.load(pb, mask=(rk[:, None] < K - k * BK) & (rn[None, :] < N), other=0.0)
        acc += tl.dot(a, b)
        pa += BK
        pb += BK * s_bk
    tl.store(c_ptr + bid * s_cb + rm[:, None] * s_cm + rn[None, :], acc.to(c_ptr.dtype.element_ty), mask=(rm[:, None] < M) & (rn[None, :] < N))


@triton.jit
def rotary_embedding(x_ptr, cos_ptr, sin_ptr, out_ptr, stride_s, HALF: tl.constexpr):
    """Rotary position embedding on [seq, heads * 2 * HALF] fp16: one program per (position, head), blocks of HALF elements."""
    s = tl.program_id(0)
    h = tl.program_id(1)
    d = tl.arange(0, HALF)
    base = s * stride_s + h * 2 * HALF
    x1 = tl.load(x_ptr + base + d).to(tl.float32)
    x2 = tl.load(x_ptr + base + HALF + d).to(tl.float32)
    c = tl.load(cos_ptr + s * HALF + d)
    sn = tl.load(sin_ptr + s * HALF + d)
    tl.store(out_ptr + base + d, (x1 * c - x2 * sn).to(tl.float16))
    tl.store(out_ptr + base + HALF + d, (x2 * c + x1 * sn).to(tl.float16))


@triton.jit
def rms_norm_rows(x_ptr, w_ptr, y_ptr, pitch, n_cols, eps, BLOCK: tl.constexpr):
    """RMSNorm of rows, one row per program: y = x / sqrt(mean(x^2) + eps) * w; 16-bit or fp32 tensors, fp32 arithmetic."""
    row = tl.program_id(0)
    c = tl.arange(0, BLOCK)
    m = c < n_cols
    x = tl.load(x_ptr + row * pitch + c, mask=m, other=0.0).to(tl.float32)
    ms = tl.sum(x * x, axis=0) / n_cols
    w = tl.load(w_ptr + c, mask=m, other=0.0).to(tl.float32)
    tl.store(y_ptr + row * pitch + c, (x * tl.rsqrt(ms + eps) * w).to(y_ptr.dtype.element_ty), mask=m)


@triton.jit
def layer_norm_dx_rows(dx_ptr, dy_ptr, x_ptr, w_ptr, mean_ptr, rstd_ptr, pitch, n_cols, BLOCK: tl.constexpr):
    """The input gradient of LayerNorm, one row per program, from the forward's saved mean and rstd:
    dx = (w dy - (xhat mean(xhat w dy) + mean(w dy))) rstd with xhat = (x - mean) rstd."""
    row = tl.program_id(0)
    c = tl.arange(0, BLOCK)
    m = c < n_cols
    x = tl.load(x_ptr + row * pitch + c, mask=m, other=0.0).to(tl.float32)
    dy = tl.load(dy_ptr + row * pitch + c, mask=m, other=0.0).to(tl.float32)
    w = tl.load(w_ptr + c, mask=m, other=0.0).to(tl.float32)
    mean = tl.load(mean_ptr + row)
    rstd = tl.load(rstd_ptr + row)
    xhat = tl.where(m, (x - mean) * rstd, 0.0)
    wdy = tl.where(m, w * dy, 0.0)
    c1 = tl.sum(xhat * wdy, axis=0) / n_cols
    c2 = tl.sum(wdy, axis=0) / n_cols
    dx = (wdy - (xhat * c1 + c2)) * rstd
    tl.store(dx_ptr + row * pitch + c, dx.to(dx_ptr.dtype.element_ty), mask=m)
