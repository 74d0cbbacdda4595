/* TEST INFRASTRUCTURE - NOT PART OF THE PRODUCT.
 *
 * CPU restatement of how the reference's CPU backend executes the five hot-path
 * kernels: the checker for the HIP kernels and the timed CPU baseline ("port").
 * Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load
 * this file's library; the product never does.
 *
 * What is restated (paths relative to the triton-shared tree):
 *   - backend/driver.py:116-133: one program at a time, serial loops over the
 *     grid, x outermost;
 *   - per masked tts.load: a malloc'd full tile, filled with `other` when one is
 *     given and the valid extent is smaller than the tile, then an element-wise
 *     copy of the leading dims[0] (x dims[1]) elements
 *     (lib/Conversion/StructuredToMemref/StructuredToMemref.cpp:192-224,794-853;
 *     copy = memrefCopy, backend/include/ExecutionEngine/CRunnerUtils.cpp:58-113);
 *   - valid extent dims = max(min(start + size, bound), start) - start in signed
 *     64-bit arithmetic (lib/Analysis/MaskAnalysis.cpp:568-585), conjunctions as a
 *     per-dimension min (MaskAnalysis.cpp:269-286);
 *   - every arith/math op as its own loop over the full tile into a fresh
 *     temporary (lib/Conversion/TritonArithToLinalg/TritonArithToLinalg.cpp:104;
 *     backend/compiler.py:84-94 applies no fusion or optimisation passes);
 *   - tt.reduce as a strictly sequential fold in index order, in f32, starting
 *     from the identity (-inf for max, 0 for add)
 *     (include/triton-shared/Conversion/TritonArithToLinalg/ConversionPatterns.hpp:
 *     1227-1286,1395-1407);
 *   - tt.dot as linalg.matmul of the operands widened to f32 into a zero tile
 *     (i, j, k loop nest, k innermost), followed by an elementwise add of the
 *     accumulator operand (ConversionPatterns.hpp:1171-1196);
 *   - arith.truncf as round-to-nearest-even (ConversionPatterns.hpp:937-938),
 *     libm expf/sqrtf, no FMA contraction (compile with -ffp-contract=off);
 *   - masked tts.store as a copy of the leading dims elements
 *     (StructuredToMemref.cpp:1163-1196); scalar stores as base[offset] = v
 *     (lib/Conversion/UnstructuredToMemref/UnstructuredToMemrefPass.cpp:115-158).
 *
 * Parity status: vec_add is pinned bit-exactly by IEEE-754 addition; softmax,
 * layer norm and the two matmuls are pinned by closed forms to the tolerances the
 * tests state (the reference's bits for those depend on its build machine's libm
 * and cannot be reproduced here); w8a16 has no reference kernel or test at all and
 * is pinned by its closed form only ("parity unpinned" by the reference).
 *
 * Lanes of a tile beyond the valid extent hold whatever malloc returned when no
 * `other` is given; like the reference, the kernels never let such lanes reach
 * memory.  To keep this file free of reads of indeterminate values, tiles are
 * allocated with calloc where the reference uses malloc.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef int64_t idx;

static idx min_i(idx a, idx b) { return a < b ? a : b; }
static idx max_i(idx a, idx b) { return a > b ? a : b; }

/* MaskAnalysis.cpp:568-585 */
static idx valid_extent(idx start, idx size, idx bound) {
  idx end = min_i(start + size, bound);
  end = max_i(end, start);
  return end - start;
}

/* ---- 16-bit float formats (exact widening, round-to-nearest-even narrowing) ---- */
static float f16_to_f32(uint16_t h) {
  uint32_t s = (uint32_t)(h >> 15) << 31, e = (h >> 10) & 31, m = h & 1023, u;
  if (e == 0) {
    if (m == 0) u = s;
    else {
      int sh = 0;
      while (!(m & 1024)) { m <<= 1; sh++; }
      u = s | ((uint32_t)(113 - sh) << 23) | ((m & 1023) << 13);
    }
  } else if (e == 31) u = s | 0x7f800000u | (m << 13);
  else u = s | ((e + 112) << 23) | (m << 13);
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static uint16_t f32_to_f16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  uint32_t s = (u >> 16) & 0x8000u, a = u & 0x7fffffffu;
  if (a > 0x7f800000u) return (uint16_t)(s | 0x7e00u);
  if (a >= 0x47800000u) return (uint16_t)(s | 0x7c00u);           /* >= 65536 (and inf) -> inf; 65520..65536 handled below */
  if (a < 0x33000001u) return (uint16_t)s;                          /* <= 2^-25 -> 0 (ties to even) */
  uint32_t e = a >> 23, m = (a & 0x7fffffu) | 0x800000u;
  if (e < 113) {                                                     /* subnormal half */
    uint32_t shift = 126 - e;                                        /* 14..24 */
    uint32_t r = m >> shift, rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (r & 1))) r++;
    return (uint16_t)(s | r);
  }
  uint32_t r = ((e - 112) << 10) | ((m >> 13) & 1023), rem = m & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (r & 1))) r++;            /* may carry into the exponent, up to inf */
  return (uint16_t)(s | r);
}
static float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static uint16_t f32_to_bf16(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1);
  return (uint16_t)(u >> 16);
}

/* exported so that tests can pin the conversions against numpy/torch */
float oracle_f16_to_f32(uint16_t h) { return f16_to_f32(h); }
uint16_t oracle_f32_to_f16(float f) { return f32_to_f16(f); }
uint16_t oracle_f32_to_bf16(float f) { return f32_to_bf16(f); }
int64_t oracle_valid_extent(int64_t start, int64_t size, int64_t bound) { return valid_extent(start, size, bound); }

/* memrefCopy of a leading 1-D / 2-D sub-block, element by element (CRunnerUtils.cpp:58-113) */
static void copy_1d(void *dst, const void *src, idx n, idx elem) {
  for (idx i = 0; i < n; i++) memcpy((char *)dst + i * elem, (const char *)src + i * elem, (size_t)elem);
}
static void copy_2d(void *dst, idx dst_pitch, const void *src, idx src_s0, idx src_s1, idx d0, idx d1, idx elem) {
  for (idx i = 0; i < d0; i++)
    for (idx j = 0; j < d1; j++)
      memcpy((char *)dst + (i * dst_pitch + j) * elem, (const char *)src + (i * src_s0 + j * src_s1) * elem, (size_t)elem);
}

/* ------------------------------------------------------------------ vec_add
 * z = x + y, BLOCK elements per program, tail masked (python/examples/test_vec_add.py:8-34). */
void ref_vec_add(const float *x, const float *y, float *z, int32_t n, int32_t BLOCK, int32_t grid_x) {
  for (int32_t pid = 0; pid < grid_x; pid++) {
    int32_t first = pid * BLOCK;                         /* arith.muli on i32 */
    idx d = valid_extent(first, BLOCK, n);
    float *tx = calloc((size_t)BLOCK, 4), *ty = calloc((size_t)BLOCK, 4), *tz = malloc((size_t)BLOCK * 4);
    copy_1d(tx, x + first, d, 4);
    copy_1d(ty, y + first, d, 4);
    for (idx i = 0; i < BLOCK; i++) tz[i] = tx[i] + ty[i]; /* linalg.generic addf over the full tile */
    copy_1d(z + first, tz, d, 4);
    free(tx); free(ty); free(tz);
  }
}

/* ------------------------------------------------------------- row softmax
 * python/examples/test_softmax.py:8-29; golden IR test/Conversion/StructuredToMemref/kernel-02-fused-softmax.mlir */
void ref_row_softmax(float *out, const float *in, int32_t in_pitch, int32_t out_pitch, int32_t n_cols, int32_t BLOCK,
                     int32_t grid_x) {
  for (int32_t pid = 0; pid < grid_x; pid++) {
    idx d = valid_extent(0, BLOCK, n_cols);
    float *row = malloc((size_t)BLOCK * 4);
    if (d < BLOCK)
      for (idx i = 0; i < BLOCK; i++) row[i] = -INFINITY; /* linalg.fill(other) guarded by scf.if */
    copy_1d(row, in + (idx)(pid * in_pitch), d, 4);
    float mx = -INFINITY;                                  /* linalg.reduce maxnumf, init -inf */
    for (idx i = 0; i < BLOCK; i++) mx = fmaxf(mx, row[i]);
    float *t0 = malloc((size_t)BLOCK * 4), *t1 = malloc((size_t)BLOCK * 4), *t2 = malloc((size_t)BLOCK * 4);
    for (idx i = 0; i < BLOCK; i++) t0[i] = mx;            /* linalg.fill (splat) */
    for (idx i = 0; i < BLOCK; i++) t1[i] = row[i] - t0[i];
    for (idx i = 0; i < BLOCK; i++) t2[i] = expf(t1[i]);
    float sum = 0.f;                                       /* linalg.reduce addf, init 0 */
    for (idx i = 0; i < BLOCK; i++) sum = sum + t2[i];
    for (idx i = 0; i < BLOCK; i++) t0[i] = sum;
    for (idx i = 0; i < BLOCK; i++) t1[i] = t2[i] / t0[i];
    copy_1d(out + (idx)(pid * out_pitch), t1, d, 4);
    free(row); free(t0); free(t1); free(t2);
  }
}

/* ---------------------------------------------------------- LayerNorm fwd
 * python/examples/test_layernorm.py:29-76; golden IR kernel-05-layer-norm-fwd.mlir.
 * is_bf16 selects the 16-bit format of X, Y, W, B. */
void ref_layer_norm_fwd(const uint16_t *X, uint16_t *Y, const uint16_t *W, const uint16_t *B, float *Mean, float *Rstd,
                        int32_t pitch, int32_t N, float eps, int32_t BLOCK, int32_t grid_x, int32_t is_bf16) {
  float (*up)(uint16_t) = is_bf16 ? bf16_to_f32 : f16_to_f32;
  uint16_t (*down)(float) = is_bf16 ? f32_to_bf16 : f32_to_f16;
  for (int32_t row = 0; row < grid_x; row++) {
    const uint16_t *x = X + (idx)(row * pitch);
    uint16_t *y = Y + (idx)(row * pitch);
    float *acc = calloc((size_t)BLOCK, 4), *tf = malloc((size_t)BLOCK * 4), *tg = malloc((size_t)BLOCK * 4);
    uint16_t *th = malloc((size_t)BLOCK * 2), *tw = malloc((size_t)BLOCK * 2), *tb = malloc((size_t)BLOCK * 2);
    uint8_t *tm = malloc((size_t)BLOCK);
    /* pass 1: lane-wise partial sums over the column blocks, then one sequential reduce */
    for (int32_t off = 0; off < N; off += BLOCK) {
      idx d = valid_extent(off, BLOCK, N);
      if (d < BLOCK) for (idx i = 0; i < BLOCK; i++) th[i] = 0;
      copy_1d(th, x + off, d, 2);
      for (idx i = 0; i < BLOCK; i++) tf[i] = up(th[i]);            /* arith.extf */
      for (idx i = 0; i < BLOCK; i++) acc[i] = acc[i] + tf[i];
    }
    float s = 0.f;
    for (idx i = 0; i < BLOCK; i++) s = s + acc[i];
    float n_f = (float)N;                                            /* arith.sitofp */
    float mean = s / n_f;
    /* pass 2 */
    for (idx i = 0; i < BLOCK; i++) acc[i] = 0.f;
    for (int32_t off = 0; off < N; off += BLOCK) {
      for (idx i = 0; i < BLOCK; i++) tm[i] = (int32_t)(off + (int32_t)i) < N; /* cmpi slt on the index tile */
      idx d = valid_extent(off, BLOCK, N);
      if (d < BLOCK) for (idx i = 0; i < BLOCK; i++) th[i] = 0;
      copy_1d(th, x + off, d, 2);
      for (idx i = 0; i < BLOCK; i++) tf[i] = up(th[i]);
      for (idx i = 0; i < BLOCK; i++) tg[i] = tf[i] - mean;
      for (idx i = 0; i < BLOCK; i++) tf[i] = tm[i] ? tg[i] : 0.f;   /* arith.select */
      for (idx i = 0; i < BLOCK; i++) tg[i] = tf[i] * tf[i];
      for (idx i = 0; i < BLOCK; i++) acc[i] = acc[i] + tg[i];
    }
    s = 0.f;
    for (idx i = 0; i < BLOCK; i++) s = s + acc[i];
    float var = s / n_f;
    float rstd = 1.0f / sqrtf(var + eps);
    Mean[row] = mean;                                                /* scalar stores */
    Rstd[row] = rstd;
    /* pass 3 */
    for (int32_t off = 0; off < N; off += BLOCK) {
      idx d = valid_extent(off, BLOCK, N);
      copy_1d(tw, W + off, d, 2);
      copy_1d(tb, B + off, d, 2);
      if (d < BLOCK) for (idx i = 0; i < BLOCK; i++) th[i] = 0;
      copy_1d(th, x + off, d, 2);
      for (idx i = 0; i < d; i++) tf[i] = up(th[i]);                 /* lanes >= d are never stored */
      for (idx i = 0; i < d; i++) tg[i] = tf[i] - mean;
      for (idx i = 0; i < d; i++) tf[i] = tg[i] * rstd;
      for (idx i = 0; i < d; i++) tg[i] = up(tw[i]);
      for (idx i = 0; i < d; i++) tf[i] = tf[i] * tg[i];
      for (idx i = 0; i < d; i++) tg[i] = up(tb[i]);
      for (idx i = 0; i < d; i++) tf[i] = tf[i] + tg[i];
      for (idx i = 0; i < d; i++) th[i] = down(tf[i]);               /* arith.truncf */
      copy_1d(y + off, th, d, 2);
    }
    free(acc); free(tf); free(tg); free(th); free(tw); free(tb); free(tm);
  }
}

/* --------------------------------------------------------- blocked matmul
 * python/examples/test_matmul.py:33-108 with M/N edge masks; golden IR
 * kernel-03-matrix-multiplication.mlir.  Runs programs [pid_begin, pid_end) of a
 * 1-D grid so that a bounded sample can be timed.  16-bit format per is_bf16. */
void ref_matmul_tiles(const uint16_t *a, const uint16_t *b, uint16_t *c, int32_t M, int32_t N, int32_t K, int32_t s_am,
                      int32_t s_ak, int32_t s_bk, int32_t s_bn, int32_t s_cm, int32_t s_cn, int32_t BM, int32_t BN,
                      int32_t BK, int32_t GROUP_M, int32_t pid_begin, int32_t pid_end, int32_t is_bf16) {
  float (*up)(uint16_t) = is_bf16 ? bf16_to_f32 : f16_to_f32;
  uint16_t (*down)(float) = is_bf16 ? f32_to_bf16 : f32_to_f16;
  for (int32_t pid = pid_begin; pid < pid_end; pid++) {
    /* scalar i32 chain of the kernel (arith.divsi truncates toward zero, as C does) */
    int32_t tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
    int32_t per_group = GROUP_M * tiles_n;
    int32_t g = pid / per_group, m0 = g * GROUP_M;
    int32_t rows_in_group = tiles_m - m0 < GROUP_M ? tiles_m - m0 : GROUP_M;
    int32_t tm = m0 + pid % rows_in_group, tn = (pid % per_group) / rows_in_group;
    idx r0 = (idx)(tm * BM), c0 = (idx)(tn * BN);
    idx dm = min_i(valid_extent(r0, BM, M), BM), dn = min_i(valid_extent(c0, BN, N), BN);
    float *acc = calloc((size_t)BM * BN, 4), *prod = malloc((size_t)BM * BN * 4);
    uint16_t *ta = malloc((size_t)BM * BK * 2), *tb = malloc((size_t)BK * BN * 2);
    idx a_off = r0 * s_am, b_off = c0 * s_bn;          /* loop-carried offsets (PtrAnalysis.cpp:1480-1602) */
    int32_t trips = (K + BK - 1) / BK;
    for (int32_t k = 0; k < trips; k++) {
      idx dk = min_i(valid_extent(0, BK, (idx)(K - k * BK)), BK);
      if (dm < BM || dk < BK) memset(ta, 0, (size_t)BM * BK * 2);   /* other = 0 */
      copy_2d(ta, BK, a + a_off, s_am, s_ak, dm, dk, 2);
      if (dk < BK || dn < BN) memset(tb, 0, (size_t)BK * BN * 2);
      copy_2d(tb, BN, b + b_off, s_bk, s_bn, dk, dn, 2);
      for (idx i = 0; i < (idx)BM * BN; i++) prod[i] = 0.f;          /* linalg.fill */
      for (idx i = 0; i < BM; i++)                                   /* linalg.matmul */
        for (idx j = 0; j < BN; j++)
          for (idx kk = 0; kk < BK; kk++) prod[i * BN + j] = prod[i * BN + j] + up(ta[i * BK + kk]) * up(tb[kk * BN + j]);
      for (idx i = 0; i < (idx)BM * BN; i++) acc[i] = prod[i] + acc[i]; /* linalg.generic addf with the C operand */
      a_off += (idx)BK * s_ak;
      b_off += (idx)BK * s_bk;
    }
    uint16_t *out = malloc((size_t)BM * BN * 2);
    for (idx i = 0; i < (idx)BM * BN; i++) out[i] = down(acc[i]);
    for (idx i = 0; i < dm; i++)
      for (idx j = 0; j < dn; j++) c[(r0 + i) * s_cm + (c0 + j) * s_cn] = out[i * BN + j];
    free(acc); free(prod); free(ta); free(tb); free(out);
  }
}

/* ------------------------------------------------- int8-weight matmul (W8A16)
 * No counterpart in the reference; same lowering rules applied to the kernel
 * triton-shared_amd/examples/kernels.py:w8a16_matmul.  2-D grid (x over M blocks,
 * y over N blocks), x outermost as in backend/driver.py:122-124; runs the
 * y-programs [y_begin, y_end) of every x. */
void ref_w8a16_matmul(const uint16_t *a, const int8_t *w, const uint16_t *s, uint16_t *c, int32_t M, int32_t N, int32_t K,
                      int32_t s_am, int32_t s_ak, int32_t s_wk, int32_t s_wn, int32_t s_cm, int32_t s_cn, int32_t BM,
                      int32_t BN, int32_t BK, int32_t grid_x, int32_t y_begin, int32_t y_end) {
  for (int32_t px = 0; px < grid_x; px++)
    for (int32_t py = y_begin; py < y_end; py++) {
      idx r0 = (idx)(px * BM), c0 = (idx)(py * BN);
      idx dm = min_i(valid_extent(r0, BM, M), BM), dn = valid_extent(c0, BN, N);
      uint16_t *scale = calloc((size_t)BN, 2);                       /* other = 0 */
      copy_1d(scale, s + c0, dn, 2);
      dn = min_i(dn, BN);
      float *acc = calloc((size_t)BM * BN, 4), *prod = malloc((size_t)BM * BN * 4);
      uint16_t *ta = malloc((size_t)BM * BK * 2), *wf = malloc((size_t)BK * BN * 2), *wd = malloc((size_t)BK * BN * 2);
      int8_t *tq = malloc((size_t)BK * BN);
      idx a_off = r0 * s_am, w_off = c0 * s_wn;
      int32_t trips = (K + BK - 1) / BK;
      for (int32_t k = 0; k < trips; k++) {
        idx dk = min_i(valid_extent(0, BK, (idx)(K - k * BK)), BK);
        if (dm < BM || dk < BK) memset(ta, 0, (size_t)BM * BK * 2);
        copy_2d(ta, BK, a + a_off, s_am, s_ak, dm, dk, 2);
        if (dk < BK || dn < BN) memset(tq, 0, (size_t)BK * BN);
        copy_2d(tq, BN, w + w_off, s_wk, s_wn, dk, dn, 1);
        for (idx i = 0; i < (idx)BK * BN; i++) wf[i] = f32_to_f16((float)tq[i]);            /* arith.sitofp i8 -> f16 */
        for (idx i = 0; i < BK; i++)                                                        /* arith.mulf on f16 */
          for (idx j = 0; j < BN; j++) wd[i * BN + j] = f32_to_f16(f16_to_f32(wf[i * BN + j]) * f16_to_f32(scale[j]));
        for (idx i = 0; i < (idx)BM * BN; i++) prod[i] = 0.f;
        for (idx i = 0; i < BM; i++)
          for (idx j = 0; j < BN; j++)
            for (idx kk = 0; kk < BK; kk++)
              prod[i * BN + j] = prod[i * BN + j] + f16_to_f32(ta[i * BK + kk]) * f16_to_f32(wd[kk * BN + j]);
        for (idx i = 0; i < (idx)BM * BN; i++) acc[i] = prod[i] + acc[i];
        a_off += (idx)BK * s_ak;
        w_off += (idx)BK * s_wk;
      }
      for (idx i = 0; i < dm; i++)
        for (idx j = 0; j < dn; j++) c[(r0 + i) * s_cm + (c0 + j) * s_cn] = f32_to_f16(acc[i * BN + j]);
      free(scale); free(acc); free(prod); free(ta); free(wf); free(wd); free(tq);
    }
}
