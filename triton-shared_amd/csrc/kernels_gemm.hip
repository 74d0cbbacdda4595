// MFMA kernel families for gfx950: 16-bit GEMM with fp32 accumulate, and the
// weight-only int8 GEMM at decode shapes (M <= 16).
//
// What they replace in the reference CPU path: per program and per K step, two
// malloc'd operand tiles filled with 0 and partially copied
// (StructuredToMemref.cpp:794-853), linalg.matmul on operands widened to f32 into
// a zero tile, an elementwise add into the loop-carried accumulator
// (ConversionPatterns.hpp:1171-1196), a truncf tile (RTNE) and a partial copy out
// (StructuredToMemref.cpp:1163-1196); the int8 variant adds a sitofp tile and a
// mulf tile per K step.  The launcher has proved that the grid of programs is a
// dense C = A*B, so these kernels choose their own tiling.
#include "kernels.h"

namespace tts {

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;

__device__ __forceinline__ uint16_t f32_to_bf16(float f) {  // round to nearest even
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1);
  return (uint16_t)(u >> 16);
}
__device__ __forceinline__ uint16_t f32_to_f16(float f) {
  _Float16 h = (_Float16)f;
  uint16_t r;
  __builtin_memcpy(&r, &h, 2);
  return r;
}

template <bool BF16>
__device__ __forceinline__ f32x16 mfma32(uint4 a, uint4 b, f32x16 c) {
  if (BF16) return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

// 8 consecutive 16-bit elements starting at p[0], zero beyond `valid`
__device__ __forceinline__ uint4 load8(const uint16_t *p, int valid, bool vec) {
  if (valid >= 8 && vec) return *reinterpret_cast<const uint4 *>(p);
  uint32_t w[4] = {0, 0, 0, 0};
  for (int i = 0; i < 8 && i < valid; i++) w[i >> 1] |= (uint32_t)p[i] << (16 * (i & 1));
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// ------------------------------------------------------------- 16-bit GEMM
// Workgroup: 256 threads = 2 x 2 wavefronts; each wavefront owns TM x TN MFMA
// tiles of 32 x 32.  A and B tiles are staged through LDS, both stored with K
// contiguous ([row][k] and [col][k], pitch BK + 8 elements so that 16-byte
// fragment reads of 32 consecutive rows hit distinct banks).  B is row-major
// [K][N] in memory; it is transposed on the way into LDS by packing the two
// K-neighbours of every column into one 32-bit word.
template <bool BF16, int TM, int TN, int BK>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(GemmParams p, int tiles_m, int tiles_n) {
  constexpr int BM = 2 * TM * 32, BN = 2 * TN * 32, PITCH = BK + 8;
  constexpr int CA = BM * BK / 8 / 256;          // 16-byte chunks of A per thread
  constexpr int UB = (BK / 2) * (BN / 8) / 256;  // 2x8 units of B per thread
  extern __shared__ __align__(16) uint16_t smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // workgroup -> output tile: consecutive ids share an XCD's L2 (ids are dealt
  // round-robin to the 8 XCDs), and within an XCD walk 8-tile-tall column groups
  int bid = blockIdx.x;
  const int nwg = tiles_m * tiles_n;
  if (nwg % 8 == 0) bid = (bid % 8) * (nwg / 8) + bid / 8;
  const int group = 8 * tiles_n;
  const int g0 = (bid / group) * 8;
  const int gh = min(tiles_m - g0, 8);
  const int tile_m = g0 + (bid % group) % gh, tile_n = (bid % group) / gh;
  const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;

  const uint16_t *__restrict__ A = (const uint16_t *)p.a;
  const uint16_t *__restrict__ B = (const uint16_t *)p.b;
  const bool a_vec = (p.lda % 8 == 0) && (((uintptr_t)A & 15) == 0);
  const bool b_vec = (p.ldb % 8 == 0) && (((uintptr_t)B & 15) == 0);
  const int K = (int)p.K;

  uint4 ra[CA], rb[UB][2];
  auto load_tiles = [&](int k0) {
#pragma unroll
    for (int j = 0; j < CA; j++) {
      int c = tid + 256 * j, row = c / (BK / 8), kc = c % (BK / 8);
      int64_t gr = m0 + row;
      int gk = k0 + kc * 8;
      ra[j] = gr < p.M ? load8(A + gr * p.lda + gk, K - gk, a_vec) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < UB; j++) {
      int u = tid + 256 * j, kp = u / (BN / 8), nc = u % (BN / 8);
      int gk = k0 + 2 * kp;
      int64_t gn = n0 + nc * 8;
      int valid = (int)min((int64_t)8, p.N - gn);
#pragma unroll
      for (int r = 0; r < 2; r++)
        rb[j][r] = (gk + r < K && valid > 0) ? load8(B + (int64_t)(gk + r) * p.ldb + gn, valid, b_vec) : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_tiles = [&](int buf) {
    uint16_t *As = smem + buf * (BM + BN) * PITCH, *Bs = As + BM * PITCH;
#pragma unroll
    for (int j = 0; j < CA; j++) {
      int c = tid + 256 * j, row = c / (BK / 8), kc = c % (BK / 8);
      *reinterpret_cast<uint4 *>(As + row * PITCH + kc * 8) = ra[j];
    }
#pragma unroll
    for (int j = 0; j < UB; j++) {
      int u = tid + 256 * j, kp = u / (BN / 8), nc = u % (BN / 8);
      uint32_t r0[4] = {rb[j][0].x, rb[j][0].y, rb[j][0].z, rb[j][0].w};
      uint32_t r1[4] = {rb[j][1].x, rb[j][1].y, rb[j][1].z, rb[j][1].w};
#pragma unroll
      for (int i = 0; i < 4; i++) {
        uint32_t lo = (r0[i] & 0xffffu) | (r1[i] << 16);          // column 2i:   k, k+1
        uint32_t hi = (r0[i] >> 16) | (r1[i] & 0xffff0000u);      // column 2i+1: k, k+1
        *reinterpret_cast<uint32_t *>(Bs + (nc * 8 + 2 * i) * PITCH + 2 * kp) = lo;
        *reinterpret_cast<uint32_t *>(Bs + (nc * 8 + 2 * i + 1) * PITCH + 2 * kp) = hi;
      }
    }
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  const int nk = (K + BK - 1) / BK;
  if (nk > 0) {
    load_tiles(0);
    store_tiles(0);
  }
  __syncthreads();
  for (int kt = 0; kt < nk; kt++) {
    const int cur = kt & 1;
    if (kt + 1 < nk) load_tiles((kt + 1) * BK);
    const uint16_t *As = smem + cur * (BM + BN) * PITCH, *Bs = As + BM * PITCH;
    const uint16_t *a_base = As + (wm * TM * 32 + (lane & 31)) * PITCH + 8 * (lane >> 5);
    const uint16_t *b_base = Bs + (wn * TN * 32 + (lane & 31)) * PITCH + 8 * (lane >> 5);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++) {
      uint4 af[TM], bf[TN];
#pragma unroll
      for (int i = 0; i < TM; i++) af[i] = *reinterpret_cast<const uint4 *>(a_base + i * 32 * PITCH + ks * 16);
#pragma unroll
      for (int j = 0; j < TN; j++) bf[j] = *reinterpret_cast<const uint4 *>(b_base + j * 32 * PITCH + ks * 16);
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = mfma32<BF16>(af[i], bf[j], acc[i][j]);
    }
    if (kt + 1 < nk) store_tiles(cur ^ 1);
    __syncthreads();
  }

  // epilogue: lane holds column (lane % 32), rows 8*(v/4) + 4*(lane/32) + v%4 of each 32x32 tile
  uint16_t *__restrict__ C = (uint16_t *)p.c;
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++) {
      int64_t col = n0 + wn * TN * 32 + j * 32 + (lane & 31);
#pragma unroll
      for (int v = 0; v < 16; v++) {
        int64_t row = m0 + wm * TM * 32 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        if (row < p.M && col < p.N) C[row * p.ldc + col] = BF16 ? f32_to_bf16(acc[i][j][v]) : f32_to_f16(acc[i][j][v]);
      }
    }
}

template <bool BF16, int TM, int TN, int BK>
hipError_t launch_gemm_cfg(const GemmParams &p, hipStream_t s) {
  constexpr int BM = 2 * TM * 32, BN = 2 * TN * 32;
  constexpr size_t lds = 2 * (size_t)(BM + BN) * (BK + 8) * 2;
  static bool configured = false;
  auto kern = gemm_mfma_kernel<BF16, TM, TN, BK>;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    configured = true;
  }
  int tiles_m = (int)((p.M + BM - 1) / BM), tiles_n = (int)((p.N + BN - 1) / BN);
  hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(256), lds, s, p, tiles_m, tiles_n);
  return hipGetLastError();
}


// ------------------------------------------- 16-bit GEMM, full-tile fast path
// For problems made of whole 256 x 256 x BK tiles with 16-byte aligned rows.
// Workgroup: 512 threads = 8 wavefronts (two per SIMD, so that one computes
// while the other waits on LDS or the barrier), wave grid 2 (M) x 4 (N), each
// wavefront 128 x 64 of C = 4 x 2 MFMA tiles.  Wavefronts 0-3 stage A (BK/8
// 16-byte chunks per thread); wavefronts 4-7 stage B: each thread loads a
// (BK/8) (k) x 8 (n) block as 16-byte rows, transposes it in registers and writes
// eight K-contiguous chunks, so that global loads are whole 128-byte row
// segments and LDS accesses are conflict-free.  DIST tiles are in flight in
// registers, so global/L2 latency is covered by DIST K steps of MFMA work.
// LDS: [2 buffers][256 A rows + 256 B columns][BK + 8] 16-bit elements.
constexpr int F_BM = 256, F_BN = 256;

template <bool BF16, int BK, int DIST, bool EARLY, int DBG>
__global__ __launch_bounds__(512) void gemm_fast_kernel(GemmParams p, int tiles_m, int tiles_n) {
  constexpr int PITCH = BK + 8, NL = BK / 8;  // NL: 16-byte loads per thread and tile
  constexpr int KS = BK / 16;
  extern __shared__ __align__(16) uint16_t smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 2, wn = wave & 3;

  int bid = blockIdx.x;
  const int nwg = tiles_m * tiles_n;
  if (nwg % 8 == 0) bid = (bid % 8) * (nwg / 8) + bid / 8;  // consecutive ids on one XCD
  const int group = 4 * tiles_n;                             // 4-tile-tall column groups
  const int g0 = (bid / group) * 4;
  const int gh = min(tiles_m - g0, 4);
  const int tile_m = g0 + (bid % group) % gh, tile_n = (bid % group) / gh;
  const int64_t m0 = (int64_t)tile_m * F_BM, n0 = (int64_t)tile_n * F_BN;

  const uint16_t *__restrict__ A = (const uint16_t *)p.a;
  const uint16_t *__restrict__ B = (const uint16_t *)p.b;
  const bool loads_a = wave < 4;
  const int lt = tid & 255;  // index among the 256 threads with the same role

  // A role: chunk c = lt + 256 j -> row c / NL, 16-byte chunk c % NL
  // B role: unit (kg = lt % 8, nc = lt / 8): rows NL kg .. NL kg + NL - 1, columns 8 nc .. 8 nc + 7
  const uint16_t *gsrc;
  int64_t gstep;  // elements between this thread's loads
  if (loads_a) {
    gsrc = A + (m0 + lt / NL) * p.lda + (lt % NL) * 8;
    gstep = (256 / NL) * p.lda;
  } else {
    gsrc = B + (int64_t)((lt & 7) * NL) * p.ldb + n0 + (lt >> 3) * 8;
    gstep = p.ldb;
  }
  auto gload = [&](int k0, uint4 (&r)[NL]) {
    const uint16_t *src = loads_a ? gsrc + k0 : gsrc + (int64_t)k0 * p.ldb;
#pragma unroll
    for (int j = 0; j < NL; j++) r[j] = *reinterpret_cast<const uint4 *>(src + j * gstep);
  };
  auto lstore = [&](int buf, uint4 (&r)[NL]) {
    uint16_t *As = smem + buf * (F_BM + F_BN) * PITCH, *Bs = As + F_BM * PITCH;
    if (loads_a) {
#pragma unroll
      for (int j = 0; j < NL; j++)
        *reinterpret_cast<uint4 *>(As + (lt / NL + (256 / NL) * j) * PITCH + (lt % NL) * 8) = r[j];
    } else {
      // r[t] = row k = NL kg + t, columns c = 0..7 (two per 32-bit word); the chunk written for
      // column c holds k = 0..NL-1 of that column
      uint32_t in[NL][4];
#pragma unroll
      for (int t = 0; t < NL; t++) { in[t][0] = r[t].x; in[t][1] = r[t].y; in[t][2] = r[t].z; in[t][3] = r[t].w; }
      uint16_t *dst = Bs + ((lt >> 3) * 8) * PITCH + (lt & 7) * NL;
#pragma unroll
      for (int c2 = 0; c2 < 4; c2++) {
        uint32_t even[NL / 2], odd[NL / 2];
#pragma unroll
        for (int tp = 0; tp < NL / 2; tp++) {
          uint32_t x = in[2 * tp][c2], y = in[2 * tp + 1][c2];
          even[tp] = __builtin_amdgcn_perm(y, x, 0x05040100u);  // [x.lo16, y.lo16]
          odd[tp] = __builtin_amdgcn_perm(y, x, 0x07060302u);   // [x.hi16, y.hi16]
        }
        if (NL == 8) {
          *reinterpret_cast<uint4 *>(dst + (2 * c2) * PITCH) = make_uint4(even[0], even[1], even[NL / 2 - 2], even[NL / 2 - 1]);
          *reinterpret_cast<uint4 *>(dst + (2 * c2 + 1) * PITCH) = make_uint4(odd[0], odd[1], odd[NL / 2 - 2], odd[NL / 2 - 1]);
        } else {
          *reinterpret_cast<uint2 *>(dst + (2 * c2) * PITCH) = make_uint2(even[0], even[1]);
          *reinterpret_cast<uint2 *>(dst + (2 * c2 + 1) * PITCH) = make_uint2(odd[0], odd[1]);
        }
      }
    }
  };

  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  const int nk = (int)(p.K / BK);
  uint4 r0[NL], r1[NL];
  // One K step.  Tile kt is in LDS buffer `cur`.  `rnew` is free and receives tile kt+DIST; `rsto`
  // holds tile kt+1, which goes to the other LDS buffer (free since the barrier that ended step kt-1).
  auto step = [&](int kt, int cur, uint4 (&rnew)[NL], uint4 (&rsto)[NL]) {
    if (!(DBG & 4) && kt + DIST < nk) gload((kt + DIST) * BK, rnew);
    if (EARLY && !(DBG & 4) && kt + 1 < nk) lstore(cur ^ 1, rsto);
    const uint16_t *As = smem + cur * (F_BM + F_BN) * PITCH, *Bs = As + F_BM * PITCH;
    const uint16_t *a_base = As + (wm * 128 + (lane & 31)) * PITCH + 8 * (lane >> 5);
    const uint16_t *b_base = Bs + (wn * 64 + (lane & 31)) * PITCH + 8 * (lane >> 5);
    uint4 af[2][4], bf[2][2];
#pragma unroll
    for (int i = 0; i < 4; i++) af[0][i] = *reinterpret_cast<const uint4 *>(a_base + i * 32 * PITCH);
#pragma unroll
    for (int j = 0; j < 2; j++) bf[0][j] = *reinterpret_cast<const uint4 *>(b_base + j * 32 * PITCH);
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const int c = ks & 1, n = c ^ 1;
      if (!(DBG & 2) && ks + 1 < KS) {
#pragma unroll
        for (int i = 0; i < 4; i++) af[n][i] = *reinterpret_cast<const uint4 *>(a_base + i * 32 * PITCH + (ks + 1) * 16);
#pragma unroll
        for (int j = 0; j < 2; j++) bf[n][j] = *reinterpret_cast<const uint4 *>(b_base + j * 32 * PITCH + (ks + 1) * 16);
      }
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
          if (DBG & 1) acc[i][j][0] += __uint_as_float(af[c][i].x ^ bf[c][j].x);
          else acc[i][j] = mfma32<BF16>(af[c][i], bf[c][j], acc[i][j]);
        }
    }
    // pin the software pipeline: the fragment reads of step ks+1 are issued before the MFMAs of step
    // ks, so that LDS latency is covered by eight MFMAs instead of being waited for
    __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
#pragma unroll
    for (int ks = 0; ks + 1 < KS; ks++) {
      __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
    if (!EARLY && !(DBG & 4) && kt + 1 < nk) lstore(cur ^ 1, rsto);
    __syncthreads();
  };
  gload(0, r0);
  if (DIST == 2 && nk > 1) gload(BK, r1);
  lstore(0, r0);
  __syncthreads();
  for (int kt = 0; kt < nk; kt += 2) {
    if (DIST == 2) {
      step(kt, 0, r0, r1);                        // tile kt was in r0, tile kt+1 is in r1
      if (kt + 1 < nk) step(kt + 1, 1, r1, r0);
    } else {
      step(kt, 0, r0, r0);
      if (kt + 1 < nk) step(kt + 1, 1, r0, r0);
    }
  }

  uint16_t *__restrict__ C = (uint16_t *)p.c;
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 2; j++) {
      int64_t col = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
      for (int v = 0; v < 16; v++) {
        int64_t row = m0 + wm * 128 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        C[row * p.ldc + col] = BF16 ? f32_to_bf16(acc[i][j][v]) : f32_to_f16(acc[i][j][v]);
      }
    }
}

template <bool BF16, int BK, int DIST, bool EARLY, int DBG = 0>
hipError_t launch_gemm_fast(const GemmParams &p, hipStream_t s) {
  constexpr size_t lds = 2 * (size_t)(F_BM + F_BN) * (BK + 8) * 2;
  static bool configured = false;
  auto kern = gemm_fast_kernel<BF16, BK, DIST, EARLY, DBG>;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    configured = true;
  }
  int tiles_m = (int)(p.M / F_BM), tiles_n = (int)(p.N / F_BN);
  hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(512), lds, s, p, tiles_m, tiles_n);
  return hipGetLastError();
}

bool gemm_fast_path_ok(const GemmParams &p) {
  return p.M % F_BM == 0 && p.N % F_BN == 0 && p.K % 64 == 0 && p.K >= 64 && p.lda % 8 == 0 && p.ldb % 8 == 0 &&
         ((uintptr_t)p.a & 15) == 0 && ((uintptr_t)p.b & 15) == 0;
}

// ------------------------------------------------------ int8-weight GEMM
// Workgroup: NW wavefronts share one 128-column slab of W and split its K range
// in interleaved steps of 32 rows.  In a step, lane (j = lane % 16, g = lane / 16)
// streams rows 8g..8g+7 of the step, 8 columns (8 bytes) each, so that a
// 16-lane group reads 128 contiguous bytes of a row.  Bytes are widened to fp16
// exactly (bit pattern 0x6400 | (b ^ 0x80) is 1152 + b), multiplied by the
// column's fp16 scale in fp16 as the Triton source does, and fed to eight
// 16x16x32 MFMAs, one per column of the lane's eight.
constexpr int W8_COLS = 128;       // slab width of the 8-byte-load kernel
constexpr int W8_COLS_WIDE = 256;  // and of the 16-byte-load kernel

__device__ __forceinline__ uint32_t pk_sub_1152_mul(uint32_t biased, uint32_t scale2) {
  f16x2 v = __builtin_bit_cast(f16x2, biased);
  f16x2 s = __builtin_bit_cast(f16x2, scale2);
  const f16x2 off = {(_Float16)1152.0f, (_Float16)1152.0f};
  v = v - off;  // exact: integers in [-128, 127]
  v = v * s;    // one fp16 rounding, as arith.mulf on f16
  return __builtin_bit_cast(uint32_t, v);
}

// FAST: K is a multiple of 32, N of 128, rows are 8/16-byte aligned: every load is unconditional,
// so that the compiler keeps all loads of a step (and of DEPTH steps) in flight.  Rows of A beyond
// M are read from row M-1: they only reach rows of the MFMA result that are never stored.
// CW: columns per lane (8: 8-byte weight loads, 128-column slabs; 16: 16-byte loads, 256-column
// slabs, FAST only).
template <int NW, int DEPTH, bool FAST, int CW>
__global__ __launch_bounds__(NW * 64) void gemm_w8a16_kernel(GemmW8A16Params p, int steps_per_slice) {
  static_assert(CW == 8 || (CW == 16 && FAST), "wide slabs exist on the unconditional path only");
  constexpr int W8_COLS = 16 * CW;
  constexpr int RW = NW > (CW == 8 ? 4 : 2) ? (CW == 8 ? 4 : 2) : NW;  // wavefronts combined per round
  using wvec = typename std::conditional<CW == 8, uint2, uint4>::type;
  __shared__ float red[RW][16][W8_COLS + 4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int j = lane & 15, g = lane >> 4;
  const int64_t n0 = (int64_t)blockIdx.x * W8_COLS;
  const int slice = blockIdx.y;
  const uint16_t *__restrict__ A = (const uint16_t *)p.a;
  const int8_t *__restrict__ W = p.w;
  const uint16_t *__restrict__ S = (const uint16_t *)p.scale;
  const int K = (int)p.K;
  const bool a_vec = (p.lda % 8 == 0) && (((uintptr_t)A & 15) == 0);
  const bool w_vec = (p.ldw % 8 == 0) && (((uintptr_t)W & 7) == 0);
  const int64_t ncol = n0 + CW * j;                      // first of this lane's CW columns
  const int ncols = (int)max((int64_t)0, min((int64_t)CW, p.N - ncol));

  uint32_t scale2[CW];
#pragma unroll
  for (int c = 0; c < CW; c++) {
    uint32_t s = c < ncols ? S[ncol + c] : 0;
    scale2[c] = s | (s << 16);
  }
  f32x4 acc[CW];
#pragma unroll
  for (int c = 0; c < CW; c++) acc[c] = (f32x4){0.f, 0.f, 0.f, 0.f};

  const int step_begin = slice * steps_per_slice;
  const int step_end = min(step_begin + steps_per_slice, (K + 31) / 32);

  const int8_t *w_lane = W + (int64_t)(8 * g) * p.ldw + ncol;
  const uint16_t *a_lane = A + (int64_t)min(j, (int)p.M - 1) * p.lda + 8 * g;
  auto load_w = [&](int step, wvec (&q)[8]) {
    if constexpr (FAST) {
      const int8_t *src = w_lane + (int64_t)step * 32 * p.ldw;
#pragma unroll
      for (int t = 0; t < 8; t++) q[t] = *reinterpret_cast<const wvec *>(src + (int64_t)t * p.ldw);
      return;
    } else {
#pragma unroll
    for (int t = 0; t < 8; t++) {
      int k = step * 32 + 8 * g + t;
      if (k < K && ncols == 8 && w_vec) {
        q[t] = *reinterpret_cast<const uint2 *>(W + (int64_t)k * p.ldw + ncol);
      } else {
        uint32_t lo = 0, hi = 0;
        if (k < K)
          for (int c = 0; c < ncols; c++) {
            uint32_t b = (uint8_t)W[(int64_t)k * p.ldw + ncol + c];
            if (c < 4) lo |= b << (8 * c);
            else hi |= b << (8 * (c - 4));
          }
        q[t] = make_uint2(lo, hi);
      }
    }
    }
  };
  auto load_a = [&](int step) {
    if (FAST) return *reinterpret_cast<const uint4 *>(a_lane + step * 32);
    int k = step * 32 + 8 * g;
    return j < p.M ? load8(A + (int64_t)j * p.lda + k, K - k, a_vec) : make_uint4(0, 0, 0, 0);
  };

  auto word = [](const wvec &v, int i) -> uint32_t {
    if constexpr (CW == 8) return i == 0 ? v.x : v.y;
    else return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w;
  };
  auto consume = [&](const wvec (&q)[8], const uint4 &af) {
#pragma unroll
    for (int c = 0; c < CW; c++) {
      uint32_t frag[4];
#pragma unroll
      for (int tp = 0; tp < 4; tp++) {
        uint32_t w0 = word(q[2 * tp], c / 4);
        uint32_t w1 = word(q[2 * tp + 1], c / 4);
        // bytes [w0.b, 0, w1.b, 0], then flip the sign bit and set the exponent: 0x6400 | (b ^ 0x80)
        uint32_t sel = 0x0c000c00u | (uint32_t)(c & 3) | ((uint32_t)(4 + (c & 3)) << 16);
        uint32_t pair = __builtin_amdgcn_perm(w1, w0, sel) ^ 0x64806480u;
        frag[tp] = pk_sub_1152_mul(pair, scale2[c]);
      }
      uint4 bfrag = make_uint4(frag[0], frag[1], frag[2], frag[3]);
      acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, af), __builtin_bit_cast(f16x8, bfrag), acc[c], 0, 0, 0);
    }
  };
  // DEPTH steps are in flight in DEPTH register sets (the loop is unrolled over them, so no
  // copies), giving a step's loads the time of DEPTH steps' arithmetic to arrive
  wvec q[DEPTH][8];
  uint4 a[DEPTH];
  int step = step_begin + wave;
#pragma unroll
  for (int d = 0; d < DEPTH; d++)
    if (step + d * NW < step_end) { load_w(step + d * NW, q[d]); a[d] = load_a(step + d * NW); }
  for (; step < step_end; step += DEPTH * NW) {
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
      if (step + d * NW < step_end) {
        consume(q[d], a[d]);
        if (step + (d + DEPTH) * NW < step_end) { load_w(step + (d + DEPTH) * NW, q[d]); a[d] = load_a(step + (d + DEPTH) * NW); }
      }
    }
  }

  // combine the wavefronts' partial tiles through LDS, RW wavefronts at a time;
  // lane holds rows 4g+v (v = 0..3) of column n0 + CW*j + c
  constexpr int ROUNDS = (NW + RW - 1) / RW;
  constexpr int PER_THREAD = (16 * W8_COLS + NW * 64 - 1) / (NW * 64);
  float total[PER_THREAD];
#pragma unroll
  for (int e = 0; e < PER_THREAD; e++) total[e] = 0.f;
  for (int r = 0; r < ROUNDS; r++) {
    if (r) __syncthreads();
    if (wave / RW == r) {
#pragma unroll
      for (int c = 0; c < CW; c++)
#pragma unroll
        for (int v = 0; v < 4; v++) red[wave % RW][4 * g + v][CW * j + c] = acc[c][v];
    }
    __syncthreads();
    const int live = min(RW, NW - RW * r);
#pragma unroll
    for (int e = 0; e < PER_THREAD; e++) {
      int idx = tid + e * NW * 64;
      if (idx < 16 * W8_COLS) {
        int m = idx / W8_COLS, n = idx % W8_COLS;
        for (int w = 0; w < live; w++) total[e] += red[w][m][n];
      }
    }
  }
  uint16_t *__restrict__ C = (uint16_t *)p.c;
#pragma unroll
  for (int e = 0; e < PER_THREAD; e++) {
    int idx = tid + e * NW * 64;
    if (idx >= 16 * W8_COLS) continue;
    int m = idx / W8_COLS;
    int64_t n = n0 + idx % W8_COLS;
    if (m >= p.M || n >= p.N) continue;
    if (p.split > 1) p.workspace[((int64_t)slice * 16 + m) * p.N + n] = total[e];
    else C[(int64_t)m * p.ldc + n] = f32_to_f16(total[e]);
  }
}

// Partial tiles cross between workgroups (and so between the XCDs' L2 caches) through agent-scope
// relaxed atomic accesses: the stores are written through to memory and the loads bypass stale
// lines, without the whole-cache write-back and invalidate that a release/acquire pair costs
// (measured: 8 us per launch at the decode shape against 3 us this way).
__device__ __forceinline__ void store_through(float4 *dst, float4 v) {
  unsigned long long *d = reinterpret_cast<unsigned long long *>(dst);
  ulonglong2 u = __builtin_bit_cast(ulonglong2, v);
  __hip_atomic_store(d, u.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(d + 1, u.y, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float4 load_through(float4 *src) {
  unsigned long long *d = reinterpret_cast<unsigned long long *>(src);
  ulonglong2 u;
  u.x = __hip_atomic_load(d, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  u.y = __hip_atomic_load(d + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return __builtin_bit_cast(float4, u);
}

// The decode shape's kernel: 256-column slabs, 16-byte weight loads (a lane holds 16 columns of
// 8 rows per step), one workgroup per (slab, K slice).  Requires K % 32 == 0, N % 256 == 0,
// 16-byte-aligned rows of W and A.
//
// Tail: the NW wavefronts' partial tiles are summed through LDS in one round (float4 per lane,
// conflict-free).  With split > 1 every workgroup writes its slice's tile through to its workspace
// slot, waits for the stores' acknowledgement, and bumps the slab's arrival counter; the workgroup
// that arrives last adds the slices in slice order (so the sum does not depend on the order of
// arrival), writes C, and resets the counter for the next launch.  No workgroup waits for another.
// The counters are zero between launches (whoever allocates them clears them once).  Launches
// that share a workspace must not overlap.
template <int NW, int DEPTH>
__global__ __launch_bounds__(NW * 64) void gemm_w8a16_wide_kernel(GemmW8A16Params p, int steps_per_slice) {
  extern __shared__ float4 w8_lds[];  // [NW][16][64]
  __shared__ int is_last;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int j = lane & 15, g = lane >> 4;
  const int slab = blockIdx.x, slice = blockIdx.y;
  const int64_t n0 = (int64_t)slab * W8_COLS_WIDE;
  const uint16_t *__restrict__ S = (const uint16_t *)p.scale;

  uint32_t scale2[16];
  {
    const uint4 *sp = reinterpret_cast<const uint4 *>(S + n0 + 16 * j);
    const bool s_vec = (((uintptr_t)S) & 15) == 0;
    uint16_t sv[16];
    if (s_vec) {
      uint4 lo = sp[0], hi = sp[1];
      uint32_t wds[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
      for (int c = 0; c < 16; c++) sv[c] = (uint16_t)(wds[c / 2] >> (16 * (c & 1)));
    } else {
#pragma unroll
      for (int c = 0; c < 16; c++) sv[c] = S[n0 + 16 * j + c];
    }
#pragma unroll
    for (int c = 0; c < 16; c++) scale2[c] = (uint32_t)sv[c] | ((uint32_t)sv[c] << 16);
  }
  f32x4 acc[16];
#pragma unroll
  for (int c = 0; c < 16; c++) acc[c] = (f32x4){0.f, 0.f, 0.f, 0.f};

  const int step_begin = slice * steps_per_slice;
  const int step_end = min(step_begin + steps_per_slice, (int)(p.K / 32));
  const int8_t *w_lane = p.w + (int64_t)(8 * g) * p.ldw + n0 + 16 * j;
  const uint16_t *a_lane = (const uint16_t *)p.a + (int64_t)min(j, (int)p.M - 1) * p.lda + 8 * g;

  auto load_w = [&](int step, uint4 (&q)[8]) {
    const int8_t *src = w_lane + (int64_t)step * 32 * p.ldw;
#pragma unroll
    for (int t = 0; t < 8; t++) q[t] = *reinterpret_cast<const uint4 *>(src + (int64_t)t * p.ldw);
  };
  auto load_a = [&](int step) { return *reinterpret_cast<const uint4 *>(a_lane + step * 32); };
  auto word = [](const uint4 &v, int i) -> uint32_t { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; };
  auto consume = [&](const uint4 (&q)[8], const uint4 &af) {
#pragma unroll
    for (int c = 0; c < 16; c++) {
      uint32_t frag[4];
#pragma unroll
      for (int tp = 0; tp < 4; tp++) {
        // bytes [w0.b, 0, w1.b, 0], then flip the sign bit and set the exponent: 0x6400 | (b ^ 0x80)
        uint32_t sel = 0x0c000c00u | (uint32_t)(c & 3) | ((uint32_t)(4 + (c & 3)) << 16);
        uint32_t pair = __builtin_amdgcn_perm(word(q[2 * tp + 1], c / 4), word(q[2 * tp], c / 4), sel) ^ 0x64806480u;
        frag[tp] = pk_sub_1152_mul(pair, scale2[c]);
      }
      uint4 bfrag = make_uint4(frag[0], frag[1], frag[2], frag[3]);
      acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, af), __builtin_bit_cast(f16x8, bfrag), acc[c], 0, 0, 0);
    }
  };
  uint4 q[DEPTH][8];
  uint4 a[DEPTH];
  int step = step_begin + wave;
#pragma unroll
  for (int d = 0; d < DEPTH; d++)
    if (step + d * NW < step_end) { load_w(step + d * NW, q[d]); a[d] = load_a(step + d * NW); }
  for (; step < step_end; step += DEPTH * NW) {
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
      if (step + d * NW < step_end) {
        consume(q[d], a[d]);
        if (step + (d + DEPTH) * NW < step_end) { load_w(step + (d + DEPTH) * NW, q[d]); a[d] = load_a(step + (d + DEPTH) * NW); }
      }
    }
  }

  // sum the wavefronts' tiles: entry (c, lane) is rows 4g..4g+3 of column n0 + 16j + c
#pragma unroll
  for (int c = 0; c < 16; c++) w8_lds[(wave * 16 + c) * 64 + lane] = __builtin_bit_cast(float4, acc[c]);
  __syncthreads();
  constexpr int PER = 1024 / (NW * 64);
  float4 tot[PER];
#pragma unroll
  for (int e = 0; e < PER; e++) {
    const int idx = tid + e * NW * 64;
    float4 t = w8_lds[idx];
#pragma unroll
    for (int w = 1; w < NW; w++) {
      float4 u = w8_lds[w * 1024 + idx];
      t.x += u.x; t.y += u.y; t.z += u.z; t.w += u.w;
    }
    tot[e] = t;
  }
  if (p.split > 1) {
    float4 *slots = reinterpret_cast<float4 *>(p.workspace) + (int64_t)slab * p.split * 1024;
#pragma unroll
    for (int e = 0; e < PER; e++) store_through(slots + slice * 1024 + tid + e * NW * 64, tot[e]);
    __builtin_amdgcn_s_waitcnt(0);  // the stores have been acknowledged: the tile is in memory
    __syncthreads();                // ... every wavefront's part of it
    if (tid == 0) {
      int *counter = p.counters + slab;
      int before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      is_last = before == p.split - 1;
      if (before == p.split - 1) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!is_last) return;
#pragma unroll
    for (int e = 0; e < PER; e++) {
      const int idx = tid + e * NW * 64;
      float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
      for (int sl = 0; sl < p.split; sl++) {
        float4 u = sl == slice ? tot[e] : load_through(slots + sl * 1024 + idx);
        if (sl == 0) t = u;
        else { t.x += u.x; t.y += u.y; t.z += u.z; t.w += u.w; }
      }
      tot[e] = t;
    }
  }
  // to row-major through LDS, then 16-byte stores of eight fp16 values
  __syncthreads();
  constexpr int PITCH = W8_COLS_WIDE + 4;
  float *tile = reinterpret_cast<float *>(w8_lds);
#pragma unroll
  for (int e = 0; e < PER; e++) {
    const int idx = tid + e * NW * 64;
    const int c = idx >> 6, jj = idx & 15, gg = (idx >> 4) & 3;
    float *dst = tile + (4 * gg) * PITCH + 16 * jj + c;
    dst[0] = tot[e].x; dst[PITCH] = tot[e].y; dst[2 * PITCH] = tot[e].z; dst[3 * PITCH] = tot[e].w;
  }
  __syncthreads();
  uint16_t *__restrict__ C = (uint16_t *)p.c;
  const bool c_vec = (p.ldc % 8 == 0) && (((uintptr_t)C & 15) == 0);
  for (int item = tid; item < 16 * (W8_COLS_WIDE / 8); item += NW * 64) {
    const int m = item / (W8_COLS_WIDE / 8), n8 = (item % (W8_COLS_WIDE / 8)) * 8;
    if (m >= p.M) continue;
    const float *src = tile + m * PITCH + n8;
    uint16_t h[8];
#pragma unroll
    for (int i = 0; i < 8; i++) h[i] = f32_to_f16(src[i]);
    uint16_t *dst = C + (int64_t)m * p.ldc + n0 + n8;
    if (c_vec) {
      *reinterpret_cast<uint4 *>(dst) = make_uint4(h[0] | (uint32_t)h[1] << 16, h[2] | (uint32_t)h[3] << 16,
                                                   h[4] | (uint32_t)h[5] << 16, h[6] | (uint32_t)h[7] << 16);
    } else {
#pragma unroll
      for (int i = 0; i < 8; i++) dst[i] = h[i];
    }
  }
}

__global__ __launch_bounds__(256) void gemm_w8a16_reduce_kernel(GemmW8A16Params p) {
  int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= p.M * p.N) return;
  int64_t m = idx / p.N, n = idx % p.N;
  float s = 0.f;
  for (int k = 0; k < p.split; k++) s += p.workspace[((int64_t)k * 16 + m) * p.N + n];
  ((uint16_t *)p.c)[m * p.ldc + n] = f32_to_f16(s);
}

constexpr int W8_WAVES = 16;

}  // namespace

hipError_t launch_gemm(const GemmParams &p, hipStream_t s, const char **name) {
  static const char *tile_env = getenv("TTS_GEMM_TILE");  // tuning aid: 128, 256 (general kernel) or unset
  if (!tile_env && gemm_fast_path_ok(p)) {
    // BK = 64, one tile in flight, LDS filled after the MFMAs: the fastest of the measured
    // combinations of BK in {32, 64}, DIST in {1, 2} and EARLY in {false, true} at 4096^3
    *name = "gemm_fast_kernel";
    return p.is_bf16 ? launch_gemm_fast<true, 64, 1, false>(p, s) : launch_gemm_fast<false, 64, 1, false>(p, s);
  }
  bool big = p.M >= 2048 && p.N >= 2048;
  if (tile_env) big = atoi(tile_env) >= 256;
  if (big) {
    *name = "gemm_mfma_kernel<256x256x32>";
    return p.is_bf16 ? launch_gemm_cfg<true, 4, 4, 32>(p, s) : launch_gemm_cfg<false, 4, 4, 32>(p, s);
  }
  *name = "gemm_mfma_kernel<128x128x64>";
  return p.is_bf16 ? launch_gemm_cfg<true, 2, 2, 64>(p, s) : launch_gemm_cfg<false, 2, 2, 64>(p, s);
}

namespace {
struct W8Config { int cw, nw, depth, split; };

// The shape decides the kernel: 256-column slabs with 16-byte weight loads when N and the
// weight pitch allow, split over K so that about one workgroup lands on each CU.
// TTS_W8=cw,nw,depth,split overrides the choice (tuning aid).
W8Config w8_config(const GemmW8A16Params &p) {
  const int64_t steps = (p.K + 31) / 32;
  W8Config c{8, 16, 2, 1};
  const bool fast = p.K % 32 == 0 && p.N % W8_COLS == 0 && p.lda % 8 == 0 && p.ldw % 8 == 0;
  if (fast && p.N % W8_COLS_WIDE == 0 && p.ldw % 16 == 0) c = W8Config{16, 8, 1, 1};
  static const char *env = getenv("TTS_W8");
  int want_split = 0;
  if (env) {
    int cw = 0, nw = 0, depth = 0;
    if (sscanf(env, "%d,%d,%d,%d", &cw, &nw, &depth, &want_split) >= 3 && (cw == 8 || (cw == 16 && c.cw == 16))) {
      c.cw = cw; c.nw = nw; c.depth = depth;
    }
  }
  const int64_t slabs = (p.N + 16 * c.cw - 1) / (16 * c.cw);
  if (want_split > 0) c.split = want_split;
  else if (slabs < 192) {
    // about one workgroup per CU; the wide kernel's LDS tile admits only one, so never more than 256 of those
    int64_t want = c.cw == 16 ? std::max<int64_t>(1, 256 / slabs) : (256 + slabs - 1) / slabs;
    int64_t most = std::max<int64_t>(1, steps / c.nw);        // keep every wavefront busy
    c.split = (int)std::max<int64_t>(1, std::min<int64_t>(std::min(want, most), 64));
  }
  return c;
}

template <int NW, int DEPTH, bool FAST>
void w8_launch(const GemmW8A16Params &p, int steps_per_slice, hipStream_t s) {
  dim3 grid((unsigned)((p.N + W8_COLS - 1) / W8_COLS), p.split);
  hipLaunchKernelGGL((gemm_w8a16_kernel<NW, DEPTH, FAST, 8>), grid, dim3(NW * 64), 0, s, p, steps_per_slice);
}

template <int NW, int DEPTH>
hipError_t w8_launch_wide(const GemmW8A16Params &p, int steps_per_slice, hipStream_t s) {
  constexpr size_t lds = (size_t)NW * 16 * 64 * sizeof(float4);
  static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_w8a16_wide_kernel<NW, DEPTH>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (attr != hipSuccess) return attr;
  dim3 grid((unsigned)(p.N / W8_COLS_WIDE), p.split);
  hipLaunchKernelGGL((gemm_w8a16_wide_kernel<NW, DEPTH>), grid, dim3(NW * 64), lds, s, p, steps_per_slice);
  return hipGetLastError();
}
}  // namespace

int gemm_w8a16_split(const GemmW8A16Params &p) { return w8_config(p).split; }

size_t gemm_w8a16_workspace_bytes(const GemmW8A16Params &p) {
  if (p.split <= 1) return 0;
  return (size_t)p.split * 16 * (size_t)((p.N + 255) / 256 * 256) * sizeof(float);  // per-slice partial tiles, 16 rows of fp32
}

size_t gemm_w8a16_counters(const GemmW8A16Params &p) { return p.split <= 1 ? 0 : (size_t)((p.N + 255) / 256); }

hipError_t launch_gemm_w8a16(const GemmW8A16Params &p, hipStream_t s, const char **name) {
  W8Config c = w8_config(p);
  const int steps = (int)((p.K + 31) / 32);
  const int sps = (steps + p.split - 1) / p.split;
  const bool fast = p.K % 32 == 0 && p.N % W8_COLS == 0 && p.lda % 8 == 0 && p.ldw % 8 == 0 &&
                    ((uintptr_t)p.a & 15) == 0 && ((uintptr_t)p.w & 7) == 0;
  const bool wide = fast && c.cw == 16 && ((uintptr_t)p.w & 15) == 0;
  if (wide) {
    *name = "gemm_w8a16_wide_kernel";
    // one step in flight per wavefront; two measured 1.2 us slower at the decode shape
    if (c.depth == 2) return w8_launch_wide<8, 2>(p, sps, s);
    return w8_launch_wide<8, 1>(p, sps, s);
  }
  *name = "gemm_w8a16_kernel";
  if (!fast) w8_launch<W8_WAVES, 2, false>(p, sps, s);
  else w8_launch<W8_WAVES, 2, true>(p, sps, s);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || p.split == 1) return e;
  int64_t outs = p.M * p.N;
  hipLaunchKernelGGL(gemm_w8a16_reduce_kernel, dim3((unsigned)((outs + 255) / 256)), dim3(256), 0, s, p);
  return hipGetLastError();
}

}  // namespace tts
