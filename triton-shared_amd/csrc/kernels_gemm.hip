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

#include <cstring>

namespace tts {

namespace {

using namespace tts_gemm_device;

struct IdentityEp {
  static constexpr int BM = 0, BN = 0;  // (no owner to look up: see the generated functor, tile_codegen.cpp)
  __device__ __forceinline__ float operator()(float x, int64_t, int64_t) const { return x; }
};

// the kernels' device code is in gemm_device.h (it is also compiled at run time, with a fused epilogue)
template <bool BF16, int TM, int TN, int BK>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(GemmParams p, int tiles_m, int tiles_n) {
  gemm_mfma_body<BF16, TM, TN, BK>(of_batch(p, 2), tiles_m, tiles_n, IdentityEp());
}

template <bool BF16, int TM, int TN, int BK>
hipError_t launch_gemm_cfg(const GemmParams &p, hipStream_t s) {
  constexpr int BM = 2 * TM * 32, BN = 2 * TN * 32;
  constexpr size_t lds = GemmStageLds<BM, BN, BK>::BYTES;
  static bool configured = false;
  auto kern = gemm_mfma_kernel<BF16, TM, TN, BK>;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    configured = true;
  }
  int tiles_m = (int)((p.M + BM - 1) / BM), tiles_n = (int)((p.N + BN - 1) / BN);
  hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n, std::max(1, p.batches)), dim3(256), lds, s, p, tiles_m, tiles_n);
  return hipGetLastError();
}


// PF: a fifth wavefront that touches B's lines ahead of the four that work (gemm_device.h); the accumulators then sit in
// the 256 registers two wavefronts of a SIMD can have each, which the 128 x 256 tile fits without spilling.
template <bool BF16, int TM, int TN, bool BT, bool AT, bool PF, bool SK>
__global__ __launch_bounds__(PF ? 320 : 256) void gemm_dma_kernel(GemmParams p, int tiles_m, int tiles_n) {
  // whole 256 x 256 tiles of row-major operands: the body on the 16 x 16 x 32 matrix instruction (gemm_device.h)
  if constexpr (TM == 4 && TN == 4 && !BT && !AT && !PF) gemm_dma16_body<BF16, IdentityEp, SK>(of_batch(p, 2), tiles_m, tiles_n, IdentityEp());
  else gemm_dma_body<BF16, TM, TN, IdentityEp, BT, AT, PF, SK>(of_batch(p, 2), tiles_m, tiles_n, IdentityEp());
}

// Adds the K slices' partial sums in slice order and narrows: four columns per thread (N is a multiple of 8).
template <bool BF16>
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(GemmParams batch) {
  const GemmParams p = of_batch(batch, 2);
  const int64_t quads = p.N / 4, idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= p.M * quads) return;
  const int64_t m = idx / quads, n = (idx % quads) * 4;
  const float4 *src = reinterpret_cast<const float4 *>(p.partial + m * p.N + n);
  float4 t = src[0];
  for (int sl = 1; sl < p.split; sl++) {
    const float4 u = src[(int64_t)sl * p.M * quads];
    t.x += u.x; t.y += u.y; t.z += u.z; t.w += u.w;
  }
  typedef float f32x4_t __attribute__((ext_vector_type(4)));
  typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
  typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));
  const f32x4_t v = {t.x, t.y, t.z, t.w};
  uint16_t *dst = (uint16_t *)p.c + m * p.ldc + n;
  const uint2 w = BF16 ? __builtin_bit_cast(uint2, __builtin_convertvector(v, bf16x4_t)) : __builtin_bit_cast(uint2, __builtin_convertvector(v, f16x4_t));
  reinterpret_cast<uint32_t *>(dst)[0] = w.x;  // (rows of C are 4-byte aligned: gemm_dma_ok)
  reinterpret_cast<uint32_t *>(dst)[1] = w.y;
}

template <bool BF16, int TM, int TN, bool BT, bool AT, bool PF = false>
hipError_t launch_gemm_dma_t(const GemmParams &p, hipStream_t s) {
  using T = DmaTile<TM, TN>;
  constexpr size_t lds = T::LDS_BYTES;
  if constexpr (!PF) {
    if (p.split > 1) {
      auto kern = gemm_dma_kernel<BF16, TM, TN, BT, AT, false, true>;
      static const hipError_t attr = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      if (attr != hipSuccess) return attr;
      int tiles_m = (int)((p.M + T::BM - 1) / T::BM), tiles_n = (int)((p.N + T::BN - 1) / T::BN);
      hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n * p.split, std::max(1, p.batches)), dim3(256), lds, s, p, tiles_m, tiles_n);
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) return e;
      hipLaunchKernelGGL(gemm_splitk_reduce_kernel<BF16>, dim3((unsigned)((p.M * (p.N / 4) + 255) / 256), std::max(1, p.batches)), dim3(256), 0, s, p);
      return hipGetLastError();
    }
  }
  // Row tiles with weight matrices of their own (p.b_block) stream B from HBM: they get the prefetching wavefront.
  if constexpr (!PF && TM == 2 && TN == 4 && !BT && !AT) {
    static const char *pf = getenv("TTS_GEMM_PREFETCH");  // tuning aid: "0" = never, "2" = for every launch of this tile
    if (pf ? pf[0] == '2' || (pf[0] != '0' && p.b_block) : p.b_block != nullptr) return launch_gemm_dma_t<BF16, TM, TN, BT, AT, true>(p, s);
  }
  auto kern = gemm_dma_kernel<BF16, TM, TN, BT, AT, PF, false>;
  static const hipError_t attr = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (attr != hipSuccess) return attr;
  int tiles_m = (int)((p.M + T::BM - 1) / T::BM), tiles_n = (int)((p.N + T::BN - 1) / T::BN);
  hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n, std::max(1, p.batches)), dim3(PF ? 320 : 256), lds, s, p, tiles_m, tiles_n);
  return hipGetLastError();
}

// one instantiation per layout of the operands in memory
template <bool BF16, int TM, int TN>
hipError_t launch_gemm_dma(const GemmParams &p, hipStream_t s) {
  if (p.a_trans) return p.b_trans ? launch_gemm_dma_t<BF16, TM, TN, true, true>(p, s) : launch_gemm_dma_t<BF16, TM, TN, false, true>(p, s);
  return p.b_trans ? launch_gemm_dma_t<BF16, TM, TN, true, false>(p, s) : launch_gemm_dma_t<BF16, TM, TN, false, false>(p, s);
}

// Whole K tiles of 32, N a multiple of 8 (whole 16-byte chunks of B rows), any M (a multiple of 8 when A is column-major);
// 16-byte aligned rows, and per-lane byte offsets that fit 32 bits.  Either operand may be column-major.  Tiles that
// stick out of C clamp their addresses and mask their stores.
bool gemm_dma_ok(const GemmParams &p, int64_t bm, int64_t bn) {
  if (p.a_trans && (p.M % 8 != 0 || p.a_rows || p.b_block)) return false;
  if ((p.a_rows || p.b_block) && bm != 128) return false;  // gathered rows: 128-row tiles (64-bit A addresses per lane)
  if (p.b_block && p.b_block_rows % bm != 0) return false;
  if (p.batches > 1 && (p.batch_a % 8 != 0 || p.batch_b % 8 != 0 || p.batch_c % 2 != 0)) return false;  // every product aligned like the first
  return p.M >= 1 && p.N >= 8 && p.N % 8 == 0 && p.K % F_BK == 0 && p.K >= F_BK && p.lda % 8 == 0 && p.ldb % 8 == 0 &&
         ((uintptr_t)p.a & 15) == 0 && ((uintptr_t)p.b & 15) == 0 && p.lda < (p.a_trans ? (1 << 25) : (1 << 22)) && p.ldb < (p.b_trans ? (1 << 22) : (1 << 25)) &&
         (!p.b_block || p.b_block_stride % 8 == 0) && p.ldc % 2 == 0 && ((uintptr_t)p.c & 3) == 0;  // C is written in 4-byte pairs
}
bool gemm_fast_path_ok(const GemmParams &p) { return !p.a_trans && !p.b_trans && gemm_dma_ok(p, F_BM, F_BN); }  // (the kernel compiled with an epilogue)

// ------------------------------------------------------------- fp32 GEMM
// tl.dot on fp32 blocks: the reference multiplies in fp32 (linalg.matmul on f32, ConversionPatterns.hpp:1128-1201; it
// ignores the dot's inputPrecision), so this kernel uses the fp32 matrix instruction (v_mfma_f32_32x32x2_f32), not a
// reduced-precision one.  Any shape and alignment, A and B row- or column-major.
// Workgroup: 128 x 128 of C, 2 x 2 wavefronts of 64 x 64 (2 x 2 MFMA tiles of 32 x 32, 64 accumulator registers), K in
// steps of 16.  Both operand tiles sit in LDS as [k][r] (r = row of A / column of B, pitch = tile + 4 floats): a lane's MFMA
// operand is element (k0 + lane / 32, r0 + lane % 32), so a wavefront reads two runs of 32 consecutive floats.
// Tiles go global -> registers -> LDS with the next tile's loads in flight during the current tile's arithmetic (two
// LDS buffers, one barrier per tile); 16-byte global loads along whichever dimension is contiguous in memory.
// T: MFMA tiles per wavefront and dimension: 2 = 128 x 128 per workgroup, 1 = 64 x 64 (for problems that give fewer than
// two of the large tiles per CU: 2048^3 ran at 57 TFLOP/s on 256 large tiles, one wavefront per SIMD).
constexpr int F32_BK = 16;

template <int T>
__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmParams batch, int tiles_m, int tiles_n) {
  const GemmParams p = of_batch(batch, 4);
  constexpr int BT = 64 * T;          // rows of A / columns of B per workgroup
  constexpr int PITCH = BT + 4;       // floats between k rows in LDS
  constexpr int CH = BT / 64;         // chunks of 4 floats per thread and operand tile (BT x 16 floats = 4 BT chunks)
  __shared__ __align__(16) float smem[2][2][F32_BK * PITCH];  // [buffer][A, B][k][r]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  int bid = blockIdx.x;
  const int nwg = tiles_m * tiles_n;
  if (nwg % 8 == 0) bid = (bid % 8) * (nwg / 8) + bid / 8;  // consecutive ids on one XCD
  const int group = 8 * tiles_n;
  const int g0 = (bid / group) * 8;
  const int gh = min(tiles_m - g0, 8);
  const int tile_m = g0 + (bid % group) % gh, tile_n = (bid % group) / gh;
  const int64_t m0 = (int64_t)tile_m * BT, n0 = (int64_t)tile_n * BT;
  const float *__restrict__ A = (const float *)p.a;
  const float *__restrict__ B = (const float *)p.b;
  const int64_t K = p.K;
  const bool a_vec = p.lda % 4 == 0 && ((uintptr_t)A & 15) == 0, b_vec = p.ldb % 4 == 0 && ((uintptr_t)B & 15) == 0;

  // An operand tile is BT r x 16 k = 4 BT chunks of 4 floats, CH per thread.  k contiguous in memory (A row-major, B
  // column-major): chunk c = (r = c / 4, k = 4 (c % 4)); r contiguous (A column-major, B row-major): (k = c / (BT / 4), r = 4 (c % (BT / 4))).
  auto load_tile = [&](float4 (&reg)[CH], const float *P, bool r_contig, int64_t ld, int64_t r_base, int64_t rows, bool vec, int64_t k0) {
#pragma unroll
    for (int j = 0; j < CH; j++) {
      const int c = tid + 256 * j;
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (r_contig) {
        const int64_t k = k0 + c / (BT / 4), r = r_base + 4 * (c % (BT / 4));
        if (k < K) {
          const float *src = P + k * ld + r;
          if (vec && r + 4 <= rows) { const float4 q = *reinterpret_cast<const float4 *>(src); v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w; }
          else
            for (int i = 0; i < 4; i++) if (r + i < rows) v[i] = src[i];
        }
      } else {
        const int64_t r = r_base + c / 4, k = k0 + 4 * (c % 4);
        if (r < rows) {
          const float *src = P + r * ld + k;
          if (vec && k + 4 <= K) { const float4 q = *reinterpret_cast<const float4 *>(src); v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w; }
          else
            for (int i = 0; i < 4; i++) if (k + i < K) v[i] = src[i];
        }
      }
      reg[j] = make_float4(v[0], v[1], v[2], v[3]);
    }
  };
  auto store_tile = [&](const float4 (&reg)[CH], float *S, bool r_contig) {
#pragma unroll
    for (int j = 0; j < CH; j++) {
      const int c = tid + 256 * j;
      if (r_contig) {
        *reinterpret_cast<float4 *>(S + (c / (BT / 4)) * PITCH + 4 * (c % (BT / 4))) = reg[j];
      } else {  // four k of one r: one float into each of four k rows
        float *dst = S + (4 * (c % 4)) * PITCH + c / 4;
        dst[0] = reg[j].x; dst[PITCH] = reg[j].y; dst[2 * PITCH] = reg[j].z; dst[3 * PITCH] = reg[j].w;
      }
    }
  };
  const bool a_r = p.a_trans != 0, b_r = p.b_trans == 0;  // r contiguous in memory
  f32x16 acc[T][T];
#pragma unroll
  for (int i = 0; i < T; i++)
#pragma unroll
    for (int j = 0; j < T; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;
  float4 ra[CH], rb[CH];
  const int64_t nk = (K + F32_BK - 1) / F32_BK;
  if (nk > 0) {
    load_tile(ra, A, a_r, p.lda, m0, p.M, a_vec, 0);
    load_tile(rb, B, b_r, p.ldb, n0, p.N, b_vec, 0);
    store_tile(ra, smem[0][0], a_r);
    store_tile(rb, smem[0][1], b_r);
  }
  __syncthreads();
  for (int64_t kt = 0; kt < nk; kt++) {
    const int cur = (int)(kt & 1);
    if (kt + 1 < nk) {
      load_tile(ra, A, a_r, p.lda, m0, p.M, a_vec, (kt + 1) * F32_BK);
      load_tile(rb, B, b_r, p.ldb, n0, p.N, b_vec, (kt + 1) * F32_BK);
    }
    const float *As = smem[cur][0] + (lane >> 5) * PITCH + wm * (32 * T) + (lane & 31);
    const float *Bs = smem[cur][1] + (lane >> 5) * PITCH + wn * (32 * T) + (lane & 31);
#pragma unroll
    for (int ks = 0; ks < F32_BK; ks += 2) {
      float af[T], bf[T];
#pragma unroll
      for (int i = 0; i < T; i++) af[i] = As[ks * PITCH + 32 * i];
#pragma unroll
      for (int j = 0; j < T; j++) bf[j] = Bs[ks * PITCH + 32 * j];
#pragma unroll
      for (int i = 0; i < T; i++)
#pragma unroll
        for (int j = 0; j < T; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < nk) {
      store_tile(ra, smem[cur ^ 1][0], a_r);
      store_tile(rb, smem[cur ^ 1][1], b_r);
    }
    __syncthreads();
  }
  // lane holds column (lane % 32), rows 8 (v / 4) + 4 (lane / 32) + v % 4 of each 32 x 32 tile
  float *__restrict__ C = (float *)p.c;
#pragma unroll
  for (int i = 0; i < T; i++)
#pragma unroll
    for (int j = 0; j < T; j++) {
      const int64_t col = n0 + wn * (32 * T) + j * 32 + (lane & 31);
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int64_t row = m0 + wm * (32 * T) + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        if (row < p.M && col < p.N) C[row * p.ldc + col] = acc[i][j][v];
      }
    }
}

hipError_t launch_gemm_f32(const GemmParams &p, hipStream_t s) {
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    return n;
  }();
  const int batches = std::max(1, p.batches);
  const int64_t big = ((p.M + 127) / 128) * ((p.N + 127) / 128) * batches;
  if (big >= 2 * cus) {
    const int tiles_m = (int)((p.M + 127) / 128), tiles_n = (int)((p.N + 127) / 128);
    hipLaunchKernelGGL(gemm_f32_kernel<2>, dim3(tiles_m * tiles_n, batches), dim3(256), 0, s, p, tiles_m, tiles_n);
  } else {
    const int tiles_m = (int)((p.M + 63) / 64), tiles_n = (int)((p.N + 63) / 64);
    hipLaunchKernelGGL(gemm_f32_kernel<1>, dim3(tiles_m * tiles_n, batches), dim3(256), 0, s, p, tiles_m, tiles_n);
  }
  return hipGetLastError();
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
// MT: groups of 16 rows of A a launch takes (1 or 2).  The weights are widened once per step and multiplied with every
// group's rows; the tails below (the sum over the wavefronts, the hand-over between K slices, the stores) run once per group.
template <int NW, int DEPTH, int MT>
__global__ __launch_bounds__(NW * 64) void gemm_w8a16_wide_kernel(GemmW8A16Params p, int first_steps, int other_steps) {
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
  f32x4 acc[MT][16];
#pragma unroll
  for (int m = 0; m < MT; m++)
#pragma unroll
    for (int c = 0; c < 16; c++) acc[m][c] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // slice 0 takes first_steps steps of 32 rows, every other slice other_steps
  const int step_begin = slice == 0 ? 0 : first_steps + (slice - 1) * other_steps;
  const int step_end = min(step_begin + (slice == 0 ? first_steps : other_steps), (int)(p.K / 32));
  const int8_t *w_lane = p.w + (int64_t)(8 * g) * p.ldw + n0 + 16 * j;
  const uint16_t *a_lane[MT];
#pragma unroll
  for (int m = 0; m < MT; m++) a_lane[m] = (const uint16_t *)p.a + (int64_t)min(16 * m + j, (int)p.M - 1) * p.lda + 8 * g;

  auto load_w = [&](int step, uint4 (&q)[8]) {
    const int8_t *src = w_lane + (int64_t)step * 32 * p.ldw;
#pragma unroll
    for (int t = 0; t < 8; t++) {
      // the weights are read once per launch: nontemporal, so that they do not displace A, the scales and the partial
      // tiles from the caches (46.2 -> 43.1 us at the decode shape with the weights coming from HBM)
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
      const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + (int64_t)t * p.ldw));
      q[t] = make_uint4(v[0], v[1], v[2], v[3]);
    }
  };
  auto load_a = [&](int step, uint4 (&af)[MT]) {
#pragma unroll
    for (int m = 0; m < MT; m++) af[m] = *reinterpret_cast<const uint4 *>(a_lane[m] + step * 32);
  };
  auto word = [](const uint4 &v, int i) -> uint32_t { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; };
  auto consume = [&](const uint4 (&q)[8], const uint4 (&af)[MT]) {
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
#pragma unroll
      for (int m = 0; m < MT; m++)
        acc[m][c] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, af[m]), __builtin_bit_cast(f16x8, bfrag), acc[m][c], 0, 0, 0);
    }
  };
  uint4 q[DEPTH][8];
  uint4 a[DEPTH][MT];
  int step = step_begin + wave;
#pragma unroll
  for (int d = 0; d < DEPTH; d++)
    if (step + d * NW < step_end) { load_w(step + d * NW, q[d]); load_a(step + d * NW, a[d]); }
  for (; step < step_end; step += DEPTH * NW) {
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
      if (step + d * NW < step_end) {
        consume(q[d], a[d]);
        if (step + (d + DEPTH) * NW < step_end) { load_w(step + (d + DEPTH) * NW, q[d]); load_a(step + (d + DEPTH) * NW, a[d]); }
      }
    }
  }

  // sum the wavefronts' tiles: entry (c, lane) is rows 4g..4g+3 (of the group) of column n0 + 16j + c
  constexpr int PER = 1024 / (NW * 64);
  float4 tot[MT][PER];
#pragma unroll
  for (int m = 0; m < MT; m++) {
    if (m) __syncthreads();  // the previous group's tiles have been read
#pragma unroll
    for (int c = 0; c < 16; c++) w8_lds[(wave * 16 + c) * 64 + lane] = __builtin_bit_cast(float4, acc[m][c]);
    __syncthreads();
#pragma unroll
    for (int e = 0; e < PER; e++) {
      const int idx = tid + e * NW * 64;
      float4 t = w8_lds[idx];
#pragma unroll
      for (int w = 1; w < NW; w++) {
        float4 u = w8_lds[w * 1024 + idx];
        t.x += u.x; t.y += u.y; t.z += u.z; t.w += u.w;
      }
      tot[m][e] = t;
    }
  }
  if (p.split > 1) {
    // a slab's slots: [slice][group][1024 float4]
    float4 *slots = reinterpret_cast<float4 *>(p.workspace) + (int64_t)slab * p.split * MT * 1024;
    int *counter = p.counters + slab;
    // tot = the slices' tiles added in slice order, whoever adds them (so the sum does not depend on who arrived when);
    // `self` is this workgroup's slice, whose tile is tot.  Up to four slices, every load is issued before the first add
    // (one round trip to memory instead of one per slice).
    auto add_slices = [&](int self) {
      constexpr int EAGER = 4;
      if (p.split <= EAGER) {
        float4 u[EAGER][MT][PER];
#pragma unroll
        for (int sl = 0; sl < EAGER; sl++)
          if (sl < p.split && sl != self) {
#pragma unroll
            for (int m = 0; m < MT; m++)
#pragma unroll
              for (int e = 0; e < PER; e++) u[sl][m][e] = load_through(slots + (sl * MT + m) * 1024 + tid + e * NW * 64);
          }
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
          for (int e = 0; e < PER; e++) {
            float4 t = self == 0 ? tot[m][e] : u[0][m][e];
#pragma unroll
            for (int sl = 1; sl < EAGER; sl++)
              if (sl < p.split) {
                const float4 v = sl == self ? tot[m][e] : u[sl][m][e];
                t.x += v.x; t.y += v.y; t.z += v.z; t.w += v.w;
              }
            tot[m][e] = t;
          }
        return;
      }
#pragma unroll
      for (int m = 0; m < MT; m++)
#pragma unroll
        for (int e = 0; e < PER; e++) {
          const int idx = tid + e * NW * 64;
          float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
          for (int sl = 0; sl < p.split; sl++) {
            float4 u = sl == self ? tot[m][e] : load_through(slots + (sl * MT + m) * 1024 + idx);
            if (sl == 0) t = u;
            else { t.x += u.x; t.y += u.y; t.z += u.z; t.w += u.w; }
          }
          tot[m][e] = t;
        }
    };
    bool others_done = false;
    if (slice == 0) {
      // Slice 0 is given slightly more of K than the others, so it usually ends last: if every other slice has arrived
      // already, nobody needs this slice's tile in memory, and the write, its acknowledgement and the counter update
      // drop out of the kernel's tail.  (If not, slice 0 goes the way of the others below.)
      if (tid == 0) is_last = __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == p.split - 1;
      __syncthreads();
      others_done = is_last;
      __syncthreads();  // is_last is written again below
    }
    if (others_done) {
      if (tid == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      add_slices(0);
    } else {
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
      for (int e = 0; e < PER; e++) store_through(slots + (slice * MT + m) * 1024 + tid + e * NW * 64, tot[m][e]);
    __builtin_amdgcn_s_waitcnt(0);  // the stores have been acknowledged: the tile is in memory
    __syncthreads();                // ... every wavefront's part of it
    if (tid == 0) {
      int before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      is_last = before == p.split - 1;
      if (before == p.split - 1) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!is_last) return;
    add_slices(slice);
    }
  }
  // to row-major through LDS, then 16-byte stores of eight fp16 values
  constexpr int PITCH = W8_COLS_WIDE + 4;
  float *tile = reinterpret_cast<float *>(w8_lds);
  uint16_t *__restrict__ C = (uint16_t *)p.c;
  const bool c_vec = (p.ldc % 8 == 0) && (((uintptr_t)C & 15) == 0);
#pragma unroll
  for (int grp = 0; grp < MT; grp++) {
    __syncthreads();
#pragma unroll
    for (int e = 0; e < PER; e++) {
      const int idx = tid + e * NW * 64;
      const int c = idx >> 6, jj = idx & 15, gg = (idx >> 4) & 3;
      float *dst = tile + (4 * gg) * PITCH + 16 * jj + c;
      dst[0] = tot[grp][e].x; dst[PITCH] = tot[grp][e].y; dst[2 * PITCH] = tot[grp][e].z; dst[3 * PITCH] = tot[grp][e].w;
    }
    __syncthreads();
    for (int item = tid; item < 16 * (W8_COLS_WIDE / 8); item += NW * 64) {
      const int m = item / (W8_COLS_WIDE / 8), n8 = (item % (W8_COLS_WIDE / 8)) * 8;
      if (16 * grp + m >= p.M) continue;
      const float *src = tile + m * PITCH + n8;
      uint16_t h[8];
#pragma unroll
      for (int i = 0; i < 8; i++) h[i] = f32_to_f16(src[i]);
      uint16_t *dst = C + (int64_t)(16 * grp + m) * p.ldc + n0 + n8;
      if (c_vec) {
        *reinterpret_cast<uint4 *>(dst) = make_uint4(h[0] | (uint32_t)h[1] << 16, h[2] | (uint32_t)h[3] << 16,
                                                     h[4] | (uint32_t)h[5] << 16, h[6] | (uint32_t)h[7] << 16);
      } else {
#pragma unroll
        for (int i = 0; i < 8; i++) dst[i] = h[i];
      }
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

namespace {
// Which direct-to-LDS tile a product runs on (null: none applies), and in how many K slices.
struct DmaCand { const char *tag; int64_t bm, bn; double eff; };
const DmaCand DMA_CANDS[4] = {{"256x256", 256, 256, 1.0}, {"128x256", 128, 256, 0.77}, {"256x128", 256, 128, 0.73}, {"128x128", 128, 128, 0.59}};
struct DmaChoice { const DmaCand *tile = nullptr; int split = 1; };

DmaChoice choose_dma(const GemmParams &p, int max_split) {
  static const char *dma_env = getenv("TTS_GEMM_DMA");      // tuning aid: "256x256", "128x256", "256x128", "128x128" or unset
  static const char *split_env = getenv("TTS_GEMM_SPLIT");  // tuning aid: the number of K slices (1 = never split)
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    return n;
  }();
  // (tiles of all the batch's products: they share the launch)
  auto tiles = [&](const DmaCand &c) { return ((p.M + c.bm - 1) / c.bm) * ((p.N + c.bn - 1) / c.bn) * std::max(1, p.batches); };
  // Among the tiles that give every CU a workgroup (128 x 128: always), the one with the least padded work per unit
  // of the tile's measured efficiency at 4096^3 (105 / 136 / 144 / 179 us): a ragged edge counts against a tile that
  // overshoots it by more.
  DmaChoice best;
  double best_cost = 0;
  for (const DmaCand &c : DMA_CANDS) {
    if (!gemm_dma_ok(p, c.bm, c.bn)) continue;
    if (dma_env ? std::string(dma_env) != c.tag : (tiles(c) < cus && c.bm + c.bn != 256)) continue;
    const double cost = (double)(tiles(c) * c.bm * c.bn) / c.eff;
    if (!best.tile || cost < best_cost) { best.tile = &c; best_cost = cost; }
  }
  if (!best.tile || max_split < 2 || p.a_rows || p.b_block) return best;
  // Too few tiles for the chip (a skinny product: M = 128 ... 1024 against N, K in the thousands): every workgroup then walks
  // all of K alone, at the pace one workgroup streams its operands, and the launch takes as long as with a fraction of
  // its rows -- 4096 x 4096 weights took 50 us at M = 128, 256, 512 and 1024 alike.  K is cut into slices so that about
  // every CU has a workgroup; each slice leaves fp32 sums that a second kernel adds.  Modelled time: the K tiles a
  // workgroup walks at the tile's measured time per K tile (times the rounds of workgroups the chip needs), the launch's
  // fixed cost, and the partial sums' way through memory (measured: 512 x 8192 x 8192 in four slices of 256 x 256 tiles
  // 79 us for a model of 82; 512 x 4096 x 4096 in four of 128 x 256 34.5 for 34.5; 128 x 4096 x 4096 in eight of
  // 128 x 128 20.9 for 22.3).
  const int64_t nk = p.K / F_BK;
  auto model = [&](const DmaCand &c, int split) {
    // per K tile and workgroup with operands from HBM (the 128 x 256 tile: 0.42 us from cache)
    const double step = c.bm + c.bn == 512 ? 0.80e-6 : c.bm + c.bn == 256 ? 0.39e-6 : c.bm == 128 ? 0.60e-6 : 0.62e-6;
    const double wgs = (double)tiles(c) * split;
    double t = std::max(1.0, wgs / cus) * (double)((nk + split - 1) / split) * step + 8e-6;
    if (split > 1) t += 1.2 * split * (double)p.M * (double)p.N * std::max(1, p.batches) * 4 / 4e12 + 3e-6;
    return t;
  };
  DmaChoice pick = best;
  double pick_t = model(*best.tile, 1);
  if (!(split_env && atoi(split_env) == 1))
    for (const DmaCand &c : DMA_CANDS) {
      if (!gemm_dma_ok(p, c.bm, c.bn) || (dma_env && std::string(dma_env) != c.tag)) continue;
      const int64_t most = std::min<int64_t>(std::min<int64_t>(std::min<int64_t>(16, max_split), nk / 8), (2 * cus + tiles(c) - 1) / tiles(c));
      for (int64_t sp = split_env ? atoi(split_env) : 2; sp <= most; sp++) {
        if ((size_t)sp * p.M * p.N * std::max(1, p.batches) * 4 > ((size_t)256 << 20)) break;
        const double t = model(c, (int)sp);
        if (t < 0.9 * pick_t || (pick.split > 1 && t < pick_t)) { pick.tile = &c; pick.split = (int)sp; pick_t = t; }
        if (split_env) break;
      }
    }
  return pick;
}
}  // namespace

int gemm_split(const GemmParams &p) {
  static const char *tile_env = getenv("TTS_GEMM_TILE");
  if (p.is_f32 || tile_env) return 1;
  return choose_dma(p, 16).split;
}
size_t gemm_workspace_bytes(const GemmParams &p) { return p.split > 1 ? (size_t)p.split * p.M * p.N * std::max(1, p.batches) * sizeof(float) : 0; }

// p.split: the most K slices p.partial has room for (what gemm_split(p) said, or fewer; 1: none).
hipError_t launch_gemm(const GemmParams &p, hipStream_t s, const char **name) {
  if (p.is_f32) {
    if (p.a_rows || p.b_block) return hipErrorInvalidValue;  // (the matcher takes gathered rows on 16-bit operands only)
    *name = "gemm_f32_kernel";
    return launch_gemm_f32(p, s);
  }
  static const char *tile_env = getenv("TTS_GEMM_TILE");  // tuning aid: set = the any-shape kernel even for whole tiles
  if (!tile_env) {
    // Whole K tiles go to the direct-to-LDS kernels.
    // at most p.split slices: what gemm_split said, or fewer when the caller's workspace holds no more (1: none)
    const DmaChoice choice = choose_dma(p, std::max(1, p.split));
    GemmParams q = p;
    q.split = choice.split;
    const DmaCand *best = choice.tile;
#define TTS_DMA(TM, TN, TAG)                                                                                  \
  do {                                                                                                        \
    *name = TAG;                                                                                              \
    return q.is_bf16 ? launch_gemm_dma<true, TM, TN>(q, s) : launch_gemm_dma<false, TM, TN>(q, s);            \
  } while (0)
    if (best && best->bm == 256 && best->bn == 256) TTS_DMA(4, 4, q.split > 1 ? "gemm_dma_kernel, K slices" : "gemm_dma_kernel");
    if (best && best->bm == 128 && best->bn == 256) TTS_DMA(2, 4, q.split > 1 ? "gemm_dma_kernel<128x256>, K slices" : "gemm_dma_kernel<128x256>");
    if (best && best->bm == 256 && best->bn == 128) TTS_DMA(4, 2, q.split > 1 ? "gemm_dma_kernel<256x128>, K slices" : "gemm_dma_kernel<256x128>");
    if (best) TTS_DMA(2, 2, q.split > 1 ? "gemm_dma_kernel<128x128>, K slices" : "gemm_dma_kernel<128x128>");
#undef TTS_DMA
  }
  // anything else: 128 x 128 x 64 tiles, two workgroups per CU (a 256 x 256 x 32 form of the same kernel measured behind it
  // at every size tried: 4096^3: 202 against 197 us; 4096 x 2048 x 2048: 112 against 56 us)
  *name = "gemm_mfma_kernel<128x128x64>";
  return p.is_bf16 ? launch_gemm_cfg<true, 2, 2, 64>(p, s) : launch_gemm_cfg<false, 2, 2, 64>(p, s);
}

int gemm_epilogue_kernel_index(const GemmParams &p) { return gemm_fast_path_ok(p) ? 0 : 1; }

// Kernel 0: whole 256 x 256 x 32 tiles; 1: any shape in 128 x 128 x 64 tiles -- compiled from gemm_device.h plus the
// epilogue functor at the first launch that needs it.
hipError_t launch_gemm_epilogue(const GemmParams &p, const std::string &epilogue, RtcModule **modules, const GemmEpilogueArgs &ep,
                                hipStream_t s, const char **name, std::string *err) {
  static const char *names[2] = {"gemm_dma_kernel + epilogue (hipRTC)", "gemm_mfma_kernel<128x128x64> + epilogue (hipRTC)"};
  const int which = gemm_epilogue_kernel_index(p);
  const int64_t tile = which == 1 ? 128 : 256;
  *name = names[which];
  if (!modules[which]) {
    const std::string source = epilogue + "#define TTS_GEMM_RTC " + std::to_string(which) + "\n#define TTS_GEMM_BF16 " + std::to_string(p.is_bf16 ? 1 : 0) +
                               "\n" + gemm_device_source();
    hipError_t e = rtc_compile(source, "gemm_rtc", &modules[which], err);
    if (e != hipSuccess) {
      if (getenv("TTS_DUMP_RTC_SOURCE")) *err += "\n--- source ---\n" + source;
      return e;
    }
  }
  struct {
    GemmParams p;
    int tiles_m, tiles_n;
    GemmEpilogueArgs ep;  // the functor: same layout as the generated struct TtsEp
  } a;
  a.p = p;
  a.tiles_m = (int)((p.M + tile - 1) / tile);
  a.tiles_n = (int)((p.N + tile - 1) / tile);
  a.ep = ep;
  return rtc_launch(modules[which], a.tiles_m * a.tiles_n, 1, 1, 256, &a, sizeof a, s);
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

template <int NW, int DEPTH, int MT = 1>
hipError_t w8_launch_wide(const GemmW8A16Params &p, int first_steps, int other_steps, hipStream_t s) {
  constexpr size_t lds = (size_t)NW * 16 * 64 * sizeof(float4);
  static const hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_w8a16_wide_kernel<NW, DEPTH, MT>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (attr != hipSuccess) return attr;
  dim3 grid((unsigned)(p.N / W8_COLS_WIDE), p.split);
  hipLaunchKernelGGL((gemm_w8a16_wide_kernel<NW, DEPTH, MT>), grid, dim3(NW * 64), lds, s, p, first_steps, other_steps);
  return hipGetLastError();
}
}  // namespace

int gemm_w8a16_split(const GemmW8A16Params &p) { return w8_config(p).split; }

size_t gemm_w8a16_workspace_bytes(const GemmW8A16Params &p) {
  if (p.split <= 1) return 0;
  // per-slice partial tiles: 16 rows of fp32, 32 when a launch takes two groups of rows
  return (size_t)p.split * (p.M > 16 ? 32 : 16) * (size_t)((p.N + 255) / 256 * 256) * sizeof(float);
}

size_t gemm_w8a16_counters(const GemmW8A16Params &p) { return p.split <= 1 ? 0 : (size_t)((p.N + 255) / 256); }

static hipError_t launch_gemm_w8a16_rows(const GemmW8A16Params &p, hipStream_t s, const char **name);

static bool w8_wide(const GemmW8A16Params &p);

// Many rows of A (a prefill-sized M): the decode kernels would read W once per 32 rows.  The weights are widened once,
// as the source does it -- w.to(f16) * scale[None, :], one fp16 rounding -- into a [K, N] fp16 matrix, and the tiled
// matmul kernels multiply (fp16 operands, fp32 accumulation: the same arithmetic as the decode kernels').  From 193
// rows up, where the passes of the decode kernel cost what widening (W read, twice its bytes written) and one tiled
// product do.  Eight columns per thread: 8-byte weight loads, 16-byte scale loads and stores.
// Measured at [8192, 28672]: 304 us at M = 129, 351 at 256, 452 at 512, 952 at 2048, against 50 us per 32 rows on the
// decode kernels: from seven launches of those on, the widened product is ahead.
constexpr int64_t W8_WIDEN_FROM_ROWS = 193;
__global__ __launch_bounds__(256) void gemm_w8a16_widen_kernel(GemmW8A16Params p) {
  const int64_t octs = p.N / 8, idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= p.K * octs) return;
  const int64_t k = idx / octs, n = (idx % octs) * 8;
  const uint2 q = *reinterpret_cast<const uint2 *>(p.w + k * p.ldw + n);
  const uint4 sv = *reinterpret_cast<const uint4 *>((const uint16_t *)p.scale + n);
  const uint32_t qs[2] = {q.x, q.y}, ss[4] = {sv.x, sv.y, sv.z, sv.w};
  uint32_t out[4];
#pragma unroll
  for (int c = 0; c < 4; c++) {
    // bytes 2c and 2c + 1 of the eight: [b0, 0, b1, 0], then 0x6400 | (b ^ 0x80) = 1152 + b as fp16 (exact), as in the decode kernels
    const uint32_t word = qs[c / 2] >> (16 * (c & 1));
    const uint32_t pair = ((word & 0xffu) | ((word & 0xff00u) << 8)) ^ 0x64806480u;
    out[c] = pk_sub_1152_mul(pair, ss[c]);
  }
  *reinterpret_cast<uint4 *>((uint16_t *)p.widened + k * p.N + n) = make_uint4(out[0], out[1], out[2], out[3]);
}
static bool w8_widens(const GemmW8A16Params &p) {
  return p.M >= W8_WIDEN_FROM_ROWS && p.N % 8 == 0 && p.ldw % 8 == 0 && ((uintptr_t)p.w & 7) == 0 && ((uintptr_t)p.scale & 15) == 0;
}

// More rows of A than a launch takes (32 on the 16-byte-load kernel, 16 on the other): the decode kernels once per
// group of rows, one launch after the other on the stream (they share the split-K workspace, which every launch leaves
// ready for the next).  W is read once per launch, so this is for the rows beside the decode shape (M = 64 at
// [8192, 28672]: two passes over W, against 13 ms on the generic family's kernel); a prefill-sized M wants the tiled
// matmul kernels on dequantised weights instead.
size_t gemm_w8a16_widened_bytes(const GemmW8A16Params &p) { return w8_widens(p) ? (size_t)p.K * p.N * 2 : 0; }

hipError_t launch_gemm_w8a16(const GemmW8A16Params &p, hipStream_t s, const char **name) {
  if (p.widened && w8_widens(p)) {
    hipLaunchKernelGGL(gemm_w8a16_widen_kernel, dim3((unsigned)((p.K * (p.N / 8) + 255) / 256)), dim3(256), 0, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    GemmParams g{};
    g.a = p.a; g.b = p.widened; g.c = p.c;
    g.M = p.M; g.N = p.N; g.K = p.K;
    g.lda = p.lda; g.ldb = p.N; g.ldc = p.ldc;
    g.split = 1;
    const char *inner = nullptr;
    e = launch_gemm(g, s, &inner);
    *name = "gemm_w8a16_widen_kernel + matmul";
    return e;
  }
  const int64_t rows = w8_wide(p) ? 32 : 16;
  if (p.M <= rows) return launch_gemm_w8a16_rows(p, s, name);
  for (int64_t m0 = 0; m0 < p.M; m0 += rows) {
    GemmW8A16Params q = p;
    q.M = std::min<int64_t>(rows, p.M - m0);
    q.a = (const uint16_t *)p.a + m0 * p.lda;
    q.c = (uint16_t *)p.c + m0 * p.ldc;
    hipError_t e = launch_gemm_w8a16_rows(q, s, name);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

static bool w8_fast(const GemmW8A16Params &p) {
  return p.K % 32 == 0 && p.N % W8_COLS == 0 && p.lda % 8 == 0 && p.ldw % 8 == 0 && ((uintptr_t)p.a & 15) == 0 && ((uintptr_t)p.w & 7) == 0;
}
static bool w8_wide(const GemmW8A16Params &p) { return w8_fast(p) && w8_config(p).cw == 16 && ((uintptr_t)p.w & 15) == 0; }

static hipError_t launch_gemm_w8a16_rows(const GemmW8A16Params &p, hipStream_t s, const char **name) {
  W8Config c = w8_config(p);
  const int steps = (int)((p.K + 31) / 32);
  const int sps = (steps + p.split - 1) / p.split;
  const bool fast = w8_fast(p);
  const bool wide = w8_wide(p);
  if (wide) {
    *name = "gemm_w8a16_wide_kernel";
    // slice 0 gets `bias` steps more than an even share (see the kernel's tail), taken evenly from the others
    int first = sps, other = sps;
    if (p.split > 1) {
      static const char *bias_env = getenv("TTS_W8_BIAS");  // tuning aid
      const int bias = bias_env ? atoi(bias_env) : 4;
      const int take = (bias + p.split - 2) / (p.split - 1);  // per other slice
      if (sps - take >= 8 && sps * p.split == steps) { first = sps + take * (p.split - 1); other = sps - take; }
    }
    // one step in flight per wavefront; two measured 1.2 us slower at the decode shape
    if (p.M > 16) return w8_launch_wide<8, 1, 2>(p, first, other, s);
    if (c.depth == 2) return w8_launch_wide<8, 2>(p, first, other, s);
    return w8_launch_wide<8, 1>(p, first, other, s);
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
