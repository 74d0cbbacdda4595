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
// For problems made of whole 256 x 256 x 32 tiles with 16-byte aligned rows.
//
// Workgroup: 256 threads = 4 wavefronts (one per SIMD), wave grid 2 x 2, each wavefront
// 128 x 128 of C = 4 x 4 MFMA tiles of 32 x 32 (256 accumulator registers).
//
// Global -> LDS without passing through registers: `global_load_lds_dwordx4` writes the 64
// lanes' 16-byte chunks to 1 KB of consecutive LDS, so the LDS layout is fixed by which global
// chunk each lane fetches.
//   A stage [256 rows][64 bytes]: position q of row r holds chunk q ^ ((r / 4) & 3) of the row's
//     four; 16-byte fragment reads of 16 consecutive rows then fall into 16 distinct slots.
//   B stage [32 k rows][512 bytes], as in memory (N contiguous): position q of row k holds chunk
//     q ^ ((k & 3) << 2).  The MFMA operand wants K contiguous per lane; `ds_read_b64_tr_b16` does
//     that transposition on the way out: within 16 lanes, lane i receives element i % 4 of the
//     8-byte rows addressed by lanes i / 4, i / 4 + 4, i / 4 + 8, i / 4 + 12.  Lane r of a group
//     therefore addresses k row r / 4, columns 4 (r % 4) .. +3 of the group's 16 columns, and
//     two reads (k 0-3, k 4-7) make one 8-element operand.
// Both layouts were checked on the device: no LDS bank conflicts (SQ_LDS_BANK_CONFLICT = 0).
//
// Pipeline: STAGES LDS stages of one K tile each.  An iteration has two phases of 16 MFMAs (the
// tile's two K halves).  Every MFMA is followed by one LDS read or one direct-to-LDS load, which
// the matrix pipe hides: phase A reads the operands of phase B, phase B those of the next
// tile's phase A; a quarter of the way through each phase one load of tile t+STAGES-1 goes out,
// into the stage of tile t-1, which every wavefront finished reading before the previous barrier.
// One barrier per tile, between the phases: it follows the wait that tells this wavefront its
// own loads of tile t+1 have landed.  Loads past the last tile fetch the last tile again, so the
// wait count is the same in every iteration.
//
// The direct-to-LDS load is issued from inline assembly: the compiler orders every later LDS
// read behind such a load with a full vmcnt wait (it cannot tell the stages apart), which
// would serialise the pipeline.  Its own counting of ordinary loads stays conservative.
constexpr int F_BM = 256, F_BN = 256, F_BK = 32, F_STAGES = 4;
constexpr int F_A_BYTES = F_BM * F_BK * 2, F_STAGE_BYTES = F_A_BYTES + F_BK * F_BN * 2;
typedef short s16x4 __attribute__((ext_vector_type(4)));
#define TTS_LDS(p) ((__attribute__((address_space(3))) void *)(p))

// s_waitcnt immediate: vmcnt in bits 3:0 and 15:14, expcnt (not waited for) in 6:4, lgkmcnt in 11:8
constexpr int waitcnt_imm(int vm, int lgkm) { return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | (lgkm << 8); }

template <bool BF16>
__global__ __launch_bounds__(256) void gemm_dma_kernel(GemmParams p, int tiles_m, int tiles_n) {
  extern __shared__ __align__(16) char dma_smem[];
  char *smem = dma_smem;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  int bid = blockIdx.x;
  const int nwg = tiles_m * tiles_n;
  if (nwg % 8 == 0) bid = (bid % 8) * (nwg / 8) + bid / 8;  // consecutive ids on one XCD
  const int group = 4 * tiles_n;                             // 4-tile-tall column groups
  const int g0 = (bid / group) * 4;
  const int gh = min(tiles_m - g0, 4);
  const int tile_m = g0 + (bid % group) % gh, tile_n = (bid % group) / gh;
  const int64_t m0 = (int64_t)tile_m * F_BM, n0 = (int64_t)tile_n * F_BN;

  // Wavefront w issues A instructions 4w..4w+3 (rows 16 ia + lane / 4) and B instructions
  // 4w..4w+3 (k rows 2 ib + lane / 32) of a tile.  Per-lane byte offsets are constant; the
  // tile's base address moves in scalar registers.
  uint32_t a_voff[4], b_voff[4];
#pragma unroll
  for (int i = 0; i < 4; i++)
    a_voff[i] = (uint32_t)(((64 * wave + 16 * i + lane / 4) * p.lda + 8 * ((lane & 3) ^ ((lane >> 4) & 3))) * 2);
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int krow = 8 * wave + 2 * i + lane / 32;
    b_voff[i] = (uint32_t)((krow * p.ldb + 8 * ((lane & 31) ^ ((krow & 3) << 2))) * 2);
  }
  const char *a_base = (const char *)((const uint16_t *)p.a + m0 * p.lda);
  const char *b_base = (const char *)((const uint16_t *)p.b + n0);
  const uint32_t lds0 = (uint32_t)(uintptr_t)TTS_LDS(smem);
  const uint32_t wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int nk = (int)(p.K / F_BK);
  auto dma = [&](const char *sbase, uint32_t voff, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds), "v"(voff), "s"(sbase) : "memory", "m0");
  };
  auto dma_one = [&](int t, int n) {  // n = 0..3: A part, 4..7: B part of tile t, into stage t % F_STAGES
    const int tc = min(t, nk - 1);
    const uint32_t st = lds0 + (t % F_STAGES) * F_STAGE_BYTES + wave_u * 4096;
    if (n < 4) dma(a_base + (int64_t)tc * F_BK * 2, a_voff[n], st + n * 1024);
    else dma(b_base + (int64_t)tc * F_BK * p.ldb * 2, b_voff[n - 4], st + F_A_BYTES + (n - 4) * 1024);
  };

  // fragment read offsets (bytes, within a stage)
  // A: row r = wm * 128 + i * 32 + lane % 32, chunk c = 2 ks + lane / 32 at position c ^ ((r / 4) & 3)
  const int ar = wm * 128 + (lane & 31);
  const int a_off = ar * 64, a_sw = (ar >> 2) & 3;
  // B: 16-lane group q = lane / 16, r16 = lane % 16: k row ks * 16 + 8 (q / 2) + 4 h + r16 / 4,
  // chunk wn * 16 + 4 j + 2 (q & 1) + (r16 % 4) / 2, byte 8 (r16 & 1) within the chunk
  const int q = lane >> 4, r16 = lane & 15;
  const int b_chunk = wn * 16 + 2 * (q & 1) + ((r16 & 3) >> 1), b_sw = (r16 >> 2) << 2;
  const int b_off = F_A_BYTES + (8 * (q >> 1) + (r16 >> 2)) * 512 + 8 * (r16 & 1);

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  uint4 af[2][4], bf[2][4];
  // one fragment read (n = 0..3: A row block n; n = 4..11: B column block (n - 4) / 2, k half (n - 4) % 2)
  auto read_one = [&](int t, int ks, int n, uint4 (&a)[4], uint4 (&b)[4]) {
    const char *st = smem + (t % F_STAGES) * F_STAGE_BYTES;
    if (n < 4) {
      a[n] = *reinterpret_cast<const uint4 *>(st + a_off + n * 2048 + (((2 * ks + (lane >> 5)) ^ a_sw) << 4));
    } else {
      const int j = (n - 4) >> 1, h = (n - 4) & 1;
      const char *bp = st + b_off + ks * 16 * 512 + (((b_chunk + 4 * j) ^ b_sw) << 4) + h * 4 * 512;
      s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)TTS_LDS(bp));
      uint2 v2 = __builtin_bit_cast(uint2, v);
      if (h == 0) { b[j].x = v2.x; b[j].y = v2.y; } else { b[j].z = v2.x; b[j].w = v2.y; }
    }
  };
  auto mfma_one = [&](int n, uint4 (&a)[4], uint4 (&b)[4]) {
    acc[n >> 2][n & 3] = mfma32<BF16>(a[n >> 2], b[n & 3], acc[n >> 2][n & 3]);
  };

  // prologue: STAGES - 1 tiles in flight; tile 0 landed; its first operands read
  for (int t = 0; t < F_STAGES - 1; t++)
#pragma unroll
    for (int n = 0; n < 8; n++) dma_one(t, n);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(8 * (F_STAGES - 2), 15));
  __syncthreads();
#pragma unroll
  for (int n = 0; n < 12; n++) read_one(0, 0, n, af[0], bf[0]);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));
  for (int t = 0; t < nk; t++) {
    // phase A: MFMAs of (tile t, first half); read (tile t, second half); first half of the loads of tile t + STAGES - 1
#pragma unroll
    for (int n = 0; n < 16; n++) {
      __builtin_amdgcn_sched_barrier(0);
      mfma_one(n, af[0], bf[0]);
      if (n < 12) read_one(t, 1, n, af[1], bf[1]);
      if ((n & 3) == 3) dma_one(t + F_STAGES - 1, n >> 2);
    }
    __builtin_amdgcn_sched_barrier(0);
    // own loads of tile t+1 have landed (later ones may be in flight); own reads of tile t are complete
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(8 * (F_STAGES - 3) + 4, 0));
    __syncthreads();
    // phase B: MFMAs of (tile t, second half); read (tile t+1, first half); the rest of the loads
#pragma unroll
    for (int n = 0; n < 16; n++) {
      __builtin_amdgcn_sched_barrier(0);
      mfma_one(n, af[1], bf[1]);
      if (n < 12) read_one(t + 1, 0, n, af[0], bf[0]);
      if ((n & 3) == 3) dma_one(t + F_STAGES - 1, (n >> 2) + 4);
    }
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));  // the surplus loads land before the LDS goes away

  // Epilogue.  A lane holds one column of each 32x32 block (rows 8 (v/4) + 4 (lane/32) + v%4 in element v).  Two rows
  // are narrowed at once (v_cvt_pk_bf16_f32 for bf16: round to nearest even, NaNs quieted), the pair is exchanged with
  // the neighbouring lane, and the even lane stores row r at columns (n, n+1), the odd lane row r+1 at (n-1, n):
  // half as many store instructions as one 2-byte store per element, and a handful of VALU ops per pair.
  uint16_t *__restrict__ C = (uint16_t *)p.c;
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  const bool odd = lane & 1;
  const uint32_t sel = odd ? 0x03020706u : 0x05040100u;  // odd: high halves of (neighbour, mine); even: low halves of (mine, neighbour)
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int64_t col = n0 + wn * 128 + j * 32 + (lane & 31) - (odd ? 1 : 0);
#pragma unroll
      for (int v = 0; v < 16; v += 2) {
        const f32x2_t pr = {acc[i][j][v], acc[i][j][v + 1]};
        const uint32_t pk = BF16 ? __builtin_bit_cast(uint32_t, __builtin_convertvector(pr, bf16x2_t))
                                 : __builtin_bit_cast(uint32_t, __builtin_convertvector(pr, f16x2_t));
        const uint32_t nb = __builtin_amdgcn_mov_dpp(pk, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]: the neighbour's pair
        const uint32_t w = __builtin_amdgcn_perm(nb, pk, sel);
        const int64_t row = m0 + wm * 128 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3) + (odd ? 1 : 0);
        __builtin_nontemporal_store(w, reinterpret_cast<uint32_t *>(&C[row * p.ldc + col]));
      }
    }
}

template <bool BF16>
hipError_t launch_gemm_dma(const GemmParams &p, hipStream_t s) {
  constexpr size_t lds = (size_t)F_STAGES * F_STAGE_BYTES;
  auto kern = gemm_dma_kernel<BF16>;
  static const hipError_t attr = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (attr != hipSuccess) return attr;
  int tiles_m = (int)(p.M / F_BM), tiles_n = (int)(p.N / F_BN);
  hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(256), lds, s, p, tiles_m, tiles_n);
  return hipGetLastError();
}

// whole tiles, 16-byte aligned rows, and per-lane byte offsets that fit 32 bits
bool gemm_fast_path_ok(const GemmParams &p) {
  return p.M % F_BM == 0 && p.N % F_BN == 0 && p.K % F_BK == 0 && p.K >= F_BK && p.lda % 8 == 0 && p.ldb % 8 == 0 &&
         ((uintptr_t)p.a & 15) == 0 && ((uintptr_t)p.b & 15) == 0 && p.lda < (1 << 22) && p.ldb < (1 << 25) &&
         p.ldc % 2 == 0 && ((uintptr_t)p.c & 3) == 0;  // C is written in 4-byte pairs
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
    for (int t = 0; t < 8; t++) {
      // the weights are read once per launch: nontemporal, so that they do not displace A, the scales and the partial
      // tiles from the caches (46.2 -> 43.1 us at the decode shape with the weights coming from HBM)
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
      const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(src + (int64_t)t * p.ldw));
      q[t] = make_uint4(v[0], v[1], v[2], v[3]);
    }
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
    *name = "gemm_dma_kernel";
    return p.is_bf16 ? launch_gemm_dma<true>(p, s) : launch_gemm_dma<false>(p, s);
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
