// Device code of the 16-bit matrix-product kernels, in a header of its own because it is compiled twice: ahead of
// time into the library (kernels_gemm.hip, results stored as they are), and at run time with hipRTC when the Triton
// kernel applies elementwise ops to the accumulator before the store (a fused activation): the generated source
// defines TTS_GEMM_RTC (which kernel: 0 whole 256 x 256 x 32 tiles, 1 any shape in 256 x 256 tiles, 2 any shape in
// 128 x 128 tiles), TTS_GEMM_BF16 and the functor TtsEp (a plain struct, passed as the kernel's last argument) that maps
// an accumulator value and its position to the value stored, then this file's text.  Nothing here may need a host header.
#pragma once
#ifdef __HIPCC_RTC__
typedef __INT64_TYPE__ int64_t;
typedef __UINT64_TYPE__ uint64_t;
typedef __UINT32_TYPE__ uint32_t;
typedef __UINT16_TYPE__ uint16_t;
typedef __UINTPTR_TYPE__ uintptr_t;
#else
#include <hip/hip_runtime.h>

#include <cstdint>
#endif

// C[M,N] = A[M,K] * B[K,N], 16-bit operands, fp32 accumulate; C is row-major, A and B row- or column-major
struct TtsGemmParams {
  const void *a, *b;
  void *c;
  int64_t M, N, K;
  int64_t lda, ldb, ldc;  // pitches in elements; the other stride of each matrix is 1
  int is_bf16;
  int a_trans, b_trans;   // A / B is column-major: element (m, k) of A is a[m + k * lda], (k, n) of B is b[k + n * ldb]
};

namespace tts_gemm_device {
typedef TtsGemmParams GemmParams;

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
// `ep(acc, row, col)` maps an accumulator value to the value that is stored at (row, col) of C (the identity for a plain
// product); it is only called for elements inside the problem.
template <bool BF16, int TM, int TN, int BK, class Ep>
__device__ __forceinline__ void gemm_mfma_body(const GemmParams &p, int tiles_m, int tiles_n, const Ep &ep) {
  constexpr int BM = 2 * TM * 32, BN = 2 * TN * 32, PITCH = BK + 8;
  constexpr int CA = BM * BK / 8 / 256;          // 16-byte chunks of A per thread
  constexpr int UB = (BK / 2) * (BN / 8) / 256;  // 2x8 units of B per thread
  #ifdef TTS_GEMM_RTC
  __shared__ __align__(16) uint16_t smem[2 * (BM + BN) * PITCH];
#else
  extern __shared__ __align__(16) uint16_t smem[];
#endif
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
  static_assert(BM == BN && CA == 2 * UB, "both operands are staged by the same two routines");

  // An operand tile is R = BM = BN rows (rows of A, columns of B) by BK values of k.  In memory either k is the
  // contiguous index (A row-major, B column-major: element (r, k) at P[r * ld + k]) or r is (A column-major, B
  // row-major: P[k * ld + r]).  Either way the tile lands in LDS as [r][k]; in the second form the two K-neighbours of
  // eight consecutive r are packed into 32-bit words on the way.
  auto load_k_contiguous = [&](uint4 (&reg)[CA], const uint16_t *P, int64_t ld, int64_t r0, int64_t rows, bool vec, int k0) {
#pragma unroll
    for (int j = 0; j < CA; j++) {
      int c = tid + 256 * j, row = c / (BK / 8), kc = c % (BK / 8);
      int64_t gr = r0 + row;
      int gk = k0 + kc * 8;
      reg[j] = gr < rows ? load8(P + gr * ld + gk, K - gk, vec) : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_k_contiguous = [&](const uint4 (&reg)[CA], uint16_t *S) {
#pragma unroll
    for (int j = 0; j < CA; j++) {
      int c = tid + 256 * j, row = c / (BK / 8), kc = c % (BK / 8);
      *reinterpret_cast<uint4 *>(S + row * PITCH + kc * 8) = reg[j];
    }
  };
  auto load_r_contiguous = [&](uint4 (&reg)[CA], const uint16_t *P, int64_t ld, int64_t r0, int64_t rows, bool vec, int k0) {
#pragma unroll
    for (int j = 0; j < UB; j++) {
      int u = tid + 256 * j, kp = u / (BN / 8), nc = u % (BN / 8);
      int gk = k0 + 2 * kp;
      int64_t gn = r0 + nc * 8;
      int valid = (int)min((int64_t)8, rows - gn);
#pragma unroll
      for (int r = 0; r < 2; r++)
        reg[2 * j + r] = (gk + r < K && valid > 0) ? load8(P + (int64_t)(gk + r) * ld + gn, valid, vec) : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_r_contiguous = [&](const uint4 (&reg)[CA], uint16_t *S) {
#pragma unroll
    for (int j = 0; j < UB; j++) {
      int u = tid + 256 * j, kp = u / (BN / 8), nc = u % (BN / 8);
      uint32_t r0[4] = {reg[2 * j].x, reg[2 * j].y, reg[2 * j].z, reg[2 * j].w};
      uint32_t r1[4] = {reg[2 * j + 1].x, reg[2 * j + 1].y, reg[2 * j + 1].z, reg[2 * j + 1].w};
#pragma unroll
      for (int i = 0; i < 4; i++) {
        uint32_t lo = (r0[i] & 0xffffu) | (r1[i] << 16);          // row 2i:   k, k+1
        uint32_t hi = (r0[i] >> 16) | (r1[i] & 0xffff0000u);      // row 2i+1: k, k+1
        *reinterpret_cast<uint32_t *>(S + (nc * 8 + 2 * i) * PITCH + 2 * kp) = lo;
        *reinterpret_cast<uint32_t *>(S + (nc * 8 + 2 * i + 1) * PITCH + 2 * kp) = hi;
      }
    }
  };
  uint4 ra[CA], rb[CA];
  auto load_tiles = [&](int k0) {
    if (p.a_trans) load_r_contiguous(ra, A, p.lda, m0, p.M, a_vec, k0);
    else load_k_contiguous(ra, A, p.lda, m0, p.M, a_vec, k0);
    if (p.b_trans) load_k_contiguous(rb, B, p.ldb, n0, p.N, b_vec, k0);
    else load_r_contiguous(rb, B, p.ldb, n0, p.N, b_vec, k0);
  };
  auto store_tiles = [&](int buf) {
    uint16_t *As = smem + buf * (BM + BN) * PITCH, *Bs = As + BM * PITCH;
    if (p.a_trans) store_r_contiguous(ra, As);
    else store_k_contiguous(ra, As);
    if (p.b_trans) store_k_contiguous(rb, Bs);
    else store_r_contiguous(rb, Bs);
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
        if (row < p.M && col < p.N) C[row * p.ldc + col] = BF16 ? f32_to_bf16(ep(acc[i][j][v], row, col)) : f32_to_f16(ep(acc[i][j][v], row, col));
      }
    }
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

template <bool BF16, class Ep>
__device__ __forceinline__ void gemm_dma_body(const GemmParams &p, int tiles_m, int tiles_n, const Ep &ep) {
  #ifdef TTS_GEMM_RTC
  __shared__ __align__(16) char dma_smem[F_STAGES * F_STAGE_BYTES];
#else
  extern __shared__ __align__(16) char dma_smem[];
#endif
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
#ifdef TTS_GEMM_RTC
    // the run-time compiler may be an older one than the library's (a process that loaded PyTorch first gets PyTorch's
    // hipRTC), and that one does not see that the tile's base address is the same in every lane: say so
    const uint64_t b = (uint64_t)(uintptr_t)sbase;
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));  // the builtin returns a signed int
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    sbase = (const char *)(uintptr_t)(((uint64_t)hi << 32) | (uint64_t)lo);
#endif
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
        const int64_t er = m0 + wm * 128 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3), ec = n0 + wn * 128 + j * 32 + (lane & 31);
        const f32x2_t pr = {ep(acc[i][j][v], er, ec), ep(acc[i][j][v + 1], er + 1, ec)};
        const uint32_t pk = BF16 ? __builtin_bit_cast(uint32_t, __builtin_convertvector(pr, bf16x2_t))
                                 : __builtin_bit_cast(uint32_t, __builtin_convertvector(pr, f16x2_t));
        const uint32_t nb = __builtin_amdgcn_mov_dpp(pk, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]: the neighbour's pair
        const uint32_t w = __builtin_amdgcn_perm(nb, pk, sel);
        const int64_t row = m0 + wm * 128 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3) + (odd ? 1 : 0);
        __builtin_nontemporal_store(w, reinterpret_cast<uint32_t *>(&C[row * p.ldc + col]));
      }
    }
}

}  // namespace tts_gemm_device

#ifdef TTS_GEMM_RTC
extern "C" __global__ __launch_bounds__(256) void gemm_rtc(TtsGemmParams p, int tiles_m, int tiles_n, TtsEp ep) {
#if TTS_GEMM_RTC == 0
  tts_gemm_device::gemm_dma_body<TTS_GEMM_BF16 != 0>(p, tiles_m, tiles_n, ep);
#elif TTS_GEMM_RTC == 1
  tts_gemm_device::gemm_mfma_body<TTS_GEMM_BF16 != 0, 4, 4, 32>(p, tiles_m, tiles_n, ep);
#else
  tts_gemm_device::gemm_mfma_body<TTS_GEMM_BF16 != 0, 2, 2, 64>(p, tiles_m, tiles_n, ep);
#endif
}
#endif
