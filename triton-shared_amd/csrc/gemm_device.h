// Device code of the 16-bit matrix-product kernels, in a header of its own because it is compiled twice: ahead of
// time into the library (kernels_gemm.hip, results stored as they are), and at run time with hipRTC when the Triton
// kernel applies elementwise ops to the accumulator before the store (a fused activation): the generated source
// defines TTS_GEMM_RTC (which kernel: 0 whole 256 x 256 x 32 tiles, 1 any shape in 128 x 128 x 64 tiles), TTS_GEMM_BF16 and the functor TtsEp (a plain struct, passed as the kernel's last argument) that maps
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

// C[M,N] = A[M,K] * B[K,N], 16-bit (or fp32) operands, fp32 accumulate; C is row-major, A and B row- or column-major
struct TtsGemmParams {
  const void *a, *b;
  void *c;
  int64_t M, N, K;
  int64_t lda, ldb, ldc;  // pitches in elements; the other stride of each matrix is 1
  int is_bf16;
  int a_trans, b_trans;   // A / B is column-major: element (m, k) of A is a[m + k * lda], (k, n) of B is b[k + n * ldb]
  // Gathered operands (null / 0 for a plain product): row m of A is row a_rows[m] of the matrix at `a` (row-major A only);
  // the rows of block m / b_block_rows multiply the matrix at b + b_block[m / b_block_rows] * b_block_stride elements,
  // or nothing at all when that id is negative (their part of C is not written).
  const int *a_rows;
  const int *b_block;
  int64_t b_block_stride;
  int b_block_rows;
  int gather_mul32;       // bit 0: a_rows[m] * lda, bit 1: id * b_block_stride is a 32-bit product that wraps, as the source computes it
  int is_f32;             // fp32 operands and result (kernels_gemm.hip: gemm_f32_kernel); is_bf16 is then 0
  // K in `split` slices, one workgroup per (tile, slice), for products with too few tiles to occupy the chip: slice s
  // leaves its fp32 sums at partial[s * M * N + m * N + n], and a second kernel adds the slices and narrows (1 = none)
  int split;
  float *partial;
  // A batch of products of one shape (grid.y of the launch = batches): batch b reads a + b * batch_a and b + b * batch_b
  // and writes c + b * batch_c (in elements); 1 / 0 for a single product
  int batches;
  int64_t batch_a, batch_b, batch_c;
};

namespace tts_gemm_device {
typedef TtsGemmParams GemmParams;

// the product of batch blockIdx.y of a launch (esize: bytes per element of the operands and of C)
__device__ __forceinline__ GemmParams of_batch(const GemmParams &p, int esize) {
  GemmParams q = p;
  const int64_t by = blockIdx.y;
  q.a = (const char *)p.a + by * p.batch_a * esize;
  q.b = (const char *)p.b + by * p.batch_b * esize;
  q.c = (char *)p.c + by * p.batch_c * esize;
  if (p.partial) q.partial = p.partial + by * (int64_t)p.split * p.M * p.N;
  return q;
}

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
// The kernel for any shape, any alignment, and operands that are row- or column-major.
// Workgroup: 256 threads = 2 x 2 wavefronts; each wavefront owns TM x TN MFMA tiles of 32 x 32.  An operand tile is
// R = BM = BN rows (rows of A, columns of B) by BK values of k and is staged through LDS (two buffers) in the form it
// has in memory, with 16-byte loads and stores where alignment allows:
//   k contiguous (A row-major, B column-major): LDS [r][k], pitch BK + 8 elements; a lane's MFMA operand (8 consecutive
//     k of row lane % 32) is one 16-byte read, and 32 consecutive rows hit distinct banks;
//   r contiguous (B row-major, A column-major): LDS [k][r], pitch R + 16 elements; `ds_read_b64_tr_b16` transposes on
//     the way out -- within 16 lanes, lane i receives element i % 4 of the 8-byte rows addressed by lanes i / 4,
//     i / 4 + 4, i / 4 + 8, i / 4 + 12, so lane j of a group addresses k row j / 4, elements 4 (j % 4) .. +3 of the
//     group's 16, and two reads (k 0-3, k 4-7) make one operand.
// Rows of A may be taken through an index vector (p.a_rows) and the base of B may depend on the block of rows
// (p.b_block): a mixture-of-experts product is this kernel with both set.
// `ep(acc, row, col)` maps an accumulator value to the value that is stored at (row, col) of C (the identity for a plain
// product); it is only called for elements inside the problem.
template <bool V>
struct BoolConstant {
  static constexpr bool value = V;
};

template <int BM, int BN, int BK>
struct GemmStageLds {
  static constexpr int A_ELEMS = (BM * (BK + 8) > BK * (BM + 16)) ? BM * (BK + 8) : BK * (BM + 16);
  static constexpr int B_ELEMS = (BN * (BK + 8) > BK * (BN + 16)) ? BN * (BK + 8) : BK * (BN + 16);
  static constexpr int BUFFER_ELEMS = A_ELEMS + B_ELEMS;
  static constexpr int BYTES = 2 * BUFFER_ELEMS * 2;
};

template <bool BF16, int TM, int TN, int BK, class Ep>
__device__ __forceinline__ void gemm_mfma_body(const GemmParams &p, int tiles_m, int tiles_n, const Ep &ep) {
  constexpr int BM = 2 * TM * 32, BN = 2 * TN * 32;
  constexpr int PK = BK + 8;   // pitch of a k-contiguous tile
  constexpr int PR = BM + 16;  // pitch of an r-contiguous tile
  constexpr int CA = BM * BK / 8 / 256;  // 16-byte chunks of an operand tile per thread
  static_assert(BM == BN, "both operands are staged by the same routines");
  using Lds = GemmStageLds<BM, BN, BK>;
#ifdef TTS_GEMM_RTC
  __shared__ __align__(16) uint16_t smem[2 * Lds::BUFFER_ELEMS];
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
  if (p.b_block) {  // the rows of this tile multiply a matrix of their own; a negative id: nothing to do for them
    const int which = p.b_block[m0 / p.b_block_rows];
    if (which < 0) return;
    B += (p.gather_mul32 & 2) ? (int64_t)(int)((uint32_t)which * (uint32_t)p.b_block_stride) : (int64_t)which * p.b_block_stride;
  }
  const bool a_vec = (p.lda % 8 == 0) && (((uintptr_t)A & 15) == 0);
  const bool b_vec = (p.ldb % 8 == 0) && (((uintptr_t)B & 15) == 0);
  const int K = (int)p.K;

  // where this thread's chunks of the tiles are: (row, k chunk) of a k-contiguous tile, (k, row chunk) of an
  // r-contiguous one; element offsets of the chunks' rows in memory (-1: outside the problem)
  int64_t a_at[CA], b_at[CA];
#pragma unroll
  for (int j = 0; j < CA; j++) {
    const int c = tid + 256 * j;
    if (p.a_trans) {
      a_at[j] = m0 + (c % (BM / 8)) * 8;  // first of 8 rows; the k row moves with the loop
    } else {
      const int64_t gr = m0 + c / (BK / 8);
      if (gr >= p.M) a_at[j] = -1;
      else if (!p.a_rows) a_at[j] = gr * p.lda;
      else a_at[j] = (p.gather_mul32 & 1) ? (int64_t)(int)((uint32_t)p.a_rows[gr] * (uint32_t)p.lda) : (int64_t)p.a_rows[gr] * p.lda;
    }
    if (p.b_trans) {
      const int64_t gn = n0 + c / (BK / 8);
      b_at[j] = gn < p.N ? gn * p.ldb : -1;
    } else {
      b_at[j] = n0 + (c % (BN / 8)) * 8;
    }
  }
  uint4 ra[CA], rb[CA];
  auto load_operand = [&](uint4 (&reg)[CA], const uint16_t *P, bool r_contiguous, const int64_t (&at)[CA], int64_t ld, int64_t rows, bool vec, int k0) {
#pragma unroll
    for (int j = 0; j < CA; j++) {
      const int c = tid + 256 * j;
      if (r_contiguous) {
        const int gk = k0 + c / (BM / 8);
        const int valid = (int)min((int64_t)8, rows - at[j]);
        reg[j] = (gk < K && valid > 0) ? load8(P + (int64_t)gk * ld + at[j], valid, vec) : make_uint4(0, 0, 0, 0);
      } else {
        const int gk = k0 + (c % (BK / 8)) * 8;
        reg[j] = at[j] >= 0 ? load8(P + at[j] + gk, K - gk, vec) : make_uint4(0, 0, 0, 0);
      }
    }
  };
  auto store_operand = [&](const uint4 (&reg)[CA], uint16_t *S, bool r_contiguous) {
#pragma unroll
    for (int j = 0; j < CA; j++) {
      const int c = tid + 256 * j;
      if (r_contiguous) *reinterpret_cast<uint4 *>(S + (c / (BM / 8)) * PR + (c % (BM / 8)) * 8) = reg[j];
      else *reinterpret_cast<uint4 *>(S + (c / (BK / 8)) * PK + (c % (BK / 8)) * 8) = reg[j];
    }
  };
  // a lane's MFMA operand for the 32 rows starting at `row0` of a staged tile, k = ks * 16 + 8 (lane / 32) .. +7
  auto fragment = [&](const uint16_t *S, bool r_contiguous, int row0, int ks) -> uint4 {
    if (!r_contiguous) return *reinterpret_cast<const uint4 *>(S + (row0 + (lane & 31)) * PK + ks * 16 + 8 * (lane >> 5));
    const int g = lane >> 4, j = lane & 15;
    const uint16_t *at = S + (ks * 16 + 8 * (g >> 1) + (j >> 2)) * PR + row0 + 16 * (g & 1) + 4 * (j & 3);
    typedef short s16x4_t __attribute__((ext_vector_type(4)));
    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t __attribute__((address_space(3))) *)((__attribute__((address_space(3))) void *)at));
    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t __attribute__((address_space(3))) *)((__attribute__((address_space(3))) void *)(at + 4 * PR)));
    const uint2 l2 = __builtin_bit_cast(uint2, lo), h2 = __builtin_bit_cast(uint2, hi);
    return make_uint4(l2.x, l2.y, h2.x, h2.y);
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  // The forms of the two operands are fixed for the launch: the loop is compiled once per combination, so that inside
  // it the loads, the LDS traffic and the MFMAs are straight-line code the compiler can overlap.
  const int nk = (K + BK - 1) / BK;
  auto sweep_k = [&](auto a_form, auto b_form) {
    constexpr bool a_r = decltype(a_form)::value, b_r = decltype(b_form)::value;  // r-contiguous in memory and in LDS
    auto load_tiles = [&](int k0) {
      load_operand(ra, A, a_r, a_at, p.lda, p.M, a_vec, k0);
      load_operand(rb, B, b_r, b_at, p.ldb, p.N, b_vec, k0);
    };
    auto store_tiles = [&](int buf) {
      uint16_t *As = smem + buf * Lds::BUFFER_ELEMS, *Bs = As + Lds::A_ELEMS;
      store_operand(ra, As, a_r);
      store_operand(rb, Bs, b_r);
    };
    if (nk > 0) {
      load_tiles(0);
      store_tiles(0);
    }
    __syncthreads();
    for (int kt = 0; kt < nk; kt++) {
      const int cur = kt & 1;
      if (kt + 1 < nk) load_tiles((kt + 1) * BK);
      const uint16_t *As = smem + cur * Lds::BUFFER_ELEMS, *Bs = As + Lds::A_ELEMS;
#pragma unroll
      for (int ks = 0; ks < BK / 16; ks++) {
        uint4 af[TM], bf[TN];
#pragma unroll
        for (int i = 0; i < TM; i++) af[i] = fragment(As, a_r, wm * TM * 32 + i * 32, ks);
#pragma unroll
        for (int j = 0; j < TN; j++) bf[j] = fragment(Bs, b_r, wn * TN * 32 + j * 32, ks);
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
          for (int j = 0; j < TN; j++) acc[i][j] = mfma32<BF16>(af[i], bf[j], acc[i][j]);
      }
      if (kt + 1 < nk) store_tiles(cur ^ 1);
      __syncthreads();
    }
  };
  if (p.a_trans) {
    if (p.b_trans) sweep_k(BoolConstant<true>(), BoolConstant<false>());
    else sweep_k(BoolConstant<true>(), BoolConstant<true>());
  } else {
    if (p.b_trans) sweep_k(BoolConstant<false>(), BoolConstant<false>());
    else sweep_k(BoolConstant<false>(), BoolConstant<true>());
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
constexpr int F_BK = 32;
// Tile geometry of the direct-to-LDS kernel: 2 x 2 wavefronts of TM x TN MFMA tiles each.
template <int TM, int TN>
struct DmaTile {
  static constexpr int BM = 2 * TM * 32, BN = 2 * TN * 32;
  static constexpr int A_BYTES = BM * F_BK * 2, B_ROW_BYTES = BN * 2, STAGE_BYTES = A_BYTES + F_BK * B_ROW_BYTES;
  static constexpr int A_DMA = BM / 64, B_DMA = BN / 64;  // direct-to-LDS instructions per wavefront and K tile
  static constexpr int DMA = A_DMA + B_DMA;
  // Four stages everywhere: 128 KB (256 x 256), 96 KB (128 x 256, 256 x 128: one workgroup per CU, which is what a
  // problem that gives fewer than one 256 x 256 tile per CU gets anyway), 64 KB (128 x 128: two per CU).  With three
  // stages the 128 x 256 tile measured 46.3 us on 4096 x 2048 x 2048 against 40.4 with four (five and six: no better).
  static constexpr int STAGES = 4;
  static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
};
constexpr int F_BM = DmaTile<4, 4>::BM, F_BN = DmaTile<4, 4>::BN, F_STAGES = DmaTile<4, 4>::STAGES;
constexpr int F_A_BYTES = DmaTile<4, 4>::A_BYTES, F_STAGE_BYTES = DmaTile<4, 4>::STAGE_BYTES;
typedef short s16x4 __attribute__((ext_vector_type(4)));
#define TTS_LDS(p) ((__attribute__((address_space(3))) void *)(p))

// s_waitcnt immediate: vmcnt in bits 3:0 and 15:14, expcnt (not waited for) in 6:4, lgkmcnt in 11:8
constexpr int waitcnt_imm(int vm, int lgkm) { return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | (lgkm << 8); }

// TM x TN = 4 x 4: the 256 x 256 tile described above.  Smaller tiles (2 x 2: 128 x 128, 2 x 4: 128 x 256, 4 x 2:
// 256 x 128) use the same stages, swizzles and phases with fewer rows and columns: an A instruction still covers 16
// rows of 64 bytes, a B instruction 1024 / (2 BN) k rows of 2 BN bytes (position q of k row k holds chunk
// q ^ ((k & 3) << 2) of the row's BN / 8).  They take A rows through an index vector and a matrix id per block of rows
// (p.a_rows, p.b_block): the A addresses are then 64-bit per lane.
// BT: B is column-major (p.b_trans: element (k, n) at b[k + n * ldb], the tutorial's `b.T` and the weight layout of a
// linear layer).  Its stage is then laid out like A's, [BN columns][64 bytes] with the same swizzle, and an operand is
// one 16-byte read; nothing needs transposing.
template <bool E> struct EdgeTile { static constexpr bool value = E; };
// AT: A is column-major (p.a_trans: element (m, k) at a[m + k * lda]).  Its stage is laid out like a row-major B's,
// [32 k rows][2 BM bytes], and read through the same transposing LDS read.
// PF: the workgroup has a fifth wavefront that fetches nothing into the stages; it touches lines of B some K tiles ahead
// of the four that work (below).
constexpr int F_PF_AHEAD = 8;
// SK: the grid holds p.split workgroups per tile; workgroup (tile, s) walks the s-th share of the K tiles and leaves its sums
// in p.partial.
template <bool BF16, int TM, int TN, class Ep, bool BT = false, bool AT = false, bool PF = false, bool SK = false>
__device__ __forceinline__ void gemm_dma_body(const GemmParams &p, int tiles_m, int tiles_n, const Ep &ep) {
  using T = DmaTile<TM, TN>;
  constexpr int BM = T::BM, BN = T::BN, STAGES = T::STAGES, A_BYTES = T::A_BYTES, STAGE_BYTES = T::STAGE_BYTES, ROWB = T::B_ROW_BYTES;
  constexpr int A_DMA = T::A_DMA, B_DMA = T::B_DMA, DMA = T::DMA;
  constexpr int B_KROWS = 1024 / ROWB;       // k rows one B instruction covers
  constexpr int B_CHUNKS = ROWB / 16;        // 16-byte chunks per k row
  constexpr bool GATHER = !(TM == 4 && TN == 4) && !AT;
  constexpr int A_ROWB = BM * 2, A_KROWS = 1024 / A_ROWB, A_CHUNKS = A_ROWB / 16;  // AT: bytes per k row, k rows per instruction, chunks per k row
  static_assert(DMA % 2 == 0, "half of a tile's loads go out in each phase");
#ifdef TTS_GEMM_RTC
  __shared__ __align__(16) char dma_smem[T::LDS_BYTES];
#else
  extern __shared__ __align__(16) char dma_smem[];
#endif
  char *smem = dma_smem;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  int bid = blockIdx.x;
  const int nwg = tiles_m * tiles_n;
  const int slice = SK ? bid / nwg : 0;
  if (SK) bid -= slice * nwg;
  if (nwg % 8 == 0) bid = (bid % 8) * (nwg / 8) + bid / 8;  // consecutive ids on one XCD
  const int group = 4 * tiles_n;                             // 4-tile-tall column groups
  const int g0 = (bid / group) * 4;
  const int gh = min(tiles_m - g0, 4);
  int tile_m = g0 + (bid % group) % gh;
  const int tile_n = (bid % group) / gh;
  int pf_share = tile_m - g0, pf_shares = gh;  // PF: this workgroup's part of the B lines its column group reads
  if (GATHER && p.b_block && tiles_m <= 256) {
    // Row tiles that multiply the same matrix should sit behind one L2: the workgroup takes the row tile whose place in
    // the order by matrix id (ties by position) is the one the tile order above gave it.  With ids 0..7 dealt round-robin
    // to 32 blocks of 128 rows, every XCD otherwise streams four of the eight matrices (measured past L2: 319 MB per
    // launch for 100 MB of operands).
    __shared__ int block_key[256], place_key[256], sorted_tile;
    if (tid < tiles_m) block_key[tid] = p.b_block[((int64_t)tid * BM) / p.b_block_rows];
    __syncthreads();
    if (tid < tiles_m) {
      const int mine = block_key[tid];
      int place = 0;
      for (int o = 0; o < tiles_m; o++) place += (block_key[o] < mine || (block_key[o] == mine && o < tid)) ? 1 : 0;
      if (place == tile_m) sorted_tile = tid;
      place_key[place] = mine;
    }
    __syncthreads();
    if (PF) {  // the row tiles of this column group that multiply the same matrix split its lines between them
      const int mine = place_key[tile_m];
      pf_share = 0, pf_shares = 0;
      for (int q = g0; q < g0 + gh; q++)
        if (place_key[q] == mine) {
          if (q < tile_m) pf_share++;
          pf_shares++;
        }
    }
    tile_m = sorted_tile;
  }
  const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;

  const char *b_base = (const char *)((const uint16_t *)p.b + (BT ? n0 * p.ldb : n0));
  int which = 0;
  if (GATHER && p.b_block) {  // the rows of this tile multiply a matrix of their own; a negative id: nothing to do for them
    which = p.b_block[m0 / p.b_block_rows];
    if (which < 0) return;
    b_base += 2 * ((p.gather_mul32 & 2) ? (int64_t)(int)((uint32_t)which * (uint32_t)p.b_block_stride) : (int64_t)which * p.b_block_stride);
  }

  const int nk_all = (int)(p.K / F_BK);
  const int k_begin = SK ? (int)((int64_t)slice * nk_all / p.split) : 0;
  const int nk = SK ? (int)((int64_t)(slice + 1) * nk_all / p.split) - k_begin : nk_all;
  // Row tiles with matrices of their own walk K from different starting tiles (matrix id tiles in, wrapping round): the
  // workgroups of a launch start together, and matrices that lie a power of two apart in memory would otherwise be read
  // at the same offsets at the same time.  (The sum over K is taken in that order; 1.5 us of 45 on the measured case.)
  const int k_first = (GATHER && p.b_block) ? (int)((uint32_t)which % (uint32_t)nk) : 0;
  if (PF && wave == 4) {
    // The working wavefronts' loads wait in the memory pipeline for as long as their lines take to arrive, and lines that
    // come from HBM (several weight matrices: nothing of B is read twice out of the Infinity Cache) take long enough that
    // more LDS stages do not help (five and six measured like four).  This wavefront asks for the lines first: a
    // 4-byte load per 128-byte line of its share of the B tile F_PF_AHEAD tiles ahead, into a patch of LDS nobody reads (a
    // load into a register would come back long after the compiler has given the register to something else).  It keeps
    // step with the others through the same barriers.  Measured on 4096 gathered rows x [8, 2048, 2048]: 50.0 -> 43.8 us
    // with operands from HBM; touching A's lines as well cost 1 us, touching every other line gained nothing.
    static_assert(!PF || (!BT && !AT), "the prefetching wavefront walks a row-major B");
    __shared__ int touched[64];
    const uint32_t sink = (uint32_t)(uintptr_t)TTS_LDS(touched);
    constexpr int LPR = ROWB / 128, LINES = F_BK * LPR;  // 128-byte lines per k row and per tile
    const int per = (LINES + pf_shares - 1) / pf_shares;
    const char *line_at[2];
    bool on[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {  // at most 128 lines per tile
      const int l = lane + 64 * h, line = pf_share * per + l;
      on[h] = l < per && line < LINES && n0 + (line % LPR) * 64 < p.N;
      line_at[h] = b_base + ((int64_t)(line / LPR) * p.ldb + (line % LPR) * 64) * 2;
    }
    auto touch = [&](int t) {
      if (t >= nk) return;
      t += k_first;
      if (t >= nk) t -= nk;
#pragma unroll
      for (int h = 0; h < 2; h++)
        if (on[h])
          asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off" : : "s"(sink), "v"(line_at[h] + (int64_t)t * F_BK * p.ldb * 2) : "memory", "m0");
    };
    for (int t = STAGES - 1; t < F_PF_AHEAD; t++) touch(t);
    __syncthreads();  // the others' barrier after the prologue ...
    for (int t = 0; t < nk; t++) {
      touch(t + F_PF_AHEAD);
      __syncthreads();  // ... and the one of every K tile
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));  // the patch of LDS goes away with the workgroup
    return;
  }

  // Wavefront w issues A instructions A_DMA w .. (rows 16 ia + lane / 4) and B instructions B_DMA w .. (k rows
  // B_KROWS ib + lane / B_CHUNKS) of a tile.  Per-lane byte offsets are constant; the tile's base address moves in
  // scalar registers (with gathered rows: per-lane 64-bit addresses that move by one K tile).
  uint32_t a_voff[A_DMA], b_voff[B_DMA];
  const char *a_lane[A_DMA];
#pragma unroll
  for (int i = 0; i < A_DMA; i++) {
    if (AT) {  // as a row-major B: k rows A_KROWS (A_DMA w + i) + lane / A_CHUNKS, chunks of rows past M fetch the last whole chunk (M % 8 == 0)
      const int krow = A_KROWS * (A_DMA * wave + i) + lane / A_CHUNKS;
      const int chunk = min((lane & (A_CHUNKS - 1)) ^ ((krow & 3) << 2), (int)((p.M - m0) / 8 - 1));
      a_voff[i] = (uint32_t)((krow * p.lda + 8 * chunk) * 2);
      continue;
    }
    // rows past M (the last row tile of a ragged problem) fetch row M - 1 again: they only reach outputs nobody stores
    const int row = min(16 * (A_DMA * wave + i) + lane / 4, (int)(p.M - 1 - m0));
    const int chunk = (lane & 3) ^ ((lane >> 4) & 3);
    a_voff[i] = (uint32_t)((row * p.lda + 8 * chunk) * 2);
    if (GATHER) {
      int64_t r = m0 + row;
      if (p.a_rows) r = (p.gather_mul32 & 1) ? (int64_t)(int)((uint32_t)p.a_rows[r] * (uint32_t)p.lda) : (int64_t)p.a_rows[r] * p.lda;
      else r *= p.lda;
      a_lane[i] = (const char *)((const uint16_t *)p.a + r + 8 * chunk);
    }
  }
#pragma unroll
  for (int i = 0; i < B_DMA; i++) {
    if (BT) {  // as A: columns 16 (B_DMA w + i) + lane / 4 of the tile, those past N fetch column N - 1
      const int col = min(16 * (B_DMA * wave + i) + lane / 4, (int)(p.N - 1 - n0));
      b_voff[i] = (uint32_t)((col * p.ldb + 8 * ((lane & 3) ^ ((lane >> 4) & 3))) * 2);
      continue;
    }
    const int krow = B_KROWS * (B_DMA * wave + i) + lane / B_CHUNKS;
    // likewise, chunks of columns past N fetch the last whole chunk of the row (N is a multiple of 8)
    const int chunk = min((lane & (B_CHUNKS - 1)) ^ ((krow & 3) << 2), (int)((p.N - n0) / 8 - 1));
    b_voff[i] = (uint32_t)((krow * p.ldb + 8 * chunk) * 2);
  }
  const char *a_base = (const char *)((const uint16_t *)p.a + (AT ? m0 : m0 * p.lda));
  const uint32_t lds0 = (uint32_t)(uintptr_t)TTS_LDS(smem);
  const uint32_t wave_u = __builtin_amdgcn_readfirstlane(wave);
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
  auto dma_lane = [&](const char *addr, uint32_t lds) {  // every lane its own 64-bit address
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(lds), "v"(addr) : "memory", "m0");
  };
  auto dma_one = [&](int t, int n) {  // n < A_DMA: A part, else B part of tile t, into stage t % STAGES
    int tc = min(t, nk - 1) + k_first;
    if (tc >= nk) tc -= nk;
    tc += k_begin;
    const uint32_t st = lds0 + (t % STAGES) * STAGE_BYTES;
    if (n < A_DMA) {
      const uint32_t at = st + (A_DMA * wave_u + n) * 1024;
      if (GATHER) dma_lane(a_lane[n] + (int64_t)tc * F_BK * 2, at);
      else dma(a_base + (AT ? (int64_t)tc * F_BK * p.lda * 2 : (int64_t)tc * F_BK * 2), a_voff[n], at);
    } else {
      dma(b_base + (BT ? (int64_t)tc * F_BK * 2 : (int64_t)tc * F_BK * p.ldb * 2), b_voff[n - A_DMA], st + A_BYTES + (B_DMA * wave_u + n - A_DMA) * 1024);
    }
  };

  // fragment read offsets (bytes, within a stage)
  // A: row r = wm * TM * 32 + i * 32 + lane % 32, chunk c = 2 ks + lane / 32 at position c ^ ((r / 4) & 3)
  const int ar = wm * TM * 32 + (lane & 31);
  const int a_off = ar * 64, a_sw = (ar >> 2) & 3;
  // B: 16-lane group q = lane / 16, r16 = lane % 16: k row ks * 16 + 8 (q / 2) + 4 h + r16 / 4,
  // chunk wn * TN * 4 + 4 j + 2 (q & 1) + (r16 % 4) / 2, byte 8 (r16 & 1) within the chunk
  const int q = lane >> 4, r16 = lane & 15;
  const int b_chunk = wn * TN * 4 + 2 * (q & 1) + ((r16 & 3) >> 1), b_sw = (r16 >> 2) << 2;
  const int b_off = A_BYTES + (8 * (q >> 1) + (r16 >> 2)) * ROWB + 8 * (r16 & 1);

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  // BT: column c = wn * TN * 32 + j * 32 + lane % 32 of the tile, chunk 2 ks + lane / 32 at position chunk ^ ((c / 4) & 3)
  const int bc = wn * TN * 32 + (lane & 31);
  const int bt_off = A_BYTES + bc * 64, bt_sw = (bc >> 2) & 3;
  // AT: as the row-major B below, with the wavefront's rows in place of its columns
  const int at_chunk = wm * TM * 4 + 2 * (q & 1) + ((r16 & 3) >> 1);
  const int at_off = (8 * (q >> 1) + (r16 >> 2)) * A_ROWB + 8 * (r16 & 1);
  constexpr int A_READS = AT ? 2 * TM : TM, READS = A_READS + (BT ? TN : 2 * TN), MFMAS = TM * TN;
  uint4 af[2][TM], bf[2][TN];
  // one fragment read (n < TM: A row block n; else B column block (n - TM) / 2, k half (n - TM) % 2)
  auto read_one = [&](int t, int ks, int n, uint4 (&a)[TM], uint4 (&b)[TN]) {
    const char *st = smem + (t % STAGES) * STAGE_BYTES;
    if (n < A_READS && AT) {
      const int i = n >> 1, h = n & 1;
      const char *ap = st + at_off + ks * 16 * A_ROWB + (((at_chunk + 4 * i) ^ b_sw) << 4) + h * 4 * A_ROWB;
      s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)TTS_LDS(ap));
      uint2 v2 = __builtin_bit_cast(uint2, v);
      if (h == 0) { a[i].x = v2.x; a[i].y = v2.y; } else { a[i].z = v2.x; a[i].w = v2.y; }
    } else if (n < A_READS) {
      a[n] = *reinterpret_cast<const uint4 *>(st + a_off + n * 2048 + (((2 * ks + (lane >> 5)) ^ a_sw) << 4));
    } else if (BT) {
      b[n - A_READS] = *reinterpret_cast<const uint4 *>(st + bt_off + (n - A_READS) * 2048 + (((2 * ks + (lane >> 5)) ^ bt_sw) << 4));
    } else {
      const int j = (n - A_READS) >> 1, h = (n - A_READS) & 1;
      const char *bp = st + b_off + ks * 16 * ROWB + (((b_chunk + 4 * j) ^ b_sw) << 4) + h * 4 * ROWB;
      s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)TTS_LDS(bp));
      uint2 v2 = __builtin_bit_cast(uint2, v);
      if (h == 0) { b[j].x = v2.x; b[j].y = v2.y; } else { b[j].z = v2.x; b[j].w = v2.y; }
    }
  };
  auto mfma_one = [&](int n, uint4 (&a)[TM], uint4 (&b)[TN]) {
    acc[n / TN][n % TN] = mfma32<BF16>(a[n / TN], b[n % TN], acc[n / TN][n % TN]);
  };
  // A phase: MFMAS matrix instructions, READS fragment reads for the next phase, DMA / 2 loads; they are dealt out
  // behind the matrix instructions as evenly as their numbers allow.
  constexpr int SLOTS = MFMAS > READS ? MFMAS : READS;
  auto phase = [&](uint4 (&a_use)[TM], uint4 (&b_use)[TN], uint4 (&a_next)[TM], uint4 (&b_next)[TN], int t_read, int ks_read, int t_load, int first_load) {
#pragma unroll
    for (int n = 0; n < SLOTS; n++) {
      __builtin_amdgcn_sched_barrier(0);
      if (n < MFMAS) mfma_one(n, a_use, b_use);
      if (n < READS) read_one(t_read, ks_read, n, a_next, b_next);
      constexpr int every = SLOTS / (DMA / 2);
      if (n % every == every - 1 && n / every < DMA / 2) dma_one(t_load, first_load + n / every);
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // prologue: STAGES - 1 tiles in flight; tile 0 landed; its first operands read
  for (int t = 0; t < STAGES - 1; t++)
#pragma unroll
    for (int n = 0; n < DMA; n++) dma_one(t, n);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(DMA * (STAGES - 2), 15));
  __syncthreads();
#pragma unroll
  for (int n = 0; n < READS; n++) read_one(0, 0, n, af[0], bf[0]);
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));
  for (int t = 0; t < nk; t++) {
    // phase A: MFMAs of (tile t, first half); read (tile t, second half); first half of the loads of tile t + STAGES - 1
    phase(af[0], bf[0], af[1], bf[1], t, 1, t + STAGES - 1, 0);
    // own loads of tile t+1 have landed (later ones may be in flight); own reads of tile t are complete
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(DMA * (STAGES - 3) + DMA / 2, 0));
    __syncthreads();
    // phase B: MFMAs of (tile t, second half); read (tile t+1, first half); the rest of the loads
    phase(af[1], bf[1], af[0], bf[0], t + 1, 0, t + STAGES - 1, DMA / 2);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));
  }
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));  // the surplus loads land before the LDS goes away

  // Epilogue.  A lane holds one column of each 32x32 block (rows 8 (v/4) + 4 (lane/32) + v%4 in element v).  Two rows
  // are narrowed at once (v_cvt_pk_bf16_f32 for bf16: round to nearest even, NaNs quieted), the pair is exchanged with
  // the neighbouring lane, and the even lane stores row r at columns (n, n+1), the odd lane row r+1 at (n-1, n):
  // half as many store instructions as one 2-byte store per element, and a handful of VALU ops per pair.
  if constexpr (SK) {
    // the slice's sums as they are: a lane's 32 x 32 block column by column, two rows of 32 consecutive floats per store
    float *__restrict__ part = p.partial + (int64_t)slice * p.M * p.N;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const int64_t col = n0 + wn * TN * 32 + j * 32 + (lane & 31);
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const int64_t row = m0 + wm * TM * 32 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
          if (row < p.M && col < p.N) part[row * p.N + col] = acc[i][j][v];
        }
      }
    return;
  }
  uint16_t *__restrict__ C = (uint16_t *)p.c;
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  const bool odd = lane & 1;
  const uint32_t sel = odd ? 0x03020706u : 0x05040100u;  // odd: high halves of (neighbour, mine); even: low halves of (mine, neighbour)
  // EDGE: the tile sticks out of C (ragged M, or N that is not a multiple of the tile): elements outside are neither
  // evaluated (the functor may read a bias or a residual at the element's position) nor stored.
  auto store_tile = [&](auto edge) {
    constexpr bool EDGE = decltype(edge)::value;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const int64_t col = n0 + wn * TN * 32 + j * 32 + (lane & 31) - (odd ? 1 : 0);
#pragma unroll
        for (int v = 0; v < 16; v += 2) {
          const int64_t er = m0 + wm * TM * 32 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3), ec = n0 + wn * TN * 32 + j * 32 + (lane & 31);
          const bool in0 = !EDGE || (er < p.M && ec < p.N), in1 = !EDGE || (er + 1 < p.M && ec < p.N);
          const f32x2_t pr = {in0 ? ep(acc[i][j][v], er, ec) : 0.f, in1 ? ep(acc[i][j][v + 1], er + 1, ec) : 0.f};
          const uint32_t pk = BF16 ? __builtin_bit_cast(uint32_t, __builtin_convertvector(pr, bf16x2_t))
                                   : __builtin_bit_cast(uint32_t, __builtin_convertvector(pr, f16x2_t));
          const uint32_t nb = __builtin_amdgcn_mov_dpp(pk, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]: the neighbour's pair
          const uint32_t w = __builtin_amdgcn_perm(nb, pk, sel);
          const int64_t row = m0 + wm * TM * 32 + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3) + (odd ? 1 : 0);
          if (!EDGE || (row < p.M && col < p.N)) __builtin_nontemporal_store(w, reinterpret_cast<uint32_t *>(&C[row * p.ldc + col]));
        }
      }
  };
  if (m0 + BM > p.M || n0 + BN > p.N) store_tile(EdgeTile<true>());
  else store_tile(EdgeTile<false>());
}


// ------------------------- the 256 x 256 tile on v_mfma_f32_16x16x32 (row-major operands, whole K tiles)
// The same tile, the same ring of four direct-to-LDS stages and the same A swizzle as gemm_dma_body<4, 4>, with the matrix
// instruction of shape 16 x 16 x 32 instead of 32 x 32 x 16.  Under the board's power limit the time of a large product is the
// energy it dissipates, and on operands of the prescribed distribution the 16 x 16 x 32 instruction sustains 0.79 of the
// peak rate from registers where 32 x 32 x 16 sustains 0.70 to 0.73 (measured with no data movement at all; on all-zero
// operands both reach 0.90); LDS and global traffic per flop are the same for both.  4096^3: 101-104 us against 104-110 for
// the 32 x 32 x 16 body in the same runs, bit for bit the same result.
//
// A wavefront's 128 x 128 part of C is 8 x 8 blocks of 16 x 16, four accumulator registers each, held transposed (the B
// operand goes in as the instruction's first source): a lane holds four consecutive columns of one row, which the epilogue
// can narrow and pack without cross-lane moves.  One K tile of 32 is one instruction's depth.
//   A operand of row block i: row 16 i + lane % 16, k 8 (lane / 16) .. +7: one 16-byte LDS read (A's swizzle is chosen
//     for the order in which such a read serves its lanes: see a_swizzle).
//   B operand of column block j: `ds_read_b64_tr_b16` twice (k 0-3 and 4-7 of the lane's octet), lane r of a 16-lane group
//     addressing k row 8 (lane / 16) + r / 4, columns 4 (r % 4) .. +3 of the block.  Two k octets share a half wavefront, so
//     the stage's swizzle also flips chunk bit 1 with k bit 3: position q of k row k holds chunk q ^ ((k & 3) << 2) ^ (((k >> 3) & 1) << 1).
// Phases of a tile t: (0) the 32 products of column blocks 0-3, with the eight reads of B blocks 4-7 of tile t and half of
// the loads of tile t + 3 behind them; wait for the own loads of tile t + 1, barrier; (1) the 32 products of column blocks
// 4-7, with the reads of all of A (8) and of B blocks 0-3 (8) of tile t + 1 and the other half of the loads.  A's operands
// alternate between two register sets (the K loop is unrolled by two), B's blocks 0-3 and 4-7 each have one.
// The matrix instruction is issued from inline assembly, in place on the accumulation registers: left to the register
// allocator (the instruction's result may overlap its addend arbitrarily, so nothing ties them) the 64 accumulators rotate
// through both register files and are copied back at the loop's end, 520 moves per two tiles.
// Epilogue: every wavefront narrows 16 rows at a time into a patch of LDS of its own (the stages are free by then) and
// stores whole 256-byte row segments with 16-byte nontemporal stores: 33.5 MB written for 33.5 MB of C where 4-byte
// stores of 64-byte segments wrote 51 MB.
// Loops over compile-time indices, and every lambda of the body below is marked always_inline: the accumulators and
// operand registers must become registers whatever the size of the epilogue functor.  (With a functor of a few hundred
// operations the inliner left the epilogue's lambda out of line, the accumulators, passed to it by reference, lived in
// scratch memory, and the compiler read them right behind matrix instructions it had not seen being issued.)
template <int V>
struct IntConstant {
  static constexpr int value = V;
};
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
  if constexpr (I < N) {
    f(IntConstant<I>());
    static_for<I + 1, N>(f);
  }
}

// SK: the grid holds p.split workgroups per tile; workgroup (tile, s) walks the s-th share of the K tiles and leaves its fp32
// sums in p.partial (a lane's four consecutive columns of a row are one 16-byte store, straight from the registers).
template <bool BF16, class Ep, bool SK = false>
__device__ __forceinline__ void gemm_dma16_body(const GemmParams &p, int tiles_m, int tiles_n, const Ep &ep) {
  using T = DmaTile<4, 4>;
  constexpr int BM = T::BM, BN = T::BN, STAGES = T::STAGES, A_BYTES = T::A_BYTES, STAGE_BYTES = T::STAGE_BYTES, ROWB = T::B_ROW_BYTES;
  constexpr int A_DMA = T::A_DMA, B_DMA = T::B_DMA, DMA = T::DMA;
  static_assert(A_DMA == 4 && B_DMA == 4 && ROWB == 512, "256 x 256 x 32 stages");
#ifdef TTS_GEMM_RTC
  __shared__ __align__(16) char dma_smem[T::LDS_BYTES];
#else
  extern __shared__ __align__(16) char dma_smem[];
#endif
  char *smem = dma_smem;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  int bid = blockIdx.x;
  const int nwg = tiles_m * tiles_n;
  const int slice = SK ? bid / nwg : 0;
  if (SK) bid -= slice * nwg;
  if (nwg % 8 == 0) bid = (bid % 8) * (nwg / 8) + bid / 8;  // consecutive ids on one XCD
  const int group = 4 * tiles_n;                             // 4-tile-tall column groups
  const int g0 = (bid / group) * 4;
  const int gh = min(tiles_m - g0, 4);
  const int tile_m = g0 + (bid % group) % gh, tile_n = (bid % group) / gh;
  const int64_t m0 = (int64_t)tile_m * BM, n0 = (int64_t)tile_n * BN;
  const char *a_base = (const char *)((const uint16_t *)p.a + m0 * p.lda);
  const char *b_base = (const char *)((const uint16_t *)p.b + n0);
  const int nk_all = (int)(p.K / F_BK);
  const int k_begin = SK ? (int)((int64_t)slice * nk_all / p.split) : 0;
  const int nk = SK ? (int)((int64_t)(slice + 1) * nk_all / p.split) - k_begin : nk_all;

  // A's swizzle: position q of row r holds chunk q ^ a_swizzle((r / 4) & 3).  A 16-byte LDS read serves sixteen lanes per
  // cycle, and not sixteen neighbours: lanes 0-3 go with 12-15, 20-23 and 24-27 (of the eight quads of a half wavefront,
  // those whose number has an even count of set bits, then the others; found by letting two lanes alone read one bank).
  // With this instruction's operand layout (lane l: row l % 16, chunk l / 16) such a cycle holds row quads 0 and 3 of one
  // chunk and 1 and 2 of the next, and the swizzle (0, 2, 3, 1) puts the four into different banks; the plain
  // (r / 4) & 3 of the 32 x 32 x 16 body, conflict-free for that body's layout, made every A read here take twice its cycles.
  auto a_swizzle = [](int row_quad) __attribute__((always_inline)) { return ((row_quad >> 1) & 1) | (((row_quad & 1) ^ ((row_quad >> 1) & 1)) << 1); };
  uint32_t a_voff[A_DMA], b_voff[B_DMA];
#pragma unroll
  for (int i = 0; i < A_DMA; i++) {
    // rows past M (the last row tile of a ragged problem) fetch row M - 1 again: they only reach outputs nobody stores
    const int row = min(16 * (A_DMA * wave + i) + lane / 4, (int)(p.M - 1 - m0));
    const int chunk = (lane & 3) ^ a_swizzle((lane >> 4) & 3);
    a_voff[i] = (uint32_t)((row * p.lda + 8 * chunk) * 2);
  }
#pragma unroll
  for (int i = 0; i < B_DMA; i++) {
    const int krow = 2 * (B_DMA * wave + i) + lane / 32;
    // likewise, chunks of columns past N fetch the last whole chunk of the row (N is a multiple of 8)
    const int chunk = min((lane & 31) ^ ((krow & 3) << 2) ^ (((krow >> 3) & 1) << 1), (int)((p.N - n0) / 8 - 1));
    b_voff[i] = (uint32_t)((krow * p.ldb + 8 * chunk) * 2);
  }
  const uint32_t lds0 = (uint32_t)(uintptr_t)TTS_LDS(smem);
  const uint32_t wave_u = __builtin_amdgcn_readfirstlane(wave);
  auto dma = [&](const char *sbase, uint32_t voff, uint32_t lds) __attribute__((always_inline)) {
#ifdef TTS_GEMM_RTC
    // (an older run-time compiler does not see that the tile's base address is the same in every lane: say so)
    const uint64_t b = (uint64_t)(uintptr_t)sbase;
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    sbase = (const char *)(uintptr_t)(((uint64_t)hi << 32) | (uint64_t)lo);
#endif
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds), "v"(voff), "s"(sbase) : "memory", "m0");
  };
  // n < A_DMA: A part, else B part of tile t, into stage t % STAGES.  Loads past the last tile fetch the last tile again, so
  // that the wait count is the same in every iteration (a scalar branch around every load and between two waits instead
  // cost 5 us of 110: sixteen branches per tile in between the matrix instructions).
  auto dma_one = [&](int t, int n) __attribute__((always_inline)) {
    const int tc = min(t, nk - 1) + k_begin;
    const uint32_t st = lds0 + (t % STAGES) * STAGE_BYTES;
    if (n < A_DMA) dma(a_base + (int64_t)tc * F_BK * 2, a_voff[n], st + (A_DMA * wave_u + n) * 1024);
    else dma(b_base + (int64_t)tc * F_BK * p.ldb * 2, b_voff[n - A_DMA], st + A_BYTES + (B_DMA * wave_u + n - A_DMA) * 1024);
  };

  const int l16 = lane & 15, q = lane >> 4;
  const int a_off = (wm * 128 + l16) * 64 + ((q ^ a_swizzle((l16 >> 2) & 3)) << 4);
  const int b_sw = ((l16 >> 2) << 2) ^ ((q & 1) << 1);
  const int b_chunk = wn * 16 + ((l16 & 3) >> 1);
  const int b_off = A_BYTES + (8 * q + (l16 >> 2)) * ROWB + 8 * (l16 & 1);

  f32x4 acc[8][8];
  static_for<0, 64>([&](auto n) __attribute__((always_inline)) { acc[n.value / 8][n.value % 8] = (f32x4){0.f, 0.f, 0.f, 0.f}; });
  uint4 A[2][8], B0[4], B1[4];
  auto read_a = [&](int t, int i, uint4 (&a)[8]) {
    a[i] = *reinterpret_cast<const uint4 *>(smem + (t % STAGES) * STAGE_BYTES + a_off + i * 1024);
  };
  auto read_b = [&](int t, int j, int h, uint4 &b) __attribute__((always_inline)) {  // column block j of the wavefront's eight, k half h of the lane's octet
    const char *bp = smem + (t % STAGES) * STAGE_BYTES + b_off + h * 4 * ROWB + (((b_chunk + 2 * j) ^ b_sw) << 4);
    s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3))) *)TTS_LDS(bp));
    uint2 v2 = __builtin_bit_cast(uint2, v);
    if (h == 0) { b.x = v2.x; b.y = v2.y; } else { b.z = v2.x; b.w = v2.y; }
  };
  typedef uint32_t u32x4_r __attribute__((ext_vector_type(4)));
  auto mfma16 = [&](int i, int j, const uint4 &a, const uint4 &b) __attribute__((always_inline)) {
    if constexpr (BF16)
      asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(__builtin_bit_cast(u32x4_r, b)), "v"(__builtin_bit_cast(u32x4_r, a)));
    else
      asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(__builtin_bit_cast(u32x4_r, b)), "v"(__builtin_bit_cast(u32x4_r, a)));
  };
  auto tile = [&](int t, uint4 (&Ac)[8], uint4 (&An)[8]) __attribute__((always_inline)) {
    static_for<0, 32>([&](auto slot) __attribute__((always_inline)) {
      constexpr int n = decltype(slot)::value;
      __builtin_amdgcn_sched_barrier(0);
      mfma16(n >> 2, n & 3, Ac[n >> 2], B0[n & 3]);
      if constexpr (n < 8) read_b(t, 4 + (n >> 1), n & 1, B1[n >> 1]);
      if constexpr (n % 8 == 7) dma_one(t + STAGES - 1, n / 8);
    });
    __builtin_amdgcn_sched_barrier(0);
    // own loads of tile t + 1 have landed (later ones may be in flight); own reads of tile t are complete
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(DMA * (STAGES - 3) + DMA / 2, 0));
    __syncthreads();
    static_for<0, 32>([&](auto slot) __attribute__((always_inline)) {
      constexpr int n = decltype(slot)::value;
      __builtin_amdgcn_sched_barrier(0);
      mfma16(n >> 2, 4 + (n & 3), Ac[n >> 2], B1[n & 3]);
      if constexpr (n < 8) read_a(t + 1, n, An);
      else if constexpr (n < 16) read_b(t + 1, (n - 8) >> 1, n & 1, B0[(n - 8) >> 1]);
      if constexpr (n % 8 == 7) dma_one(t + STAGES - 1, 4 + n / 8);
    });
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));
  };

  // prologue: STAGES - 1 tiles in flight; tile 0 landed; its first operands read
  for (int t = 0; t < STAGES - 1; t++) static_for<0, DMA>([&](auto n) __attribute__((always_inline)) { dma_one(t, n.value); });
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(DMA * (STAGES - 2), 15));
  __syncthreads();
  static_for<0, 8>([&](auto i) __attribute__((always_inline)) { read_a(0, i.value, A[0]); });
  static_for<0, 4>([&](auto j) __attribute__((always_inline)) {
    read_b(0, j.value, 0, B0[j.value]);
    read_b(0, j.value, 1, B0[j.value]);
  });
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0));
  int t = 0;
  for (; t + 1 < nk; t += 2) {  // two tiles per turn: A's register sets take turns
    tile(t, A[0], A[1]);
    tile(t + 1, A[1], A[0]);
  }
  if (t < nk) tile(t, A[0], A[1]);
  // The compiler does not know that the assembly above issued matrix instructions, so it leaves no wait states between
  // one of them and a read of its result (the epilogue's, or a spill the register allocator places right behind the
  // loop).  The sixteen accumulators the last tile wrote last pass through this statement, so whatever reads them comes
  // after its wait states; the others were written at least sixteen instructions (256 cycles) earlier.
  asm volatile("s_nop 15\n\ts_nop 15"
               : "+a"(acc[4][4]), "+a"(acc[4][5]), "+a"(acc[4][6]), "+a"(acc[4][7]), "+a"(acc[5][4]), "+a"(acc[5][5]), "+a"(acc[5][6]), "+a"(acc[5][7]),
                 "+a"(acc[6][4]), "+a"(acc[6][5]), "+a"(acc[6][6]), "+a"(acc[6][7]), "+a"(acc[7][4]), "+a"(acc[7][5]), "+a"(acc[7][6]), "+a"(acc[7][7])
               :
               : "memory");
  // Every wavefront has read its last operands: the last tile's stage is free.  The other three still receive the surplus
  // loads of the last iterations, which nobody waits for before the kernel's end.
  __syncthreads();

  // acc[i][j][v] is C(row 16 i + lane % 16, column 16 j + 4 (lane / 16) + v) of the wavefront's part
  if constexpr (SK) {
    float *__restrict__ part = p.partial + (int64_t)slice * p.M * p.N;
    static_for<0, 64>([&](auto bc) __attribute__((always_inline)) {
      constexpr int i = decltype(bc)::value / 8, j = decltype(bc)::value % 8;
      const int64_t row = m0 + wm * 128 + i * 16 + l16, col = n0 + wn * 128 + j * 16 + 4 * q;
      if (row < p.M && col < p.N) *reinterpret_cast<f32x4 *>(part + row * p.N + col) = acc[i][j];  // (N is a multiple of 8)
    });
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));  // the surplus loads land before the LDS goes away
    return;
  }
  uint16_t *__restrict__ C = (uint16_t *)p.c;
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  constexpr int PITCH = 272;  // bytes per staged row of 128 columns
  // (one patch of 16 rows per wavefront, in the last tile's stage; a wavefront's LDS accesses complete in order, so the
  // next 16 rows' writes come after this 16 rows' reads)
  static_assert(4 * 16 * PITCH <= STAGE_BYTES, "the four wavefronts' patches fit one stage");
  char *mine = smem + ((nk + STAGES - 1) % STAGES) * STAGE_BYTES + wave * (16 * PITCH);
  // A fused epilogue evaluates the stored value with the ids of the Triton program that owns the element (Ep::BM x Ep::BN
  // blocks; 0: no functor).  Blocks of 16 x 16 never straddle two owners, and a wavefront's 128 x 128 part has GI x GJ of
  // them: they are looked up once each, and what the functor computes from the program's ids alone is then the same
  // expression on the same values for every element of an owner, which the compiler evaluates once.  (Looked up per
  // element, every one of the 256 evaluations per lane is separate code: a functor with the tutorial's grouped tile
  // order and a bias per row and column took eight minutes to compile.)
  constexpr int EBM = Ep::BM, EBN = Ep::BN;
  constexpr bool OWNED = EBM >= 16 && EBN >= 16 && (128 % EBM == 0 || EBM % 128 == 0) && (128 % EBN == 0 || EBN % 128 == 0);
  constexpr int GI = OWNED && EBM < 128 ? 128 / EBM : 1, GJ = OWNED && EBN < 128 ? 128 / EBN : 1;
  int owner[GI][GJ];
  if constexpr (OWNED)
    static_for<0, GI * GJ>([&](auto gc) __attribute__((always_inline)) {
      constexpr int gi = decltype(gc)::value / GJ, gj = decltype(gc)::value % GJ;
      const int64_t r0 = m0 + wm * 128 + gi * (128 / GI), c0 = n0 + wn * 128 + gj * (128 / GJ);
      owner[gi][gj] = (r0 < p.M && c0 < p.N) ? ep.tile_pid[(r0 / EBM) * ep.tiles_n + c0 / EBN] : 0;  // (outside C: nobody's)
    });
  auto value = [&](auto ic, auto jc, float a, int64_t row, int64_t col) __attribute__((always_inline)) -> float {
    if constexpr (OWNED) return ep.at(owner[decltype(ic)::value * 16 / (128 / GI)][decltype(jc)::value * 16 / (128 / GJ)], a, (int)(row % EBM), (int)(col % EBN));
    else return ep(a, row, col);
  };
  // this lane's chunk of row lane / 16 of the wavefront's part
  uint16_t *c_lane = C + (m0 + wm * 128 + (lane >> 4)) * p.ldc + n0 + wn * 128 + (lane & 15) * 8;
  auto store_tile = [&](auto edge) __attribute__((always_inline)) {
    // EDGE: the tile sticks out of C (ragged M, or N that is not a multiple of the tile): elements outside are neither
    // evaluated (the functor may read a bias or a residual at the element's position) nor stored.
    constexpr bool EDGE = decltype(edge)::value;
    // rows and columns of the wavefront's part that lie inside C (N is a multiple of 8: a lane's four columns, and a
    // stored chunk's eight, are inside or outside together)
    const int rows_left = (int)min((int64_t)128, p.M - (m0 + wm * 128)), cols_left = (int)min((int64_t)128, p.N - (n0 + wn * 128));
    static_for<0, 8>([&](auto ic) __attribute__((always_inline)) {
      constexpr int i = decltype(ic)::value;
      char *reg = mine;
      const int64_t er = m0 + wm * 128 + i * 16 + l16;
      const bool row_in = !EDGE || i * 16 + l16 < rows_left;
      static_for<0, 8>([&](auto jc) __attribute__((always_inline)) {
        constexpr int j = decltype(jc)::value;
        const int64_t ec = n0 + wn * 128 + j * 16 + 4 * q;
        const bool in = !EDGE || (row_in && j * 16 + 4 * q < cols_left);
        float o[4];
        static_for<0, 4>([&](auto vc) __attribute__((always_inline)) {
          constexpr int v = decltype(vc)::value;
          o[v] = in ? value(ic, jc, acc[i][j][v], er, ec + v) : 0.f;
        });
        const f32x2_t p01 = {o[0], o[1]}, p23 = {o[2], o[3]};
        uint2 w;
        if (BF16) {
          w.x = __builtin_bit_cast(uint32_t, __builtin_convertvector(p01, bf16x2_t));
          w.y = __builtin_bit_cast(uint32_t, __builtin_convertvector(p23, bf16x2_t));
        } else {
          w.x = __builtin_bit_cast(uint32_t, __builtin_convertvector(p01, f16x2_t));
          w.y = __builtin_bit_cast(uint32_t, __builtin_convertvector(p23, f16x2_t));
        }
        *reinterpret_cast<uint2 *>(reg + l16 * PITCH + (j * 16 + 4 * q) * 2) = w;
      });
      // (a wavefront's LDS accesses complete in order: its reads below see its writes above)
      uint4 chunk[4];
      static_for<0, 4>([&](auto kc) __attribute__((always_inline)) {
        constexpr int k = decltype(kc)::value;
        chunk[k] = *reinterpret_cast<const uint4 *>(reg + (4 * k + (lane >> 4)) * PITCH + (lane & 15) * 16);
      });
      static_for<0, 4>([&](auto kc) __attribute__((always_inline)) {
        constexpr int k = decltype(kc)::value;
        const int row = 4 * k + (lane >> 4), ch = lane & 15;  // row of the sixteen, 16-byte chunk of the row
        // (rows of C need only be 4-byte aligned: a store of four dwords wants dword alignment, no more)
        typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
        const u32x4_a4 w = {chunk[k].x, chunk[k].y, chunk[k].z, chunk[k].w};
        if (!EDGE || (i * 16 + row < rows_left && ch * 8 < cols_left))
          __builtin_nontemporal_store(w, reinterpret_cast<u32x4_a4 *>(c_lane + (int64_t)(i * 16 + 4 * k) * p.ldc));
      });
    });
  };
  if (m0 + BM > p.M || n0 + BN > p.N) store_tile(EdgeTile<true>());
  else store_tile(EdgeTile<false>());
  __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 15));  // the surplus loads land before the LDS goes away
}

}  // namespace tts_gemm_device

#ifdef TTS_GEMM_RTC
extern "C" __global__ __launch_bounds__(256) void gemm_rtc(TtsGemmParams p, int tiles_m, int tiles_n, TtsEp ep) {
#if TTS_GEMM_RTC == 0
  tts_gemm_device::gemm_dma16_body<TTS_GEMM_BF16 != 0>(p, tiles_m, tiles_n, ep);
#else
  tts_gemm_device::gemm_mfma_body<TTS_GEMM_BF16 != 0, 2, 2, 64>(p, tiles_m, tiles_n, ep);
#endif
}
#endif
