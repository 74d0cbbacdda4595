// Memory-bound kernel families for gfx950: masked 1-D elementwise map, row
// softmax, LayerNorm forward.  One Triton program maps to one workgroup (map1d,
// layernorm) or one wavefront (softmax); every kernel covers the whole grid in
// one launch.
//
// What they replace in the reference CPU path, per program: a malloc'd tile per
// masked load filled with `other` and a partial element-wise copy
// (StructuredToMemref.cpp:794-853, CRunnerUtils.cpp:58-113), one scalar loop
// nest per linalg op with a full-tile temporary in between, sequential
// reductions (ConversionPatterns.hpp:1395-1407), and a partial copy back
// (StructuredToMemref.cpp:1163-1196).  Here a tile lives in registers, masking is
// a per-lane predicate derived from the same valid extent, and the elementwise
// ops are fused.  Compiled with -ffp-contract=off: the reference requests no
// FMA contraction and no fast-math (backend/compiler.py:127-129,172-173).
#include "kernels.h"

#include <type_traits>

namespace tts {

namespace {

constexpr int WAVE = 64;

__device__ __forceinline__ int64_t affine(const Affine &a, int px, int py, int pz) {
  return a.c0 + a.c[0] * px + a.c[1] * py + a.c[2] * pz;
}

// The program a workgroup runs.  The device's grid holds 65535 along y and z, the reference's launcher loops over any
// extents (backend/driver.py:116-133): for such grids the launch is one-dimensional and the kernel numbers the programs
// itself, x fastest (lin_gx != 0).
struct ProgramId {
  int x, y, z;
};
__device__ __forceinline__ ProgramId program_id(int lin_gx, int lin_gy) {
  if (!lin_gx) return {(int)blockIdx.x, (int)blockIdx.y, (int)blockIdx.z};
  const int64_t lin = blockIdx.x;
  return {(int)(lin % lin_gx), (int)((lin / lin_gx) % lin_gy), (int)(lin / ((int64_t)lin_gx * lin_gy))};
}
// the launch grid for gx x gy x gz programs (and what the kernel needs to number them)
template <class P>
dim3 program_grid(P &p, int gx, int gy, int gz) {
  if (gy <= 65535 && gz <= 65535) return dim3(gx, gy, gz);
  p.lin_gx = gx;
  p.lin_gy = gy;
  return dim3((unsigned)((int64_t)gx * gy * gz));
}

// Wavefront reductions with DPP cross-lane operands (no LDS round trips): quad swaps, half-row and
// row mirrors leave every lane of a 16-lane row with the row's result; row_bcast15 / row_bcast31 fold
// the four rows into lane 63, which is then broadcast.  Lanes a step does not write take the
// reduction's identity.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float v, float identity) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(identity), __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}
__device__ __forceinline__ float lane63(float v) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63)); }

__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_move<0xB1, 0xf>(v, 0.f);   // quad_perm [1,0,3,2]
  v += dpp_move<0x4E, 0xf>(v, 0.f);   // quad_perm [2,3,0,1]
  v += dpp_move<0x141, 0xf>(v, 0.f);  // row_half_mirror
  v += dpp_move<0x140, 0xf>(v, 0.f);  // row_mirror
  v += dpp_move<0x142, 0xa>(v, 0.f);  // row_bcast15 into rows 1 and 3
  v += dpp_move<0x143, 0xc>(v, 0.f);  // row_bcast31 into rows 2 and 3
  return lane63(v);
}
template <bool NAN_PROP>
__device__ __forceinline__ float fmax_sel(float a, float b) {
  if (NAN_PROP) return (a != a || b != b) ? __builtin_nanf("") : fmaxf(a, b);
  return fmaxf(a, b);  // arith.maxnumf: a NaN operand loses
}
template <bool NAN_PROP>
__device__ __forceinline__ float wave_max(float v) {
  v = fmax_sel<NAN_PROP>(v, dpp_move<0xB1, 0xf>(v, -INFINITY));
  v = fmax_sel<NAN_PROP>(v, dpp_move<0x4E, 0xf>(v, -INFINITY));
  v = fmax_sel<NAN_PROP>(v, dpp_move<0x141, 0xf>(v, -INFINITY));
  v = fmax_sel<NAN_PROP>(v, dpp_move<0x140, 0xf>(v, -INFINITY));
  v = fmax_sel<NAN_PROP>(v, dpp_move<0x142, 0xa>(v, -INFINITY));
  v = fmax_sel<NAN_PROP>(v, dpp_move<0x143, 0xc>(v, -INFINITY));
  return lane63(v);
}

// ------------------------------------------------------------------ map1d
template <int OP>
__device__ __forceinline__ float apply(float a, float b) {
  if (OP == 0) return a + b;
  if (OP == 1) return a - b;
  if (OP == 2) return a * b;
  if (OP == 3) return a / b;
  if (OP == 4) return (a != a || b != b) ? __builtin_nanf("") : fmaxf(a, b);
  return (a != a || b != b) ? __builtin_nanf("") : fminf(a, b);
}

typedef float f32x4_t __attribute__((ext_vector_type(4)));
// Outputs are written once and not read again by the kernel: nontemporal stores keep them from
// displacing the inputs in L2 / Infinity Cache (LayerNorm [4096, 8192]: 29.2 -> 27.4 us from HBM,
// 23.3 -> 21.3 us with the input cached).  Nontemporal loads: nothing gained for LayerNorm and softmax (and the cached
// case lost), 4 % for the two-input map at N = 2^28 and 7 % for the int8 weight stream, which use them.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void ntstore(uint4 *p, uint4 v) {
  u32x4_t w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, reinterpret_cast<u32x4_t *>(p));
}
__device__ __forceinline__ void ntstore(float4 *p, float4 v) {
  f32x4_t w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, reinterpret_cast<f32x4_t *>(p));
}

template <int OP, bool SWAP>
__global__ __launch_bounds__(256) void map1d_f32_kernel(Map1DParams p) {
  const ProgramId id = program_id(p.lin_gx, p.lin_gy);
  const int px = id.x, py = id.y, pz = id.z;
  const float *__restrict__ x = p.x + affine(p.xo, px, py, pz);
  const float *__restrict__ y = p.y + affine(p.yo, px, py, pz);
  float *__restrict__ z = p.z + affine(p.zo, px, py, pz);
  int d = p.block;
  if (p.masked) {
    int64_t left = p.bound - affine(p.m_start, px, py, pz);
    d = left < 0 ? 0 : left < p.block ? (int)left : p.block;
  }
  const bool vec = (((uintptr_t)x | (uintptr_t)y | (uintptr_t)z) & 15) == 0;
  for (int i = threadIdx.x * 4; i < d; i += 256 * 4) {
    if (vec && i + 4 <= d) {
      const f32x4_t av = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(x + i));  // read once: no need to keep them cached
      const f32x4_t bv = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t *>(y + i));
      const float4 a = make_float4(av[0], av[1], av[2], av[3]), b = make_float4(bv[0], bv[1], bv[2], bv[3]);
      float4 r;
      if (SWAP) {
        r.x = apply<OP>(b.x, a.x); r.y = apply<OP>(b.y, a.y); r.z = apply<OP>(b.z, a.z); r.w = apply<OP>(b.w, a.w);
      } else {
        r.x = apply<OP>(a.x, b.x); r.y = apply<OP>(a.y, b.y); r.z = apply<OP>(a.z, b.z); r.w = apply<OP>(a.w, b.w);
      }
      ntstore(reinterpret_cast<float4 *>(z + i), r);
    } else {
      for (int j = i; j < i + 4 && j < d; j++) z[j] = SWAP ? apply<OP>(y[j], x[j]) : apply<OP>(x[j], y[j]);
    }
  }
}

template <int OP>
hipError_t launch_map1d_op(const Map1DParams &p, dim3 grid, hipStream_t s) {
  if (p.swap) hipLaunchKernelGGL((map1d_f32_kernel<OP, true>), grid, dim3(256), 0, s, p);
  else hipLaunchKernelGGL((map1d_f32_kernel<OP, false>), grid, dim3(256), 0, s, p);
  return hipGetLastError();
}

// fp16 / bf16 <-> fp32 (narrowing rounds to nearest even, as arith.truncf)
template <bool BF16>
struct Half;
template <>
struct Half<false> {
  static __device__ __forceinline__ float up(uint16_t h) {
    _Float16 f;
    __builtin_memcpy(&f, &h, 2);
    return (float)f;
  }
  static __device__ __forceinline__ uint16_t down(float f) {  // arith.truncf, round to nearest even
    _Float16 h = (_Float16)f;
    uint16_t r;
    __builtin_memcpy(&r, &h, 2);
    return r;
  }
};
template <>
struct Half<true> {
  static __device__ __forceinline__ float up(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }
  static __device__ __forceinline__ uint16_t down(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // NaN stays NaN
    u += 0x7fffu + ((u >> 16) & 1);
    return (uint16_t)(u >> 16);
  }
};

__device__ __forceinline__ float block_sum_256(float v, float *red) {
  v = wave_sum(v);
  __syncthreads();  // red may still be read from the previous use
  if (threadIdx.x % WAVE == 0) red[threadIdx.x / WAVE] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

// ---------------------------------------------------------------- softmax
// T threads share one row; thread t holds elements t, t+T, ... (NPL of them).
// VEC (block == NPL * T, NPL % 4 == 0, d_in >= 4): thread t holds the four-element chunks t, t+T, ...
// of a grid laid on the 16-byte boundaries of memory instead, and moves each with one aligned 16-byte
// access (the grid starts up to three elements before the row; see the loads below).
typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

// IO: the element type of the rows in memory (0 fp16, 1 bf16, 2 fp32); a 16-bit row is widened after the load and narrowed
// before the store, as its Triton source does, and its VEC path moves whole 16-byte chunks of eight elements (the
// launcher picks it for rows that are multiples of 8 elements long and start 16-byte aligned).
template <int NPL, int WAVES, bool NAN_PROP, bool VEC, int WG = 256, int IO = 2>
__global__ __launch_bounds__(WG) void softmax_f32_kernel(SoftmaxParams p, int gx, int gy, int64_t programs) {
  using E = typename std::conditional<IO == 2, float, uint16_t>::type;
  auto up = [](E e) -> float {
    if constexpr (IO == 2) return e;
    else return Half<IO == 1>::up(e);
  };
  auto down = [](float f) -> E {
    if constexpr (IO == 2) return f;
    else return Half<IO == 1>::down(f);
  };
  static_assert(WAVES == 1 || WG == WAVES * WAVE, "rows that span wavefronts meet in red[], one row per workgroup");
  constexpr int T = WAVES * WAVE;
  constexpr int ROWS_PER_WG = WG / T;
  __shared__ float red[WAVES];
  const int sub = threadIdx.x / T, t = threadIdx.x % T;
  const int64_t prog = (int64_t)blockIdx.x * ROWS_PER_WG + sub;
  const bool active = prog < programs;
  int px = 0, py = 0, pz = 0;
  if (active) {
    if (gy == 1 && programs == gx) px = (int)prog;  // 1-D grid: no divisions
    else { px = (int)(prog % gx); py = (int)((prog / gx) % gy); pz = (int)(prog / ((int64_t)gx * gy)); }
  }
  const E *__restrict__ in = (const E *)p.in + affine(p.in_off, px, py, pz);
  E *__restrict__ out = (E *)p.out + affine(p.out_off, px, py, pz);
  const int d_in = active ? (int)p.d_in : 0, d_out = active ? (int)p.d_out : 0;
  // fp32 rows moved in 16-byte chunks: elements between the 16-byte boundary at or below the row's start and the row
  const int lead = (VEC && IO == 2 && active) ? (int)(((uintptr_t)in >> 2) & 3) : 0;
  // lanes beyond d_in hold `other` and take part in the reductions, as a filled
  // tile does; lanes beyond the block do not exist
  float v[NPL];
  if constexpr (VEC && IO != 2) {
    // thread t holds the eight-element chunks t, t+T, ...; a chunk is whole or absent (an absent one reads the row's start)
#pragma unroll
    for (int j = 0; j < NPL / 8; j++) {
      const int i0 = 8 * (t + j * T);
      const bool present = i0 < d_in;
      const uint4 raw = *reinterpret_cast<const uint4 *>(in + (present ? i0 : 0));
      const uint32_t q[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int k = 0; k < 4; k++) {
        v[8 * j + 2 * k] = present ? up((uint16_t)(q[k] & 0xffff)) : p.other;
        v[8 * j + 2 * k + 1] = present ? up((uint16_t)(q[k] >> 16)) : p.other;
      }
    }
  } else if constexpr (VEC) {
    // The chunk grid lies on 16-byte boundaries of memory: it starts `lead` elements before the row (rows of 781 floats are
    // 3124 bytes apart, so a row starts 0, 4, 8 or 12 bytes past a boundary), every chunk is one aligned 16-byte load, and
    // chunks past the row's end are not loaded at all.  Slots outside the row -- before its first element, after its last
    // -- hold `other`: together they are the block's padding, block - d_in slots, as in a filled tile.  (The bytes read
    // before the row and after it lie in the same aligned 16 bytes as an element of the row, so they are mapped.)
    const f32x4_t *grid = reinterpret_cast<const f32x4_t *>(in - lead);
    const int slots = lead + d_in;
    f32x4_t win[NPL / 4];
#pragma unroll
    for (int j = 0; j < NPL / 4; j++) {
      win[j] = (f32x4_t){p.other, p.other, p.other, p.other};
      if (4 * (t + j * T) < slots) win[j] = grid[t + j * T];
    }
#pragma unroll
    for (int j = 0; j < NPL / 4; j++) {
      const int s0 = 4 * (t + j * T);
#pragma unroll
      for (int c = 0; c < 4; c++) v[4 * j + c] = (s0 + c >= lead && s0 + c < slots) ? win[j][c] : p.other;
    }
  } else {
#pragma unroll
    for (int j = 0; j < NPL; j++) {
      int i = t + j * T;
      v[j] = i < d_in ? up(in[i]) : p.other;
    }
  }
  float m = -INFINITY;
#pragma unroll
  for (int j = 0; j < NPL; j++)
    if (VEC || t + j * T < p.block) m = fmax_sel<NAN_PROP>(m, v[j]);
  m = wave_max<NAN_PROP>(m);
  if (WAVES > 1) {
    if (t % WAVE == 0) red[t / WAVE] = m;
    __syncthreads();
    m = red[0];
#pragma unroll
    for (int w = 1; w < WAVES; w++) m = fmax_sel<NAN_PROP>(m, red[w]);
    __syncthreads();
  }
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < NPL; j++) {
    // exp through the hardware exp2 (1 ulp) of a product rounded once: relative error below 1e-5
    // even at the smallest normal result; a row of 781 elements costs 40 instructions per lane
    // this way against some 300 through libm's expf, which made the kernel ALU-bound
    v[j] = __builtin_amdgcn_exp2f((v[j] - m) * 1.44269504088896341f);
    if (VEC || t + j * T < p.block) sum += v[j];
  }
  sum = wave_sum(sum);
  if (WAVES > 1) {
    if (t % WAVE == 0) red[t / WAVE] = sum;
    __syncthreads();
    sum = red[0];
#pragma unroll
    for (int w = 1; w < WAVES; w++) sum += red[w];
  }
  const float rsum = 1.0f / sum;  // one division per lane; the products are within 1.5 ulp of the quotients
  if constexpr (VEC && IO != 2) {
#pragma unroll
    for (int j = 0; j < NPL / 8; j++) {
      const int i0 = 8 * (t + j * T);
      uint32_t o[4];
#pragma unroll
      for (int k = 0; k < 4; k++)
        o[k] = (uint32_t)down(v[8 * j + 2 * k] * rsum) | ((uint32_t)down(v[8 * j + 2 * k + 1] * rsum) << 16);
      if (i0 < d_out) ntstore(reinterpret_cast<uint4 *>(out + i0), make_uint4(o[0], o[1], o[2], o[3]));
    }
  } else if constexpr (VEC) {
    // slot s of the grid is element s - lead of the row; the output row's chunks are aligned stores when it sits at the
    // same offset from a 16-byte boundary as the input row (dword-aligned ones otherwise)
    E *ogrid = out - lead;
    const int oslots = lead + d_out;
#pragma unroll
    for (int j = 0; j < NPL / 4; j++) {
      const int s0 = 4 * (t + j * T);
      f32x4_a4 w;
#pragma unroll
      for (int c = 0; c < 4; c++) w[c] = v[4 * j + c] * rsum;
      if (s0 >= lead && s0 + 4 <= oslots) __builtin_nontemporal_store(w, reinterpret_cast<f32x4_a4 *>(ogrid + s0));
      else
#pragma unroll
        for (int c = 0; c < 4; c++)
          if (s0 + c >= lead && s0 + c < oslots) ogrid[s0 + c] = w[c];
    }
  } else {
#pragma unroll
    for (int j = 0; j < NPL; j++) {
      int i = t + j * T;
      if (i < d_out) out[i] = down(v[j] * rsum);
    }
  }
}

template <int NPL, int WAVES, int WG, int IO>
hipError_t launch_softmax_io(const SoftmaxParams &p, int gx, int gy, int gz, hipStream_t s) {
  int64_t programs = (int64_t)gx * gy * gz;
  int rows_per_wg = WG / (WAVES * WAVE);
  dim3 grid((unsigned)((programs + rows_per_wg - 1) / rows_per_wg));
  constexpr int EPC = IO == 2 ? 4 : 8;  // elements per 16-byte chunk
  constexpr bool CAN_VEC = NPL % EPC == 0;
  // (fp32: a row's chunk grid starts up to 3 elements before the row and its NPL * T slots must hold the row as well: rows
  // that fill the block to its last three elements must start on 16-byte boundaries, all of them)
  auto rows_on_boundaries = [&](const Affine &a, const void *base) {
    return (a.c0 | a.c[0] | a.c[1] | a.c[2]) % 4 == 0 && ((uintptr_t)base & 15) == 0;
  };
  bool vec = CAN_VEC && p.block == NPL * WAVES * WAVE && p.d_in >= 4 &&
             (IO != 2 || p.d_in + 3 <= p.block || rows_on_boundaries(p.in_off, p.in));
  if (IO != 2) {  // whole chunks of aligned rows only
    auto aligned = [](const Affine &a) { return (a.c0 | a.c[0] | a.c[1] | a.c[2]) % 8 == 0; };
    vec = vec && p.d_in % 8 == 0 && p.d_out % 8 == 0 && aligned(p.in_off) && aligned(p.out_off) && (((uintptr_t)p.in | (uintptr_t)p.out) & 15) == 0;
  }
  if (vec) {
    if (p.propagate_nan) hipLaunchKernelGGL((softmax_f32_kernel<NPL, WAVES, true, CAN_VEC, WG, IO>), grid, dim3(WG), 0, s, p, gx, gy, programs);
    else hipLaunchKernelGGL((softmax_f32_kernel<NPL, WAVES, false, CAN_VEC, WG, IO>), grid, dim3(WG), 0, s, p, gx, gy, programs);
    return hipGetLastError();
  }
  if (p.propagate_nan) hipLaunchKernelGGL((softmax_f32_kernel<NPL, WAVES, true, false, WG, IO>), grid, dim3(WG), 0, s, p, gx, gy, programs);
  else hipLaunchKernelGGL((softmax_f32_kernel<NPL, WAVES, false, false, WG, IO>), grid, dim3(WG), 0, s, p, gx, gy, programs);
  return hipGetLastError();
}

template <int NPL, int WAVES, int WG = 256>
hipError_t launch_softmax_cfg(const SoftmaxParams &p, int gx, int gy, int gz, hipStream_t s) {
  if (p.elem_kind == 2) return launch_softmax_io<NPL, WAVES, WG, 2>(p, gx, gy, gz, s);
  if (p.elem_kind == 1) return launch_softmax_io<NPL, WAVES, WG, 1>(p, gx, gy, gz, s);
  return launch_softmax_io<NPL, WAVES, WG, 0>(p, gx, gy, gz, s);
}

// -------------------------------------------------------------- layernorm
// The element type of x, y, w and b: 0 fp16, 1 bf16, 2 fp32.  A chunk is the 16 bytes a thread moves at once: EPC elements.
template <int KIND>
struct LnType {
  using elem = uint16_t;
  static constexpr int EPC = 8;
  static __device__ __forceinline__ float up(uint16_t h) { return Half<KIND == 1>::up(h); }
  static __device__ __forceinline__ uint16_t down(float f) { return Half<KIND == 1>::down(f); }
  static __device__ __forceinline__ void unpack(const uint32_t (&q)[4], float (&v)[8]) {
#pragma unroll
    for (int k = 0; k < 4; k++) {
      v[2 * k] = up((uint16_t)(q[k] & 0xffff));
      v[2 * k + 1] = up((uint16_t)(q[k] >> 16));
    }
  }
  static __device__ __forceinline__ uint4 pack(const float (&y)[8]) {
    uint32_t o[4];
#pragma unroll
    for (int k = 0; k < 4; k++) o[k] = (uint32_t)down(y[2 * k]) | ((uint32_t)down(y[2 * k + 1]) << 16);
    return make_uint4(o[0], o[1], o[2], o[3]);
  }
};
template <>
struct LnType<2> {
  using elem = float;
  static constexpr int EPC = 4;
  static __device__ __forceinline__ float up(float x) { return x; }
  static __device__ __forceinline__ float down(float f) { return f; }
  static __device__ __forceinline__ void unpack(const uint32_t (&q)[4], float (&v)[4]) {
#pragma unroll
    for (int k = 0; k < 4; k++) v[k] = __uint_as_float(q[k]);
  }
  static __device__ __forceinline__ uint4 pack(const float (&y)[4]) {
    return make_uint4(__float_as_uint(y[0]), __float_as_uint(y[1]), __float_as_uint(y[2]), __float_as_uint(y[3]));
  }
};

// One workgroup per row.  The row is read from HBM once and kept in registers
// as fp32 (CPT chunks of EPC elements per thread); the Triton source's three
// passes over the row all read these registers.
// FAST: N is a multiple of EPC and every row of x, y, w, b starts 16-byte aligned, so a chunk is
// either whole or absent and all loads are unconditional (an absent chunk re-reads chunk 0 and is
// zeroed), which lets the compiler keep the CPT loads of a thread in flight together.
template <int KIND, int CPT, bool FAST>
__global__ __launch_bounds__(256, CPT <= 4 ? 8 : 4) void layernorm_fwd_kernel(LayerNormParams p) {
  using T = LnType<KIND>;
  using E = typename T::elem;
  constexpr int EPC = T::EPC;
  __shared__ float red[4];
  const ProgramId id = program_id(p.lin_gx, p.lin_gy);
  const int px = id.x, py = id.y, pz = id.z;
  const E *__restrict__ x = (const E *)p.x + affine(p.x_off, px, py, pz);
  const E *__restrict__ w = (const E *)p.w + affine(p.w_off, px, py, pz);
  const E *__restrict__ b = (const E *)p.b + affine(p.b_off, px, py, pz);
  E *__restrict__ y = (E *)p.y + affine(p.y_off, px, py, pz);
  const int N = (int)p.N;
  const bool vec = (((uintptr_t)x | (uintptr_t)w | (uintptr_t)b | (uintptr_t)y) & 15) == 0;
  float v[CPT][EPC];
#pragma unroll
  for (int c = 0; c < CPT; c++) {
    int i0 = (threadIdx.x + c * 256) * EPC;
    if (FAST) {
      const bool present = i0 < N;
      uint4 raw = *reinterpret_cast<const uint4 *>(x + (present ? i0 : 0));
      const uint32_t q[4] = {raw.x, raw.y, raw.z, raw.w};
      T::unpack(q, v[c]);
#pragma unroll
      for (int k = 0; k < EPC; k++) v[c][k] = present ? v[c][k] : 0.f;
    } else if (vec && i0 + EPC <= N) {
      uint4 raw = *reinterpret_cast<const uint4 *>(x + i0);
      const uint32_t q[4] = {raw.x, raw.y, raw.z, raw.w};
      T::unpack(q, v[c]);
    } else {
#pragma unroll
      for (int k = 0; k < EPC; k++) v[c][k] = i0 + k < N ? T::up(x[i0 + k]) : 0.f;  // other = 0
    }
  }
  const float n_f = (float)N;  // arith.sitofp
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < CPT; c++)
#pragma unroll
    for (int k = 0; k < EPC; k++) s += v[c][k];
  const float mean = block_sum_256(s, red) / n_f;
  float s2 = 0.f;
#pragma unroll
  for (int c = 0; c < CPT; c++) {
    int i0 = (threadIdx.x + c * 256) * EPC;
#pragma unroll
    for (int k = 0; k < EPC; k++) {
      float d = i0 + k < N ? v[c][k] - mean : 0.f;  // tl.where(cols < N, x - mean, 0)
      s2 += d * d;
    }
  }
  const float var = block_sum_256(s2, red) / n_f;
  const float rstd = 1.0f / sqrtf(var + p.eps);
  if (threadIdx.x == 0) {
    p.mean[affine(p.mean_off, px, py, pz)] = mean;
    p.rstd[affine(p.rstd_off, px, py, pz)] = rstd;
  }
#pragma unroll
  for (int c = 0; c < CPT; c++) {
    int i0 = (threadIdx.x + c * 256) * EPC;
    if (FAST ? i0 < N : (vec && i0 + EPC <= N)) {
      uint4 wr = *reinterpret_cast<const uint4 *>(w + i0);
      uint4 br = *reinterpret_cast<const uint4 *>(b + i0);
      const uint32_t wq[4] = {wr.x, wr.y, wr.z, wr.w}, bq[4] = {br.x, br.y, br.z, br.w};
      float wv[EPC], bv[EPC], o[EPC];
      T::unpack(wq, wv);
      T::unpack(bq, bv);
#pragma unroll
      for (int k = 0; k < EPC; k++) o[k] = (v[c][k] - mean) * rstd * wv[k] + bv[k];
      ntstore(reinterpret_cast<uint4 *>(y + i0), T::pack(o));
    } else {
#pragma unroll
      for (int k = 0; k < EPC; k++)
        if (i0 + k < N) y[i0 + k] = T::down((v[c][k] - mean) * rstd * T::up(w[i0 + k]) + T::up(b[i0 + k]));
    }
  }
}

// The same row arithmetic in a workgroup that walks rows blockIdx.x, blockIdx.x + gridDim.x, ...: the weight and bias
// chunks a thread needs are read once and stay in registers (packed), and the loads of the next row are issued before
// the current row is reduced, so a workgroup always has a row in flight while it computes and stores another.
// Measured on fp16 [4096, 8192] with the rows coming from HBM: one workgroup per row 27.4 us; 1024 / 512 / 256
// workgroups walking rows 26.3 / 25.0 / 24.4 us (a plain copy of the same bytes: 23.4 us).  What the row-per-workgroup
// kernel loses is the 32 KB of w and b that every row fetches again through L2: taking those loads out of it, and
// nothing else, gives 23.8 us.  512 or 1024 threads per workgroup, a third row in flight and nontemporal row loads
// gain nothing or lose.  [8192, 8192]: 51.7 -> 44.8 us (6.0 TB/s).
// For one-dimensional grids, rows of exactly CPT * 256 chunks starting 16-byte aligned, w and b the same for every row.
template <int KIND, int CPT>
__global__ __launch_bounds__(256) void layernorm_fwd_persistent_kernel(LayerNormParams p, int rows) {
  using T = LnType<KIND>;
  using E = typename T::elem;
  constexpr int EPC = T::EPC;
  __shared__ float red[2][2][4];  // [which reduction][row parity][wavefront]: one barrier per reduction
  const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
  const int N = (int)p.N;
  const E *__restrict__ xb = (const E *)p.x + p.x_off.c0;
  E *__restrict__ yb = (E *)p.y + p.y_off.c0;
  const E *__restrict__ w = (const E *)p.w + p.w_off.c0;
  const E *__restrict__ b = (const E *)p.b + p.b_off.c0;
  uint4 wq[CPT], bq[CPT];
#pragma unroll
  for (int c = 0; c < CPT; c++) {
    wq[c] = *reinterpret_cast<const uint4 *>(w + (tid + c * 256) * EPC);
    bq[c] = *reinterpret_cast<const uint4 *>(b + (tid + c * 256) * EPC);
  }
  // A row's loads are issued from inline assembly and waited for by hand (row_landed): left to the compiler, the wait
  // for a row also waits for the next row's loads, issued just before (it does not count memory operations across the
  // loop's back edge), and the rows do not overlap.
  auto load_row = [&](u32x4_t (&q)[CPT], int r) {
    const E *x = xb + (int64_t)r * p.x_off.c[0];
#pragma unroll
    for (int c = 0; c < CPT; c++) {
      const E *src = x + (tid + c * 256) * EPC;
      asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(q[c]) : "v"(src) : "memory");
    }
  };
  // Waits until at most `newer` vector memory operations issued after the row's loads are outstanding (they complete in
  // order, so the row has landed), and ties the row's registers to the wait so that no use moves above it.
  auto row_landed = [&](u32x4_t (&q)[CPT], int newer) {
    switch (newer) {  // a constant after inlining; the instruction takes an immediate
      case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
      case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
      case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
      case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
      case 16: asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); break;
      default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
#pragma unroll
    for (int c = 0; c < CPT; c++) asm volatile("" : "+v"(q[c]) : : "memory");
  };
  auto block_sum = [&](float v, int which, int parity) {
    v = wave_sum(v);
    if (lane == 0) red[which][parity][wave] = v;
    __syncthreads();
    return (red[which][parity][0] + red[which][parity][1]) + (red[which][parity][2] + red[which][parity][3]);
  };
  const float n_f = (float)N;  // arith.sitofp
  auto process = [&](const u32x4_t (&raw)[CPT], int r, int parity) {
    float v[CPT][EPC];
#pragma unroll
    for (int c = 0; c < CPT; c++) {
      const uint32_t q[4] = {raw[c][0], raw[c][1], raw[c][2], raw[c][3]};
      T::unpack(q, v[c]);
    }
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < CPT; c++)
#pragma unroll
      for (int k = 0; k < EPC; k++) s += v[c][k];
    const float mean = block_sum(s, 0, parity) / n_f;
    float s2 = 0.f;
#pragma unroll
    for (int c = 0; c < CPT; c++)
#pragma unroll
      for (int k = 0; k < EPC; k++) {
        const float d = v[c][k] - mean;
        s2 += d * d;
      }
    const float var = block_sum(s2, 1, parity) / n_f;
    const float rstd = 1.0f / sqrtf(var + p.eps);
    E *y = yb + (int64_t)r * p.y_off.c[0];
#pragma unroll
    for (int c = 0; c < CPT; c++) {
      // (the optimiser widens w and b to fp32 once, outside the row loop: 16 registers per chunk, which a workgroup
      // that has a CU's register file nearly to itself can afford, and four operations per element and row saved)
      const uint32_t wr[4] = {wq[c].x, wq[c].y, wq[c].z, wq[c].w}, br[4] = {bq[c].x, bq[c].y, bq[c].z, bq[c].w};
      float wv[EPC], bv[EPC], o[EPC];
      T::unpack(wr, wv);
      T::unpack(br, bv);
#pragma unroll
      for (int k = 0; k < EPC; k++) o[k] = (v[c][k] - mean) * rstd * wv[k] + bv[k];
      ntstore(reinterpret_cast<uint4 *>(y + (tid + c * 256) * EPC), T::pack(o));
    }
    if (tid == 0) {
      p.mean[p.mean_off.c0 + (int64_t)r * p.mean_off.c[0]] = mean;
      p.rstd[p.rstd_off.c0 + (int64_t)r * p.rstd_off.c[0]] = rstd;
    }
  };
  // Two register sets take turns, so that no row is copied from one to the other (a copy would wait for the loads).
  // Past the last row a workgroup loads the last row again: the loads are unconditional, hence countable.  Between a
  // row's loads and its use lie the next row's CPT loads and, from the second row on, the previous row's CPT stores
  // (every wavefront issues all of them: the rows are whole) -- plus the two statistics stores of the first wavefront,
  // which only make its wait stricter than necessary.
  int r = blockIdx.x;
  if (r >= rows) return;
  const int step = gridDim.x, last = rows - 1;
  u32x4_t even[CPT], odd[CPT];
  load_row(even, r);
  load_row(odd, min(r + step, last));
  row_landed(even, CPT);
  process(even, r, 0);
  r += step;
  while (r < rows) {
    load_row(even, min(r + step, last));
    row_landed(odd, 2 * CPT);
    process(odd, r, 1);
    r += step;
    if (r >= rows) break;
    load_row(odd, min(r + step, last));
    row_landed(even, 2 * CPT);
    process(even, r, 0);
    r += step;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the surplus loads of the last row land before the registers go away
}

// Rows too long for the register file: three passes over global memory, the
// second and third served by L2.
template <int KIND>
__global__ __launch_bounds__(256) void layernorm_fwd_long_kernel(LayerNormParams p) {
  using T = LnType<KIND>;
  using E = typename T::elem;
  __shared__ float red[4];
  const ProgramId id = program_id(p.lin_gx, p.lin_gy);
  const int px = id.x, py = id.y, pz = id.z;
  const E *__restrict__ x = (const E *)p.x + affine(p.x_off, px, py, pz);
  const E *__restrict__ w = (const E *)p.w + affine(p.w_off, px, py, pz);
  const E *__restrict__ b = (const E *)p.b + affine(p.b_off, px, py, pz);
  E *__restrict__ y = (E *)p.y + affine(p.y_off, px, py, pz);
  const int64_t N = p.N;
  const float n_f = (float)(int)N;
  float s = 0.f;
  for (int64_t i = threadIdx.x; i < N; i += 256) s += T::up(x[i]);
  const float mean = block_sum_256(s, red) / n_f;
  float s2 = 0.f;
  for (int64_t i = threadIdx.x; i < N; i += 256) {
    float d = T::up(x[i]) - mean;
    s2 += d * d;
  }
  const float var = block_sum_256(s2, red) / n_f;
  const float rstd = 1.0f / sqrtf(var + p.eps);
  if (threadIdx.x == 0) {
    p.mean[affine(p.mean_off, px, py, pz)] = mean;
    p.rstd[affine(p.rstd_off, px, py, pz)] = rstd;
  }
  for (int64_t i = threadIdx.x; i < N; i += 256)
    y[i] = T::down((T::up(x[i]) - mean) * rstd * T::up(w[i]) + T::up(b[i]));
}

template <int KIND>
hipError_t launch_layernorm_t(const LayerNormParams &p, dim3 grid, hipStream_t s, const char **name) {
  constexpr int EPC = LnType<KIND>::EPC;
  int64_t chunks = (p.N + EPC - 1) / EPC;
  auto aligned = [](const Affine &a) { return (a.c0 | a.c[0] | a.c[1] | a.c[2]) % EPC == 0; };
  const bool fast = p.N % EPC == 0 && aligned(p.x_off) && aligned(p.y_off) && aligned(p.w_off) && aligned(p.b_off) &&
                    (((uintptr_t)p.x | (uintptr_t)p.y | (uintptr_t)p.w | (uintptr_t)p.b) & 15) == 0;
  // Rows walked by persistent workgroups (see layernorm_fwd_persistent_kernel): whole rows of 256, 512, 1024 or (fp32)
  // 2048 chunks in one-dimensional grids with enough rows to amortise the walk (fewer, and the workgroup-per-row kernel
  // measured faster), w and b the same for every row.  About 32 KB of row loads in flight per CU: one workgroup per CU
  // for rows of 16 KB and more, four for 8 KB, eight for 4 KB (measured best of 1, 2, 4 and 8 per CU on fp16 [8192, 4096]
  // and [16384, 2048]: 25.5 us against 26.3 and 26.5 us against 31.1 for a workgroup per row).
  static const char *ln_env = getenv("TTS_LN");  // tuning aid: "0" = always one workgroup per row; "G" = G persistent workgroups
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    return n;
  }();
  const int cpt = chunks == 256 ? 1 : chunks == 512 ? 2 : chunks == 1024 ? 4 : (chunks == 2048 && KIND == 2) ? 8 : 0;
  int persistent_grid = cus * (cpt == 1 ? 8 : cpt == 2 ? 4 : 1);
  int64_t min_rows = (int64_t)persistent_grid * (cpt >= 4 ? 16 : 8);
  if (ln_env) {
    persistent_grid = atoi(ln_env);
    min_rows = 2 * (int64_t)persistent_grid;
  }
  auto row_invariant = [](const Affine &a) { return (a.c[0] | a.c[1] | a.c[2]) == 0; };
  if (fast && cpt && persistent_grid > 0 && !p.lin_gx && grid.y == 1 && grid.z == 1 && (int64_t)grid.x >= min_rows && row_invariant(p.w_off) &&
      row_invariant(p.b_off)) {
    const int rows = (int)grid.x;
    const dim3 pg((unsigned)persistent_grid);
    if (cpt == 1) hipLaunchKernelGGL((layernorm_fwd_persistent_kernel<KIND, 1>), pg, dim3(256), 0, s, p, rows);
    else if (cpt == 2) hipLaunchKernelGGL((layernorm_fwd_persistent_kernel<KIND, 2>), pg, dim3(256), 0, s, p, rows);
    else if (cpt == 4) hipLaunchKernelGGL((layernorm_fwd_persistent_kernel<KIND, 4>), pg, dim3(256), 0, s, p, rows);
    else if constexpr (KIND == 2) hipLaunchKernelGGL((layernorm_fwd_persistent_kernel<KIND, 8>), pg, dim3(256), 0, s, p, rows);
    *name = "layernorm_fwd_persistent_kernel";
    return hipGetLastError();
  }
#define TTS_LN(CPT)                                                                                          \
  do {                                                                                                       \
    if (fast) hipLaunchKernelGGL((layernorm_fwd_kernel<KIND, CPT, true>), grid, dim3(256), 0, s, p);        \
    else hipLaunchKernelGGL((layernorm_fwd_kernel<KIND, CPT, false>), grid, dim3(256), 0, s, p);            \
    *name = "layernorm_fwd_kernel<" #CPT ">";                                                                \
  } while (0)
  if (chunks <= 256) TTS_LN(1);
  else if (chunks <= 512) TTS_LN(2);
  else if (chunks <= 1024) TTS_LN(4);
  else if (chunks <= 2048) TTS_LN(8);
  else { hipLaunchKernelGGL((layernorm_fwd_long_kernel<KIND>), grid, dim3(256), 0, s, p); *name = "layernorm_fwd_long_kernel"; }
#undef TTS_LN
  return hipGetLastError();
}

// -------------------------------------------------------------- fused map
// The interpreter's registers are float4 slots in LDS, one column per lane (a lane only ever
// touches its own column: no bank conflicts, no barriers), because registers indexed by a
// run-time number would live in scratch memory.  Fetch and dispatch are scalar: all lanes run
// the same instruction.
typedef uint16_t u16x4_a2 __attribute__((ext_vector_type(4), aligned(2)));

template <class F>
__device__ __forceinline__ float4 map4(float4 a, F f) { return make_float4(f(a.x), f(a.y), f(a.z), f(a.w)); }
template <class F>
__device__ __forceinline__ float4 map4(float4 a, float4 b, F f) { return make_float4(f(a.x, b.x), f(a.y, b.y), f(a.z, b.z), f(a.w, b.w)); }
template <class F>
__device__ __forceinline__ float4 map4(float4 a, float4 b, float4 c, F f) {
  return make_float4(f(a.x, b.x, c.x), f(a.y, b.y, c.y), f(a.z, b.z, c.z), f(a.w, b.w, c.w));
}
__device__ __forceinline__ float as_bool(bool b) { return b ? 1.0f : 0.0f; }

__device__ __forceinline__ float4 mapn_load(const void *base, int type, int i, int valid, float other) {
  float v[4] = {other, other, other, other};
  if (type == 0) {
    const float *p = (const float *)base + i;
    if (valid >= 4) {
      f32x4_a4 w = *reinterpret_cast<const f32x4_a4 *>(p);
      return make_float4(w[0], w[1], w[2], w[3]);
    }
    for (int e = 0; e < valid; e++) v[e] = p[e];
  } else {
    const uint16_t *p = (const uint16_t *)base + i;
    uint16_t h[4] = {0, 0, 0, 0};
    if (valid >= 4) {
      u16x4_a2 w = *reinterpret_cast<const u16x4_a2 *>(p);
      h[0] = w[0]; h[1] = w[1]; h[2] = w[2]; h[3] = w[3];
    } else {
      for (int e = 0; e < valid; e++) h[e] = p[e];
    }
    for (int e = 0; e < 4; e++)
      if (e < valid) v[e] = type == 1 ? Half<false>::up(h[e]) : Half<true>::up(h[e]);
  }
  return make_float4(v[0], v[1], v[2], v[3]);
}

__device__ __forceinline__ void mapn_store(void *base, int type, int i, int valid, float4 r) {
  float v[4] = {r.x, r.y, r.z, r.w};
  if (type == 0) {
    float *p = (float *)base + i;
    if (valid >= 4) {
      f32x4_a4 w = {v[0], v[1], v[2], v[3]};
      __builtin_nontemporal_store(w, reinterpret_cast<f32x4_a4 *>(p));
    } else {
      for (int e = 0; e < valid; e++) p[e] = v[e];
    }
  } else {
    uint16_t *p = (uint16_t *)base + i;
    uint16_t h[4];
    for (int e = 0; e < 4; e++) h[e] = type == 1 ? Half<false>::down(v[e]) : Half<true>::down(v[e]);
    if (valid >= 4) {
      u16x4_a2 w = {h[0], h[1], h[2], h[3]};
      __builtin_nontemporal_store(w, reinterpret_cast<u16x4_a2 *>(p));
    } else {
      for (int e = 0; e < valid; e++) p[e] = h[e];
    }
  }
}

// One wavefront per program.  A lane owns MAPN_CHUNKS four-element chunks per pass over the block (chunk j
// starts at element 4 * (lane + 64 j)), so that fetching and dispatching an instruction (a lane read and a
// tree of scalar compares, about a hundred cycles) is paid once per 1024 elements.
constexpr int MAPN_CHUNKS = 4, MAPN_PASS = 64 * 4 * MAPN_CHUNKS;

template <class F>
__device__ __forceinline__ void mapn_apply1(float4 (&r)[MAPN_CHUNKS], const float4 (&a)[MAPN_CHUNKS], F f) {
#pragma unroll
  for (int j = 0; j < MAPN_CHUNKS; j++) r[j] = map4(a[j], f);
}
template <class F>
__device__ __forceinline__ void mapn_apply2(float4 (&r)[MAPN_CHUNKS], const float4 (&a)[MAPN_CHUNKS], const float4 (&b)[MAPN_CHUNKS], F f) {
#pragma unroll
  for (int j = 0; j < MAPN_CHUNKS; j++) r[j] = map4(a[j], b[j], f);
}
template <class F>
__device__ __forceinline__ void mapn_apply3(float4 (&r)[MAPN_CHUNKS], const float4 (&a)[MAPN_CHUNKS], const float4 (&b)[MAPN_CHUNKS],
                                            const float4 (&c)[MAPN_CHUNKS], F f) {
#pragma unroll
  for (int j = 0; j < MAPN_CHUNKS; j++) r[j] = map4(a[j], b[j], c[j], f);
}

template <int N_IN>
__global__ __launch_bounds__(64) void mapn_kernel(MapNParams p) {
  extern __shared__ float4 mapn_regs[];  // [n_regs][MAPN_CHUNKS][64]
  const int lane = threadIdx.x;
  const int px = blockIdx.x, py = blockIdx.y, pz = blockIdx.z;
  int d = p.block;
  if (p.masked) {
    int64_t left = p.bound - affine(p.m_start, px, py, pz);
    d = left < 0 ? 0 : left < p.block ? (int)left : p.block;
  }
  const uint2 my_ins = lane < MAPN_MAX_INS ? reinterpret_cast<const uint2 *>(p.ins)[lane] : make_uint2(0, 0);
  const uint32_t my_imm = lane < MAPN_MAX_IMM ? __float_as_uint(p.imm[lane]) : 0u;
  const char *in[N_IN];
#pragma unroll
  for (int k = 0; k < N_IN; k++) in[k] = (const char *)p.in[k] + affine(p.in_off[k], px, py, pz) * (p.in_type[k] == 0 ? 4 : 2);
  auto reg = [&](int r, int j) -> float4 & { return mapn_regs[(r * MAPN_CHUNKS + j) * 64 + lane]; };
  for (int i0 = 0; i0 < d; i0 += MAPN_PASS) {
    float4 v[N_IN][MAPN_CHUNKS];
#pragma unroll
    for (int k = 0; k < N_IN; k++)
#pragma unroll
      for (int j = 0; j < MAPN_CHUNKS; j++) {
        const int i = i0 + 4 * (lane + 64 * j);
        v[k][j] = mapn_load(in[k], p.in_type[k], i, d - i, p.in_other[k]);
      }
#pragma unroll
    for (int k = 0; k < N_IN; k++)
#pragma unroll
      for (int j = 0; j < MAPN_CHUNKS; j++) reg(p.in_reg[k], j) = v[k][j];
    float4 prev[MAPN_CHUNKS];
#pragma unroll
    for (int j = 0; j < MAPN_CHUNKS; j++) prev[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int t = 0; t < p.n_ins; t++) {
      // instruction words and immediates sit one per lane in two registers; a lane read makes them scalar
      const uint32_t w0 = __builtin_amdgcn_readlane(my_ins.x, t), w1 = __builtin_amdgcn_readlane(my_ins.y, t);
      const int op = w0 & 255, dst = (w0 >> 8) & 255, ia = (w0 >> 16) & 255, ib = w0 >> 24;
      const int ic = w1 & 255, kinds = (w1 >> 8) & 255, round = (w1 >> 16) & 255;
      auto fetch = [&](float4 (&o)[MAPN_CHUNKS], int kind, int idx) {
        if (kind == MS_PREV) {
#pragma unroll
          for (int j = 0; j < MAPN_CHUNKS; j++) o[j] = prev[j];
        } else if (kind == MS_IMM) {
          float c = __uint_as_float(__builtin_amdgcn_readlane(my_imm, idx));
#pragma unroll
          for (int j = 0; j < MAPN_CHUNKS; j++) o[j] = make_float4(c, c, c, c);
        } else {
#pragma unroll
          for (int j = 0; j < MAPN_CHUNKS; j++) o[j] = reg(idx, j);
        }
      };
      float4 a[MAPN_CHUNKS], b[MAPN_CHUNKS], c[MAPN_CHUNKS], r[MAPN_CHUNKS];
      fetch(a, kinds & 3, ia);
      const bool unary = op == MO_MOV || (op >= MO_NEG && op <= MO_CEIL);
      if (!unary) fetch(b, (kinds >> 2) & 3, ib);
      else
#pragma unroll
        for (int j = 0; j < MAPN_CHUNKS; j++) b[j] = a[j];
      if (op == MO_FMA || op == MO_SELECT) fetch(c, (kinds >> 4) & 3, ic);
      else
#pragma unroll
        for (int j = 0; j < MAPN_CHUNKS; j++) c[j] = a[j];
#pragma unroll
      for (int j = 0; j < MAPN_CHUNKS; j++) r[j] = a[j];
      switch (op) {
        case MO_MOV: break;
        case MO_ADD: mapn_apply2(r, a, b, [](float x, float y) { return x + y; }); break;
        case MO_SUB: mapn_apply2(r, a, b, [](float x, float y) { return x - y; }); break;
        case MO_MUL: mapn_apply2(r, a, b, [](float x, float y) { return x * y; }); break;
        case MO_DIV: mapn_apply2(r, a, b, [](float x, float y) { return x / y; }); break;
        case MO_MAXNUM: mapn_apply2(r, a, b, [](float x, float y) { return fmaxf(x, y); }); break;
        case MO_MINNUM: mapn_apply2(r, a, b, [](float x, float y) { return fminf(x, y); }); break;
        case MO_MAXIMUM: mapn_apply2(r, a, b, [](float x, float y) { return apply<4>(x, y); }); break;
        case MO_MINIMUM: mapn_apply2(r, a, b, [](float x, float y) { return apply<5>(x, y); }); break;
        case MO_NEG: mapn_apply1(r, a, [](float x) { return -x; }); break;
        case MO_ABS: mapn_apply1(r, a, [](float x) { return fabsf(x); }); break;
        case MO_EXP: mapn_apply1(r, a, [](float x) { return expf(x); }); break;
        case MO_EXP2: mapn_apply1(r, a, [](float x) { return exp2f(x); }); break;
        case MO_LOG: mapn_apply1(r, a, [](float x) { return logf(x); }); break;
        case MO_LOG2: mapn_apply1(r, a, [](float x) { return log2f(x); }); break;
        case MO_SQRT: mapn_apply1(r, a, [](float x) { return sqrtf(x); }); break;
        case MO_RSQRT: mapn_apply1(r, a, [](float x) { return 1.0f / sqrtf(x); }); break;
        case MO_SIN: mapn_apply1(r, a, [](float x) { return sinf(x); }); break;
        case MO_COS: mapn_apply1(r, a, [](float x) { return cosf(x); }); break;
        case MO_TANH: mapn_apply1(r, a, [](float x) { return tanhf(x); }); break;
        case MO_ERF: mapn_apply1(r, a, [](float x) { return erff(x); }); break;
        case MO_FLOOR: mapn_apply1(r, a, [](float x) { return floorf(x); }); break;
        case MO_CEIL: mapn_apply1(r, a, [](float x) { return ceilf(x); }); break;
        case MO_FMA: mapn_apply3(r, a, b, c, [](float x, float y, float z) { return fmaf(x, y, z); }); break;
        case MO_SELECT: mapn_apply3(r, a, b, c, [](float s, float x, float y) { return s != 0.f ? x : y; }); break;
        case MO_AND: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(x != 0.f && y != 0.f); }); break;
        case MO_OR: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(x != 0.f || y != 0.f); }); break;
        case MO_XOR: mapn_apply2(r, a, b, [](float x, float y) { return as_bool((x != 0.f) != (y != 0.f)); }); break;
        case MO_CMP_OEQ: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(x == y); }); break;
        case MO_CMP_ONE: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(x < y || x > y); }); break;
        case MO_CMP_OLT: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(x < y); }); break;
        case MO_CMP_OLE: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(x <= y); }); break;
        case MO_CMP_OGT: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(x > y); }); break;
        case MO_CMP_OGE: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(x >= y); }); break;
        case MO_CMP_UNE: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(!(x == y)); }); break;
        case MO_CMP_UEQ: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(!(x < y || x > y)); }); break;
        case MO_CMP_ULT: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(!(x >= y)); }); break;
        case MO_CMP_ULE: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(!(x > y)); }); break;
        case MO_CMP_UGT: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(!(x <= y)); }); break;
        case MO_CMP_UGE: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(!(x < y)); }); break;
        case MO_CMP_ORD: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(x == x && y == y); }); break;
        case MO_CMP_UNO: mapn_apply2(r, a, b, [](float x, float y) { return as_bool(x != x || y != y); }); break;
      }
      if (round == 1) mapn_apply1(r, r, [](float x) { return Half<false>::up(Half<false>::down(x)); });
      else if (round == 2) mapn_apply1(r, r, [](float x) { return Half<true>::up(Half<true>::down(x)); });
#pragma unroll
      for (int j = 0; j < MAPN_CHUNKS; j++) prev[j] = r[j];
      if (!(kinds & 64))
#pragma unroll
        for (int j = 0; j < MAPN_CHUNKS; j++) reg(dst, j) = r[j];
    }
    for (int o = 0; o < p.n_out; o++) {
      char *out = (char *)p.out[o] + affine(p.out_off[o], px, py, pz) * (p.out_type[o] == 0 ? 4 : 2);
#pragma unroll
      for (int j = 0; j < MAPN_CHUNKS; j++) {
        const int i = i0 + 4 * (lane + 64 * j);
        mapn_store(out, p.out_type[o], i, d - i, reg(p.out_reg[o], j));
      }
    }
  }
}

template <int N_IN>
hipError_t launch_mapn_n(const MapNParams &p, dim3 grid, hipStream_t s) {
  hipLaunchKernelGGL((mapn_kernel<N_IN>), grid, dim3(64), (size_t)p.n_regs * MAPN_CHUNKS * 64 * sizeof(float4), s, p);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_map1d(const Map1DParams &params, int gx, int gy, int gz, hipStream_t s, const char **name) {
  Map1DParams p = params;
  const dim3 grid = program_grid(p, gx, gy, gz);
  *name = "map1d_f32_kernel";
  switch (p.op) {
    case 0: return launch_map1d_op<0>(p, grid, s);
    case 1: return launch_map1d_op<1>(p, grid, s);
    case 2: return launch_map1d_op<2>(p, grid, s);
    case 3: return launch_map1d_op<3>(p, grid, s);
    case 4: return launch_map1d_op<4>(p, grid, s);
    case 5: return launch_map1d_op<5>(p, grid, s);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_mapn(const MapNParams &p, int gx, int gy, int gz, hipStream_t s, const char **name) {
  dim3 grid(gx, gy, gz);
  *name = "mapn_kernel";
  switch (p.n_in) {
    case 1: return launch_mapn_n<1>(p, grid, s);
    case 2: return launch_mapn_n<2>(p, grid, s);
    case 3: return launch_mapn_n<3>(p, grid, s);
    case 4: return launch_mapn_n<4>(p, grid, s);
    case 5: return launch_mapn_n<5>(p, grid, s);
    case 6: return launch_mapn_n<6>(p, grid, s);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_softmax(const SoftmaxParams &p, int gx, int gy, int gz, hipStream_t s, const char **name) {
  *name = "softmax_f32_kernel";
  int b = p.block;
  if (b <= 64) return launch_softmax_cfg<1, 1>(p, gx, gy, gz, s);
  if (b <= 128) return launch_softmax_cfg<2, 1>(p, gx, gy, gz, s);
  if (b <= 256) return launch_softmax_cfg<4, 1>(p, gx, gy, gz, s);
  if (b <= 512) return launch_softmax_cfg<8, 1>(p, gx, gy, gz, s);
  if (b <= 1024) return launch_softmax_cfg<16, 1>(p, gx, gy, gz, s);  // 4 rows per workgroup: 64 ... 1024 threads measured within 3 % of each other, 256 best
  if (b <= 2048) return launch_softmax_cfg<32, 1>(p, gx, gy, gz, s);
  if (b <= 4096) return launch_softmax_cfg<16, 4>(p, gx, gy, gz, s);
  if (b <= 8192) return launch_softmax_cfg<32, 4>(p, gx, gy, gz, s);
  if (b <= 16384) return launch_softmax_cfg<64, 4>(p, gx, gy, gz, s);
  // longer rows: more wavefronts per row, still one pass over memory with the row in registers
  if (b <= 32768) return launch_softmax_cfg<64, 8, 512>(p, gx, gy, gz, s);
  if (b <= 65536) return launch_softmax_cfg<64, 16, 1024>(p, gx, gy, gz, s);
  return hipErrorInvalidValue;
}

hipError_t launch_layernorm(const LayerNormParams &params, int gx, int gy, int gz, hipStream_t s, const char **name) {
  LayerNormParams p = params;
  const dim3 grid = program_grid(p, gx, gy, gz);
  return p.elem_kind == 2 ? launch_layernorm_t<2>(p, grid, s, name) : p.elem_kind == 1 ? launch_layernorm_t<1>(p, grid, s, name) : launch_layernorm_t<0>(p, grid, s, name);
}

}  // namespace tts
