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

namespace tts {

namespace {

constexpr int WAVE = 64;

__device__ __forceinline__ int64_t affine(const Affine &a, int px, int py, int pz) {
  return a.c0 + a.c[0] * px + a.c[1] * py + a.c[2] * pz;
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
// 23.3 -> 21.3 us with the input cached; nontemporal loads gained nothing and lost the cached case).
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
  const int px = blockIdx.x, py = blockIdx.y, pz = blockIdx.z;
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
      float4 a = *reinterpret_cast<const float4 *>(x + i);
      float4 b = *reinterpret_cast<const float4 *>(y + i);
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

// ---------------------------------------------------------------- softmax
// T threads share one row; thread t holds elements t, t+T, ... (NPL of them).
// VEC (block == NPL * T, NPL % 4 == 0, d_in >= 4): thread t holds the four-element chunks t, t+T, ...
// instead and moves each with one 16-byte access.  Rows need no 16-byte alignment for that (global
// accesses of several dwords only need dword alignment).  Every load is unconditional: a chunk that
// sticks out of the row is read from the row's last four elements and shifted into place.
typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

template <int NPL, int WAVES, bool NAN_PROP, bool VEC>
__global__ __launch_bounds__(256) void softmax_f32_kernel(SoftmaxParams p, int gx, int gy, int64_t programs) {
  constexpr int T = WAVES * WAVE;
  constexpr int ROWS_PER_WG = 256 / T;
  __shared__ float red[4];
  const int sub = threadIdx.x / T, t = threadIdx.x % T;
  const int64_t prog = (int64_t)blockIdx.x * ROWS_PER_WG + sub;
  const bool active = prog < programs;
  int px = 0, py = 0, pz = 0;
  if (active) {
    if (gy == 1 && programs == gx) px = (int)prog;  // 1-D grid: no divisions
    else { px = (int)(prog % gx); py = (int)((prog / gx) % gy); pz = (int)(prog / ((int64_t)gx * gy)); }
  }
  const float *__restrict__ in = p.in + affine(p.in_off, px, py, pz);
  float *__restrict__ out = p.out + affine(p.out_off, px, py, pz);
  const int d_in = active ? (int)p.d_in : 0, d_out = active ? (int)p.d_out : 0;
  // lanes beyond d_in hold `other` and take part in the reductions, as a filled
  // tile does; lanes beyond the block do not exist
  float v[NPL];
  if constexpr (VEC) {
    const int last = max(d_in - 4, 0);  // inactive rows (d_in == 0) read the first row's start and store nothing
    f32x4_a4 win[NPL / 4];
#pragma unroll
    for (int j = 0; j < NPL / 4; j++) win[j] = *reinterpret_cast<const f32x4_a4 *>(in + min(4 * (t + j * T), last));
#pragma unroll
    for (int j = 0; j < NPL / 4; j++) {
      const int i0 = 4 * (t + j * T);
      const int shift = i0 - min(i0, last);  // chunk element c is window[c + shift]
      const f32x4_a4 w = win[j];
#pragma unroll
      for (int c = 0; c < 4; c++) {
        float x = p.other;
        if (shift == 0) x = w[c];
#pragma unroll
        for (int sft = 1; sft < 4; sft++)
          if (c + sft < 4 && shift == sft) x = w[c + sft];
        v[4 * j + c] = i0 + c < d_in ? x : p.other;
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < NPL; j++) {
      int i = t + j * T;
      v[j] = i < d_in ? in[i] : p.other;
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
  if constexpr (VEC) {
#pragma unroll
    for (int j = 0; j < NPL / 4; j++) {
      const int i0 = 4 * (t + j * T);
      f32x4_a4 w;
#pragma unroll
      for (int c = 0; c < 4; c++) w[c] = v[4 * j + c] * rsum;
      if (i0 + 4 <= d_out) __builtin_nontemporal_store(w, reinterpret_cast<f32x4_a4 *>(out + i0));
      else
#pragma unroll
        for (int c = 0; c < 4; c++)
          if (i0 + c < d_out) out[i0 + c] = w[c];
    }
  } else {
#pragma unroll
    for (int j = 0; j < NPL; j++) {
      int i = t + j * T;
      if (i < d_out) out[i] = v[j] * rsum;
    }
  }
}

template <int NPL, int WAVES>
hipError_t launch_softmax_cfg(const SoftmaxParams &p, int gx, int gy, int gz, hipStream_t s) {
  int64_t programs = (int64_t)gx * gy * gz;
  int rows_per_wg = 256 / (WAVES * WAVE);
  dim3 grid((unsigned)((programs + rows_per_wg - 1) / rows_per_wg));
  constexpr bool CAN_VEC = NPL % 4 == 0;
  if (CAN_VEC && p.block == NPL * WAVES * WAVE && p.d_in >= 4) {
    if (p.propagate_nan) hipLaunchKernelGGL((softmax_f32_kernel<NPL, WAVES, true, CAN_VEC>), grid, dim3(256), 0, s, p, gx, gy, programs);
    else hipLaunchKernelGGL((softmax_f32_kernel<NPL, WAVES, false, CAN_VEC>), grid, dim3(256), 0, s, p, gx, gy, programs);
    return hipGetLastError();
  }
  if (p.propagate_nan) hipLaunchKernelGGL((softmax_f32_kernel<NPL, WAVES, true, false>), grid, dim3(256), 0, s, p, gx, gy, programs);
  else hipLaunchKernelGGL((softmax_f32_kernel<NPL, WAVES, false, false>), grid, dim3(256), 0, s, p, gx, gy, programs);
  return hipGetLastError();
}

// -------------------------------------------------------------- layernorm
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

// One workgroup per row.  The row is read from HBM once and kept in registers
// as fp32 (CPT chunks of 8 elements per thread); the Triton source's three
// passes over the row all read these registers.
// FAST: N is a multiple of 8 and every row of x, y, w, b starts 16-byte aligned, so a chunk is
// either whole or absent and all loads are unconditional (an absent chunk re-reads chunk 0 and is
// zeroed), which lets the compiler keep the CPT loads of a thread in flight together.
template <bool BF16, int CPT, bool FAST>
__global__ __launch_bounds__(256, CPT <= 4 ? 8 : 4) void layernorm_fwd_kernel(LayerNormParams p) {
  __shared__ float red[4];
  const int px = blockIdx.x, py = blockIdx.y, pz = blockIdx.z;
  const uint16_t *__restrict__ x = (const uint16_t *)p.x + affine(p.x_off, px, py, pz);
  const uint16_t *__restrict__ w = (const uint16_t *)p.w + affine(p.w_off, px, py, pz);
  const uint16_t *__restrict__ b = (const uint16_t *)p.b + affine(p.b_off, px, py, pz);
  uint16_t *__restrict__ y = (uint16_t *)p.y + affine(p.y_off, px, py, pz);
  const int N = (int)p.N;
  const bool vec = (((uintptr_t)x | (uintptr_t)w | (uintptr_t)b | (uintptr_t)y) & 15) == 0;
  float v[CPT][8];
#pragma unroll
  for (int c = 0; c < CPT; c++) {
    int i0 = (threadIdx.x + c * 256) * 8;
    if (FAST) {
      const bool present = i0 < N;
      uint4 raw = *reinterpret_cast<const uint4 *>(x + (present ? i0 : 0));
      uint32_t q[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int k = 0; k < 4; k++) {
        v[c][2 * k] = present ? Half<BF16>::up((uint16_t)(q[k] & 0xffff)) : 0.f;
        v[c][2 * k + 1] = present ? Half<BF16>::up((uint16_t)(q[k] >> 16)) : 0.f;
      }
    } else if (vec && i0 + 8 <= N) {
      uint4 raw = *reinterpret_cast<const uint4 *>(x + i0);
      uint32_t q[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int k = 0; k < 4; k++) {
        v[c][2 * k] = Half<BF16>::up((uint16_t)(q[k] & 0xffff));
        v[c][2 * k + 1] = Half<BF16>::up((uint16_t)(q[k] >> 16));
      }
    } else {
#pragma unroll
      for (int k = 0; k < 8; k++) v[c][k] = i0 + k < N ? Half<BF16>::up(x[i0 + k]) : 0.f;  // other = 0
    }
  }
  const float n_f = (float)N;  // arith.sitofp
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < CPT; c++)
#pragma unroll
    for (int k = 0; k < 8; k++) s += v[c][k];
  const float mean = block_sum_256(s, red) / n_f;
  float s2 = 0.f;
#pragma unroll
  for (int c = 0; c < CPT; c++) {
    int i0 = (threadIdx.x + c * 256) * 8;
#pragma unroll
    for (int k = 0; k < 8; k++) {
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
    int i0 = (threadIdx.x + c * 256) * 8;
    if (FAST ? i0 < N : (vec && i0 + 8 <= N)) {
      uint4 wr = *reinterpret_cast<const uint4 *>(w + i0);
      uint4 br = *reinterpret_cast<const uint4 *>(b + i0);
      uint32_t wq[4] = {wr.x, wr.y, wr.z, wr.w}, bq[4] = {br.x, br.y, br.z, br.w}, o[4];
#pragma unroll
      for (int k = 0; k < 4; k++) {
        float y0 = (v[c][2 * k] - mean) * rstd * Half<BF16>::up((uint16_t)(wq[k] & 0xffff)) +
                   Half<BF16>::up((uint16_t)(bq[k] & 0xffff));
        float y1 = (v[c][2 * k + 1] - mean) * rstd * Half<BF16>::up((uint16_t)(wq[k] >> 16)) +
                   Half<BF16>::up((uint16_t)(bq[k] >> 16));
        o[k] = (uint32_t)Half<BF16>::down(y0) | ((uint32_t)Half<BF16>::down(y1) << 16);
      }
      ntstore(reinterpret_cast<uint4 *>(y + i0), make_uint4(o[0], o[1], o[2], o[3]));
    } else {
#pragma unroll
      for (int k = 0; k < 8; k++)
        if (i0 + k < N)
          y[i0 + k] = Half<BF16>::down((v[c][k] - mean) * rstd * Half<BF16>::up(w[i0 + k]) + Half<BF16>::up(b[i0 + k]));
    }
  }
}

// Rows too long for the register file: three passes over global memory, the
// second and third served by L2.
template <bool BF16>
__global__ __launch_bounds__(256) void layernorm_fwd_long_kernel(LayerNormParams p) {
  __shared__ float red[4];
  const int px = blockIdx.x, py = blockIdx.y, pz = blockIdx.z;
  const uint16_t *__restrict__ x = (const uint16_t *)p.x + affine(p.x_off, px, py, pz);
  const uint16_t *__restrict__ w = (const uint16_t *)p.w + affine(p.w_off, px, py, pz);
  const uint16_t *__restrict__ b = (const uint16_t *)p.b + affine(p.b_off, px, py, pz);
  uint16_t *__restrict__ y = (uint16_t *)p.y + affine(p.y_off, px, py, pz);
  const int64_t N = p.N;
  const float n_f = (float)(int)N;
  float s = 0.f;
  for (int64_t i = threadIdx.x; i < N; i += 256) s += Half<BF16>::up(x[i]);
  const float mean = block_sum_256(s, red) / n_f;
  float s2 = 0.f;
  for (int64_t i = threadIdx.x; i < N; i += 256) {
    float d = Half<BF16>::up(x[i]) - mean;
    s2 += d * d;
  }
  const float var = block_sum_256(s2, red) / n_f;
  const float rstd = 1.0f / sqrtf(var + p.eps);
  if (threadIdx.x == 0) {
    p.mean[affine(p.mean_off, px, py, pz)] = mean;
    p.rstd[affine(p.rstd_off, px, py, pz)] = rstd;
  }
  for (int64_t i = threadIdx.x; i < N; i += 256)
    y[i] = Half<BF16>::down((Half<BF16>::up(x[i]) - mean) * rstd * Half<BF16>::up(w[i]) + Half<BF16>::up(b[i]));
}

template <bool BF16>
hipError_t launch_layernorm_t(const LayerNormParams &p, dim3 grid, hipStream_t s, const char **name) {
  int64_t chunks = (p.N + 7) / 8;
  auto aligned = [](const Affine &a) { return (a.c0 | a.c[0] | a.c[1] | a.c[2]) % 8 == 0; };
  const bool fast = p.N % 8 == 0 && aligned(p.x_off) && aligned(p.y_off) && aligned(p.w_off) && aligned(p.b_off) &&
                    (((uintptr_t)p.x | (uintptr_t)p.y | (uintptr_t)p.w | (uintptr_t)p.b) & 15) == 0;
#define TTS_LN(CPT)                                                                                          \
  do {                                                                                                       \
    if (fast) hipLaunchKernelGGL((layernorm_fwd_kernel<BF16, CPT, true>), grid, dim3(256), 0, s, p);        \
    else hipLaunchKernelGGL((layernorm_fwd_kernel<BF16, CPT, false>), grid, dim3(256), 0, s, p);            \
    *name = "layernorm_fwd_kernel<" #CPT ">";                                                                \
  } while (0)
  if (chunks <= 256) TTS_LN(1);
  else if (chunks <= 512) TTS_LN(2);
  else if (chunks <= 1024) TTS_LN(4);
  else if (chunks <= 2048) TTS_LN(8);
  else { hipLaunchKernelGGL((layernorm_fwd_long_kernel<BF16>), grid, dim3(256), 0, s, p); *name = "layernorm_fwd_long_kernel"; }
#undef TTS_LN
  return hipGetLastError();
}

}  // namespace

hipError_t launch_map1d(const Map1DParams &p, int gx, int gy, int gz, hipStream_t s, const char **name) {
  dim3 grid(gx, gy, gz);
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

hipError_t launch_softmax(const SoftmaxParams &p, int gx, int gy, int gz, hipStream_t s, const char **name) {
  *name = "softmax_f32_kernel";
  int b = p.block;
  if (b <= 64) return launch_softmax_cfg<1, 1>(p, gx, gy, gz, s);
  if (b <= 128) return launch_softmax_cfg<2, 1>(p, gx, gy, gz, s);
  if (b <= 256) return launch_softmax_cfg<4, 1>(p, gx, gy, gz, s);
  if (b <= 512) return launch_softmax_cfg<8, 1>(p, gx, gy, gz, s);
  if (b <= 1024) return launch_softmax_cfg<16, 1>(p, gx, gy, gz, s);
  if (b <= 2048) return launch_softmax_cfg<32, 1>(p, gx, gy, gz, s);
  if (b <= 4096) return launch_softmax_cfg<16, 4>(p, gx, gy, gz, s);
  if (b <= 8192) return launch_softmax_cfg<32, 4>(p, gx, gy, gz, s);
  if (b <= 16384) return launch_softmax_cfg<64, 4>(p, gx, gy, gz, s);
  return hipErrorInvalidValue;
}

hipError_t launch_layernorm(const LayerNormParams &p, int gx, int gy, int gz, hipStream_t s, const char **name) {
  dim3 grid(gx, gy, gz);
  return p.is_bf16 ? launch_layernorm_t<true>(p, grid, s, name) : launch_layernorm_t<false>(p, grid, s, name);
}

}  // namespace tts
