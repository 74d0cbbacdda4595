// Launch interface of the hand-written gfx950 kernels, one per kernel family.
// Parameter blocks are plain data resolved by the launcher from the plan's
// bindings; the kernels know nothing about Triton.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>

#include "gemm_device.h"
#include "mapn_isa.h"

namespace tts {

// value(pid) = c0 + cx*pid.x + cy*pid.y + cz*pid.z, in elements
struct Affine {
  int64_t c0 = 0;
  int64_t c[3] = {0, 0, 0};
};

// z[off_z(p)+i] = x[off_x(p)+i] op y[off_y(p)+i],  0 <= i < extent(p)
// extent(p) = masked ? clamp(bound - m_start(p), 0, block) : block
struct Map1DParams {
  const float *x, *y;
  float *z;
  Affine xo, yo, zo, m_start;
  int64_t bound;
  int block;
  int masked;
  int op;    // 0 add 1 sub 2 mul 3 div 4 maximum 5 minimum
  int swap;  // operands of `op` are (y, x)
  int lin_gx = 0, lin_gy = 0;  // set by the launch: a one-dimensional launch numbers the programs of a grid this wide and tall itself
};
hipError_t launch_map1d(const Map1DParams &p, int gx, int gy, int gz, hipStream_t s, const char **kernel_name);

// Fused elementwise map over one-dimensional blocks: out_j[off(p)+i] = f_j(in_0[..+i], ..., scalars), 0 <= i < extent(p).
// f is a straight-line program over 32-bit registers, one instruction per elementwise op of the
// Triton kernel (linalg.generic bodies in the reference, TritonArithToLinalg.cpp:104), run by an
// interpreter inside the kernel.  Narrow float types live in registers as fp32 and are rounded
// (RTNE) after every op whose Triton result type is narrow, which gives the same values as
// computing in the narrow type.  i1 values are 0.0f / 1.0f.
struct MapNParams {
  const void *in[MAPN_MAX_IN];
  void *out[MAPN_MAX_OUT];
  Affine in_off[MAPN_MAX_IN], out_off[MAPN_MAX_OUT], m_start;
  int64_t bound;
  int block, masked;
  int n_in, n_out, n_ins, n_regs;
  uint8_t in_type[MAPN_MAX_IN], out_type[MAPN_MAX_OUT];  // 0 fp32, 1 fp16, 2 bf16
  uint8_t in_reg[MAPN_MAX_IN], out_reg[MAPN_MAX_OUT];
  float in_other[MAPN_MAX_IN];
  float imm[MAPN_MAX_IMM];
  MapIns ins[MAPN_MAX_INS];
};
hipError_t launch_mapn(const MapNParams &p, int gx, int gy, int gz, hipStream_t s, const char **kernel_name);

// Kernels compiled at run time with hipRTC (fused_rtc.hip): a compiled module with one entry point.
struct RtcModule;
hipError_t rtc_compile(const std::string &source, const char *entry, RtcModule **out, std::string *err);
hipError_t rtc_launch(RtcModule *m, int gx, int gy, int gz, int block, void *args, size_t size, hipStream_t s);
int rtc_resident_workgroups(RtcModule *m);  // how many workgroups of 256 threads of this kernel a CU holds at once (asked once, then kept)
const char *gemm_device_source();  // the text of gemm_device.h
void rtc_release(RtcModule *m);
// The fused map's register program printed as HIP source and compiled once.
hipError_t fused_map_compile(const MapNParams &p, RtcModule **out, std::string *err);
hipError_t fused_map_launch(RtcModule *m, const MapNParams &p, int gx, int gy, int gz, hipStream_t s);
std::string fused_map_source(const MapNParams &p);

// out[off_out(p)+i] = softmax(row)[i], i < d_out, where row[i] = i < d_in ? in[off_in(p)+i] : other, i < block
struct SoftmaxParams {
  const void *in;
  void *out;
  Affine in_off, out_off;
  int64_t d_in, d_out;
  int block;
  float other;
  int propagate_nan;  // the max reduction is arith.maximumf rather than arith.maxnumf
  int elem_kind;      // the element type of in and out: 0 fp16, 1 bf16, 2 fp32 (the arithmetic is fp32 either way)
};
hipError_t launch_softmax(const SoftmaxParams &p, int gx, int gy, int gz, hipStream_t s, const char **kernel_name);

// LayerNorm forward over rows of N elements (fp16, bf16 or fp32 I/O, fp32 statistics)
struct LayerNormParams {
  const void *x, *w, *b;
  void *y;
  float *mean, *rstd;
  Affine x_off, y_off, w_off, b_off, mean_off, rstd_off;
  int64_t N;
  float eps;
  int elem_kind;  // the element type of x, y, w and b: 0 fp16, 1 bf16, 2 fp32
  int lin_gx = 0, lin_gy = 0;  // set by the launch: a one-dimensional launch numbers the programs of a grid this wide and tall itself
};
hipError_t launch_layernorm(const LayerNormParams &p, int gx, int gy, int gz, hipStream_t s, const char **kernel_name);

// C[M,N] = A[M,K] * B[K,N], 16-bit inputs, fp32 accumulate, 16-bit output (RTNE)
using GemmParams = ::TtsGemmParams;  // gemm_device.h
// p.split = at most gemm_split(p) K slices (1: none) with p.partial = gemm_workspace_bytes(p) bytes of device memory for them
int gemm_split(const GemmParams &p);
size_t gemm_workspace_bytes(const GemmParams &p);
hipError_t launch_gemm(const GemmParams &p, hipStream_t s, const char **kernel_name);
// The same product with elementwise ops fused into the epilogue: `epilogue` is the source of the functor (match.h:
// gemm_epilogue_source), `modules` the plan's two slots for the kernels compiled from it (one per tiling, filled at
// the first launch that needs it), `args` / `args_size` the generic families' argument block.
struct RtcModule;
// The epilogue functor as the kernel receives it (the generated `struct TtsEp` has this layout): every kernel argument
// by index, then what it takes to find the Triton program that owns an element -- tile_pid[(row / BM) * tiles_n +
// col / BN] is that program's linear id x + gx * (y + gy * z) in the Triton launch grid (device memory).
struct GemmEpilogueArgs {
  void *ptr[32];
  long long ival[32];
  double fval[32];
  const int *tile_pid;
  int tiles_n, gx, gy, gz;
};
int gemm_epilogue_kernel_index(const GemmParams &p);  // which of `modules` a launch of this shape uses
hipError_t launch_gemm_epilogue(const GemmParams &p, const std::string &epilogue, RtcModule **modules, const GemmEpilogueArgs &ep,
                                hipStream_t s, const char **kernel_name, std::string *err);

// C[M,N] = A[M,K] * (f16(W[K,N]) * scale[N]), A/scale/C fp16, W int8, fp32 accumulate, M <= 16
struct GemmW8A16Params {
  const void *a;
  const int8_t *w;
  const void *scale;
  void *c;
  int64_t M, N, K;
  int64_t lda, ldw, ldc;
  float *workspace;        // split-K partial sums, gemm_w8a16_workspace_bytes() large, or null when split == 1
  int *counters;           // gemm_w8a16_counters() arrival counters, zero between launches (clear them once)
  int split;
  void *widened;           // gemm_w8a16_widened_bytes() of device memory for the weights as fp16 (many rows of A), or null
};
int gemm_w8a16_split(const GemmW8A16Params &p);  // how many K slices the kernel wants (from shapes and pitches)
size_t gemm_w8a16_workspace_bytes(const GemmW8A16Params &p);
size_t gemm_w8a16_counters(const GemmW8A16Params &p);
size_t gemm_w8a16_widened_bytes(const GemmW8A16Params &p);  // 0: this shape runs on the decode kernels
hipError_t launch_gemm_w8a16(const GemmW8A16Params &p, hipStream_t s, const char **kernel_name);

}  // namespace tts
