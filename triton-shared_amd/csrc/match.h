// Pattern matcher: structured program -> kernel family + symbolic bindings.
//
// The reference lowers the structured program generically (mlir-opt pipeline,
// backend/compiler.py:75-124) and runs it one Triton program at a time
// (backend/driver.py:116-133).  This backend instead recognises the shape of
// the whole structured program and hands the whole grid to one hand-written
// gfx950 kernel of the matching family.  A program that matches no family is
// refused (tts::Unsupported); nothing falls back to the CPU.
#pragma once
#include <map>
#include <string>

#include "structured.h"

namespace tts {

enum class Family { Map1D, RowSoftmax, LayerNormFwd, Gemm, GemmW8A16, FusedMap, TileProgram };
const char *family_name(Family f);

// value(pid) = c0 + cx*pid.x + cy*pid.y + cz*pid.z ; all four are index
// expressions that do not read the program id.
struct Lin {
  int c0 = -1;
  int coef[3] = {-1, -1, -1};
  int orig = -1;  // the expression the form was derived from (loop offsets taken as 0)
};

struct Plan {
  Program prog;
  Family family;
  std::string signature;            // normalised op listing the family was recognised from
  std::map<std::string, int> e;     // named index expressions
  std::map<std::string, Lin> lin;   // named pid-linear forms
  std::map<std::string, int64_t> k; // named compile-time constants (block sizes, arg indices)
  std::map<std::string, double> f;  // named float constants
  std::string source;               // TileProgram: the HIP source of the program's kernel; Gemm: of its epilogue functor, if any
  std::string fallback_source;      // Gemm, GemmW8A16: the same program as a TileProgram kernel (empty if that family declines it),
                                    // for launches whose strides, sizes or grid the matrix-product kernels do not take
};

// Generic family: HIP source for a program of structured loads, elementwise ops and stores
// (tile_codegen.cpp).  Throws Unsupported for anything else.  The kernel's argument block holds
// every kernel argument by index: { void *ptr[N]; long long ival[N]; double fval[N]; }, N = TILE_MAX_ARGS.
constexpr int TILE_MAX_ARGS = 32;
std::string tile_program_source(const Program &p, bool allow_persistent = true);  // (persistent: see tile_program_is_persistent)
bool tile_program_is_persistent(const std::string &source);  // the kernel walks the programs itself: any one-dimensional launch, lgx/lgy/lgz = the grid
bool tile_program_swaps_grid(const std::string &source);  // the launcher exchanges the grid's x and y for this source (when y fits)
// Matmul family with ops between the K loop and the store: the source of the functor that applies them to one
// accumulator value (tile_codegen.cpp), compiled at run time together with the kernels of gemm_device.h.
std::string gemm_epilogue_source(const Program &p, const std::vector<const SOp *> &ops, int acc, int out, int64_t BM, int64_t BN);

// Normalised listing of a program's ops (no shapes, no expression ids).
std::string signature(const Program &p);

// Recognises the family and extracts its bindings.  Throws Unsupported.
Plan make_plan(Program &&p);

}  // namespace tts
