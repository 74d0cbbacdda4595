// Run-time specialisation of a fused elementwise map: the register program that the planner
// assembled for the interpreter kernel (mapn_isa.h) is printed as straight-line HIP source inside
// a fixed mover (the load / predicate / store code of the hand-written map kernels) and compiled
// once per plan with hipRTC, at the first launch -- the point at which the reference compiles
// its launcher with g++ (backend/driver.py:274-345).  Every instruction becomes the same C
// expression the interpreter evaluates, with contraction off, so both paths give identical bits.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <hip/hiprtc.h>
#include <sys/stat.h>
#include <unistd.h>
#include <cstdio>
#include <cstdlib>

#include <sstream>
#include <string>

#include "kernels.h"

namespace tts {

namespace {

// the argument block of the generated kernel; its text below must describe the same layout
struct RtcArgs {
  const void *in[MAPN_MAX_IN];
  void *out[MAPN_MAX_OUT];
  long long in_off[MAPN_MAX_IN][4], out_off[MAPN_MAX_OUT][4], m_start[4];
  long long bound;
  int block, masked;
  float other[MAPN_MAX_IN];
  float imm[MAPN_MAX_IMM];
  // the programs of the gx x gy x gz grid are counted along x first (order 0) or along y first (1)
  int order, gx, gy;
  long long programs;
};

// Threads per program (as a shift) and programs per workgroup: a block's 16-byte chunks rounded up to a power of two share
// the 256 threads of a workgroup with the neighbouring programs' when there are 32 or fewer of them, that is when a
// program would leave half a wavefront or more idle.  (Programs of one or two wavefronts are better off alone: their
// addresses then stay in scalar registers; two programs of 128 chunks per workgroup measured 73 us against 69 on
// silu(x) * y, fp16, N = 2^26.)
struct Packing {
  int tpp_shift = 8, ppw = 1, threads = 256;
};
Packing packing_of(const MapNParams &p) {
  bool narrow = true;
  for (int k = 0; k < p.n_in; k++) narrow = narrow && p.in_type[k] != 0;
  for (int j = 0; j < p.n_out; j++) narrow = narrow && p.out_type[j] != 0;
  const int chunks = (p.block + (narrow ? 8 : 4) - 1) / (narrow ? 8 : 4);
  Packing k;
  if (chunks <= 32) {
    k.tpp_shift = 0;
    while ((1 << k.tpp_shift) < chunks) k.tpp_shift++;
    k.ppw = 256 >> k.tpp_shift;
  } else {
    // as many threads as the block has chunks, in whole wavefronts: idle wavefronts would only take up room
    k.threads = std::min(256, (chunks + 63) / 64 * 64);
  }
  return k;
}

const char *PRELUDE = R"SRC(
struct Args {
  const void *in[%IN%];
  void *out[%OUT%];
  long long in_off[%IN%][4], out_off[%OUT%][4], m_start[4];
  long long bound;
  int block, masked;
  float other[%IN%];
  float imm[%IMM%];
  int order, gx, gy;
  long long programs;
};
static_assert(sizeof(Args) == %SIZE%, "argument block layout");
// inputs are read once and outputs written once: nontemporal both ways (gelu(x + b), fp32, N = 2^26: 132 -> 123 us)
constexpr int W = %W%;  // elements per thread and pass: 4, or 8 when every tensor is 16 bits wide (16-byte accesses either way)
typedef float f4 __attribute__((ext_vector_type(4), aligned(4)));
typedef unsigned short hw __attribute__((ext_vector_type(W)));
#define affine(a) ((a)[0] + (a)[1] * pidx + (a)[2] * pidy + (a)[3] * pidz)
__device__ inline float up_f16(unsigned short h) { _Float16 f; __builtin_memcpy(&f, &h, 2); return (float)f; }
// The empty asm hides where f comes from: the compiler otherwise folds a multiplication into the narrowing (v_fma_mixlo_f16
// with an addend of +0), which rounds once instead of twice and turns a product of -0 into +0.
__device__ inline unsigned short down_f16(float f) { asm("" : "+v"(f)); _Float16 h = (_Float16)f; unsigned short r; __builtin_memcpy(&r, &h, 2); return r; }
// for values that an fp16 holds exactly (whatever has the type f16 here): nothing to round, so nothing to hide, and the
// compiler may cancel this against the widening before it
__device__ inline unsigned short down_f16_exact(float f) { _Float16 h = (_Float16)f; unsigned short r; __builtin_memcpy(&r, &h, 2); return r; }
__device__ inline float up_bf16(unsigned short h) { __bf16 b; __builtin_memcpy(&b, &h, 2); return (float)b; }
// the hardware conversion (v_cvt_pk_bf16_f32: round to nearest even); NaNs keep their sign and high payload bits
__device__ inline unsigned short down_bf16(float f) {
  if (f != f) return (unsigned short)((__float_as_uint(f) >> 16) | 0x40);
  __bf16 h = (__bf16)f; unsigned short r; __builtin_memcpy(&r, &h, 2); return r;
}
__device__ inline float maximum_f(float a, float b) { return (a != a || b != b) ? __builtin_nanf("") : fmaxf(a, b); }
__device__ inline float minimum_f(float a, float b) { return (a != a || b != b) ? __builtin_nanf("") : fminf(a, b); }
__device__ inline float as_bool(bool b) { return b ? 1.0f : 0.0f; }
__device__ inline void load_f32(float (&v)[W], const void *base, int i, int valid, float other) {
  const float *p = (const float *)base + i;
  if (valid >= 4) { f4 w = __builtin_nontemporal_load((const f4 *)p); v[0] = w[0]; v[1] = w[1]; v[2] = w[2]; v[3] = w[3]; return; }
  for (int e = 0; e < 4; e++) v[e] = e < valid ? p[e] : other;
}
template <bool BF16>
__device__ inline void load_h(float (&v)[W], const void *base, int i, int valid, float other) {
  const unsigned short *p = (const unsigned short *)base + i;
  unsigned short h[W];
  for (int e = 0; e < W; e++) h[e] = 0;
  if (valid >= W && (((unsigned long long)p) & (2 * W - 1)) == 0) { hw w = __builtin_nontemporal_load((const hw *)p); for (int e = 0; e < W; e++) h[e] = w[e]; }
  else for (int e = 0; e < W && e < valid; e++) h[e] = p[e];
  for (int e = 0; e < W; e++) v[e] = e < valid ? (BF16 ? up_bf16(h[e]) : up_f16(h[e])) : other;
}
__device__ inline void store_f32(void *base, int i, int valid, const float (&v)[W]) {
  float *p = (float *)base + i;
  if (valid >= 4) { f4 w = {v[0], v[1], v[2], v[3]}; __builtin_nontemporal_store(w, (f4 *)p); return; }
  for (int e = 0; e < valid; e++) p[e] = v[e];
}
template <bool BF16>
__device__ inline void store_h(void *base, int i, int valid, const float (&v)[W]) {
  unsigned short *p = (unsigned short *)base + i;
  hw w;
  for (int e = 0; e < W; e++) w[e] = BF16 ? down_bf16(v[e]) : down_f16_exact(v[e]);  // (stored values have been rounded to the type already)
  if (valid >= W && (((unsigned long long)p) & (2 * W - 1)) == 0) { __builtin_nontemporal_store(w, (hw *)p); return; }
  for (int e = 0; e < W && e < valid; e++) p[e] = w[e];
}
)SRC";

std::string replace_all(std::string s, const std::string &from, const std::string &to) {
  for (size_t pos = 0; (pos = s.find(from, pos)) != std::string::npos; pos += to.size()) s.replace(pos, from.size(), to);
  return s;
}

std::string expression(int op, const std::string &a, const std::string &b, const std::string &c) {
  switch (op) {
    case MO_MOV: return a;
    case MO_ADD: return a + " + " + b;
    case MO_SUB: return a + " - " + b;
    case MO_MUL: return a + " * " + b;
    case MO_DIV: return a + " / " + b;
    case MO_MAXNUM: return "fmaxf(" + a + ", " + b + ")";
    case MO_MINNUM: return "fminf(" + a + ", " + b + ")";
    case MO_MAXIMUM: return "maximum_f(" + a + ", " + b + ")";
    case MO_MINIMUM: return "minimum_f(" + a + ", " + b + ")";
    case MO_NEG: return "-" + a;
    case MO_ABS: return "fabsf(" + a + ")";
    case MO_EXP: return "expf(" + a + ")";
    case MO_EXP2: return "exp2f(" + a + ")";
    case MO_LOG: return "logf(" + a + ")";
    case MO_LOG2: return "log2f(" + a + ")";
    case MO_SQRT: return "sqrtf(" + a + ")";
    case MO_RSQRT: return "1.0f / sqrtf(" + a + ")";
    case MO_SIN: return "sinf(" + a + ")";
    case MO_COS: return "cosf(" + a + ")";
    case MO_TANH: return "tanhf(" + a + ")";
    case MO_ERF: return "erff(" + a + ")";
    case MO_FLOOR: return "floorf(" + a + ")";
    case MO_CEIL: return "ceilf(" + a + ")";
    case MO_FMA: return "fmaf(" + a + ", " + b + ", " + c + ")";
    case MO_SELECT: return a + " != 0.f ? " + b + " : " + c;
    case MO_AND: return "as_bool(" + a + " != 0.f && " + b + " != 0.f)";
    case MO_OR: return "as_bool(" + a + " != 0.f || " + b + " != 0.f)";
    case MO_XOR: return "as_bool((" + a + " != 0.f) != (" + b + " != 0.f))";
    case MO_CMP_OEQ: return "as_bool(" + a + " == " + b + ")";
    case MO_CMP_ONE: return "as_bool(" + a + " < " + b + " || " + a + " > " + b + ")";
    case MO_CMP_OLT: return "as_bool(" + a + " < " + b + ")";
    case MO_CMP_OLE: return "as_bool(" + a + " <= " + b + ")";
    case MO_CMP_OGT: return "as_bool(" + a + " > " + b + ")";
    case MO_CMP_OGE: return "as_bool(" + a + " >= " + b + ")";
    case MO_CMP_UNE: return "as_bool(!(" + a + " == " + b + "))";
    case MO_CMP_UEQ: return "as_bool(!(" + a + " < " + b + " || " + a + " > " + b + "))";
    case MO_CMP_ULT: return "as_bool(!(" + a + " >= " + b + "))";
    case MO_CMP_ULE: return "as_bool(!(" + a + " > " + b + "))";
    case MO_CMP_UGT: return "as_bool(!(" + a + " <= " + b + "))";
    case MO_CMP_UGE: return "as_bool(!(" + a + " < " + b + "))";
    case MO_CMP_ORD: return "as_bool(" + a + " == " + a + " && " + b + " == " + b + ")";
    case MO_CMP_UNO: return "as_bool(" + a + " != " + a + " || " + b + " != " + b + ")";
  }
  return "0.f";
}

std::string source_of(const MapNParams &p) {
  std::string src = PRELUDE;
  src = replace_all(src, "%IN%", std::to_string(MAPN_MAX_IN));
  src = replace_all(src, "%OUT%", std::to_string(MAPN_MAX_OUT));
  src = replace_all(src, "%IMM%", std::to_string(MAPN_MAX_IMM));
  src = replace_all(src, "%SIZE%", std::to_string(sizeof(RtcArgs)));
  bool narrow = true;
  for (int k = 0; k < p.n_in; k++) narrow = narrow && p.in_type[k] != 0;
  for (int j = 0; j < p.n_out; j++) narrow = narrow && p.out_type[j] != 0;
  src = replace_all(src, "%W%", narrow ? "8" : "4");
  std::ostringstream os;
  os << src;
  // The launch is one-dimensional: a workgroup takes ppw consecutive programs (blocks of a few dozen elements would
  // otherwise each occupy a wavefront of mostly idle lanes, and a launch of them is bound by the rate at which
  // workgroups start), counted along the grid axis on which the first output advances least, so that workgroups
  // that run at the same time write neighbouring memory.
  os << "extern \"C\" __global__ __launch_bounds__(256) void fused_map(const Args p) {\n"
     << "  constexpr int TPP_SHIFT = " << packing_of(p).tpp_shift << ", PPW = " << packing_of(p).ppw << ";\n"
     << "  const int lane = PPW == 1 ? (int)threadIdx.x : (int)(threadIdx.x & ((1 << TPP_SHIFT) - 1));\n"
     << "  const long long prog = PPW == 1 ? (long long)blockIdx.x : (long long)blockIdx.x * PPW + (threadIdx.x >> TPP_SHIFT);\n"
     << "  if (PPW > 1 && prog >= p.programs) return;\n"
     << "  long long pidx = prog, pidy = 0, pidz = 0;\n"
     << "  if (p.programs != p.gx) {\n"
     << "    if (p.programs <= 0xffffffffLL) {\n"
     << "      const unsigned l = (unsigned)prog, n0 = p.order ? p.gy : p.gx, n1 = p.order ? p.gx : p.gy;\n"
     << "      const unsigned a0 = l % n0, r = l / n0, a1 = r % n1;\n"
     << "      pidz = r / n1; pidx = p.order ? a1 : a0; pidy = p.order ? a0 : a1;\n"
     << "    } else {\n"
     << "      const long long n0 = p.order ? p.gy : p.gx, n1 = p.order ? p.gx : p.gy;\n"
     << "      const long long a0 = prog % n0, r = prog / n0, a1 = r % n1;\n"
     << "      pidz = r / n1; pidx = p.order ? a1 : a0; pidy = p.order ? a0 : a1;\n"
     << "    }\n"
     << "  }\n"
     << "  int d = p.block;\n"
     << "  if (p.masked) { long long left = p.bound - affine(p.m_start); d = left < 0 ? 0 : left < p.block ? (int)left : p.block; }\n";
  for (int k = 0; k < p.n_in; k++)
    os << "  const char *in" << k << " = (const char *)p.in[" << k << "] + affine(p.in_off[" << k << "]) * " << (p.in_type[k] == 0 ? 4 : 2) << ";\n";
  for (int j = 0; j < p.n_out; j++)
    os << "  char *out" << j << " = (char *)p.out[" << j << "] + affine(p.out_off[" << j << "]) * " << (p.out_type[j] == 0 ? 4 : 2) << ";\n";
  os << "  for (int i = W * lane; i < d; i += (W << TPP_SHIFT)) {\n    const int valid = d - i;\n";
  for (int r = 0; r < p.n_regs; r++) os << "    float r" << r << "[W];\n";
  os << "    float prev[W];\n    for (int e = 0; e < W; e++) prev[e] = 0.f;\n";
  for (int k = 0; k < p.n_in; k++) {
    const char *fn = p.in_type[k] == 0 ? "load_f32" : p.in_type[k] == 1 ? "load_h<false>" : "load_h<true>";
    os << "    " << fn << "(r" << (int)p.in_reg[k] << ", in" << k << ", i, valid, p.other[" << k << "]);\n";
  }
  for (int t = 0; t < p.n_ins; t++) {
    const MapIns &ins = p.ins[t];
    auto operand = [&](int kind, int idx) {
      if (kind == MS_PREV) return std::string("prev[e]");
      if (kind == MS_IMM) return "p.imm[" + std::to_string(idx) + "]";
      return "r" + std::to_string(idx) + "[e]";
    };
    std::string e = expression(ins.op, operand(ins.kinds & 3, ins.a), operand((ins.kinds >> 2) & 3, ins.b), operand((ins.kinds >> 4) & 3, ins.c));
    os << "    { float t[W];\n      for (int e = 0; e < W; e++) { float v = " << e << ";";
    if (ins.round == 1) os << " v = up_f16(down_f16(v));";
    if (ins.round == 2) os << " v = up_bf16(down_bf16(v));";
    os << " t[e] = v; }\n      for (int e = 0; e < W; e++) { prev[e] = t[e];";
    if (!(ins.kinds & 64)) os << " r" << (int)ins.dst << "[e] = t[e];";
    os << " } }\n";
  }
  for (int j = 0; j < p.n_out; j++) {
    const char *fn = p.out_type[j] == 0 ? "store_f32" : p.out_type[j] == 1 ? "store_h<false>" : "store_h<true>";
    os << "    " << fn << "(out" << j << ", i, valid, r" << (int)p.out_reg[j] << ");\n";
  }
  os << "  }\n}\n";
  return os.str();
}

}  // namespace

struct RtcModule {
  hipModule_t module = nullptr;
  hipFunction_t fn = nullptr;
  int resident = 0;  // workgroups of 256 threads a CU holds at once (0: not asked yet)
};

std::string fused_map_source(const MapNParams &p) { return source_of(p); }

namespace {
// Compiled code objects are kept on disk, as the reference keeps its compiled launchers in Triton's cache
// (backend/driver.py:274-282,344-345): <dir>/<hash of source, options and hipRTC version>.hsaco, with <dir> =
// $TTS_RTC_CACHE, else $TRITON_CACHE_DIR/tts_rtc, else $HOME/.triton/cache/tts_rtc.  TTS_RTC_CACHE=off disables it.
// (no packed fp32 instructions, as in the library's own build: the compiler forms them from ordinary float code otherwise)
const char *const RTC_OPTS[] = {"--offload-arch=gfx950", "-O3", "-ffp-contract=off", "-fhip-fp32-correctly-rounded-divide-sqrt",
                                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};

std::string cache_dir() {
  const char *own = getenv("TTS_RTC_CACHE");
  if (own) return std::string(own) == "off" ? "" : own;
  if (const char *t = getenv("TRITON_CACHE_DIR")) return std::string(t) + "/tts_rtc";
  if (const char *h = getenv("HOME")) return std::string(h) + "/.triton/cache/tts_rtc";
  return "";
}

std::string cache_key(const std::string &source) {
  int major = 0, minor = 0;
  hiprtcVersion(&major, &minor);
  std::string all = source + "\n" + std::to_string(major) + "." + std::to_string(minor);
  for (const char *o : RTC_OPTS) all += std::string("\n") + o;
  uint64_t h1 = 1469598103934665603ull, h2 = 0x9E3779B97F4A7C15ull;  // two FNV-1a style passes: 128 bits of name
  for (unsigned char c : all) {
    h1 = (h1 ^ c) * 1099511628211ull;
    h2 = (h2 + c) * 0x100000001B3ull ^ (h2 >> 29);
  }
  char buf[40];
  snprintf(buf, sizeof buf, "%016llx%016llx", (unsigned long long)h1, (unsigned long long)h2);
  return buf;
}

bool read_file(const std::string &path, std::string *out) {
  FILE *f = fopen(path.c_str(), "rb");
  if (!f) return false;
  std::string data;
  char chunk[65536];
  size_t n;
  while ((n = fread(chunk, 1, sizeof chunk, f)) > 0) data.append(chunk, n);
  fclose(f);
  if (data.empty()) return false;
  *out = std::move(data);
  return true;
}

void write_file(const std::string &dir, const std::string &name, const std::string &data) {
  // best effort: mkdir -p, write to a temporary name, rename (so that a concurrent reader never sees half a file)
  for (size_t i = 1; i <= dir.size(); i++)
    if (i == dir.size() || dir[i] == '/') mkdir(dir.substr(0, i).c_str(), 0777);
  const std::string tmp = dir + "/" + name + ".tmp" + std::to_string((long)getpid());
  FILE *f = fopen(tmp.c_str(), "wb");
  if (!f) return;
  const bool ok = fwrite(data.data(), 1, data.size(), f) == data.size();
  if (fclose(f) != 0 || !ok || rename(tmp.c_str(), (dir + "/" + name).c_str()) != 0) remove(tmp.c_str());
}
}  // namespace

static hipError_t rtc_compile_with(const std::string &source, const char *entry, RtcModule **out, std::string *err, bool use_cache) {
  auto *m = new RtcModule;
  const std::string dir = use_cache ? cache_dir() : "", name = dir.empty() ? "" : cache_key(source) + ".hsaco";
  std::string code;
  const bool cached = !dir.empty() && read_file(dir + "/" + name, &code);
  if (!cached) {
    hiprtcProgram prog;
    if (hiprtcCreateProgram(&prog, source.c_str(), "kernel.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS) {
      *err = "hiprtcCreateProgram failed";
      delete m;
      return hipErrorUnknown;
    }
    // no contraction into fmas, IEEE division and square root: the reference's loops are plain scalar C semantics
    hiprtcResult r = hiprtcCompileProgram(prog, (int)(sizeof RTC_OPTS / sizeof RTC_OPTS[0]), RTC_OPTS);
    if (r != HIPRTC_SUCCESS) {
      size_t n = 0;
      hiprtcGetProgramLogSize(prog, &n);
      std::string log(n, '\0');
      if (n) hiprtcGetProgramLog(prog, &log[0]);
      *err = std::string("hipRTC: ") + hiprtcGetErrorString(r) + "\n" + log;
      hiprtcDestroyProgram(&prog);
      delete m;
      return hipErrorUnknown;
    }
    size_t size = 0;
    hiprtcGetCodeSize(prog, &size);
    code.assign(size, '\0');
    hiprtcGetCode(prog, &code[0]);
    hiprtcDestroyProgram(&prog);
  }
  hipError_t e = hipModuleLoadData(&m->module, code.data());
  if (e == hipSuccess) e = hipModuleGetFunction(&m->fn, m->module, entry);
  if (e != hipSuccess && cached) {  // a damaged cache file: forget it and compile
    if (m->module) (void)hipModuleUnload(m->module);
    delete m;
    remove((dir + "/" + name).c_str());
    return rtc_compile_with(source, entry, out, err, false);
  }
  if (e != hipSuccess) {
    *err = std::string("loading the compiled kernel: ") + hipGetErrorString(e);
    if (m->module) (void)hipModuleUnload(m->module);
    delete m;
    return e;
  }
  if (!cached && !dir.empty()) write_file(dir, name, code);
  if (getenv("TTS_RTC_REPORT")) {  // tuning aid: what the run-time compiler made of the kernel
    int regs = -1, scratch = -1, lds = -1;
    (void)hipFuncGetAttribute(&regs, HIP_FUNC_ATTRIBUTE_NUM_REGS, m->fn);
    (void)hipFuncGetAttribute(&scratch, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, m->fn);
    (void)hipFuncGetAttribute(&lds, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, m->fn);
    int major = 0, minor = 0;
    hiprtcVersion(&major, &minor);
    fprintf(stderr, "tts rtc: %s: %d registers, %d bytes of scratch per lane, %d bytes of LDS, %zu bytes of code (%s, hipRTC %d.%d)\n", entry, regs,
            scratch, lds, code.size(), cached ? "from the cache" : "compiled", major, minor);
  }
  *out = m;
  return hipSuccess;
}

hipError_t rtc_compile(const std::string &source, const char *entry, RtcModule **out, std::string *err) {
  return rtc_compile_with(source, entry, out, err, true);
}

void rtc_release(RtcModule *m) {
  if (!m) return;
  if (m->module) (void)hipModuleUnload(m->module);
  delete m;
}

hipError_t rtc_launch(RtcModule *m, int gx, int gy, int gz, int block, void *args, size_t size, hipStream_t s) {
  void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, args, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
  return hipModuleLaunchKernel(m->fn, gx, gy, gz, block, 1, 1, 0, s, nullptr, config);
}

int rtc_resident_workgroups(RtcModule *m) {
  if (m->resident == 0) {
    int n = 0;
    m->resident = hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&n, m->fn, 256, 0) == hipSuccess && n > 0 ? n : 1;
  }
  return m->resident;
}

const char *gemm_device_source() {
  static const char *text =
#include "gemm_device.inc"
      ;
  return text;
}

hipError_t fused_map_compile(const MapNParams &p, RtcModule **out, std::string *err) { return rtc_compile(source_of(p), "fused_map", out, err); }

hipError_t fused_map_launch(RtcModule *m, const MapNParams &p, int gx, int gy, int gz, hipStream_t s) {
  RtcArgs a{};
  auto put = [](long long (&dst)[4], const Affine &src) {
    dst[0] = src.c0;
    for (int i = 0; i < 3; i++) dst[1 + i] = src.c[i];
  };
  for (int k = 0; k < p.n_in; k++) {
    a.in[k] = p.in[k];
    put(a.in_off[k], p.in_off[k]);
    a.other[k] = p.in_other[k];
  }
  for (int j = 0; j < p.n_out; j++) {
    a.out[j] = p.out[j];
    put(a.out_off[j], p.out_off[j]);
  }
  put(a.m_start, p.m_start);
  a.bound = p.bound;
  a.block = p.block;
  a.masked = p.masked;
  for (int q = 0; q < MAPN_MAX_IMM; q++) a.imm[q] = p.imm[q];
  a.programs = (long long)gx * gy * gz;
  a.gx = gx;
  a.gy = gy;
  // count along y first when the first output (or, without one, the first input) advances less per step of y than of x
  const Affine &lead = p.n_out ? p.out_off[0] : p.in_off[0];
  a.order = gy > 1 && lead.c[1] != 0 && (lead.c[0] == 0 || std::llabs(lead.c[1]) < std::llabs(lead.c[0])) ? 1 : 0;
  const Packing k = packing_of(p);
  const long long groups = (a.programs + k.ppw - 1) / k.ppw;
  if (groups > 0x7fffffffLL) return hipErrorInvalidValue;
  return rtc_launch(m, (int)groups, 1, 1, k.threads, &a, sizeof a, s);
}

}  // namespace tts
