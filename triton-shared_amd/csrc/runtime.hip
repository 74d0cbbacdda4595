// C ABI (include/tts_hip.h) and the launcher: resolves a plan's symbolic
// bindings for the scalar arguments and grid of one launch, checks what the
// whole-grid kernels assume, and enqueues one kernel for the whole grid.
//
// The reference runs `for x, for y, for z: kernel(args, grid, x, y, z)` on the
// calling thread (backend/driver.py:116-133).  Here the per-program index
// arithmetic the reference executes inside each program (offsets, valid
// extents) is evaluated on the host once per distinct (scalars, grid) and
// cached; the device kernels receive closed forms of it.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <array>
#include <cstring>
#include <list>
#include <map>
#include <memory>
#include <mutex>
#include <set>
#include <sstream>
#include <unordered_map>

#include "../../include/tts_hip.h"
#include "kernels.h"
#include "match.h"

using namespace tts;

namespace {

thread_local std::string g_error;

tts_status fail(tts_status st, const std::string &msg) {
  g_error = msg;
  return st;
}

char *dup_string(const std::string &s) {
  char *p = (char *)malloc(s.size() + 1);
  memcpy(p, s.c_str(), s.size() + 1);
  return p;
}

struct Invalid : std::runtime_error {
  using std::runtime_error::runtime_error;
};

// What tts_launch_noalloc refuses.  Not an Unsupported: a launch that the matrix-product families decline for a reason of
// their own goes on to the generic family's kernel and its binding is cached as such, whereas this refusal says nothing
// about the launch -- the same launch through tts_launch must still find the family's kernel, so nothing is cached.
struct WouldAllocate : std::runtime_error {
  using std::runtime_error::runtime_error;
};

thread_local bool g_no_alloc = false;  // set while tts_launch_noalloc runs on this thread
void may_allocate(const char *what) {
  if (g_no_alloc)
    throw WouldAllocate(std::string("tts_launch_noalloc: this launch needs ") + what + ", which allocates; run it once through tts_launch first");
}

// Everything a launch needs besides the pointers, resolved for one (scalars, grid).
struct Bound {
  Family family;
  Map1DParams map1d{};
  SoftmaxParams softmax{};
  LayerNormParams layernorm{};
  GemmParams gemm{};
  GemmW8A16Params w8{};
  MapNParams mapn{};
  bool empty = false;  // nothing to do (e.g. zero trip count with nothing stored)
  bool fallback = false;  // the family's kernels do not take this launch; the generic family's kernel for the same program runs it
  std::string describe;
  // matrix products with a fused epilogue: which program owns which BM x BN tile (device memory, owned by the binding)
  int *tile_pid = nullptr;
  int tiles_n = 0;
  Bound() = default;
  Bound(const Bound &) = delete;
  Bound &operator=(const Bound &) = delete;
  ~Bound() {
    if (tile_pid) (void)hipFree(tile_pid);
  }
};

}  // namespace

struct tts_plan {
  Plan plan;
  std::string family;
  std::vector<int> arg_kinds;
  // bindings per (grid, scalar arguments), least recently used last; the oldest goes when there are more than 256
  struct CacheEntry {
    std::shared_ptr<Bound> bound;
    std::list<std::string>::iterator pos;
  };
  std::unordered_map<std::string, CacheEntry> cache;
  std::list<std::string> lru;
  std::mutex mu;
  const char *last_kernel = "";
  // Split-K partial sums and arrival counters (device memory, owned by the plan), one set per stream the plan has been
  // launched on: launches on one stream run one after the other, launches on different streams may overlap and must
  // not share them.  Counters are zero between launches.
  struct SplitK {
    void *widened = nullptr;  // the int8-weight product's weights as fp16, for launches with many rows
    size_t widened_bytes = 0;
    float *workspace = nullptr;
    size_t workspace_bytes = 0;
    int *counters = nullptr;
    size_t counters_count = 0;
  };
  std::unordered_map<void *, SplitK> split_k;
  // Buffers a stream has outgrown.  Launches already enqueued (by this or another thread) may still use them, so they are
  // neither freed nor reused before the plan goes: growing never waits for the device.  A buffer grows to at least twice
  // its size, so the retired ones of a stream together are smaller than the one in use.
  std::vector<void *> retired;
  // A buffer of at least `need` bytes in *buf (of *have bytes); called with `mu` held.
  hipError_t grow(void **buf, size_t *have, size_t need) {
    if (*have >= need) return hipSuccess;
    size_t got = std::max(need, 2 * *have);
    void *fresh = nullptr;
    hipError_t e = hipMalloc(&fresh, got);
    if (e != hipSuccess && got > need) {
      (void)hipGetLastError();
      got = need;
      e = hipMalloc(&fresh, got);
    }
    if (e != hipSuccess) return e;
    if (*buf) retired.push_back(*buf);
    *buf = fresh;
    *have = got;
    return hipSuccess;
  }
  RtcModule *fused = nullptr;  // the kernel compiled for this plan at its first launch (fused maps, tile programs)
  bool fused_is_plain = false; // a tile program whose source is persistent but whose kernel with a workgroup per program was kept
  RtcModule *gemm_rtc[2] = {nullptr, nullptr};  // matrix products with a fused epilogue: one kernel per tiling
  RtcModule *fallback = nullptr;  // the generic family's kernel for a matrix-product plan (launches the product kernels decline)
  ~tts_plan() {
    for (auto &kv : split_k) {
      if (kv.second.workspace) (void)hipFree(kv.second.workspace);
      if (kv.second.widened) (void)hipFree(kv.second.widened);
      if (kv.second.counters) (void)hipFree(kv.second.counters);
    }
    for (void *p : retired) (void)hipFree(p);
    rtc_release(fused);
    rtc_release(fallback);
    for (RtcModule *m : gemm_rtc) rtc_release(m);
  }
};

namespace {

struct Resolver {
  const Plan &pl;
  const ExprPool &X;
  std::vector<int64_t> ints;
  std::vector<double> floats;
  int g[3];
  Resolver(const Plan &p, const tts_arg *args, int n, int gx, int gy, int gz) : pl(p), X(p.prog.pool), g{gx, gy, gz} {
    ints.assign(n, 0);
    floats.assign(n, 0.0);
    for (int i = 0; i < n; i++) {
      if (args[i].kind == TTS_ARG_INT) ints[i] = args[i].v.i;
      if (args[i].kind == TTS_ARG_FLOAT) floats[i] = args[i].v.f;
    }
  }
  EvalEnv env(int px = 0, int py = 0, int pz = 0) const {
    EvalEnv e;
    e.args = ints.data();
    e.pid[0] = px; e.pid[1] = py; e.pid[2] = pz;
    e.nprog[0] = g[0]; e.nprog[1] = g[1]; e.nprog[2] = g[2];
    e.iv.assign(pl.prog.num_loops, 0);
    e.iter.assign(pl.prog.num_loops, {});
    e.result.assign(pl.prog.num_loops, {});
    return e;
  }
  int64_t ev(const std::string &name, const EvalEnv &e) const { return X.eval(pl.e.at(name), e); }
  int64_t ev0(const std::string &name) const { return ev(name, env()); }
  Affine affine(const std::string &name) const {
    const Lin &l = pl.lin.at(name);
    EvalEnv e = env();
    Affine a;
    a.c0 = X.eval(l.c0, e);
    for (int k = 0; k < 3; k++) a.c[k] = X.eval(l.coef[k], e);
    if (l.orig >= 0) {
      // the linear form was derived looking through i32 -> index extensions; confirm at every corner of the grid
      // (a coefficient may be negative, so the extreme offset can sit at any of them) that no 32-bit product wrapped
      for (int corner = 0; corner < 8; corner++) {
        const int px = (corner & 1) ? g[0] - 1 : 0, py = (corner & 2) ? g[1] - 1 : 0, pz = (corner & 4) ? g[2] - 1 : 0;
        if (((corner & 1) && g[0] == 1) || ((corner & 2) && g[1] == 1) || ((corner & 4) && g[2] == 1)) continue;  // same program as another corner
        EvalEnv at = env(px, py, pz);
        int64_t want = X.eval(l.orig, at);
        int64_t got = a.c0 + a.c[0] * px + a.c[1] * py + a.c[2] * pz;
        if (want != got)
          throw Invalid("32-bit overflow in the kernel's index arithmetic for '" + name + "' at program (" + std::to_string(px) + ", " +
                        std::to_string(py) + ", " + std::to_string(pz) + ") of the grid");
      }
    }
    return a;
  }
};

std::string show(const Affine &a) {
  std::ostringstream os;
  os << a.c0 << "+" << a.c[0] << "*x+" << a.c[1] << "*y+" << a.c[2] << "*z";
  return os.str();
}

void bind_map1d(const Resolver &r, Bound &b) {
  Map1DParams &p = b.map1d;
  p.xo = r.affine("x_off");
  p.yo = r.affine("y_off");
  p.zo = r.affine("z_off");
  p.block = (int)r.pl.k.at("block");
  p.masked = (int)r.pl.k.at("masked");
  p.op = (int)r.pl.k.at("op");
  p.swap = (int)r.pl.k.at("swap");
  if (p.masked) {
    p.m_start = r.affine("m_start");
    p.bound = r.ev0("bound");
  }
  std::ostringstream os;
  os << "kernel=map1d_f32\nop=" << p.op << "\nswap=" << p.swap << "\nblock=" << p.block << "\nmasked=" << p.masked
     << "\nx_off=" << show(p.xo) << "\ny_off=" << show(p.yo) << "\nz_off=" << show(p.zo) << "\nm_start=" << show(p.m_start)
     << "\nbound=" << p.bound << "\n";
  b.describe = os.str();
}

void bind_fused_map(const Resolver &r, Bound &b) {
  MapNParams &p = b.mapn;
  const auto &k = r.pl.k;
  p.block = (int)k.at("block");
  p.masked = (int)k.at("masked");
  p.n_in = (int)k.at("n_in");
  p.n_out = (int)k.at("n_out");
  p.n_ins = (int)k.at("n_ins");
  p.n_regs = (int)k.at("n_regs");
  if (p.masked) {
    p.m_start = r.affine("m_start");
    p.bound = r.ev0("bound");
  }
  std::ostringstream os;
  os << "kernel=mapn\nblock=" << p.block << "\nmasked=" << p.masked << "\nbound=" << p.bound << "\nm_start=" << show(p.m_start)
     << "\nregs=" << p.n_regs << "\n";
  for (int i = 0; i < p.n_in; i++) {
    std::string n = "in" + std::to_string(i);
    p.in_off[i] = r.affine(n + "_off");
    p.in_type[i] = (uint8_t)k.at(n + "_type");
    p.in_reg[i] = (uint8_t)k.at(n + "_reg");
    p.in_other[i] = (float)r.pl.f.at(n + "_other");
    os << n << "_off=" << show(p.in_off[i]) << "\n";
  }
  for (int j = 0; j < p.n_out; j++) {
    std::string n = "out" + std::to_string(j);
    p.out_off[j] = r.affine(n + "_off");
    p.out_type[j] = (uint8_t)k.at(n + "_type");
    p.out_reg[j] = (uint8_t)k.at(n + "_reg");
    os << n << "_off=" << show(p.out_off[j]) << "\n";
  }
  for (int q = 0; q < (int)k.at("n_imm"); q++) {
    int64_t arg = k.at("imm" + std::to_string(q) + "_arg");
    p.imm[q] = arg >= 0 ? (float)r.floats.at(arg) : (float)r.pl.f.at("imm" + std::to_string(q));
  }
  for (int t = 0; t < p.n_ins; t++) {
    uint64_t w = (uint64_t)k.at("ins" + std::to_string(t));
    MapIns &ins = p.ins[t];
    ins.op = w & 255; ins.dst = (w >> 8) & 255; ins.a = (w >> 16) & 255; ins.b = (w >> 24) & 255;
    ins.c = (w >> 32) & 255; ins.kinds = (w >> 40) & 255; ins.round = (w >> 48) & 255; ins.pad = 0;
    auto src = [&](int kind, int idx) {
      return kind == MS_PREV ? std::string("prev") : kind == MS_IMM ? "#" + std::to_string(p.imm[idx]) : "r" + std::to_string(idx);
    };
    os << "ins" << t << "=op" << (int)ins.op << " " << ((ins.kinds & 64) ? std::string("prev") : "r" + std::to_string(ins.dst)) << " <- "
       << src(ins.kinds & 3, ins.a) << ", " << src((ins.kinds >> 2) & 3, ins.b) << ", " << src((ins.kinds >> 4) & 3, ins.c)
       << (ins.round ? (ins.round == 1 ? " ->f16" : " ->bf16") : "") << "\n";
  }
  b.describe = os.str();
}

void bind_softmax(const Resolver &r, Bound &b) {
  SoftmaxParams &p = b.softmax;
  p.in_off = r.affine("in_off");
  p.out_off = r.affine("out_off");
  p.d_in = r.ev0("in_dims");
  p.d_out = r.ev0("out_dims");
  p.block = (int)r.pl.k.at("block");
  p.other = (float)r.pl.f.at("other");
  p.propagate_nan = r.pl.signature.find("maximumf") != std::string::npos;
  p.elem_kind = (int)r.pl.k.at("elem_kind");
  if (p.block > 65536) throw Unsupported("row_softmax: block sizes above 65536 are not implemented");
  std::ostringstream os;
  os << "kernel=softmax_f32\nelem=" << (p.elem_kind == 2 ? "f32" : p.elem_kind == 1 ? "bf16" : "f16") << "\nblock=" << p.block << "\nd_in=" << p.d_in << "\nd_out=" << p.d_out << "\nother=" << p.other
     << "\nin_off=" << show(p.in_off) << "\nout_off=" << show(p.out_off) << "\n";
  b.describe = os.str();
}

void bind_layernorm(const Resolver &r, Bound &b) {
  LayerNormParams &p = b.layernorm;
  p.x_off = r.affine("x_off");
  p.y_off = r.affine("y_off");
  p.w_off = r.affine("w_off");
  p.b_off = r.affine("b_off");
  p.mean_off = r.affine("mean_off");
  p.rstd_off = r.affine("rstd_off");
  p.N = r.ev0("N");
  p.eps = (float)r.floats.at(r.pl.k.at("eps_arg"));
  p.elem_kind = (int)r.pl.k.at("elem_kind");
  if (p.N > INT32_MAX) throw Invalid("layernorm_fwd: N does not fit 32 bits");
  std::ostringstream os;
  os << "kernel=layernorm_fwd\nN=" << p.N << "\neps=" << p.eps << "\nelem=" << (p.elem_kind == 2 ? "f32" : p.elem_kind == 1 ? "bf16" : "f16") << "\nx_off=" << show(p.x_off)
     << "\ny_off=" << show(p.y_off) << "\nw_off=" << show(p.w_off) << "\nb_off=" << show(p.b_off)
     << "\nmean_off=" << show(p.mean_off) << "\nrstd_off=" << show(p.rstd_off) << "\n";
  b.describe = os.str();
}

// Shared by both GEMM families: evaluates every program's tile origin and
// operand offsets, and proves that the grid of programs is exactly a dense
// C[M,N] = A[M,K] * B[K,N] tiled BM x BN, so that one kernel with its own
// tiling may compute it.
struct DenseGemm {
  int64_t M, N, K, lda, ldb, ldc;
  bool a_trans = false, b_trans = false;  // column-major operands (the tutorial's `b.T`): the pitch is the other stride
  std::vector<int> tile_pid;  // per BM x BN tile (row-major over the tile grid): linear id of the program that computes it
  int tiles_n = 0;
  // a batch of products of this shape: product b reads A and B and writes C batch_a * b, batch_b * b, batch_c * b elements further on
  int64_t batches = 1, batch_a = 0, batch_b = 0, batch_c = 0;
};

DenseGemm prove_dense_gemm(const Resolver &r, const char *F) {
  const Plan &pl = r.pl;
  const ExprPool &X = r.X;
  const int64_t BM = pl.k.at("BM"), BN = pl.k.at("BN"), BK = pl.k.at("BK");
  const int loop = (int)pl.k.at("loop");
  DenseGemm d;
  d.M = r.ev0("M");
  d.N = r.ev0("N");
  const int64_t sam = r.ev0("sam"), sak = r.ev0("sak"), sbk = r.ev0("sbk"), sbn = r.ev0("sbn"), scn = r.ev0("scn");
  d.ldc = r.ev0("scm");
  auto need = [&](bool ok, const std::string &why) {
    if (!ok) throw Unsupported(std::string(F) + ": " + why);
  };
  // the reference's lowering takes any strides (StructuredToMemref.cpp:105-138); these kernels want one stride of each
  // operand to be 1 and C row-major
  need(sak == 1 || sam == 1, "neither stride of A is 1");
  need(sbn == 1 || sbk == 1, "neither stride of B is 1");
  need(scn == 1, "the inner stride of C is not 1");
  d.a_trans = sak != 1;
  d.b_trans = sbn != 1;
  d.lda = d.a_trans ? sak : sam;
  d.ldb = d.b_trans ? sbn : sbk;
  need(d.M > 0 && d.N > 0, "empty problem");
  // a pitch of 0 is a broadcast operand, which the kernels read correctly; a negative one would become an unsigned byte
  // offset in the kernels, and rows of C that overlap or run backwards are not a dense product
  need(d.lda >= 0 && d.ldb >= 0, "a negative pitch of A or B");
  need(d.ldc > 0, "a pitch of C that is not positive");
  // K: the loop must sweep K in full blocks followed by at most one partial block
  int64_t trip = r.ev0("trip");
  need(trip >= 0 && trip < (1 << 24), "unreasonable K trip count");
  d.K = 0;
  {
    EvalEnv e = r.env();
    for (int64_t k = 0; k < trip; k++) {
      e.iv[loop] = k;
      int64_t kd = X.eval(pl.e.at("kdim"), e);
      need(kd == BK || (k == trip - 1 && kd >= 0), "the K mask does not describe a contiguous sweep of K");
      d.K += kd;
    }
  }
  need(r.ev0("a_kstep") == BK * sak && r.ev0("b_kstep") == BK * sbk, "operand pointers do not advance by one K block per iteration");
  // wraparound operands: the period is the whole matrix, so rows (columns) inside the problem are not affected
  const bool a_wraps = pl.e.count("a_mod"), b_wraps = pl.e.count("b_mod");
  if (a_wraps) need(r.ev0("a_mod") == d.M * sam, "A rows wrap around with a period other than M");
  if (b_wraps) need(r.ev0("b_mod") == d.N * sbn, "B columns wrap around with a period other than N");
  // tiles: every program's origin, offsets consistent with a dense layout, exact cover
  // A grid with a whole multiple of that many programs may be a batch of products (a batch index on another grid axis,
  // tutorial-style bmm): the programs then fall into groups that differ by constant offsets into A, B and C, each group
  // an exact cover of its own C, the offsets in arithmetic progression, the C's apart.
  const int64_t tm = (d.M + BM - 1) / BM, tn = (d.N + BN - 1) / BN;
  const int64_t programs = (int64_t)r.g[0] * r.g[1] * r.g[2];
  need(programs % (tm * tn) == 0 && programs >= tm * tn, "the grid does not have one program per output tile");
  d.batches = programs / (tm * tn);
  need(d.batches == 1 || (!a_wraps && !b_wraps), "a batch of products with wrapped operands");
  need(d.batches <= 65535, "more than 65535 products in a batch");
  std::map<std::array<int64_t, 3>, int> batch_of;  // offsets (A, B, C) of a product beyond those of a single one -> its place in `seen`
  std::vector<std::vector<char>> seen;
  d.tile_pid.assign(tm * tn, 0);
  d.tiles_n = (int)tn;
  for (int z = 0; z < r.g[2]; z++)
    for (int y = 0; y < r.g[1]; y++)
      for (int x = 0; x < r.g[0]; x++) {
        EvalEnv e = r.env(x, y, z);
        int64_t r0 = r.ev("r0", e), c0 = r.ev("c0", e);
        need(r0 >= 0 && c0 >= 0 && r0 % BM == 0 && c0 % BN == 0 && r0 / BM < tm && c0 / BN < tn, "a program's tile origin is off the tile grid");
        const std::array<int64_t, 3> off = {r.ev("a_base", e) - r0 * sam, r.ev("b_base", e) - c0 * sbn, r.ev("c_base", e) - (r0 * d.ldc + c0)};
        if (d.batches == 1) {
          need(off[0] == 0, "A tile offset is not row0 * its row stride");
          need(off[1] == 0, "B tile offset is not col0 * its column stride");
          need(off[2] == 0, "C tile offset is not row0 * ldc + col0");
        }
        auto at = batch_of.find(off);
        if (at == batch_of.end()) {
          need((int64_t)batch_of.size() < d.batches, "the programs do not fall into products of one shape");
          at = batch_of.emplace(off, (int)seen.size()).first;
          seen.emplace_back(tm * tn, 0);
        }
        char &s = seen[at->second][(r0 / BM) * tn + c0 / BN];
        need(!s, "two programs compute the same output tile");
        s = 1;
        if (d.batches == 1) d.tile_pid[(r0 / BM) * tn + c0 / BN] = x + r.g[0] * (y + r.g[1] * z);
        if (a_wraps) need(r.ev("a_wrapped", e) == r0 * sam, "the wrapped part of A's offset is not row0 * its row stride");
        if (b_wraps) need(r.ev("b_wrapped", e) == c0 * sbn, "the wrapped part of B's offset is not col0 * its column stride");
      }
  if (d.batches > 1) {
    // (every product has tm * tn distinct tiles, and there are batches * tm * tn programs: all covers are exact)
    need((int64_t)batch_of.size() == d.batches, "the programs do not fall into products of one shape");
    std::vector<std::array<int64_t, 3>> offs;
    for (auto &kv : batch_of) offs.push_back(kv.first);
    std::sort(offs.begin(), offs.end(), [](const std::array<int64_t, 3> &a, const std::array<int64_t, 3> &b) { return a[2] < b[2]; });
    need(offs[0][0] == 0 && offs[0][1] == 0 && offs[0][2] == 0, "the first product of a batch does not start at the arguments' addresses");
    d.batch_a = offs[1][0];
    d.batch_b = offs[1][1];
    d.batch_c = offs[1][2];
    for (int64_t b = 0; b < d.batches; b++)
      need(offs[b][0] == b * d.batch_a && offs[b][1] == b * d.batch_b && offs[b][2] == b * d.batch_c, "the products of a batch are not evenly spaced");
    need(d.batch_c >= (d.M - 1) * d.ldc + d.N, "the results of a batch's products overlap");
  }
  return d;
}

// The product with gathered rows (match.cpp: try_gemm_gathered): one program per BM x BN tile of C, rows of A through an
// index vector at rows_ptr + row0, the matrix of a block of BM rows picked by the id at block_ptr + row0 / BM.
void bind_gemm_gathered(const Resolver &r, Bound &b) {
  const Plan &pl = r.pl;
  const char *F = "gemm (gathered rows)";
  auto need = [&](bool ok, const std::string &why) {
    if (!ok) throw Unsupported(std::string(F) + ": " + why);
  };
  const int64_t BM = pl.k.at("BM"), BN = pl.k.at("BN"), BK = pl.k.at("BK");
  GemmParams &p = b.gemm;
  p.M = r.ev0("M"); p.N = r.ev0("N"); p.K = r.ev0("K");
  p.lda = r.ev0("sam"); p.ldb = r.ev0("sbk"); p.ldc = r.ev0("scm");
  p.is_bf16 = (int)pl.k.at("is_bf16");
  need(p.M > 0 && p.N > 0 && p.K >= 0, "empty problem");
  need(BM % 128 == 0, "blocks of rows that are not whole 128-row kernel tiles");
  need(r.ev0("b_kstep") == BK * p.ldb, "the B pointer does not advance by one K block per iteration");
  need(p.lda >= 0 && p.lda <= INT32_MAX && p.ldb >= 0, "negative or oversized pitches");
  const int64_t tm = (p.M + BM - 1) / BM, tn = (p.N + BN - 1) / BN;
  need((int64_t)r.g[0] * r.g[1] * r.g[2] == tm * tn, "the grid does not have one program per output tile");
  std::vector<char> seen(tm * tn, 0);
  for (int z = 0; z < r.g[2]; z++)
    for (int y = 0; y < r.g[1]; y++)
      for (int x = 0; x < r.g[0]; x++) {
        EvalEnv e = r.env(x, y, z);
        const int64_t r0 = r.ev("r0", e), c0 = r.ev("c0", e);
        need(r0 >= 0 && c0 >= 0 && r0 % BM == 0 && c0 % BN == 0 && r0 / BM < tm && c0 / BN < tn, "a program's tile origin is off the tile grid");
        char &s = seen[(r0 / BM) * tn + c0 / BN];
        need(!s, "two programs compute the same output tile");
        s = 1;
        need(r.ev("block_off", e) == r0 / BM, "the matrix id of a block of rows is not read from ids[row0 / BM]");
        need(r.ev("c_base", e) == r0 * p.ldc + c0, "C tile offset is not row0 * ldc + col0");
      }
  p.b_block_rows = (int)BM;
  p.b_block_stride = r.ev0("block_stride");
  p.gather_mul32 = 1 | (pl.k.at("mul32") ? 2 : 0);
  std::ostringstream os;
  os << "kernel=gemm_mfma\ngathered=1\nM=" << p.M << "\nN=" << p.N << "\nK=" << p.K << "\nlda=" << p.lda << "\nldb=" << p.ldb << "\nldc=" << p.ldc
     << "\nbf16=" << p.is_bf16 << "\nblock_rows=" << p.b_block_rows << "\nblock_stride=" << p.b_block_stride << "\n";
  b.describe = os.str();
}

void bind_gemm(const Resolver &r, Bound &b) {
  if (r.pl.k.count("gathered")) return bind_gemm_gathered(r, b);
  DenseGemm d = prove_dense_gemm(r, "gemm");
  GemmParams &p = b.gemm;
  p.M = d.M; p.N = d.N; p.K = d.K; p.lda = d.lda; p.ldb = d.ldb; p.ldc = d.ldc;
  p.a_trans = d.a_trans; p.b_trans = d.b_trans;
  p.is_bf16 = (int)r.pl.k.at("is_bf16");
  p.is_f32 = r.pl.k.count("is_f32") ? (int)r.pl.k.at("is_f32") : 0;
  p.batches = (int)d.batches; p.batch_a = d.batch_a; p.batch_b = d.batch_b; p.batch_c = d.batch_c;
  if (p.is_f32 && !r.pl.source.empty()) throw Unsupported("gemm: a fused epilogue on fp32 operands");
  if (p.batches > 1 && !r.pl.source.empty()) throw Unsupported("gemm: a fused epilogue on a batch of products");
  if (!r.pl.source.empty()) {  // a fused epilogue looks up the program that owns an element
    may_allocate("a table of tile owners on the device");
    hipError_t e = hipMalloc((void **)&b.tile_pid, d.tile_pid.size() * sizeof(int));
    if (e == hipSuccess) e = hipMemcpy(b.tile_pid, d.tile_pid.data(), d.tile_pid.size() * sizeof(int), hipMemcpyHostToDevice);
    if (e != hipSuccess) throw std::runtime_error(std::string("gemm: tile table: ") + hipGetErrorString(e));
    b.tiles_n = d.tiles_n;
  }
  std::ostringstream os;
  os << "kernel=gemm_mfma\nM=" << p.M << "\nN=" << p.N << "\nK=" << p.K << "\nlda=" << p.lda << "\nldb=" << p.ldb
     << "\nldc=" << p.ldc << "\nbf16=" << p.is_bf16 << "\nf32=" << p.is_f32 << "\na_trans=" << p.a_trans << "\nb_trans=" << p.b_trans << "\n";
  if (p.batches > 1) os << "batches=" << p.batches << "\nbatch_a=" << p.batch_a << "\nbatch_b=" << p.batch_b << "\nbatch_c=" << p.batch_c << "\n";
  b.describe = os.str();
}

void bind_w8a16(const Resolver &r, Bound &b) {
  DenseGemm d = prove_dense_gemm(r, "gemm_w8a16");
  if (d.a_trans || d.b_trans) throw Unsupported("gemm_w8a16: only row-major operands are implemented");
  if (d.batches > 1) throw Unsupported("gemm_w8a16: a batch of products");
  GemmW8A16Params &p = b.w8;
  p.M = d.M; p.N = d.N; p.K = d.K; p.lda = d.lda; p.ldw = d.ldb; p.ldc = d.ldc;
  p.split = gemm_w8a16_split(p);
  std::ostringstream os;
  os << "kernel=gemm_w8a16\nM=" << p.M << "\nN=" << p.N << "\nK=" << p.K << "\nlda=" << p.lda << "\nldw=" << p.ldw
     << "\nldc=" << p.ldc << "\nsplit=" << p.split << "\n";
  b.describe = os.str();
}

std::shared_ptr<Bound> resolve(tts_plan *h, int gx, int gy, int gz, const tts_arg *args, int n) {
  if (n != (int)h->arg_kinds.size())
    throw Invalid("expected " + std::to_string(h->arg_kinds.size()) + " kernel arguments, got " + std::to_string(n));
  std::string key;
  key.reserve(16 + 8 * n);
  int g[3] = {gx, gy, gz};
  key.append((const char *)g, sizeof g);
  for (int i = 0; i < n; i++) {
    if (args[i].kind != h->arg_kinds[i])
      throw Invalid("kernel argument " + std::to_string(i) + " has the wrong kind (pointer/integer/float)");
    if (args[i].kind != TTS_ARG_PTR) key.append((const char *)&args[i].v, 8);
  }
  std::lock_guard<std::mutex> lock(h->mu);
  auto it = h->cache.find(key);
  if (it != h->cache.end()) {
    h->lru.splice(h->lru.begin(), h->lru, it->second.pos);
    return it->second.bound;
  }
  auto b = std::make_shared<Bound>();
  b->family = h->plan.family;
  Resolver r(h->plan, args, n, gx, gy, gz);
  switch (b->family) {
    case Family::Map1D: bind_map1d(r, *b); break;
    case Family::RowSoftmax: bind_softmax(r, *b); break;
    case Family::LayerNormFwd: bind_layernorm(r, *b); break;
    case Family::Gemm:
    case Family::GemmW8A16:
      // what these families can only check now (strides, M, the grid's shape) may fail for a launch that is a valid
      // Triton program all the same: the generic family's kernel for the same program runs it
      try {
        if (b->family == Family::Gemm) bind_gemm(r, *b);
        else bind_w8a16(r, *b);
      } catch (const Unsupported &e) {
        if (h->plan.fallback_source.empty()) throw;
        b->fallback = true;
        b->describe = std::string("kernel=tile_program\nfallback_reason=") + e.what() + "\n";
      }
      break;
    case Family::FusedMap: bind_fused_map(r, *b); break;
    case Family::TileProgram: b->describe = "kernel=tile_program\n"; break;
  }
  h->lru.push_front(key);
  h->cache[key] = {b, h->lru.begin()};
  if (h->cache.size() > 256) {  // launches in flight hold their own reference to the binding they use
    h->cache.erase(h->lru.back());
    h->lru.pop_back();
  }
  return b;
}

template <class T>
T *ptr_arg(const tts_arg *args, const Plan &pl, const char *name) {
  return (T *)args[pl.k.at(name)].v.ptr;
}

template <class F>
tts_status guarded(F &&f) {
  try {
    return f();
  } catch (const Unsupported &e) {
    return fail(TTS_UNSUPPORTED, e.what());
  } catch (const WouldAllocate &e) {
    return fail(TTS_UNSUPPORTED, e.what());
  } catch (const Invalid &e) {
    return fail(TTS_INVALID, e.what());
  } catch (const std::exception &e) {
    return fail(TTS_INVALID, e.what());
  }
}

const char *PLAN_MAGIC = "tts.plan 1";

// ---- tts_launch_noalloc: the split-K scratch memory of callers that cannot allocate
// Partial tiles first, arrival counters behind them.  One copy of the array per GPU, held until the process ends.
constexpr size_t NOALLOC_WORKSPACE_BYTES = (size_t)8 << 20;
constexpr size_t NOALLOC_COUNTERS = 4096;
constexpr int NOALLOC_MAX_DEVICES = 64;

}  // namespace

// In host code this name is only a handle for hipGetSymbolAddress: the device address is looked up once per device
// (noalloc_scratch) and that pointer is what kernels and copies receive.
static __device__ __align__(256) unsigned char scratch[NOALLOC_WORKSPACE_BYTES + NOALLOC_COUNTERS * sizeof(int)];

namespace {

__global__ void clear_ints_kernel(int *p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// the current device's copy of `scratch`
unsigned char *noalloc_scratch() {
  static std::mutex mu;
  static unsigned char *ptrs[NOALLOC_MAX_DEVICES] = {};
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) throw std::runtime_error(std::string("hipGetDevice: ") + hipGetErrorString(e));
  if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) throw Invalid("tts_launch_noalloc: device ordinal out of range");
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) throw std::runtime_error(std::string("hipGetSymbolAddress(scratch): ") + hipGetErrorString(e));
    ptrs[dev] = (unsigned char *)p;
  }
  return ptrs[dev];
}

}  // namespace

extern "C" {

const char *tts_last_error(void) { return g_error.c_str(); }
void tts_free(void *p) { free(p); }

tts_status tts_ttir_to_structured(const char *ttir_text, char **out) {
  if (!ttir_text || !out) return fail(TTS_INVALID, "null argument");
  return guarded([&]() {
    Func f = parse_ttir(ttir_text);
    Program p = lower_ttir(f);
    *out = dup_string(print_program(p));
    return TTS_OK;
  });
}

tts_status tts_structured_to_plan(const char *structured_text, char **out_plan, size_t *out_len, char **out_name) {
  if (!structured_text || !out_plan || !out_len) return fail(TTS_INVALID, "null argument");
  return guarded([&]() {
    Program p = read_program(structured_text);
    std::string name = p.name;
    Plan pl = make_plan(std::move(p));  // refuses here, at compile time, if no family matches
    std::string bytes = std::string(PLAN_MAGIC) + " family=" + family_name(pl.family) + "\n" + structured_text;
    *out_plan = dup_string(bytes);
    *out_len = bytes.size();
    if (out_name) *out_name = dup_string(name);
    return TTS_OK;
  });
}

tts_status tts_plan_load(const char *plan_bytes, size_t len, tts_plan **out) {
  if (!plan_bytes || !out) return fail(TTS_INVALID, "null argument");
  return guarded([&]() {
    std::string text(plan_bytes, len);
    if (text.rfind(PLAN_MAGIC, 0) != 0) throw Invalid("not a tts launch plan");
    size_t nl = text.find('\n');
    std::string header = text.substr(0, nl);
    auto h = std::make_unique<tts_plan>();
    h->plan = make_plan(read_program(text.substr(nl + 1)));
    h->family = family_name(h->plan.family);
    if (header.find("family=" + h->family) == std::string::npos) throw Invalid("plan header and plan body disagree on the kernel family");
    for (auto &t : h->plan.prog.arg_types)
      h->arg_kinds.push_back(t.ptr ? TTS_ARG_PTR : t.is_float() ? TTS_ARG_FLOAT : TTS_ARG_INT);
    *out = h.release();
    return TTS_OK;
  });
}

void tts_plan_destroy(tts_plan *plan) { delete plan; }
const char *tts_plan_kernel_name(const tts_plan *plan) { return plan->plan.prog.name.c_str(); }
const char *tts_plan_family(const tts_plan *plan) { return plan->family.c_str(); }
const char *tts_plan_signature(const tts_plan *plan) { return plan->plan.signature.c_str(); }
int tts_plan_num_args(const tts_plan *plan) { return (int)plan->arg_kinds.size(); }
int tts_plan_arg_kind(const tts_plan *plan, int i) {
  return i >= 0 && i < (int)plan->arg_kinds.size() ? plan->arg_kinds[i] : -1;
}
const char *tts_plan_last_kernel(const tts_plan *plan) { return plan->last_kernel; }

tts_status tts_plan_describe_launch(tts_plan *plan, int gx, int gy, int gz, const tts_arg *args, int n, char **out) {
  if (!plan || !out || (n > 0 && !args)) return fail(TTS_INVALID, "null argument");
  return guarded([&]() {
    if ((int64_t)gx * gy * gz <= 0) {
      *out = dup_string("kernel=none\n");
      return TTS_OK;
    }
    auto b = resolve(plan, gx, gy, gz, args, n);
    *out = dup_string("family=" + plan->family + "\n" + b->describe);
    return TTS_OK;
  });
}

}  // extern "C"

namespace {

int compute_units() {  // of the current device (256 when the query fails)
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    return n;
  }();
  return cus;
}

// tts_launch and tts_launch_noalloc (no_alloc: nothing below may allocate device memory or compile)
tts_status launch_impl(tts_plan *plan, int gx, int gy, int gz, void *stream, const tts_arg *args, int n, bool no_alloc) {
  if (!plan || (n > 0 && !args)) return fail(TTS_INVALID, "null argument");
  struct Flag {
    bool saved;
    explicit Flag(bool v) : saved(g_no_alloc) { g_no_alloc = v; }
    ~Flag() { g_no_alloc = saved; }
  } flag(no_alloc);
  return guarded([&]() {
    if (gx < 0 || gy < 0 || gz < 0) throw Invalid("negative grid");
    if ((int64_t)gx * gy * gz == 0) return TTS_OK;  // backend/driver.py:117
    auto b = resolve(plan, gx, gy, gz, args, n);
    const Plan &pl = plan->plan;
    {
      // The device's grid holds 65535 along y and z; the reference's launcher loops over any extents
      // (backend/driver.py:116-133).  For larger ones every family launches one-dimensionally and numbers its programs
      // itself, as the compiled fused map and the row softmax always do (the matrix products use tilings of their own);
      // only the fused map's interpreter (a tuning aid) is left out.
      const char *mode = getenv("TTS_FUSED_MAP");
      const bool interpreter = pl.family == Family::FusedMap && !b->fallback && mode && std::string(mode) == "interpreter";
      if ((gy > 65535 || gz > 65535) && interpreter) throw Unsupported("grid y/z extents above 65535 on the fused map's interpreter");
      if ((int64_t)gx * gy * gz > INT32_MAX) throw Unsupported("more than 2^31 - 1 programs in a launch");
    }
    hipStream_t s = (hipStream_t)stream;
    hipError_t err = hipSuccess;
    const char *kname = "";
    // one workgroup of 256 threads per Triton program, on the kernel generated for the program (compiled at its first use)
    auto run_tile_program = [&](RtcModule **slot, const std::string &source) -> tts_status {
      struct { void *ptr[TILE_MAX_ARGS]; long long ival[TILE_MAX_ARGS]; double fval[TILE_MAX_ARGS]; int swap_xy, lgx, lgy, lgz; } a{};
      for (int i = 0; i < n; i++) {
        if (args[i].kind == TTS_ARG_PTR) a.ptr[i] = args[i].v.ptr;
        else if (args[i].kind == TTS_ARG_INT) a.ival[i] = args[i].v.i;
        else a.fval[i] = args[i].v.f;
      }
      bool persistent = false;
      {
        std::lock_guard<std::mutex> lock(plan->mu);
        if (!*slot) {
          may_allocate("to compile the program's kernel");
          std::string why;
          hipError_t ce = rtc_compile(source, "tile_program", slot, &why);
          if (ce != hipSuccess) return fail(TTS_HIP_ERROR, "tile_program: " + why + "\n--- source ---\n" + source);
          // A persistent kernel keeps what its programs share in registers.  When that costs it workgroups per CU (fewer
          // than four fit), the kernel with a workgroup per program is compiled as well, and kept unless fewer of it fit
          // (LayerNorm's input gradient on rows of 8192: 2 against 3 per CU, 50 us against 41).
          if (slot == &plan->fused && tile_program_is_persistent(source) && rtc_resident_workgroups(*slot) < 4) {
            const std::string plain = tile_program_source(pl.prog, false);
            RtcModule *other = nullptr;
            if (rtc_compile(plain, "tile_program", &other, &why) == hipSuccess && rtc_resident_workgroups(other) >= rtc_resident_workgroups(*slot)) {
              rtc_release(*slot);
              *slot = other;
              plan->fused_is_plain = true;
            } else if (other) {
              rtc_release(other);
            }
          }
        }
        persistent = tile_program_is_persistent(source) && !(slot == &plan->fused && plan->fused_is_plain);
      }
      kname = "tile_program (hipRTC)";
      // the program asks for neighbouring workgroups along program_id(1) (tile_codegen.cpp); grid.y holds 65535 at most
      a.swap_xy = tile_program_swaps_grid(source) && gy > 1 && gx <= 65535 ? 1 : 0;
      if (persistent) {
        // as many workgroups as the device holds at once, four per CU at most, walk the programs (RMSNorm of 4096 rows:
        // 768 / 1024 / 2048 workgroups took 26.5 / 25.6 / 26.2 us; a kernel whose registers admit three per CU runs a
        // quarter of 1024 workgroups after the others)
        a.swap_xy = 0;
        a.lgx = gx; a.lgy = gy; a.lgz = gz;
        const int64_t per_cu = std::min(4, rtc_resident_workgroups(*slot));
        err = rtc_launch(*slot, (int)std::min<int64_t>((int64_t)gx * gy * gz, per_cu * compute_units()), 1, 1, 256, &a, sizeof a, s);
      } else if ((a.swap_xy ? gx : gy) > 65535 || gz > 65535) {  // the kernel numbers the programs itself (x fastest)
        a.swap_xy = 0;
        a.lgx = gx; a.lgy = gy; a.lgz = gz;
        err = rtc_launch(*slot, (int)((int64_t)gx * gy * gz), 1, 1, 256, &a, sizeof a, s);
      } else {
        err = a.swap_xy ? rtc_launch(*slot, gy, gx, gz, 256, &a, sizeof a, s) : rtc_launch(*slot, gx, gy, gz, 256, &a, sizeof a, s);
      }
      return TTS_OK;
    };
    if (b->fallback) {
      tts_status st = run_tile_program(&plan->fallback, pl.fallback_source);
      if (st != TTS_OK) return st;
      plan->last_kernel = kname;
      if (err != hipSuccess) return fail(TTS_HIP_ERROR, std::string("kernel launch failed: ") + hipGetErrorString(err));
      return TTS_OK;
    }
    switch (b->family) {
      case Family::Map1D: {
        Map1DParams p = b->map1d;
        p.x = ptr_arg<const float>(args, pl, "x_arg");
        p.y = ptr_arg<const float>(args, pl, "y_arg");
        p.z = ptr_arg<float>(args, pl, "z_arg");
        err = launch_map1d(p, gx, gy, gz, s, &kname);
        break;
      }
      case Family::FusedMap: {
        MapNParams p = b->mapn;
        for (int i = 0; i < p.n_in; i++) p.in[i] = ptr_arg<const void>(args, pl, ("in" + std::to_string(i) + "_arg").c_str());
        for (int j = 0; j < p.n_out; j++) p.out[j] = ptr_arg<void>(args, pl, ("out" + std::to_string(j) + "_arg").c_str());
        // TTS_FUSED_MAP=interpreter keeps the program on the interpreter kernel; otherwise it is compiled
        // into a kernel of its own at the plan's first launch (scalar arguments stay arguments: one compile per plan)
        const char *mode = getenv("TTS_FUSED_MAP");
        if (mode && std::string(mode) == "interpreter") {
          err = launch_mapn(p, gx, gy, gz, s, &kname);
          break;
        }
        {
          std::lock_guard<std::mutex> lock(plan->mu);
          if (!plan->fused) {
            may_allocate("to compile the fused map's kernel");
            std::string why;
            hipError_t ce = fused_map_compile(p, &plan->fused, &why);
            if (ce != hipSuccess) return fail(TTS_HIP_ERROR, "fused_map: " + why);
          }
        }
        kname = "fused_map (hipRTC)";
        err = fused_map_launch(plan->fused, p, gx, gy, gz, s);
        break;
      }
      case Family::TileProgram: {
        tts_status st = run_tile_program(&plan->fused, pl.source);
        if (st != TTS_OK) return st;
        break;
      }
      case Family::RowSoftmax: {
        SoftmaxParams p = b->softmax;
        p.in = ptr_arg<const void>(args, pl, "in_arg");
        p.out = ptr_arg<void>(args, pl, "out_arg");
        err = launch_softmax(p, gx, gy, gz, s, &kname);
        break;
      }
      case Family::LayerNormFwd: {
        LayerNormParams p = b->layernorm;
        p.x = ptr_arg<const void>(args, pl, "x_arg");
        p.y = ptr_arg<void>(args, pl, "y_arg");
        p.w = ptr_arg<const void>(args, pl, "w_arg");
        p.b = ptr_arg<const void>(args, pl, "b_arg");
        p.mean = ptr_arg<float>(args, pl, "mean_arg");
        p.rstd = ptr_arg<float>(args, pl, "rstd_arg");
        err = launch_layernorm(p, gx, gy, gz, s, &kname);
        break;
      }
      case Family::Gemm: {
        GemmParams p = b->gemm;
        p.a = ptr_arg<const void>(args, pl, "a_arg");
        p.b = ptr_arg<const void>(args, pl, "b_arg");
        p.c = ptr_arg<void>(args, pl, "c_arg");
        if (pl.k.count("gathered")) {
          p.a_rows = ptr_arg<const int>(args, pl, "rows_arg");
          p.b_block = ptr_arg<const int>(args, pl, "block_arg");
        }
        p.split = 1;
        p.partial = nullptr;
        if (pl.source.empty()) {
          // a product with too few tiles for the chip runs in K slices, whose partial sums need memory: the stream's
          // workspace (as for the int8-weight product), or the static array of the call that may not allocate, when
          // they fit there (else that call runs the product without slices)
          const int want = gemm_split(p);
          if (want > 1) {
            p.split = want;
            const size_t need = gemm_workspace_bytes(p);
            if (no_alloc) {  // as many slices as the static array holds
              const size_t one = (size_t)p.M * p.N * std::max(1, p.batches) * sizeof(float);
              p.split = (int)std::min<size_t>((size_t)want, NOALLOC_WORKSPACE_BYTES / one);
              if (p.split > 1) p.partial = reinterpret_cast<float *>(noalloc_scratch());
              else p.split = 1;
            } else {
              std::lock_guard<std::mutex> lock(plan->mu);
              tts_plan::SplitK &sk = plan->split_k[stream];
              hipError_t e = plan->grow((void **)&sk.workspace, &sk.workspace_bytes, need);
              if (e != hipSuccess) return fail(TTS_HIP_ERROR, std::string("hipMalloc(split-K workspace): ") + hipGetErrorString(e));
              p.partial = sk.workspace;
            }
          }
          err = launch_gemm(p, s, &kname);
          break;
        }
        static_assert(TILE_MAX_ARGS == 32, "GemmEpilogueArgs holds 32 arguments");
        GemmEpilogueArgs a{};
        for (int i = 0; i < n; i++) {
          if (args[i].kind == TTS_ARG_PTR) a.ptr[i] = args[i].v.ptr;
          else if (args[i].kind == TTS_ARG_INT) a.ival[i] = args[i].v.i;
          else a.fval[i] = args[i].v.f;
        }
        a.tile_pid = b->tile_pid;
        a.tiles_n = b->tiles_n;
        a.gx = gx;
        a.gy = gy;
        a.gz = gz;
        std::string why;
        if (no_alloc) {
          const GemmParams &gp = p;
          const int which = gemm_epilogue_kernel_index(gp);
          std::lock_guard<std::mutex> lock(plan->mu);
          if (!plan->gemm_rtc[which]) may_allocate("to compile the matrix product with its fused epilogue");
        }
        {
          std::lock_guard<std::mutex> lock(plan->mu);
          err = launch_gemm_epilogue(p, pl.source, plan->gemm_rtc, a, s, &kname, &why);
        }
        if (err != hipSuccess && !why.empty()) return fail(TTS_HIP_ERROR, "gemm epilogue: " + why);
        break;
      }
      case Family::GemmW8A16: {
        GemmW8A16Params p = b->w8;
        p.a = ptr_arg<const void>(args, pl, "a_arg");
        p.w = ptr_arg<const int8_t>(args, pl, "b_arg");
        p.scale = ptr_arg<const void>(args, pl, "s_arg");
        p.c = ptr_arg<void>(args, pl, "c_arg");
        if (p.split > 1 && no_alloc) {
          const size_t need = gemm_w8a16_workspace_bytes(p), ncount = gemm_w8a16_counters(p);
          if (need > NOALLOC_WORKSPACE_BYTES || ncount > NOALLOC_COUNTERS)
            throw Unsupported("tts_launch_noalloc: the split-K partial tiles of this shape need " + std::to_string(need) + " bytes and " +
                              std::to_string(ncount) + " counters; the static scratch array holds " +
                              std::to_string(NOALLOC_WORKSPACE_BYTES) + " bytes and " + std::to_string(NOALLOC_COUNTERS) + " counters");
          unsigned char *base = noalloc_scratch();
          p.workspace = reinterpret_cast<float *>(base);
          p.counters = reinterpret_cast<int *>(base + NOALLOC_WORKSPACE_BYTES);
          // every call on this GPU shares the array: the counters start at zero whatever the last call left there
          // (a fill kernel rather than hipMemsetAsync, so that the call may be captured into a graph)
          if (ncount) {
            hipLaunchKernelGGL(clear_ints_kernel, dim3((unsigned)((ncount + 255) / 256)), dim3(256), 0, s, p.counters, (int)ncount);
            hipError_t e = hipGetLastError();
            if (e != hipSuccess) return fail(TTS_HIP_ERROR, std::string("clearing the split-K counters: ") + hipGetErrorString(e));
          }
        } else if (p.split > 1) {
          const size_t need = gemm_w8a16_workspace_bytes(p), ncount = gemm_w8a16_counters(p);
          std::lock_guard<std::mutex> lock(plan->mu);
          tts_plan::SplitK &sk = plan->split_k[stream];
          hipError_t e = plan->grow((void **)&sk.workspace, &sk.workspace_bytes, need);
          if (e != hipSuccess) return fail(TTS_HIP_ERROR, std::string("hipMalloc(split-K workspace): ") + hipGetErrorString(e));
          if (sk.counters_count < ncount) {
            // (new counters start at zero; the old ones, which launches in flight may still be bumping, are retired)
            int *fresh = nullptr;
            const size_t count = std::max(ncount, 2 * sk.counters_count);
            e = hipMalloc((void **)&fresh, count * sizeof(int));
            if (e == hipSuccess) e = hipMemset(fresh, 0, count * sizeof(int));
            if (e == hipSuccess) e = hipDeviceSynchronize();  // the fill has landed before a launch on any stream reads the counters
            if (e != hipSuccess) return fail(TTS_HIP_ERROR, std::string("hipMalloc(split-K counters): ") + hipGetErrorString(e));
            if (sk.counters) plan->retired.push_back(sk.counters);
            sk.counters = fresh;
            sk.counters_count = count;
          }
          p.workspace = sk.workspace;
          p.counters = sk.counters;
        }
        p.widened = nullptr;
        if (!no_alloc) {  // (the call that may not allocate stays on the decode kernels, a launch per 32 rows)
          const size_t need = gemm_w8a16_widened_bytes(p);
          if (need) {
            std::lock_guard<std::mutex> lock(plan->mu);
            tts_plan::SplitK &sk = plan->split_k[stream];
            hipError_t e = plan->grow(&sk.widened, &sk.widened_bytes, need);
            if (e != hipSuccess) return fail(TTS_HIP_ERROR, std::string("hipMalloc(widened weights): ") + hipGetErrorString(e));
            p.widened = sk.widened;
          }
        }
        err = launch_gemm_w8a16(p, s, &kname);
        break;
      }
    }
    plan->last_kernel = kname;
    if (err != hipSuccess) return fail(TTS_HIP_ERROR, std::string("kernel launch failed: ") + hipGetErrorString(err));
    return TTS_OK;
  });
}

}  // namespace

extern "C" {

tts_status tts_launch(tts_plan *plan, int gx, int gy, int gz, void *stream, const tts_arg *args, int n) {
  return launch_impl(plan, gx, gy, gz, stream, args, n, false);
}

tts_status tts_launch_noalloc(tts_plan *plan, int gx, int gy, int gz, void *stream, const tts_arg *args, int n) {
  return launch_impl(plan, gx, gy, gz, stream, args, n, true);
}

}  // extern "C"
