// Family recognition and binding extraction: see match.h.
#include "match.h"

#include "mapn_isa.h"

#include <functional>
#include <set>
#include <sstream>

namespace tts {

static std::string generic_fallback(const Program &p);

const char *family_name(Family f) {
  switch (f) {
    case Family::Map1D: return "map1d";
    case Family::RowSoftmax: return "row_softmax";
    case Family::LayerNormFwd: return "layernorm_fwd";
    case Family::Gemm: return "gemm";
    case Family::GemmW8A16: return "gemm_w8a16";
    case Family::FusedMap: return "fused_map";
    case Family::TileProgram: return "tile_program";
  }
  return "?";
}

// ---------------------------------------------------------------- signature

std::string signature(const Program &p) {
  std::map<int, int> num;  // value id -> normalised number
  auto V = [&](int v) {
    auto it = num.find(v);
    if (it == num.end()) return std::string("v?");
    return "v" + std::to_string(it->second);
  };
  auto def = [&](int v) {
    int n = (int)num.size();
    num[v] = n;
    return "v" + std::to_string(n);
  };
  std::ostringstream os;
  std::function<void(const std::vector<SOp> &)> walk = [&](const std::vector<SOp> &ops) {
    for (auto &s : ops) {
      auto operands = [&]() {
        std::string r = "(";
        for (size_t i = 0; i < s.operands.size(); i++) r += (i ? "," : "") + V(s.operands[i]);
        return r + ")";
      };
      auto acc = [&]() {
        std::string r = ":" + s.acc.elem + ".r" + std::to_string(s.acc.sizes.size());
        if (!s.acc.dims.empty()) r += ".m";
        if (s.acc.has_other) r += ".o";
        return r;
      };
      switch (s.kind) {
        case SK::Load: os << def(s.result) << "=load" << acc() << ";"; break;
        case SK::ScalarLoad: os << def(s.result) << "=sload" << acc() << ";"; break;
        case SK::Store: os << "store" << acc() << operands() << ";"; break;
        case SK::ScalarStore: os << "sstore" << acc() << operands() << ";"; break;
        case SK::Map: {
          std::string o = operands();
          os << def(s.result) << "=" << s.name << ":" << p.values[s.result].dtype << o << ";";
          break;
        }
        case SK::Splat: { std::string o = operands(); os << def(s.result) << "=splat" << o << ";"; break; }
        case SK::Const: os << def(s.result) << "=const:" << p.values[s.result].dtype << ";"; break;
        case SK::Iota: os << def(s.result) << "=iota;"; break;
        case SK::FromIndex: os << def(s.result) << "=index;"; break;
        case SK::ScalarArg: os << def(s.result) << "=farg;"; break;
        case SK::Reduce: {
          std::string o = operands();
          if (s.results.empty()) os << def(s.result);
          for (size_t j = 0; j < s.results.size(); j++) os << (j ? "," : "") << def(s.results[j]);
          os << "=reduce." << s.name << "." << s.axis << o << ";";
          break;
        }
        case SK::Scan: {
          std::string o = operands();
          for (size_t j = 0; j < s.results.size(); j++) os << (j ? "," : "") << def(s.results[j]);
          os << "=scan." << s.name << "." << s.axis << o << ";";
          break;
        }
        case SK::Dot: { std::string o = operands(); os << def(s.result) << "=dot" << o << ";"; break; }
        case SK::ExpandDims: { std::string o = operands(); os << def(s.result) << "=expand." << s.axis << o << ";"; break; }
        case SK::Broadcast: { std::string o = operands(); os << def(s.result) << "=bcast" << o << ";"; break; }
        case SK::If: {
          os << (s.ival ? "unless" : "if") << operands() << "{";
          walk(s.body);
          os << "};";
          break;
        }
        case SK::For: {
          os << "for[";
          for (size_t j = 0; j < s.tile_args.size(); j++) {
            std::string init = V(s.tile_inits[j]);
            os << (j ? "," : "") << def(s.tile_args[j]) << "<-" << init;
          }
          os << "]{";
          walk(s.body);
          os << "yield(";
          for (size_t j = 0; j < s.tile_yields.size(); j++) os << (j ? "," : "") << V(s.tile_yields[j]);
          os << ")}";
          if (!s.results.empty()) {
            os << "->";
            for (size_t j = 0; j < s.results.size(); j++) os << (j ? "," : "") << def(s.results[j]);
          }
          os << ";";
          break;
        }
      }
    }
  };
  walk(p.body);
  return os.str();
}

// ------------------------------------------------------------ expr helpers

namespace {

struct LinIv : Lin {
  int iv = -1;  // coefficient of the designated loop's induction variable
};

struct Matcher {
  Program &P;
  ExprPool &X;
  explicit Matcher(Program &p) : P(p), X(p.pool) { index_ops(P.body); }

  int c64(int64_t v) { return X.constant(v, 64); }

  bool pid_free(int e) { return !X.depends_on(e, EK::Pid); }
  bool loop_free(int e) {
    return !X.depends_on(e, EK::IV) && !X.depends_on(e, EK::Iter) && !X.depends_on(e, EK::Result);
  }
  bool is_const(int e, int64_t want) {
    int64_t v;
    return X.is_const(e, &v) && v == want;
  }

  // Decomposes e into c0 + sum coef[a]*pid[a] + iv*IV(loop) with parts that read
  // neither the program id nor any loop state.  Sign extension is looked
  // through: a 32-bit product that overflowed would differ, which the launcher
  // rules out by evaluating the original expression at the last program of the
  // grid and comparing.
  bool linear(int e, LinIv &out, int loop = -1) {
    const Expr x = X.at(e);
    auto zero = [&](LinIv &l) {
      l.c0 = c64(0);
      for (int a = 0; a < 3; a++) l.coef[a] = c64(0);
      l.iv = c64(0);
    };
    if (pid_free(e) && loop_free(e)) {
      zero(out);
      out.c0 = X.to_index(e);
      return true;
    }
    if (x.k == EK::Pid) {
      zero(out);
      out.coef[x.a] = c64(1);
      return true;
    }
    if (x.k == EK::IV && x.a == loop) {
      zero(out);
      out.iv = c64(1);
      return true;
    }
    if (x.k == EK::Sext) return linear(x.a, out, loop);
    if (x.k == EK::Add || x.k == EK::Sub) {
      LinIv l, r;
      if (!linear(x.a, l, loop) || !linear(x.b, r, loop)) return false;
      out.c0 = X.bin(x.k, l.c0, r.c0);
      for (int a = 0; a < 3; a++) out.coef[a] = X.bin(x.k, l.coef[a], r.coef[a]);
      out.iv = X.bin(x.k, l.iv, r.iv);
      return true;
    }
    if (x.k == EK::Mul) {
      bool fa = pid_free(x.a) && loop_free(x.a), fb = pid_free(x.b) && loop_free(x.b);
      if (!fa && !fb) return false;
      int free_side = fa ? x.a : x.b, other = fa ? x.b : x.a;
      LinIv l;
      if (!linear(other, l, loop)) return false;
      int s = X.to_index(free_side);
      out.c0 = X.bin(EK::Mul, l.c0, s);
      for (int a = 0; a < 3; a++) out.coef[a] = X.bin(EK::Mul, l.coef[a], s);
      out.iv = X.bin(EK::Mul, l.iv, s);
      return true;
    }
    return false;
  }

  // Recognises the valid extent MaskAnalysis derives for `start + arange(size) <
  // bound`:  max(start, min(start+size, bound)) - start, possibly wrapped in
  // min(size, .) by a conjunction with a broadcast mask.
  bool extent(int e, int64_t size, int &start, int &bound) {
    for (int guard = 0; guard < 4; guard++) {
      const Expr x = X.at(e);
      if (x.k != EK::MinS) break;
      int64_t v;
      if (X.is_const(x.a, &v) && v == size) e = x.b;
      else if (X.is_const(x.b, &v) && v == size) e = x.a;
      else break;
    }
    const Expr x = X.at(e);
    auto min_with_end = [&](int m, int s, int &b) {
      const Expr mm = X.at(m);
      if (mm.k != EK::MinS) return false;
      int end = X.bin(EK::Add, s, c64(size));
      if (mm.a == end) { b = mm.b; return true; }
      if (mm.b == end) { b = mm.a; return true; }
      return false;
    };
    if (x.k == EK::Sub) {
      int s = x.b;
      const Expr mx = X.at(x.a);
      if (mx.k != EK::MaxS) return false;
      int m = mx.a == s ? mx.b : mx.b == s ? mx.a : -1;
      if (m < 0) return false;
      if (!min_with_end(m, s, bound)) return false;
      start = s;
      return true;
    }
    if (x.k == EK::MaxS) {  // start == 0: the subtraction folded away
      int zero = c64(0);
      int m = x.a == zero ? x.b : x.b == zero ? x.a : -1;
      if (m < 0) return false;
      if (!min_with_end(m, zero, bound)) return false;
      start = zero;
      return true;
    }
    return false;
  }

  int sum(const std::vector<int> &v) {
    int s = c64(0);
    for (int e : v) s = X.bin(EK::Add, s, X.to_index(e));
    return s;
  }

  // flattened views of the program
  std::vector<SOp *> accesses, loops, all;
  void index_ops(std::vector<SOp> &ops) {
    for (auto &s : ops) {
      all.push_back(&s);
      if (s.kind == SK::Load || s.kind == SK::Store || s.kind == SK::ScalarLoad || s.kind == SK::ScalarStore)
        accesses.push_back(&s);
      if (s.kind == SK::For) {
        loops.push_back(&s);
        index_ops(s.body);
      }
      if (s.kind == SK::If) index_ops(s.body);
    }
  }
  std::vector<SOp *> of_kind(SK k) {
    std::vector<SOp *> r;
    for (auto s : all)
      if (s->kind == k) r.push_back(s);
    return r;
  }
};

[[noreturn]] void refuse(const char *family, const std::string &why) {
  throw Unsupported(std::string("the program has the op structure of family '") + family + "' but " + why);
}

void no_wrap(Matcher &m, const char *family) {
  for (SOp *a : m.accesses)
    for (int e : a->acc.mods)
      if (e >= 0) refuse(family, "it addresses memory modulo a size (wraparound), which only the matmul family implements");
}

void unit_stride(Matcher &m, const Access &a, const char *family) {
  if (!m.is_const(a.strides.back(), 1)) refuse(family, "its innermost stride is not 1");
}

Lin as_lin(const LinIv &l, int orig) {
  Lin r = (Lin)l;
  r.orig = orig;
  return r;
}

// ------------------------------------------------------------------ map1d
// load, load, one binary f32 op, store: z[i] = x[i] op y[i] over each program's block.
bool try_map1d(Plan &pl) {
  Matcher m(pl.prog);
  if (m.all.size() != 4) return false;
  SOp *l0 = m.all[0], *l1 = m.all[1], *op = m.all[2], *st = m.all[3];
  if (l0->kind != SK::Load || l1->kind != SK::Load || op->kind != SK::Map || st->kind != SK::Store) return false;
  static const std::map<std::string, int> ops = {{"arith.addf", 0}, {"arith.subf", 1}, {"arith.mulf", 2},
                                                 {"arith.divf", 3}, {"arith.maximumf", 4}, {"arith.minimumf", 5}};
  auto it = ops.find(op->name);
  if (it == ops.end() || op->operands.size() != 2) return false;
  bool direct = op->operands[0] == l0->result && op->operands[1] == l1->result;
  bool swapped = op->operands[0] == l1->result && op->operands[1] == l0->result;
  if (!direct && !swapped) return false;
  if (st->operands[0] != op->result) return false;
  const char *F = "map1d";
  no_wrap(m, F);
  for (SOp *a : {l0, l1, st}) {
    if (a->acc.sizes.size() != 1) return false;
    if (a->acc.elem != "f32") refuse(F, "its element type is " + a->acc.elem + " (only f32 is implemented)");
    if (a->acc.sizes[0] != st->acc.sizes[0]) return false;
    unit_stride(m, a->acc, F);
    if (a->acc.dims != st->acc.dims) refuse(F, "its loads and its store are masked differently");
  }
  int64_t B = st->acc.sizes[0];
  pl.family = Family::Map1D;
  pl.k["op"] = it->second;
  pl.k["swap"] = swapped;
  pl.k["block"] = B;
  pl.k["x_arg"] = l0->acc.base_arg;
  pl.k["y_arg"] = l1->acc.base_arg;
  pl.k["z_arg"] = st->acc.base_arg;
  const char *names[] = {"x_off", "y_off", "z_off"};
  int i = 0;
  for (SOp *a : {l0, l1, st}) {
    LinIv l;
    if (!m.linear(a->acc.offsets[0], l)) refuse(F, "a block offset is not linear in the program id");
    pl.lin[names[i++]] = as_lin(l, a->acc.offsets[0]);
  }
  pl.k["masked"] = !st->acc.dims.empty();
  if (!st->acc.dims.empty()) {
    int start, bound;
    if (!m.extent(st->acc.dims[0], B, start, bound)) refuse(F, "its mask is not of the form start+arange < bound");
    LinIv l;
    if (!m.linear(start, l)) refuse(F, "its mask start is not linear in the program id");
    if (!m.pid_free(bound) || !m.loop_free(bound)) refuse(F, "its mask bound depends on the program id");
    pl.lin["m_start"] = as_lin(l, start);
    pl.e["bound"] = bound;
  }
  return true;
}

// ------------------------------------------------------------ row softmax
const char *SIG_SOFTMAX =
    "v0=load:f32.r1.m.o;v1=reduce.arith.{MAX}.0(v0);v2=splat(v1);v3=arith.subf:f32(v0,v2);v4=math.exp:f32(v3);"
    "v5=reduce.arith.addf.0(v4);v6=splat(v5);v7=arith.divf:f32(v4,v6);store:f32.r1.m(v7);";

std::string subst(std::string s, const std::string &key, const std::string &val) {
  for (size_t p = s.find(key); p != std::string::npos; p = s.find(key, p + val.size())) s.replace(p, key.size(), val);
  return s;
}

// the same arithmetic on rows of fp16 / bf16: widened after the load, narrowed before the store
const char *SIG_SOFTMAX_16 =
    "v0=load:{T}.r1.m.o;v1=arith.extf:f32(v0);v2=reduce.arith.{MAX}.0(v1);v3=splat(v2);v4=arith.subf:f32(v1,v3);v5=math.exp:f32(v4);"
    "v6=reduce.arith.addf.0(v5);v7=splat(v6);v8=arith.divf:f32(v5,v7);v9=arith.truncf:{T}(v8);store:{T}.r1.m(v9);";

bool try_softmax(Plan &pl) {
  bool known = false;
  for (const char *mx : {"maxnumf", "maximumf"}) {
    known = known || pl.signature == subst(SIG_SOFTMAX, "{MAX}", mx);
    for (const char *t : {"f16", "bf16"}) known = known || pl.signature == subst(subst(SIG_SOFTMAX_16, "{MAX}", mx), "{T}", t);
  }
  if (!known) return false;
  const char *F = "row_softmax";
  Matcher m(pl.prog);
  SOp *ld = m.accesses.at(0), *st = m.accesses.at(1);
  no_wrap(m, F);
  unit_stride(m, ld->acc, F);
  unit_stride(m, st->acc, F);
  if (ld->acc.sizes != st->acc.sizes) refuse(F, "its load and store blocks differ in size");
  if (ld->acc.sizes[0] > 65536) refuse(F, "its rows are longer than the 65536 elements the row kernel keeps in registers");
  pl.family = Family::RowSoftmax;
  pl.k["block"] = ld->acc.sizes[0];
  pl.k["in_arg"] = ld->acc.base_arg;
  pl.k["out_arg"] = st->acc.base_arg;
  pl.f["other"] = ld->acc.other_f;
  if (ld->acc.elem != st->acc.elem) refuse(F, "its input and output differ in element type");
  pl.k["elem_kind"] = ld->acc.elem == "f32" ? 2 : ld->acc.elem == "bf16" ? 1 : 0;
  LinIv li, lo;
  if (!m.linear(ld->acc.offsets[0], li) || !m.linear(st->acc.offsets[0], lo))
    refuse(F, "a row offset is not linear in the program id");
  pl.lin["in_off"] = as_lin(li, ld->acc.offsets[0]);
  pl.lin["out_off"] = as_lin(lo, st->acc.offsets[0]);
  for (SOp *a : {ld, st})
    if (!m.pid_free(a->acc.dims[0]) || !m.loop_free(a->acc.dims[0])) refuse(F, "its column mask depends on the program id");
  pl.e["in_dims"] = ld->acc.dims[0];
  pl.e["out_dims"] = st->acc.dims[0];
  return true;
}

// ---------------------------------------------------------- layernorm fwd
const char *SIG_LAYERNORM = 
    "v0=const:f32;v1=const:f32;v2=iota;v3=index;v4=splat(v3);for[v5<-v1]{v6=load:{T}.r1.m.o;v7=arith.extf"
    ":f32(v6);v8=arith.addf:f32(v5,v7);yield(v8)}->v9;v10=reduce.arith.addf.0(v9);v11=index;v12=arith.sit"
    "ofp:f32(v11);v13=arith.divf:f32(v10,v12);v14=splat(v13);for[v15<-v1]{v16=index;v17=splat(v16);v18=ar"
    "ith.addi:i32(v17,v2);v19=arith.cmpi.slt:i1(v18,v4);v20=load:{T}.r1.m.o;v21=arith.extf:f32(v20);v22=a"
    "rith.subf:f32(v21,v14);v23=arith.select:f32(v19,v22,v1);v24=arith.mulf:f32(v23,v23);v25=arith.addf:f"
    "32(v15,v24);yield(v25)}->v26;v27=reduce.arith.addf.0(v26);v28=arith.divf:f32(v27,v12);v29=farg;v30=a"
    "rith.addf:f32(v28,v29);v31=math.sqrt:f32(v30);v32=arith.divf:f32(v0,v31);sstore:f32.r0(v13);sstore:f"
    "32.r0(v32);v33=splat(v32);for[]{v34=load:{T}.r1.m;v35=load:{T}.r1.m;v36=load:{T}.r1.m.o;v37=arith.ex"
    "tf:f32(v36);v38=arith.subf:f32(v37,v14);v39=arith.mulf:f32(v38,v33);v40=arith.extf:f32(v34);v41=arit"
    "h.mulf:f32(v39,v40);v42=arith.extf:f32(v35);v43=arith.addf:f32(v41,v42);v44=arith.truncf:{T}(v43);st"
    "ore:{T}.r1.m(v44);yield()};";

// the same program on fp32 tensors: no widening or narrowing casts
const char *SIG_LAYERNORM_F32 =
    "v0=const:f32;v1=const:f32;v2=iota;v3=index;v4=splat(v3);for[v5<-v1]{v6=load:f32.r1.m.o;v7=arith.addf:f32(v5,v6);yield(v7)}->v8;"
    "v9=reduce.arith.addf.0(v8);v10=index;v11=arith.sitofp:f32(v10);v12=arith.divf:f32(v9,v11);v13=splat(v12);for[v14<-v1]{v15=index;"
    "v16=splat(v15);v17=arith.addi:i32(v16,v2);v18=arith.cmpi.slt:i1(v17,v4);v19=load:f32.r1.m.o;v20=arith.subf:f32(v19,v13);"
    "v21=arith.select:f32(v18,v20,v1);v22=arith.mulf:f32(v21,v21);v23=arith.addf:f32(v14,v22);yield(v23)}->v24;"
    "v25=reduce.arith.addf.0(v24);v26=arith.divf:f32(v25,v11);v27=farg;v28=arith.addf:f32(v26,v27);v29=math.sqrt:f32(v28);"
    "v30=arith.divf:f32(v0,v29);sstore:f32.r0(v12);sstore:f32.r0(v30);v31=splat(v30);for[]{v32=load:f32.r1.m;v33=load:f32.r1.m;"
    "v34=load:f32.r1.m.o;v35=arith.subf:f32(v34,v13);v36=arith.mulf:f32(v35,v31);v37=arith.mulf:f32(v36,v32);v38=arith.addf:f32(v37,v33);"
    "store:f32.r1.m(v38);yield()};";

bool try_layernorm(Plan &pl) {
  if (pl.signature != subst(SIG_LAYERNORM, "{T}", "f16") && pl.signature != subst(SIG_LAYERNORM, "{T}", "bf16") && pl.signature != SIG_LAYERNORM_F32)
    return false;
  const char *F = "layernorm_fwd";
  Matcher m(pl.prog);
  if (m.loops.size() != 3 || m.accesses.size() != 8) return false;
  no_wrap(m, F);
  SOp *x0 = m.accesses[0], *x1 = m.accesses[1], *mean_st = m.accesses[2], *rstd_st = m.accesses[3];
  SOp *w = m.accesses[4], *b = m.accesses[5], *x2 = m.accesses[6], *y = m.accesses[7];
  int64_t B = x0->acc.sizes[0];
  ExprPool &X = pl.prog.pool;
  int N = m.loops[0]->ub;
  for (size_t i = 0; i < 3; i++) {
    SOp *lp = m.loops[i];
    if (lp->ub != N) refuse(F, "its three column loops have different bounds");
    if (!m.is_const(lp->lb, 0) || !m.is_const(lp->step, B)) refuse(F, "a column loop does not run from 0 in steps of the block size");
  }
  if (!m.pid_free(N) || !m.loop_free(N)) refuse(F, "its column count depends on the program id");
  int Nidx = X.to_index(N);
  // every block access: unit stride, same block, extent = clamp(N - iv)
  SOp *blocks[] = {x0, x1, w, b, x2, y};
  int loop_of[] = {0, 1, 2, 2, 2, 2};
  const char *names[] = {"x_off", "x_off1", "w_off", "b_off", "x_off2", "y_off"};
  for (int i = 0; i < 6; i++) {
    SOp *a = blocks[i];
    int loop = m.loops[loop_of[i]]->loop;
    if (a->acc.sizes.size() != 1 || a->acc.sizes[0] != B) refuse(F, "its blocks differ in size");
    unit_stride(m, a->acc, F);
    int start, bound;
    if (a->acc.dims.empty() || !m.extent(a->acc.dims[0], B, start, bound)) refuse(F, "a column mask is not start+arange < N");
    if (start != X.to_index(X.iv(loop, 32)) || bound != Nidx) refuse(F, "a column mask is not (loop offset + arange) < N");
    LinIv l;
    if (!m.linear(a->acc.offsets[0], l, loop) || !m.is_const(l.iv, 1)) refuse(F, "a block offset is not row offset + loop offset");
    pl.lin[names[i]] = as_lin(l, a->acc.offsets[0]);
  }
  auto same = [&](const Lin &a, const Lin &c) {
    return a.c0 == c.c0 && a.coef[0] == c.coef[0] && a.coef[1] == c.coef[1] && a.coef[2] == c.coef[2];
  };
  if (!same(pl.lin["x_off"], pl.lin["x_off1"]) || !same(pl.lin["x_off"], pl.lin["x_off2"]))
    refuse(F, "its three passes read different rows");
  if (x0->acc.base_arg != x1->acc.base_arg || x0->acc.base_arg != x2->acc.base_arg) refuse(F, "its three passes read different tensors");
  for (SOp *a : {x0, x1, x2})
    if (!a->acc.has_other || a->acc.other_f != 0.0) refuse(F, "its input loads do not pad with 0");
  // the select mask of the variance pass and the float N: every integer that
  // reaches the data path must be the loop offset or N
  auto from_index = m.of_kind(SK::FromIndex);
  for (SOp *fi : from_index) {
    int e = fi->expr;
    bool is_n = e == N;
    bool is_iv = X.at(e).k == EK::IV && X.at(e).a == m.loops[1]->loop;
    if (!is_n && !is_iv) refuse(F, "an unexpected integer feeds its arithmetic");
  }
  for (SOp *io : m.of_kind(SK::Iota))
    if (io->ival != 0) refuse(F, "its lane index does not start at 0");
  auto consts = m.of_kind(SK::Const);
  if (consts.size() != 2 || consts[0]->fval != 1.0 || consts[1]->fval != 0.0) refuse(F, "its constants are not 1 and 0");
  for (SOp *s : {mean_st, rstd_st}) {
    LinIv l;
    if (!m.linear(s->acc.offsets[0], l)) refuse(F, "a statistics offset is not linear in the program id");
    pl.lin[s == mean_st ? "mean_off" : "rstd_off"] = as_lin(l, s->acc.offsets[0]);
  }
  pl.family = Family::LayerNormFwd;
  pl.k["block"] = B;
  pl.k["x_arg"] = x0->acc.base_arg;
  pl.k["y_arg"] = y->acc.base_arg;
  pl.k["w_arg"] = w->acc.base_arg;
  pl.k["b_arg"] = b->acc.base_arg;
  pl.k["mean_arg"] = mean_st->acc.base_arg;
  pl.k["rstd_arg"] = rstd_st->acc.base_arg;
  pl.k["eps_arg"] = m.of_kind(SK::ScalarArg).at(0)->ival;
  pl.k["elem_kind"] = x0->acc.elem == "f32" ? 2 : x0->acc.elem == "bf16" ? 1 : 0;
  for (SOp *a : {x1, x2, w, b, y})
    if (a->acc.elem != x0->acc.elem) refuse(F, "its tensors differ in element type");
  pl.e["N"] = N;
  return true;
}

// ------------------------------------------------------------------- gemm
const char *SIG_GEMM = 
    "v0=const:f32;for[v1<-v0]{v2=load:{T}.r2.m.o;v3=load:{T}.r2.m.o;v4=dot(v2,v3,v1);yield(v4)}->v5;v6=ar"
    "ith.truncf:{T}(v5);store:{T}.r2.m(v6);";
const char *SIG_W8A16 = 
    "v0=const:f32;v1=load:f16.r1.m.o;v2=expand.0(v1);v3=bcast(v2);for[v4<-v0]{v5=load:f16.r2.m.o;v6=load:"
    "i8.r2.m.o;v7=arith.sitofp:f16(v6);v8=arith.mulf:f16(v7,v3);v9=dot(v5,v8,v4);yield(v9)}->v10;v11=arit"
    "h.truncf:f16(v10);store:f16.r2.m(v11);";

// Loop-carried pointer state of a 2-D block: strides must not change, offsets
// advance by a loop-invariant amount per iteration.
struct Carried2D {
  int base = -1;   // sum of the offsets at iteration 0
  int kstep = -1;  // sum of the per-iteration advances
  int stride[2] = {-1, -1};
  int init[2] = {-1, -1};  // per-dim offset at iteration 0
};

bool carried_state(Matcher &m, SOp *loop, const Access &a, Carried2D &out) {
  ExprPool &X = m.X;
  auto slot_of = [&](int e) -> IntIter * {
    for (auto &it : loop->int_iters)
      if (it.iter_expr == e) return &it;
    return nullptr;
  };
  std::vector<int> inits, steps;
  for (int e : a.offsets) {
    IntIter *it = slot_of(e);
    if (!it) {
      if (!m.loop_free(e)) return false;
      inits.push_back(e);
      continue;
    }
    inits.push_back(it->init);
    if (it->next == it->iter_expr) continue;
    const Expr n = X.at(it->next);
    if (n.k != EK::Add) return false;
    int delta = n.a == it->iter_expr ? n.b : n.b == it->iter_expr ? n.a : -1;
    if (delta < 0 || !m.loop_free(delta) || !m.pid_free(delta)) return false;
    steps.push_back(delta);
  }
  for (int d = 0; d < 2; d++) {
    int e = a.strides[d];
    IntIter *it = slot_of(e);
    if (it) {
      if (it->next != it->iter_expr) return false;
      e = it->init;
    }
    if (!m.loop_free(e) || !m.pid_free(e)) return false;
    out.stride[d] = e;
  }
  out.base = m.sum(inits);
  out.kstep = m.sum(steps);
  for (size_t d = 0; d < 2 && d < inits.size(); d++) out.init[d] = inits[d];
  return true;
}

// the same program on fp32 blocks: the accumulator is stored as it is
const char *SIG_GEMM_F32 = "v0=const:f32;for[v1<-v0]{v2=load:f32.r2.m.o;v3=load:f32.r2.m.o;v4=dot(v2,v3,v1);yield(v4)}->v5;store:f32.r2.m(v5);";

bool try_gemm(Plan &pl, bool w8a16) {
  std::string sig = pl.signature;
  std::string T;
  if (!w8a16) {
    if (sig == subst(SIG_GEMM, "{T}", "bf16")) T = "bf16";
    else if (sig == subst(SIG_GEMM, "{T}", "f16")) T = "f16";
    else if (sig == SIG_GEMM_F32) T = "f32";
    else return false;
  } else {
    if (sig != SIG_W8A16) return false;
    T = "f16";
  }
  const char *F = w8a16 ? "gemm_w8a16" : "gemm";
  Matcher m(pl.prog);
  if (m.loops.size() != 1) return false;
  SOp *loop = m.loops[0];
  size_t o = w8a16 ? 1 : 0;
  if (m.accesses.size() != 3 + o) return false;
  SOp *A = m.accesses[o], *Bm = m.accesses[o + 1], *C = m.accesses[o + 2];
  if (A->acc.sizes.size() != 2 || Bm->acc.sizes.size() != 2 || C->acc.sizes.size() != 2) return false;
  int64_t BM = A->acc.sizes[0], BK = A->acc.sizes[1], BN = Bm->acc.sizes[1];
  if (Bm->acc.sizes[0] != BK || C->acc.sizes[0] != BM || C->acc.sizes[1] != BN) refuse(F, "its block shapes do not compose");
  if (!m.is_const(loop->lb, 0) || !m.is_const(loop->step, 1)) refuse(F, "its K loop does not count 0,1,2,...");
  if (!m.pid_free(loop->ub)) refuse(F, "its K trip count depends on the program id");
  Carried2D ca, cb;
  if (!carried_state(m, loop, A->acc, ca) || !carried_state(m, loop, Bm->acc, cb))
    refuse(F, "its operand pointers do not advance by a constant per K step");
  for (int e : C->acc.strides)
    if (!m.pid_free(e) || !m.loop_free(e)) refuse(F, "its output strides depend on the program id");
  // masks: rows against M, columns against N, K against what is left
  // Rows of A / columns of B beyond the problem are either masked off (other = 0) or, as in the
  // stock tutorial kernel, read modulo M / N (test_matmul.py:74-75): those lanes only reach
  // outputs that the store masks off, so both forms are the same dense product.  The launcher
  // checks that the period is M * lda (N) and that the tile origin itself does not wrap.
  auto wraps = [&](const Access &a, size_t dim) { return a.mods.size() == 2 && a.mods[dim] >= 0; };
  const bool a_wraps = wraps(A->acc, 0), b_wraps = wraps(Bm->acc, 1);
  if (wraps(A->acc, 1) || wraps(Bm->acc, 0) || !C->acc.mods.empty()) refuse(F, "it wraps an address around in K or in the output");
  int r0, Mb, c0, Nb, r0c, Mc, c0c, Nc;
  if (C->acc.dims.size() != 2 || !m.extent(C->acc.dims[0], BM, r0c, Mc) || !m.extent(C->acc.dims[1], BN, c0c, Nc))
    refuse(F, "its output is not masked as (row0+arange < M) & (col0+arange < N)");
  if (A->acc.dims.size() != 2 || Bm->acc.dims.size() != 2) refuse(F, "its operand loads carry no K mask");
  if (a_wraps) {
    if (!m.is_const(A->acc.dims[0], BM)) refuse(F, "its A rows are both wrapped and masked");
    r0 = r0c; Mb = Mc;
  } else if (!m.extent(A->acc.dims[0], BM, r0, Mb)) refuse(F, "its A rows are not masked as row0+arange < M");
  if (b_wraps) {
    if (!m.is_const(Bm->acc.dims[1], BN)) refuse(F, "its B columns are both wrapped and masked");
    c0 = c0c; Nb = Nc;
  } else if (!m.extent(Bm->acc.dims[1], BN, c0, Nb)) refuse(F, "its B columns are not masked as col0+arange < N");
  if (r0 != r0c || c0 != c0c || Mb != Mc || Nb != Nc) refuse(F, "its operand masks and its output mask disagree");
  if (A->acc.dims[1] != Bm->acc.dims[0]) refuse(F, "A and B mask the K dimension differently");
  if (!m.pid_free(A->acc.dims[1])) refuse(F, "its K mask depends on the program id");
  for (int e : {Mb, Nb})
    if (!m.pid_free(e) || !m.loop_free(e)) refuse(F, "its problem size depends on the program id");
  for (SOp *a : {A, Bm})
    if (!a->acc.has_other || a->acc.other_f != 0.0 || a->acc.other_i != 0) refuse(F, "its operand loads do not pad with 0");
  auto consts = m.of_kind(SK::Const);
  if (consts.size() != 1 || consts[0]->fval != 0.0) refuse(F, "its accumulator does not start at 0");
  if (w8a16) {
    SOp *S = m.accesses[0];
    int s0, Ns;
    if (S->acc.sizes.size() != 1 || S->acc.sizes[0] != BN || S->acc.dims.empty() || !m.extent(S->acc.dims[0], BN, s0, Ns) ||
        s0 != c0 || Ns != Nb || S->acc.offsets[0] != c0)
      refuse(F, "its scale vector is not indexed and masked like the output columns");
    unit_stride(m, S->acc, F);
    pl.k["s_arg"] = S->acc.base_arg;
  }
  pl.family = w8a16 ? Family::GemmW8A16 : Family::Gemm;
  pl.k["BM"] = BM;
  pl.k["BN"] = BN;
  pl.k["BK"] = BK;
  pl.k["a_arg"] = A->acc.base_arg;
  pl.k["b_arg"] = Bm->acc.base_arg;
  pl.k["c_arg"] = C->acc.base_arg;
  pl.k["is_bf16"] = T == "bf16";
  pl.k["is_f32"] = T == "f32";
  pl.k["loop"] = loop->loop;
  pl.e["a_base"] = ca.base;
  pl.e["a_kstep"] = ca.kstep;
  pl.e["sam"] = ca.stride[0];
  pl.e["sak"] = ca.stride[1];
  pl.e["b_base"] = cb.base;
  pl.e["b_kstep"] = cb.kstep;
  pl.e["sbk"] = cb.stride[0];
  pl.e["sbn"] = cb.stride[1];
  pl.e["c_base"] = m.sum(C->acc.offsets);
  pl.e["scm"] = C->acc.strides[0];
  pl.e["scn"] = C->acc.strides[1];
  pl.e["r0"] = r0;
  pl.e["c0"] = c0;
  pl.e["M"] = Mb;
  pl.e["N"] = Nb;
  pl.e["kdim"] = A->acc.dims[1];
  pl.e["trip"] = loop->ub;
  if (a_wraps) { pl.e["a_mod"] = A->acc.mods[0]; pl.e["a_wrapped"] = ca.init[0]; }
  if (b_wraps) { pl.e["b_mod"] = Bm->acc.mods[1]; pl.e["b_wrapped"] = cb.init[1]; }
  return true;
}

// ----------------------------------------------------- gemm, gathered operands
// The product of a mixture-of-experts layer (test/Conversion/TritonToUnstructured/unstructured_ptr_used_in_loop.mlir
// has its shape): program (pm, pn) reads an id from memory -- negative: return at once --, takes BM rows of A through an
// index vector, multiplies them with the matrix b + id * stride, and stores a BM x BN tile of C.  The reference lowers
// the row gather to a loop of per-row copies (StructuredToMemref.cpp:855-993) and runs the rest as any other tiled
// product; here the matrix-product kernel takes the index vector and the table of ids as they are.
// The op structure is pinned by the signature; what the ops' leaves must be is checked here.
const char *SIG_GEMM_GATHERED =
    "v0=const:f32;v1=const:i32;v2=sload:i32.r0;v3=index;unless(v3){v4=iota;v5=index;v6=splat(v5);v7=arith.addi:i32(v6,v4);v8=index;"
    "v9=splat(v8);v10=arith.cmpi.slt:i1(v7,v9);v11=load:i32.r1.m.o;v12=iota;v13=expand.1(v11);v14=index;v15=splat(v14);v16=arith.mu"
    "li:i32(v13,v15);v17=expand.0(v12);v18=bcast(v17);v19=expand.1(v10);v20=bcast(v19);v21=arith.extsi:i64(v16);v22=bcast(v21);v23="
    "arith.extsi:i64(v18);v24=arith.addi:i64(v22,v23);for[v25<-v24,v26<-v0]{v27=index;v28=splat(v27);v29=arith.cmpi.slt:i1(v17,v28)"
    ";v30=bcast(v29);v31=arith.andi:i1(v20,v30);v32=load:{T}.r2.o;v33=load:{T}.r2.m.o;v34=dot(v32,v33,v26);v35=arith.extsi:i64(v1);"
    "v36=arith.addi:i64(v25,v35);yield(v36,v34)}->v37,v38;v39=arith.truncf:{T}(v38);store:{T}.r2.m(v39);};";

bool try_gemm_gathered(Plan &pl) {
  std::string T;
  if (pl.signature == subst(SIG_GEMM_GATHERED, "{T}", "bf16")) T = "bf16";
  else if (pl.signature == subst(SIG_GEMM_GATHERED, "{T}", "f16")) T = "f16";
  else return false;
  const char *F = "gemm (gathered rows)";
  Matcher m(pl.prog);
  ExprPool &X = m.X;
  if (m.all.size() != 39 || m.loops.size() != 1) return false;
  SOp *acc0 = m.all[0], *step = m.all[1], *id = m.all[2], *cond = m.all[3], *unless = m.all[4], *lane_m = m.all[5], *row0 = m.all[6],
      *n_rows = m.all[9], *rows = m.all[12], *lane_k = m.all[13], *pitch = m.all[15], *loop = m.all[26], *k_left = m.all[27],
      *k_ok = m.all[31], *A = m.all[32], *Bm = m.all[33], *C = m.all[38];
  if (A->acc.sizes.size() != 2 || Bm->acc.sizes.size() != 2 || C->acc.sizes.size() != 2) return false;
  const int64_t BM = A->acc.sizes[0], BK = A->acc.sizes[1], BN = Bm->acc.sizes[1];
  if (Bm->acc.sizes[0] != BK || C->acc.sizes[0] != BM || C->acc.sizes[1] != BN) refuse(F, "its block shapes do not compose");
  if (acc0->fval != 0.0) refuse(F, "its accumulator does not start at 0");
  if (BM % 128 != 0) refuse(F, "its blocks of rows are not whole 128-row kernel tiles");
  if (step->ival != BK) refuse(F, "its row pointers do not advance by one K block per iteration");
  if (unless->kind != SK::If || unless->ival != 1) return false;
  // the id and the early return
  if (id->acc.offsets.size() != 1 || id->acc.gather >= 0 || id->acc.mask_value >= 0) refuse(F, "its matrix id is not read from a plain address");
  {
    const Expr c = X.at(cond->expr);
    if (c.k != EK::CmpSel || c.val != 0 || X.at(c.a).k != EK::Data || X.at(c.a).a != id->result || !m.is_const(c.b, 0) || !m.is_const(c.c, 1) ||
        !m.is_const(c.d, 0))
      refuse(F, "its early return is not `id < 0`");
  }
  // rows: which = rows_ptr[row0 + arange(BM)], masked against n_rows
  if (lane_m->ival != 0 || lane_k->ival != 0) refuse(F, "its lane indices do not start at 0");
  const int r0 = X.to_index(row0->expr), Mb = X.to_index(n_rows->expr);
  {
    int start, bound;
    if (rows->acc.gather >= 0 || rows->acc.mask_value >= 0 || rows->acc.sizes.size() != 1 || rows->acc.sizes[0] != BM || !m.is_const(rows->acc.strides[0], 1) ||
        X.to_index(rows->acc.offsets[0]) != r0 || rows->acc.dims.size() != 1 || !m.extent(rows->acc.dims[0], BM, start, bound) || start != r0 || bound != Mb ||
        rows->acc.other_i != 0 || !rows->acc.mods.empty())
      refuse(F, "its index vector is not rows_ptr[row0 + arange] masked against the row count");
  }
  if (!m.pid_free(Mb) || !m.loop_free(Mb) || !m.pid_free(pitch->expr) || !m.loop_free(pitch->expr)) refuse(F, "its row count or row pitch depends on the program id");
  // the K loop: k0 = 0, BK, ... < K; the K mask is arange(BK) < K - k0
  if (!m.is_const(loop->lb, 0) || !m.is_const(loop->step, BK) || !m.pid_free(loop->ub)) refuse(F, "its K loop is not range(0, K, BK)");
  {
    const Expr l = X.at(k_left->expr);
    if (l.k != EK::Sub || l.a != loop->ub || X.at(l.b).k != EK::IV || X.at(l.b).a != loop->loop) refuse(F, "its K mask is not arange < K - k0");
  }
  // A: gathered through the carried block of offsets, masked by (row ok) & (k ok), padded with 0
  if (A->acc.gather != loop->tile_args.at(0) || A->acc.mask_value != k_ok->result || !A->acc.has_other || A->acc.other_f != 0.0 || A->acc.other_value >= 0 ||
      A->acc.offsets.size() != 1 || !m.is_const(A->acc.offsets[0], 0))
    refuse(F, "its A rows are not read through the carried offsets with the row and K masks, padded with 0");
  // B: a structured block below the matrix the id picks
  if (Bm->acc.gather >= 0 || Bm->acc.mask_value >= 0 || !Bm->acc.mods.empty() || !C->acc.mods.empty()) refuse(F, "its B or C block is not structured");
  Carried2D cb;
  if (!carried_state(m, loop, Bm->acc, cb)) refuse(F, "its B pointer does not advance by a constant per K step");
  int block_stride = -1;
  bool mul32 = false;
  {
    int e = cb.init[0];
    if (X.at(e).k == EK::Sext) { e = X.at(e).a; mul32 = true; }
    const Expr mu = X.at(e);
    if (mu.k != EK::Mul) refuse(F, "its B base is not id * stride");
    auto is_id = [&](int x) { return X.at(x).k == EK::Data && X.at(x).a == id->result; };
    if (is_id(mu.a)) block_stride = mu.b;
    else if (is_id(mu.b)) block_stride = mu.a;
    else refuse(F, "its B base is not id * stride");
    if (mu.bits != 32) mul32 = false;
    if (!m.pid_free(block_stride) || !m.loop_free(block_stride) || X.depends_on(block_stride, EK::Data)) refuse(F, "its matrix stride is not a launch constant");
  }
  const int c0 = X.to_index(cb.init[1]);
  if (X.depends_on(c0, EK::Data) || !m.loop_free(c0)) refuse(F, "its column origin depends on data");
  if (!m.is_const(cb.stride[1], 1)) refuse(F, "B's inner stride is not 1");
  int c0b, Nb, r0c, Mc, c0c, Nc;
  if (Bm->acc.dims.size() != 2 || !m.pid_free(Bm->acc.dims[0]) || !m.extent(Bm->acc.dims[1], BN, c0b, Nb) || c0b != c0)
    refuse(F, "its B block is not masked as (K left) x (col0 + arange < N)");
  if (C->acc.dims.size() != 2 || !m.extent(C->acc.dims[0], BM, r0c, Mc) || !m.extent(C->acc.dims[1], BN, c0c, Nc) || r0c != r0 || Mc != Mb || c0c != c0 || Nc != Nb)
    refuse(F, "its output is not masked as (row0 + arange < rows) & (col0 + arange < N)");
  if (!m.pid_free(Nb) || !m.loop_free(Nb)) refuse(F, "its column count depends on the program id");
  if (!m.is_const(C->acc.strides[1], 1)) refuse(F, "C's inner stride is not 1");
  if (!Bm->acc.has_other || Bm->acc.other_f != 0.0) refuse(F, "its B block does not pad with 0");
  if (A->acc.elem != T || Bm->acc.elem != T || C->acc.elem != T) return false;
  LinIv lid;
  if (!m.linear(id->acc.offsets[0], lid)) refuse(F, "the address of its matrix id is not linear in the program id");
  pl.family = Family::Gemm;
  pl.k["gathered"] = 1;
  pl.k["BM"] = BM; pl.k["BN"] = BN; pl.k["BK"] = BK;
  pl.k["a_arg"] = A->acc.base_arg;
  pl.k["b_arg"] = Bm->acc.base_arg;
  pl.k["c_arg"] = C->acc.base_arg;
  pl.k["rows_arg"] = rows->acc.base_arg;
  pl.k["block_arg"] = id->acc.base_arg;
  pl.k["is_bf16"] = T == "bf16";
  pl.k["mul32"] = mul32;
  pl.e["r0"] = r0;
  pl.e["c0"] = c0;
  pl.e["M"] = Mb;
  pl.e["N"] = Nb;
  pl.e["K"] = loop->ub;
  pl.e["sam"] = pitch->expr;
  pl.e["sbk"] = cb.stride[0];
  pl.e["b_kstep"] = cb.kstep;
  pl.e["scm"] = C->acc.strides[0];
  pl.e["c_base"] = m.sum(C->acc.offsets);
  pl.e["block_off"] = X.to_index(id->acc.offsets[0]);
  pl.e["block_stride"] = block_stride;
  return true;
}

}  // namespace

// ------------------------------------------------------------- fused map
// Any straight-line program of one-dimensional loads, elementwise ops, constants, splatted scalar
// arguments and stores over blocks of one size becomes a register program for the interpreter
// kernel: one instruction per elementwise op (the reference runs one linalg.generic loop per op,
// TritonArithToLinalg.cpp:104; here they run back to back on values that stay on chip).
bool try_fused_map(Plan &pl) {
  Matcher m(pl.prog);
  const char *F = "fused_map";
  if (!m.loops.empty() || m.accesses.empty()) return false;
  std::vector<SOp *> loads, stores;
  int64_t B = -1;
  for (SOp *s : m.all) {
    switch (s->kind) {
      case SK::Load: loads.push_back(s); break;
      case SK::Store: stores.push_back(s); break;
      case SK::Map: case SK::Splat: case SK::Const: case SK::ScalarArg: break;
      default: return false;
    }
    if (s->kind == SK::Load || s->kind == SK::Store) {
      if (s->acc.sizes.size() != 1) return false;
      if (B < 0) B = s->acc.sizes[0];
      if (s->acc.sizes[0] != B) return false;
    }
  }
  if (stores.empty() || B <= 0) return false;
  {
    // the kernel performs every load before the first store: a load from an argument that an earlier store wrote has
    // to see that store, which only the generic family's phases arrange
    std::set<int> stored;
    for (SOp *s : m.all) {
      if (s->kind == SK::Load && stored.count(s->acc.base_arg)) return false;
      if (s->kind == SK::Store) stored.insert(s->acc.base_arg);
    }
  }
  for (SOp *s : m.all)
    if (s->result >= 0) {
      const Value &v = pl.prog.values[s->result];
      if (!(v.shape.empty() || (v.shape.size() == 1 && v.shape[0] == B))) return false;
    }
  no_wrap(m, F);
  if ((int)loads.size() > MAPN_MAX_IN) refuse(F, "it has more than " + std::to_string(MAPN_MAX_IN) + " block loads");
  if (loads.empty()) refuse(F, "it loads nothing");
  if ((int)stores.size() > MAPN_MAX_OUT) refuse(F, "it has more than " + std::to_string(MAPN_MAX_OUT) + " block stores");
  auto type_code = [&](const std::string &t) -> int {
    if (t == "f32") return 0;
    if (t == "f16") return 1;
    if (t == "bf16") return 2;
    refuse(F, "element type " + t + " (fp32, fp16 and bf16 are implemented)");
  };
  const std::vector<int> &dims = stores[0]->acc.dims;
  for (SOp *a : m.accesses) {
    unit_stride(m, a->acc, F);
    if (a->acc.dims != dims) refuse(F, "its loads and stores are masked differently");
  }
  // liveness: position of the last use of every value
  std::map<int, size_t> last_use;
  for (size_t i = 0; i < m.all.size(); i++)
    for (int v : m.all[i]->operands) last_use[v] = m.all[i]->kind == SK::Store ? SIZE_MAX : std::max(last_use[v], i);
  // (the kernel stores after the whole program has run, so a stored value keeps its register to the end)
  static const std::map<std::string, int> ops = {
      {"arith.addf", MO_ADD}, {"arith.subf", MO_SUB}, {"arith.mulf", MO_MUL}, {"arith.divf", MO_DIV},
      {"arith.maxnumf", MO_MAXNUM}, {"arith.minnumf", MO_MINNUM}, {"arith.maximumf", MO_MAXIMUM}, {"arith.minimumf", MO_MINIMUM},
      {"arith.negf", MO_NEG}, {"math.absf", MO_ABS}, {"math.exp", MO_EXP}, {"math.exp2", MO_EXP2}, {"math.log", MO_LOG},
      {"math.log2", MO_LOG2}, {"math.sqrt", MO_SQRT}, {"math.rsqrt", MO_RSQRT}, {"math.sin", MO_SIN}, {"math.cos", MO_COS},
      {"math.tanh", MO_TANH}, {"math.erf", MO_ERF}, {"math.floor", MO_FLOOR}, {"math.ceil", MO_CEIL}, {"math.fma", MO_FMA},
      {"arith.select", MO_SELECT}, {"arith.andi", MO_AND}, {"arith.ori", MO_OR}, {"arith.xori", MO_XOR},
      {"arith.cmpf.oeq", MO_CMP_OEQ}, {"arith.cmpf.one", MO_CMP_ONE}, {"arith.cmpf.olt", MO_CMP_OLT}, {"arith.cmpf.ole", MO_CMP_OLE},
      {"arith.cmpf.ogt", MO_CMP_OGT}, {"arith.cmpf.oge", MO_CMP_OGE}, {"arith.cmpf.une", MO_CMP_UNE}, {"arith.cmpf.ueq", MO_CMP_UEQ},
      {"arith.cmpf.ult", MO_CMP_ULT}, {"arith.cmpf.ule", MO_CMP_ULE}, {"arith.cmpf.ugt", MO_CMP_UGT}, {"arith.cmpf.uge", MO_CMP_UGE},
      {"arith.cmpf.ord", MO_CMP_ORD}, {"arith.cmpf.uno", MO_CMP_UNO}, {"arith.extf", MO_MOV}, {"arith.truncf", MO_MOV}};
  // operands: a value lives in a register, is the result of the instruction before, or is an immediate
  struct Where { int kind = -1, idx = 0; };
  std::map<int, int> reg_of;          // value -> register
  std::map<int, int> imm_of;          // value -> immediate index
  std::map<int, int> scalar_arg_of;   // scalar value -> kernel argument index
  std::vector<char> busy(MAPN_MAX_REGS, 0);
  auto alloc = [&]() {
    for (int r = 0; r < MAPN_MAX_REGS; r++)
      if (!busy[r]) { busy[r] = 1; return r; }
    refuse(F, "it keeps more than " + std::to_string(MAPN_MAX_REGS) + " block values alive at once");
  };
  // the kernel performs every load before the first instruction, so loaded values get their
  // registers first; such a register is reused only after its loaded value has died
  for (SOp *s : loads) reg_of[s->result] = alloc();
  // positions of the ops that become instructions, and per value the positions that read it
  std::vector<size_t> map_pos;
  std::map<int, std::vector<size_t>> readers;
  for (size_t i = 0; i < m.all.size(); i++) {
    if (m.all[i]->kind == SK::Map) map_pos.push_back(i);
    for (int v : m.all[i]->operands) readers[v].push_back(i);
  }
  auto next_map_after = [&](size_t pos) -> size_t {
    for (size_t q : map_pos)
      if (q > pos) return q;
    return SIZE_MAX;
  };
  int n_ins = 0, n_imm = 0, n_in = 0, n_out = 0, n_regs = (int)loads.size();
  int prev_value = -1;
  auto new_imm = [&](double value, int arg) {
    if (n_imm >= MAPN_MAX_IMM) refuse(F, "it has more than " + std::to_string(MAPN_MAX_IMM) + " constants and scalar arguments");
    pl.f["imm" + std::to_string(n_imm)] = value;
    pl.k["imm" + std::to_string(n_imm) + "_arg"] = arg;
    return n_imm++;
  };
  auto round_of = [&](int value) {
    const std::string &t = pl.prog.values[value].dtype;
    return t == "f16" ? 1 : t == "bf16" ? 2 : 0;
  };
  auto release_dead = [&](size_t pos, const std::vector<int> &operands) {
    for (int v : operands) {
      auto it = reg_of.find(v);
      if (it != reg_of.end() && last_use[v] == pos) busy[it->second] = 0;
    }
  };
  for (size_t i = 0; i < m.all.size(); i++) {
    SOp *s = m.all[i];
    switch (s->kind) {
      case SK::ScalarArg: scalar_arg_of[s->result] = (int)s->ival; break;
      case SK::Load: {
        LinIv l;
        if (!m.linear(s->acc.offsets[0], l)) refuse(F, "a block offset is not linear in the program id");
        std::string n = "in" + std::to_string(n_in++);
        pl.lin[n + "_off"] = as_lin(l, s->acc.offsets[0]);
        pl.k[n + "_arg"] = s->acc.base_arg;
        pl.k[n + "_type"] = type_code(s->acc.elem);
        pl.f[n + "_other"] = s->acc.has_other ? s->acc.other_f : 0.0;
        pl.k[n + "_reg"] = reg_of.at(s->result);
        if (!last_use.count(s->result)) busy[reg_of.at(s->result)] = 0;
        break;
      }
      case SK::Const: {
        const Value &v = pl.prog.values[s->result];
        if (v.dtype[0] == 'i' && v.dtype != "i1") refuse(F, "integer block constants are not implemented");
        imm_of[s->result] = new_imm(v.dtype == "i1" ? (double)(s->ival != 0) : s->fval, -1);
        break;
      }
      case SK::Splat: {
        auto it = scalar_arg_of.find(s->operands.at(0));
        if (it == scalar_arg_of.end()) refuse(F, "it splats something other than a floating-point kernel argument");
        if (round_of(s->result)) refuse(F, "it splats a scalar argument into a narrow float type");
        imm_of[s->result] = new_imm(0.0, it->second);
        break;
      }
      case SK::Map: {
        auto it = ops.find(s->name);
        if (it == ops.end()) refuse(F, "elementwise op " + s->name + " is not implemented");
        const Value &rv = pl.prog.values[s->result];
        if (rv.dtype != "f32" && rv.dtype != "f16" && rv.dtype != "bf16" && rv.dtype != "i1")
          refuse(F, "elementwise op " + s->name + " on " + rv.dtype + " is not implemented");
        if (s->operands.size() > 3) refuse(F, "elementwise op " + s->name + " has more than three operands");
        int src[3] = {0, 0, 0}, kind[3] = {MS_REG, MS_REG, MS_REG};
        for (size_t q = 0; q < s->operands.size(); q++) {
          const int v = s->operands[q];
          const std::string &ot = pl.prog.values[v].dtype;
          if (ot != "f32" && ot != "f16" && ot != "bf16" && ot != "i1") refuse(F, "elementwise op " + s->name + " on " + ot + " is not implemented");
          if (imm_of.count(v)) { kind[q] = MS_IMM; src[q] = imm_of[v]; }
          else if (v == prev_value) { kind[q] = MS_PREV; }
          else if (reg_of.count(v)) { kind[q] = MS_REG; src[q] = reg_of[v]; }
          else refuse(F, "an operand of " + s->name + " is not a block value");
        }
        release_dead(i, s->operands);  // the result may take the register of an operand that dies here
        // the result goes to the register file unless its only reader is the next instruction
        const auto &rd = readers[s->result];
        const size_t nxt = next_map_after(i);
        bool only_next = !rd.empty();
        for (size_t q : rd) only_next = only_next && q == nxt && m.all[q]->kind == SK::Map;
        int dst = 0;
        if (!only_next && !rd.empty()) {
          dst = alloc();
          reg_of[s->result] = dst;
          n_regs = std::max(n_regs, dst + 1);
        }
        if (n_ins >= MAPN_MAX_INS) refuse(F, "it has more than " + std::to_string(MAPN_MAX_INS) + " elementwise ops");
        const int kinds = kind[0] | (kind[1] << 2) | (kind[2] << 4) | ((only_next || rd.empty()) ? 64 : 0);
        pl.k["ins" + std::to_string(n_ins++)] = (int64_t)it->second | ((int64_t)dst << 8) | ((int64_t)src[0] << 16) | ((int64_t)src[1] << 24) |
                                                ((int64_t)src[2] << 32) | ((int64_t)kinds << 40) | ((int64_t)round_of(s->result) << 48);
        prev_value = s->result;
        break;
      }
      case SK::Store: {
        LinIv l;
        if (!m.linear(s->acc.offsets[0], l)) refuse(F, "a block offset is not linear in the program id");
        const int v = s->operands.at(0);
        if (!reg_of.count(v)) refuse(F, "it stores something that is not a computed or loaded block value");
        if (pl.prog.values[v].dtype != s->acc.elem) refuse(F, "a stored value and its destination differ in type");
        std::string n = "out" + std::to_string(n_out++);
        pl.lin[n + "_off"] = as_lin(l, s->acc.offsets[0]);
        pl.k[n + "_arg"] = s->acc.base_arg;
        pl.k[n + "_type"] = type_code(s->acc.elem);
        pl.k[n + "_reg"] = reg_of[v];
        break;
      }
      default: return false;
    }
  }
  pl.family = Family::FusedMap;
  pl.k["block"] = B;
  pl.k["n_in"] = n_in;
  pl.k["n_out"] = n_out;
  pl.k["n_ins"] = n_ins;
  pl.k["n_imm"] = n_imm;
  pl.k["n_regs"] = n_regs;
  pl.k["masked"] = !dims.empty();
  if (!dims.empty()) {
    int start, bound;
    if (!m.extent(dims[0], B, start, bound)) refuse(F, "its mask is not of the form start+arange < bound");
    LinIv l;
    if (!m.linear(start, l)) refuse(F, "its mask start is not linear in the program id");
    if (!m.pid_free(bound) || !m.loop_free(bound)) refuse(F, "its mask bound depends on the program id");
    pl.lin["m_start"] = as_lin(l, start);
    pl.e["bound"] = bound;
  }
  return true;
}

// Anything made of structured loads, elementwise ops and stores that no hand-written family took.
bool try_tile_program(Plan &pl) {
  Matcher m(pl.prog);
  if (m.accesses.empty()) return false;
  pl.source = tile_program_source(pl.prog);  // throws Unsupported with the reason
  pl.family = Family::TileProgram;
  return true;
}

// A tiled matmul whose accumulator goes through elementwise ops before the store (the tutorial kernel's fused
// activation, test_matmul.py:98-99; a bias, a residual): what stands between the K loop and the store is taken out as an
// epilogue functor, and what is left -- the loop, a narrowing cast, the store -- is matched as the plain product.
// What the matrix-product families check only at launch (strides, M, the grid) may fail for a launch that the
// generic family runs all the same: its kernel for the same program, if it takes the program.
static std::string generic_fallback(const Program &p) {
  try {
    return tile_program_source(p);
  } catch (const Unsupported &) {
    return std::string();
  }
}

static bool try_gemm_with_epilogue(Plan &pl) {
  const Program &P = pl.prog;
  int loop_at = -1, store_at = -1;
  for (size_t i = 0; i < P.body.size(); i++) {
    const SK k = P.body[i].kind;
    if (k == SK::For) {
      if (loop_at >= 0) return false;
      loop_at = (int)i;
    } else if (k == SK::Store) {
      if (store_at >= 0) return false;
      store_at = (int)i;
    } else if (k != SK::Map && k != SK::Const && k != SK::Splat && k != SK::ScalarArg && k != SK::FromIndex && k != SK::Load && k != SK::Iota &&
               k != SK::ExpandDims && k != SK::Broadcast) {
      return false;
    }
  }
  if (loop_at < 0 || store_at != (int)P.body.size() - 1 || store_at < loop_at) return false;
  const SOp &loop = P.body[loop_at], &st = P.body[store_at];
  if (loop.results.size() != 1 || loop.results[0] < 0 || st.operands.empty()) return false;
  const int acc = loop.results[0], out = st.operands[0];
  const std::string T = st.acc.elem;
  if ((T != "bf16" && T != "f16") || P.values[acc].dtype != "f32" || P.values[out].shape != P.values[acc].shape) return false;
  if (store_at == loop_at + 2 && P.body[loop_at + 1].kind == SK::Map && P.body[loop_at + 1].name == "arith.truncf" &&
      P.body[loop_at + 1].operands.at(0) == acc)
    return false;  // the plain product: nothing to take out
  // the product without the epilogue
  Program Q = P;
  Value narrowed = P.values[acc];
  narrowed.dtype = T;
  Q.values.push_back(narrowed);
  SOp cast;
  cast.kind = SK::Map;
  cast.name = "arith.truncf";
  cast.operands = {acc};
  cast.result = (int)Q.values.size() - 1;
  SOp store = st;
  store.operands[0] = cast.result;
  // values the loop reads keep their definitions; what only the epilogue read goes
  std::set<int> used;
  std::function<void(const SOp &)> reads = [&](const SOp &s) {
    for (int v : s.operands) used.insert(v);
    for (int v : s.tile_inits) used.insert(v);
    for (int v : {s.acc.gather, s.acc.mask_value, s.acc.other_value})
      if (v >= 0) used.insert(v);
    for (auto &b : s.body) reads(b);
  };
  reads(loop);
  std::vector<SOp> kept;
  for (int i = loop_at - 1; i >= 0; i--) {
    const SOp &s = P.body[i];
    if (s.result >= 0 && !used.count(s.result)) continue;
    reads(s);
    kept.insert(kept.begin(), s);
  }
  Q.body = kept;
  Q.body.push_back(loop);
  Q.body.push_back(cast);
  Q.body.push_back(store);
  Plan q;
  q.prog = std::move(Q);
  q.signature = signature(q.prog);
  try {
    if (!try_gemm(q, false)) return false;
    std::vector<const SOp *> ops;
    for (auto &s : P.body)
      if (s.kind != SK::For && s.kind != SK::Store) ops.push_back(&s);
    q.source = gemm_epilogue_source(P, ops, acc, out, q.k.at("BM"), q.k.at("BN"));
  } catch (const Unsupported &) {
    return false;  // not this shape of program: the other families get their turn
  }
  q.fallback_source = generic_fallback(P);
  pl = std::move(q);
  return true;
}

Plan make_plan(Program &&p) {
  Plan pl;
  pl.prog = std::move(p);
  pl.signature = signature(pl.prog);
  // the hand-written families read their operands through structured accesses only: a program with a gather or a
  // scatter goes to the generic family
  if (pl.prog.body.empty()) {  // nothing with an effect on memory is left: an empty kernel keeps the launch's place in the stream
    pl.source = tile_program_source(pl.prog);
    pl.family = Family::TileProgram;
    return pl;
  }
  {
    // one unstructured shape the matrix-product kernels take: a product whose A rows come through an index vector and
    // whose B matrix is picked by an id read from memory (the generic family's kernel stays behind it for launches
    // those kernels decline)
    bool taken = false;
    try {
      taken = try_gemm_gathered(pl);
    } catch (const Unsupported &) {
      pl.k.clear(); pl.e.clear(); pl.lin.clear(); pl.f.clear();
    }
    if (taken) {
      pl.fallback_source = generic_fallback(pl.prog);
      return pl;
    }
  }
  bool unstructured = pl.prog.pool.has_data();  // addresses that depend on loaded values: nothing the host could check or bind
  {
    Matcher m(pl.prog);
    for (SOp *a : m.accesses) unstructured = unstructured || a->acc.gather >= 0 || a->acc.other_value >= 0 || a->acc.mask_value >= 0;
  }
  if (unstructured) {
    if (try_tile_program(pl)) return pl;
    throw Unsupported("a program with gathers, scatters or masks and fill values that are data is outside the hand-written families; signature: " + pl.signature);
  }
  // A program with the op structure of a hand-written family but a detail that family declines (another element
  // type, a strided load, a block too long) goes on to the families after it; the first refusal is the one reported
  // if none of them takes it.
  std::string first_refusal;
  auto reset = [&]() { pl.k.clear(); pl.e.clear(); pl.lin.clear(); pl.f.clear(); };
  for (bool (*attempt)(Plan &) : {try_map1d, try_softmax, try_layernorm}) {
    try {
      if (attempt(pl)) return pl;
    } catch (const Unsupported &e) {
      if (first_refusal.empty()) first_refusal = e.what();
      reset();
    }
  }
  if (!first_refusal.empty()) {
    try {
      if (try_fused_map(pl)) return pl;
    } catch (const Unsupported &) {
      reset();
    }
    try {
      if (try_tile_program(pl)) return pl;
    } catch (const Unsupported &) {
    }
    throw Unsupported(first_refusal);
  }
  if (try_gemm_with_epilogue(pl)) return pl;
  std::string gemm_refusal;
  try {
    if (try_gemm(pl, false) || try_gemm(pl, true)) {
      pl.fallback_source = generic_fallback(pl.prog);
      return pl;
    }
  } catch (const Unsupported &e) {
    // shaped like a tiled matmul but outside what those kernels take: the generic family may run it (small tiles);
    // if not, the matmul family's reason is the one to report
    gemm_refusal = e.what();
    pl.k.clear(); pl.e.clear(); pl.lin.clear(); pl.f.clear();
  }
  if (!gemm_refusal.empty()) {
    try {
      if (try_tile_program(pl)) return pl;
    } catch (const Unsupported &) {
    }
    throw Unsupported(gemm_refusal);
  }
  try {
    if (try_fused_map(pl)) return pl;
  } catch (const Unsupported &) {
    // what the vectorised one-dimensional map declines (integer data, loads and stores masked differently, ...) the
    // generic family may still take
    pl.k.clear(); pl.e.clear(); pl.lin.clear(); pl.f.clear();
  }
  if (try_tile_program(pl)) return pl;
  throw Unsupported("no hand-written kernel family matches this structured program; signature: " + pl.signature);
}

}  // namespace tts
