// Structured program -> HIP source: the generic family behind the hand-tuned ones.  It takes whatever
// program of block loads and stores (structured, wrapped, gathered / scattered), elementwise ops,
// reductions, scans, index shuffles, small matrix products, loops and branches no other family took.
//
// What the reference does with such a program: one memref copy per load/store
// (StructuredToMemref.cpp:748-853,1163-1196, wraparound as two chunks :263-487, gathers and scatters as
// loops over rows :855-993,1034-1157), one linalg.generic loop per elementwise op
// (TritonArithToLinalg.cpp:104), linalg.reduce / linalg.matmul (ConversionPatterns.hpp:1128-1440),
// scf.for / scf.if around them.
// Here one workgroup of 256 threads runs one program.  Thread t owns elements t, t + 256, ... of every
// block (row-major); the ops of a body are fused into loops over the elements, index expressions are
// printed from the expression pool with their i32 / index widths, and the source is compiled with
// hipRTC at the plan's first launch.
//
// Order of memory effects.  The reference finishes every load of a body before the op after it
// starts.  A fused element loop keeps that order per element only, which differs when a store
// writes what another element's load reads (an in-place shift).  Blocks of up to 16384 elements are
// therefore run in two phases -- every load of a run of ops into per-thread registers, a barrier,
// then ops and stores; larger blocks are fused in one loop and accepted only when no store's base
// argument is also a load's.
//
// Values.  A block value lives in one of four places: nowhere (an elementwise op is written out where
// its result is used), the owning threads' registers (loads of a two-phase run, loop-carried blocks,
// results of matrix products and of `if`), LDS (results of reductions and scans, small blocks of another
// shape than the run's), or memory (a load of another shape that found no room in LDS is read again
// where it is used; the program is refused if its base is also stored to).  Registers can only be named
// for the element the thread owns: any other element, behind a transpose say, is computed again.
//
// Loads are written so that they issue back to back: a wavefront's loads complete in order, so a load
// whose address waits for another load's result, or a select between a loaded value and `other` right
// after the load, serialises the whole run (see the notes at the two places).
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>
#include <set>
#include <sstream>

#include "match.h"

namespace tts {

namespace {

constexpr int64_t HAZARD_MAX = 65536;     // elements; the limit for blocks that must run in two phases
constexpr int64_t TWO_PHASE_MAX = 16384;  // elements; 64 registers per thread and held block value

struct Gen {
  const Program &P;
  std::ostringstream os;
  std::map<int, const SOp *> def;          // value id -> defining op
  std::map<int, std::string> var;          // value id -> C variable holding it at the current element
  int indent = 1;
  std::set<int> all_inline_bases, all_store_bases;  // checked against each other at the end
  // Arguments the program reads anywhere, and arguments a scalar store writes anywhere (collected before the body is
  // written, so that an access in a later iteration of a loop counts): a scalar store is one thread's, every read is
  // all threads', so the two are kept apart by barriers wherever they may touch the same argument.
  std::set<int> read_bases_anywhere, scalar_store_bases_anywhere;
  std::map<int, int> uses;  // value id -> how many operands of the program name it
  std::map<int, std::vector<const SOp *>> users;  // value id -> the ops that name it
  void collect_bases(const std::vector<SOp> &ops) {
    for (const SOp &s : ops) {
      if (s.kind == SK::Load || s.kind == SK::ScalarLoad) read_bases_anywhere.insert(s.acc.base_arg);
      if (s.kind == SK::ScalarStore) scalar_store_bases_anywhere.insert(s.acc.base_arg);
      for (int v : s.operands) uses[v]++, users[v].push_back(&s);
      for (int v : s.tile_inits) uses[v]++, users[v].push_back(&s);
      for (int v : s.tile_yields) uses[v]++, users[v].push_back(&s);
      for (int v : {s.acc.gather, s.acc.mask_value, s.acc.other_value})
        if (v >= 0) uses[v]++, users[v].push_back(&s);
      if (s.kind == SK::For || s.kind == SK::If) collect_bases(s.body);
    }
  }
  // Does computing v take a transcendental function, a division or a square root?  (Worth a register per element to a
  // value that is used twice: every use of a value that has no register writes its whole expression out again.)
  bool costly(int v, int depth = 0) {
    auto d = def.find(v);
    if (d == def.end() || depth > 24 || var.count(v) || held.count(v)) return false;
    const SOp &o = *d->second;
    if (o.kind == SK::Map) {
      static const char *heavy[] = {"math.exp", "math.log", "math.sqrt", "math.rsqrt", "arith.divf", "math.erf", "math.tanh", "math.sin", "math.cos",
                                    "math.pow", "tt.precise", "extern.", "arith.remf", "arith.divsi", "arith.divui", "arith.remsi", "arith.remui"};
      for (const char *h : heavy)
        if (o.name.rfind(h, 0) == 0) return true;
    }
    if (o.kind != SK::Map && o.kind != SK::Broadcast && o.kind != SK::ExpandDims && o.kind != SK::Splat) return false;
    for (int x : o.operands)
      if (costly(x, depth + 1)) return true;
    return false;
  }
  // Is v only ever read element by element, by ops over blocks of its own shape (through any chain of elementwise ops,
  // down to block stores)?  Then the thread that owns an element is the only one that needs it.
  bool read_in_place_only(int v, const std::vector<int64_t> &shape, int depth = 0) {
    if (depth > 32) return false;
    auto u = users.find(v);
    if (u == users.end()) return true;
    for (const SOp *o : u->second) {
      if (o->kind == SK::Store) {
        if (o->acc.sizes != shape || o->acc.gather == v) return false;  // (offsets of a scatter are read by index expressions)
        continue;
      }
      if (o->kind != SK::Map || o->result < 0 || val(o->result).shape != shape) return false;
      if (o->name.rfind("tt.", 0) == 0 && o->name != "tt.clampf.none" && o->name != "tt.clampf.all" && o->name != "tt.precise_sqrt" && o->name != "tt.precise_divf" &&
          o->name != "tt.mulhiui" && o->name != "tt.bitcast")
        return false;  // transposes, reshapes, joins and the like read other elements
      if (!read_in_place_only(o->result, shape, depth + 1)) return false;
    }
    return true;
  }
  std::vector<int> kept_by_scan;  // results of the last scan that stay in the owning threads' registers (see reduce())
  std::ostringstream fns;                           // combiner functions of reductions and scans (before the kernel)
  std::ostringstream decl;                          // LDS arrays holding their results (top of the kernel)
  size_t pool_bytes = 0, out_bytes = 0;             // staging pool shared by all reductions; result arrays
  bool uses_mfma = false;
  bool uses_dummy = false;  // wide loads of invalid groups read this instead

  explicit Gen(const Program &p) : P(p) {}

  [[noreturn]] void no(const std::string &why) { throw Unsupported("tile_program: " + why); }
  std::string pad() const { return std::string(2 * indent, ' '); }

  static std::string ctype(const std::string &t) {
    if (t == "f32" || t == "f16" || t == "bf16") return "float";
    if (t == "i1") return "bool";
    if (t == "i8") return "signed char";
    if (t == "i16") return "short";
    if (t == "i32") return "int";
    if (t == "i64") return "long long";
    if (t == "f64") return "double";
    throw Unsupported("tile_program: element type " + t);
  }
  static std::string memtype(const std::string &t) {
    if (t == "f32") return "float";
    if (t == "f16" || t == "bf16") return "unsigned short";
    return ctype(t);
  }
  static bool is_float(const std::string &t) { return t[0] == 'f' || t[0] == 'b'; }
  static bool is16(const std::string &t) { return t == "f16" || t == "bf16"; }
  static int mem_bytes(const std::string &t) { return t == "i8" ? 1 : is16(t) ? 2 : 4; }  // of the element types vector_access takes

  // ---- index expressions -------------------------------------------------
  // name_index_exprs: every operation node of the pool becomes a local (`const long long x<id> = ...;` in index_locals,
  // operands before their users), and ex() returns the local's name: a caller that evaluates its expression many times on
  // the same leaves (the matrix-product epilogue, once per accumulator element) then has the shared part in one place.
  bool name_index_exprs = false;
  std::ostringstream index_locals;
  std::map<int, std::string> named_exprs;
  std::string ex(int id) {
    if (!name_index_exprs) return ex_text(id);
    const EK k = P.pool.at(id).k;
    if (k == EK::Const || k == EK::Arg || k == EK::Pid || k == EK::NProg || k == EK::IV || k == EK::Iter || k == EK::Result || k == EK::Data)
      return ex_text(id);
    auto it = named_exprs.find(id);
    if (it != named_exprs.end()) return it->second;
    const std::string text = ex_text(id);  // (names the operands first)
    const std::string name = "x" + std::to_string(id);
    index_locals << "    const long long " << name << " = " << text << ";\n";
    named_exprs[id] = name;
    return name;
  }
  std::string ex_text(int id) {
    const Expr &e = P.pool.at(id);
    auto w = [&](const std::string &s) { return e.bits == 32 ? "(long long)(int)(" + s + ")" : "(" + s + ")"; };
    auto u = [&](const char *op) {  // wrapping arithmetic through unsigned
      return e.bits == 32 ? "(long long)(int)((unsigned)" + ex(e.a) + " " + op + " (unsigned)" + ex(e.b) + ")"
                          : "(long long)((unsigned long long)" + ex(e.a) + " " + op + " (unsigned long long)" + ex(e.b) + ")";
    };
    switch (e.k) {
      case EK::Const: return "(" + std::to_string(e.val) + "LL)";
      case EK::Arg: return w("p.ival[" + std::to_string(e.a) + "]");
      case EK::Pid: return std::string("pid") + "xyz"[e.a];
      case EK::NProg: return std::string("np") + "xyz"[e.a];
      case EK::IV: return "iv" + std::to_string(e.a);
      case EK::Iter: return "it" + std::to_string(e.a) + "_" + std::to_string(e.b);
      case EK::Result: return "res" + std::to_string(e.a) + "_" + std::to_string(e.b);
      case EK::Data: return w("(long long)" + at(e.a, "0", "0"));
      case EK::Add: return u("+");
      case EK::Sub: return u("-");
      case EK::Mul: return u("*");
      case EK::DivS: return e.bits == 32 ? "sdiv32(" + ex(e.a) + ", " + ex(e.b) + ")" : "(sdiv(" + ex(e.a) + ", " + ex(e.b) + "))";
      case EK::RemS: return e.bits == 32 ? "srem32(" + ex(e.a) + ", " + ex(e.b) + ")" : "(srem(" + ex(e.a) + ", " + ex(e.b) + "))";
      case EK::MinS: return "smin(" + ex(e.a) + ", " + ex(e.b) + ")";
      case EK::MaxS: return "smax(" + ex(e.a) + ", " + ex(e.b) + ")";
      case EK::Sext: return ex(e.a);
      case EK::Trunc: return "(long long)(int)" + ex(e.a);
      case EK::CmpSel: {
        static const char *ps[] = {"<", "<=", ">", ">=", "==", "!="};
        return "(" + ex(e.a) + " " + ps[e.val] + " " + ex(e.b) + " ? " + ex(e.c) + " : " + ex(e.d) + ")";
      }
    }
    return "0";
  }

  // ---- shapes ------------------------------------------------------------
  const Value &val(int v) const { return P.values.at(v); }
  static int64_t count(const std::vector<int64_t> &s) {
    int64_t n = 1;
    for (auto d : s) n *= d;
    return n;
  }

  // Blocks of rank above 2 are addressed like rank-2 blocks: i1 is the index along the last dimension and i0 the
  // row-major index over all the others.  Where an op needs the index along one dimension, i0 is taken apart with
  // divisions by constants, and put together again for the operand.
  using Idx = std::vector<std::string>;
  static Idx split_index(const std::vector<int64_t> &shape, const std::string &i0, const std::string &i1) {
    const size_t r = shape.size();
    if (r == 0) return {};
    if (r == 1) return {i0};
    if (r == 2) return {i0, i1};
    Idx ix(r);
    ix[r - 1] = i1;
    int64_t below = 1;  // product of the leading dimensions after d
    for (size_t d = r - 1; d-- > 0;) {
      std::string e = below == 1 ? i0 : "(" + i0 + " / " + std::to_string(below) + ")";
      ix[d] = shape[d] == 1 ? "0" : d == 0 ? e : "(" + e + " % " + std::to_string(shape[d]) + ")";
      below *= shape[d];
    }
    return ix;
  }
  static std::pair<std::string, std::string> join_index(const std::vector<int64_t> &shape, const Idx &ix) {
    const size_t r = shape.size();
    if (r == 0) return {"0", "0"};
    if (r == 1) return {ix[0], "0"};
    if (r == 2) return {ix[0], ix[1]};
    std::string lead;
    int64_t below = 1;
    for (size_t d = r - 1; d-- > 0;) {
      if (ix[d] != "0") lead = (below == 1 ? ix[d] : ix[d] + " * " + std::to_string(below)) + (lead.empty() ? "" : " + " + lead);
      below *= shape[d];
    }
    return {lead.empty() ? "0" : "(" + lead + ")", ix[r - 1]};
  }
  std::string at_index(int v, const Idx &ix) {
    auto ij = join_index(val(v).shape, ix);
    return at(v, ij.first, ij.second);
  }
  static std::string linear(const std::vector<int64_t> &shape, const std::string &i0, const std::string &i1) {
    return shape.empty() ? "0" : shape.size() == 1 ? i0 : "(" + i0 + " * " + std::to_string(shape.back()) + " + " + i1 + ")";
  }

  // C expression for element (i0, i1) of value v; rank-1 values use i0, scalars neither
  std::string at(int v, const std::string &i0, const std::string &i1) {
    auto it = var.find(v);
    if (it != var.end()) {
      // a named value is the element the thread owns in the current loop; any other element (behind a transpose or a
      // reshape) is computed again from its definition
      const auto &sh = val(v).shape;
      if (sh.empty() || (i0 == cur_i0 && (sh.size() < 2 || i1 == cur_i1))) return it->second;
    }
    {
      auto lc = lds_copy.find(v);
      if (lc != lds_copy.end()) return lc->second + "[" + linear(val(v).shape, i0, i1) + "]";
    }
    auto d = def.find(v);
    if (d == def.end()) {
      auto mi = mirror.find(v);
      if (mi != mirror.end()) return mi->second + "[" + linear(val(v).shape, i0, i1) + "]";
      no("a loop-carried block value used in a loop over another block shape");
    }
    const SOp &s = *d->second;
    const Value &V = val(v);
    auto idx = [&](const std::vector<int64_t> &shape, size_t dim) -> std::string {
      // index along `dim` of a value of this shape, seen from the enclosing element
      if (shape[dim] == 1) return "0";
      return shape.size() == 1 ? i0 : dim == 0 ? i0 : i1;
    };
    switch (s.kind) {
      case SK::ScalarArg: return (V.dtype == "f64" ? "p.fval[" : "(float)p.fval[") + std::to_string(s.ival) + "]";
      case SK::FromIndex: return "(" + ctype(V.dtype) + ")" + ex(s.expr);
      case SK::Const:
        if (V.dtype == "f64") {
          std::ostringstream c;
          if (s.fval != s.fval) return "__builtin_nan(\"\")";
          if (s.fval == 1.0 / 0.0) return "__builtin_inf()";
          if (s.fval == -1.0 / 0.0) return "(-__builtin_inf())";
          c << std::hexfloat << s.fval;
          return "(" + c.str() + ")";
        }
        if (is_float(V.dtype)) {
          std::ostringstream c;
          c.precision(9);
          if (s.fval != s.fval) return "__builtin_nanf(\"\")";
          if (s.fval == 1.0 / 0.0) return "__builtin_inff()";
          if (s.fval == -1.0 / 0.0) return "(-__builtin_inff())";
          c << std::hexfloat << (float)s.fval << "f";
          return "(" + c.str() + ")";
        }
        return "(" + ctype(V.dtype) + ")(" + std::to_string(s.ival) + "LL)";
      case SK::Splat: return at(s.operands.at(0), "0", "0");
      case SK::Iota: return "(int)(" + std::to_string(s.ival) + " + " + i0 + ")";
      case SK::ExpandDims: {
        // operand has one dimension fewer; element (i0, i1) reads the operand at the index of the kept dimension
        const Value &O = val(s.operands.at(0));
        if (O.shape.size() + 1 != V.shape.size()) no("expand_dims that adds more than one dimension");
        if (V.shape.size() == 2) return at(s.operands[0], s.axis == 0 ? i1 : i0, "0");
        Idx ix = split_index(V.shape, i0, i1);
        ix.erase(ix.begin() + s.axis);
        return at_index(s.operands[0], ix);
      }
      case SK::Broadcast: {
        const Value &O = val(s.operands.at(0));
        if (O.shape.size() != V.shape.size()) no("broadcast that changes the rank");
        if (O.shape.size() == 1) return at(s.operands[0], O.shape[0] == 1 ? "0" : i0, "0");
        if (O.shape.size() == 2) return at(s.operands[0], O.shape[0] == 1 ? "0" : i0, O.shape[1] == 1 ? "0" : i1);
        if (O.shape == V.shape) return at(s.operands[0], i0, i1);
        Idx ix = split_index(V.shape, i0, i1);
        for (size_t d = 0; d < ix.size(); d++)
          if (O.shape[d] == 1) ix[d] = "0";
        return at_index(s.operands[0], ix);
      }
      case SK::Load: {
        // a load that is not of the run's block shape (an index vector, a row of scales): from its copy in LDS when the
        // run staged one, else read where it is used (the program is then refused if anything stores to its base)
        if (staged.count(v)) return staged_at(v, i0, i1);
        all_inline_bases.insert(s.acc.base_arg);
        std::string pred, addr = address(s.acc, i0, i1, pred);
        const std::string rd = mem_read(s.acc, addr);
        return "(" + (pred.empty() ? rd : "(" + pred + ") ? " + rd + " : " + other_of(s.acc, i0, i1)) + ")";
      }
      case SK::ScalarLoad: no("internal: scalar load without a variable");
      case SK::Reduce: case SK::Scan: {
        size_t j = 0;
        for (size_t q = 0; q < s.results.size(); q++)
          if (s.results[q] == v) j = q;
        const std::string arr = "out" + std::to_string(s.result) + "_" + std::to_string(j);
        return arr + "[" + linear(V.shape, i0, i1) + "]";
      }
      case SK::Map: {
        if (s.name.rfind("tt.trans", 0) == 0) {  // "tt.trans" (rank 2, order (1, 0)) or "tt.trans.<order>": result dim d is operand dim order[d]
          const Value &O = val(s.operands.at(0));
          if (O.shape.size() != V.shape.size()) no("tt.trans that changes the rank");
          if (s.name == "tt.trans") {
            if (V.shape.size() != 2) no("tt.trans of a block of rank above 2 without an order");
            return at(s.operands[0], i1, i0);
          }
          std::vector<size_t> order;
          for (size_t q = 8; q < s.name.size(); q++)
            if (isdigit((unsigned char)s.name[q])) order.push_back((size_t)(s.name[q] - '0'));
          if (order.size() != V.shape.size()) no("tt.trans with an order of another rank than the block");
          const Idx ix = split_index(V.shape, i0, i1);
          Idx ox(order.size());
          for (size_t d = 0; d < order.size(); d++) {
            if (order[d] >= order.size() || O.shape[order[d]] != V.shape[d]) no("tt.trans whose order does not fit the shapes");
            ox[order[d]] = ix[d];
          }
          return at_index(s.operands[0], ox);
        }
        if (s.name == "tt.cat") {  // two rank-1 blocks end to end
          const int64_t na = val(s.operands.at(0)).shape.at(0);
          return "(" + i0 + " < " + std::to_string(na) + " ? " + at(s.operands[0], i0, "0") + " : " +
                 at(s.operands.at(1), "(" + i0 + " - " + std::to_string(na) + ")", "0") + ")";
        }
        if (s.name == "tt.join")  // [N] and [N] -> [N, 2]
          return "(" + i1 + " == 0 ? " + at(s.operands.at(0), i0, "0") + " : " + at(s.operands.at(1), i0, "0") + ")";
        if (s.name == "tt.split.0" || s.name == "tt.split.1") return at(s.operands.at(0), i0, s.name.substr(9));
        if (s.name == "tt.unsplat") return at(s.operands.at(0), "0", "0");
        if (s.name == "tt.reshape") {  // row-major element order is kept
          const Value &O = val(s.operands.at(0));
          const std::string lin = linear(V.shape, i0, i1);
          if (O.shape.size() >= 2) return at(s.operands[0], "(" + lin + " / " + std::to_string(O.shape.back()) + ")", "(" + lin + " % " + std::to_string(O.shape.back()) + ")");
          return at(s.operands[0], O.shape.empty() ? "0" : lin, "0");
        }
        std::vector<std::string> a;
        for (int o : s.operands) {
          const Value &O = val(o);
          if (O.shape.size() == V.shape.size()) {
            a.push_back(O.shape.size() > 2    ? at(o, i0, i1)
                        : O.shape.size() == 2 ? at(o, idx(O.shape, 0), idx(O.shape, 1))
                        : O.shape.size() == 1 ? at(o, idx(O.shape, 0), "0")
                                              : at(o, "0", "0"));
          } else if (O.shape.empty()) a.push_back(at(o, "0", "0"));
          else no("an elementwise op whose operands differ in rank");
        }
        return "(" + map_expr(s, a) + ")";
      }
      default: no("internal: value without an inline form");
    }
  }

  std::string rounded(const std::string &dtype, const std::string &e) {
    if (dtype == "f16") return "up_f16(down_f16(" + e + "))";
    if (dtype == "bf16") return "up_bf16(down_bf16(" + e + "))";
    return e;
  }

  std::string map_expr(const SOp &s, const std::vector<std::string> &a) {
    const std::string &n = s.name;
    const std::string &rt = val(s.result).dtype;
    const std::string ot = s.operands.empty() ? rt : val(s.operands[0]).dtype;
    auto need = [&](size_t k) { if (a.size() != k) no("elementwise op " + n + " with " + std::to_string(a.size()) + " operands"); };
    auto fl = [&](const std::string &e) { return rounded(rt, e); };
    auto wrapi = [&](const char *op) {  // wrapping integer arithmetic in the result type
      const std::string T = ctype(rt), U = rt == "i64" ? "unsigned long long" : "unsigned";
      return "(" + T + ")((" + U + ")" + a[0] + " " + op + " (" + U + ")" + a[1] + ")";
    };
    static const std::map<std::string, const char *> bin_f = {{"arith.addf", "+"}, {"arith.subf", "-"}, {"arith.mulf", "*"}, {"arith.divf", "/"}};
    static const std::map<std::string, const char *> fn2 = {{"arith.maxnumf", "fmaxf"}, {"arith.minnumf", "fminf"},
                                                            {"arith.maximumf", "maximum_f"}, {"arith.minimumf", "minimum_f"}};
    static const std::map<std::string, const char *> fn1 = {
        {"math.absf", "fabsf"}, {"math.exp", "expf"}, {"math.exp2", "exp2f"}, {"math.log", "logf"}, {"math.log2", "log2f"},
        {"math.sqrt", "sqrtf"}, {"math.sin", "sinf"}, {"math.cos", "cosf"}, {"math.tanh", "tanhf"}, {"math.erf", "erff"},
        {"math.floor", "floorf"}, {"math.ceil", "ceilf"}};
    static const std::map<std::string, const char *> cmpf = {
        {"oeq", "A == B"}, {"one", "A < B || A > B"}, {"olt", "A < B"}, {"ole", "A <= B"}, {"ogt", "A > B"}, {"oge", "A >= B"},
        {"une", "!(A == B)"}, {"ueq", "!(A < B || A > B)"}, {"ult", "!(A >= B)"}, {"ule", "!(A > B)"}, {"ugt", "!(A <= B)"},
        {"uge", "!(A < B)"}, {"ord", "A == A && B == B"}, {"uno", "A != A || B != B"}};
    static const std::map<std::string, const char *> cmpi = {{"slt", "<"}, {"sle", "<="}, {"sgt", ">"}, {"sge", ">="}, {"eq", "=="}, {"ne", "!="}};
    if (rt == "f64" || ot == "f64") {  // double precision: the same ops through the double-precision library names
      auto plain = [](std::string f) { f.pop_back(); return f; };  // "sqrtf" -> "sqrt"
      if (bin_f.count(n)) { need(2); return a[0] + " " + bin_f.at(n) + " " + a[1]; }
      if (n == "arith.maxnumf" || n == "arith.minnumf") { need(2); return std::string(n == "arith.maxnumf" ? "fmax(" : "fmin(") + a[0] + ", " + a[1] + ")"; }
      if (n == "arith.maximumf" || n == "arith.minimumf") { need(2); return std::string(n == "arith.maximumf" ? "maximum_d(" : "minimum_d(") + a[0] + ", " + a[1] + ")"; }
      if (fn1.count(n)) { need(1); return plain(fn1.at(n)) + "(" + a[0] + ")"; }
      if (n == "math.rsqrt") { need(1); return "1.0 / sqrt(" + a[0] + ")"; }
      if (n == "math.fma") { need(3); return "fma(" + a[0] + ", " + a[1] + ", " + a[2] + ")"; }
      if (n == "arith.extf" || n == "arith.sitofp") { need(1); return "(double)" + a[0]; }
      if (n == "arith.uitofp") { need(1); return "(double)(" + std::string(ot == "i64" ? "unsigned long long" : ot == "i8" ? "unsigned char" : ot == "i16" ? "unsigned short" : "unsigned") + ")" + a[0]; }
      if (n == "arith.truncf") { need(1); return fl("(float)" + a[0]); }
      if (n == "tt.precise_sqrt") { need(1); return "sqrt(" + a[0] + ")"; }
      if (n == "tt.precise_divf") { need(2); return a[0] + " / " + a[1]; }
      if (n == "arith.remf") { need(2); return "fmod(" + a[0] + ", " + a[1] + ")"; }
      if (n == "tt.clampf.none") { need(3); return "fmin(fmax(" + a[0] + ", " + a[1] + "), " + a[2] + ")"; }
      if (n == "tt.clampf.all") { need(3); return "minimum_d(maximum_d(" + a[0] + ", " + a[1] + "), " + a[2] + ")"; }
      if (n == "tt.bitcast" || n == "arith.bitcast") {
        need(1);
        if (rt == ot) return a[0];
        if (rt == "f64" && ot == "i64") return "__longlong_as_double(" + a[0] + ")";
        if (rt == "i64" && ot == "f64") return "__double_as_longlong(" + a[0] + ")";
        no("a bitcast between f64 and " + (rt == "f64" ? ot : rt));
      }
      if (n.rfind("extern.", 0) == 0) no("double-precision function " + n.substr(7));
      // negation, select, comparisons and conversions to integers read the same for every width: below
    }
    if (bin_f.count(n)) { need(2); return fl(a[0] + " " + bin_f.at(n) + " " + a[1]); }
    if (fn2.count(n)) { need(2); return fl(std::string(fn2.at(n)) + "(" + a[0] + ", " + a[1] + ")"); }
    if (fn1.count(n)) { need(1); return fl(std::string(fn1.at(n)) + "(" + a[0] + ")"); }
    if (n == "arith.negf") { need(1); return "-" + a[0]; }
    if (n == "math.rsqrt") { need(1); return fl("1.0f / sqrtf(" + a[0] + ")"); }
    if (n == "math.fma") { need(3); return fl("fmaf(" + a[0] + ", " + a[1] + ", " + a[2] + ")"); }
    if (n == "arith.select") { need(3); return a[0] + " ? " + a[1] + " : " + a[2]; }
    if (n == "arith.extf") { need(1); return a[0]; }
    if (n == "arith.truncf") { need(1); return fl(a[0]); }
    if (n == "arith.sitofp") { need(1); return fl("(float)" + a[0]); }
    if (n == "arith.fptosi") { need(1); return "(" + ctype(rt) + ")" + a[0]; }
    if (n == "arith.extsi" || n == "arith.trunci") { need(1); return "(" + ctype(rt) + ")" + a[0]; }
    if (n == "arith.extui") { need(1); return ot == "i1" ? "(" + ctype(rt) + ")(" + a[0] + " ? 1 : 0)" : "(" + ctype(rt) + ")(unsigned " + ctype(ot) + ")" + a[0]; }
    if (n == "arith.addi") { need(2); return rt == "i1" ? a[0] + " != " + a[1] : wrapi("+"); }
    if (n == "arith.subi") { need(2); return rt == "i1" ? a[0] + " != " + a[1] : wrapi("-"); }
    if (n == "arith.muli") { need(2); return rt == "i1" ? a[0] + " && " + a[1] : wrapi("*"); }
    if (n == "arith.divsi") { need(2); return "(" + ctype(rt) + ")sdiv(" + a[0] + ", " + a[1] + ")"; }
    if (n == "arith.remsi") { need(2); return "(" + ctype(rt) + ")srem(" + a[0] + ", " + a[1] + ")"; }
    if (n == "arith.minsi") { need(2); return "(" + ctype(rt) + ")smin(" + a[0] + ", " + a[1] + ")"; }
    if (n == "arith.maxsi") { need(2); return "(" + ctype(rt) + ")smax(" + a[0] + ", " + a[1] + ")"; }
    if (n == "arith.maxui" || n == "arith.minui") {
      need(2);
      const std::string U = rt == "i64" ? "unsigned long long" : "unsigned";
      return "(" + ctype(rt) + ")((" + U + ")" + a[0] + (n == "arith.maxui" ? " > (" : " < (") + U + ")" + a[1] + " ? " + a[0] + " : " + a[1] + ")";
    }
    {
      const std::string U = (rt == "i64" || ot == "i64") ? "unsigned long long" : ot == "i8" ? "unsigned char" : ot == "i16" ? "unsigned short" : "unsigned";
      const int bits = ot == "i64" ? 64 : ot == "i8" ? 8 : ot == "i16" ? 16 : 32;
      if (n == "arith.divui") { need(2); return "(" + ctype(rt) + ")((" + U + ")" + a[1] + " == 0 ? 0 : (" + U + ")" + a[0] + " / (" + U + ")" + a[1] + ")"; }
      if (n == "arith.remui") { need(2); return "(" + ctype(rt) + ")((" + U + ")" + a[1] + " == 0 ? 0 : (" + U + ")" + a[0] + " % (" + U + ")" + a[1] + ")"; }
      // shifts by the width or more are undefined in the source dialect; the amount is taken modulo the width here
      const std::string amount = "((" + U + ")" + (a.size() > 1 ? a[1] : std::string("0")) + " & " + std::to_string(bits - 1) + ")";
      if (n == "arith.shli") { need(2); return "(" + ctype(rt) + ")((" + U + ")" + a[0] + " << " + amount + ")"; }
      if (n == "arith.shrui") { need(2); return "(" + ctype(rt) + ")((" + U + ")" + a[0] + " >> " + amount + ")"; }
      if (n == "arith.shrsi") { need(2); return "(" + ctype(rt) + ")(" + a[0] + " >> " + amount + ")"; }
      static const std::map<std::string, const char *> cmpu = {{"ult", "<"}, {"ule", "<="}, {"ugt", ">"}, {"uge", ">="}};
      if (n.rfind("arith.cmpi.", 0) == 0 && cmpu.count(n.substr(11))) {
        need(2);
        return "(" + U + ")" + a[0] + " " + cmpu.at(n.substr(11)) + " (" + U + ")" + a[1];
      }
      if (n == "arith.uitofp") { need(1); return fl("(float)(" + U + ")" + a[0]); }
      if (n == "arith.fptoui") { need(1); return "(" + ctype(rt) + ")(" + (rt == "i64" ? std::string("unsigned long long") : std::string("unsigned")) + ")" + a[0]; }
      if (n == "tt.mulhiui") {
        need(2);
        if (rt == "i64") return "(long long)__umul64hi((unsigned long long)" + a[0] + ", (unsigned long long)" + a[1] + ")";
        return "(int)(((unsigned long long)(unsigned)" + a[0] + " * (unsigned long long)(unsigned)" + a[1] + ") >> 32)";
      }
      if (n == "math.absi") { need(1); return "(" + ctype(rt) + ")(" + a[0] + " < 0 ? (" + U + ")0 - (" + U + ")" + a[0] + " : (" + U + ")" + a[0] + ")"; }
    }
    if (n.rfind("extern.__nv_", 0) == 0) {  // the fp32 libdevice names: the device math library's function of the same name
      static const std::set<std::string> fns = {"acosf", "acoshf", "asinf", "asinhf", "atan2f", "atanf", "atanhf", "ceilf", "cosf", "coshf",
                                                "erff", "exp2f", "expf", "fabsf", "floorf", "log10f", "log1pf", "logf", "log2f", "powf",
                                                "rsqrtf", "sinf", "sinhf", "sqrtf", "tanf", "tanhf", "truncf", "fmodf", "expm1f", "cbrtf"};
      const std::string fn = n.substr(12);
      if (!fns.count(fn) || rt != "f32") no("extern function " + n.substr(7));
      std::string call = fn + "(";
      for (size_t q = 0; q < a.size(); q++) call += (q ? ", " : "") + a[q];
      return call + ")";
    }
    if (n == "tt.bitcast" || n == "arith.bitcast") {
      need(1);
      if (is_float(ot) == is_float(rt)) return a[0];                           // same class (signedness only): the bits are the value
      if (ot != "f32" && rt != "f32") no("a bitcast between 16-bit floats and integers");
      return is_float(rt) ? "__int_as_float(" + a[0] + ")" : "__float_as_int(" + a[0] + ")";
    }
    // correctly rounded whatever the compiler's defaults: the fp64 result rounds to the fp32 one (53 >= 2 * 24 + 2 bits)
    if (n == "tt.precise_sqrt") { need(1); return fl("(float)sqrt((double)" + a[0] + ")"); }
    if (n == "tt.precise_divf") { need(2); return fl("(float)((double)" + a[0] + " / (double)" + a[1] + ")"); }
    if (n == "arith.remf") { need(2); return fl("fmodf(" + a[0] + ", " + a[1] + ")"); }
    if (n == "tt.clampf.none") { need(3); return fl("fminf(fmaxf(" + a[0] + ", " + a[1] + "), " + a[2] + ")"); }
    if (n == "tt.clampf.all") { need(3); return fl("minimum_f(maximum_f(" + a[0] + ", " + a[1] + "), " + a[2] + ")"); }
    if (n == "arith.andi") { need(2); return rt == "i1" ? a[0] + " && " + a[1] : "(" + ctype(rt) + ")(" + a[0] + " & " + a[1] + ")"; }
    if (n == "arith.ori") { need(2); return rt == "i1" ? a[0] + " || " + a[1] : "(" + ctype(rt) + ")(" + a[0] + " | " + a[1] + ")"; }
    if (n == "arith.xori") { need(2); return rt == "i1" ? a[0] + " != " + a[1] : "(" + ctype(rt) + ")(" + a[0] + " ^ " + a[1] + ")"; }
    if (n.rfind("arith.cmpf.", 0) == 0 && cmpf.count(n.substr(11))) {
      need(2);
      std::string t = cmpf.at(n.substr(11)), out;
      for (char c : t) out += c == 'A' ? "(" + a[0] + ")" : c == 'B' ? "(" + a[1] + ")" : std::string(1, c);
      return out;
    }
    if (n.rfind("arith.cmpi.", 0) == 0 && cmpi.count(n.substr(11))) { need(2); return a[0] + " " + cmpi.at(n.substr(11)) + " " + a[1]; }
    no("elementwise op " + n + " is not implemented");
  }

  // ---- accesses ----------------------------------------------------------
  // element offset and validity of an access at (i0, i1); fills `pred` ("" = always)
  std::string address(const Access &a, const std::string &i0, const std::string &i1, std::string &pred) {
    std::string sum;
    pred.clear();
    if (a.gather >= 0) {  // per-element offsets and mask are data
      if (a.mask_value >= 0) pred = at(a.mask_value, i0, i1);
      return ex(a.offsets.at(0)) + " + (long long)" + at(a.gather, i0, i1);
    }
    const Idx ix = split_index(a.sizes, i0, i1);
    for (size_t d = 0; d < a.sizes.size(); d++) {
      const std::string &i = ix[d];
      std::string term = "(" + ex(a.offsets[d]) + " + " + i + " * " + ex(a.strides[d]) + ")";
      if (!a.mods.empty() && a.mods[d] >= 0) term = "wrap(" + term + ", " + ex(a.mods[d]) + ")";
      sum += (d ? " + " : "") + term;
      // (An index lies in [0, size): comparing it with the extent clamped to that range is the same, and the clamped
      // extent is a 32-bit value that is the same in every lane, where the extent itself is a 64-bit one.  For extents
      // that do not change inside a loop, where it measured faster: LayerNorm's dx on fp16 [4096, 8192] 51 -> 45 us;
      // a softmax over rows read in pieces, whose extents follow the loop, 284 -> 306 us with it.)
      if (!a.dims.empty()) {
        const bool fixed = !P.pool.depends_on(a.dims[d], EK::IV) && !P.pool.depends_on(a.dims[d], EK::Iter);
        pred += std::string(pred.empty() ? "" : " && ") + i + " < " +
                (fixed ? "(int)smin(smax(" + ex(a.dims[d]) + ", 0LL), " + std::to_string(a.sizes[d]) + "LL)" : ex(a.dims[d]));
      }
    }
    if (a.sizes.empty()) sum = ex(a.offsets.at(0));
    return sum;
  }

  std::string mem_read(const Access &a, const std::string &addr) {
    const std::string ptr = "((const " + memtype(a.elem) + " *)p.ptr[" + std::to_string(a.base_arg) + "])[" + addr + "]";
    if (a.elem == "f16") return "up_f16(" + ptr + ")";
    if (a.elem == "bf16") return "up_bf16(" + ptr + ")";
    return ptr;
  }
  static bool raw16(const SOp &o) {  // a masked load of f16 / bf16: widened in the fill loop (see the two-phase loads)
    return (o.acc.elem == "f16" || o.acc.elem == "bf16") && (!o.acc.dims.empty() || o.acc.mask_value >= 0);
  }
  std::string other_of(const Access &a, const std::string &i0 = "0", const std::string &i1 = "0") {
    if (a.other_value >= 0) return at(a.other_value, i0, i1);
    if (!a.has_other) return a.elem == "f64" ? "0.0" : is_float(a.elem) ? "0.f" : "(" + ctype(a.elem) + ")0";
    if (a.elem == "f64") {
      if (a.other_f != a.other_f) return "__builtin_nan(\"\")";
      if (a.other_f == 1.0 / 0.0) return "__builtin_inf()";
      if (a.other_f == -1.0 / 0.0) return "(-__builtin_inf())";
      std::ostringstream c;
      c << std::hexfloat << a.other_f;
      return "(" + c.str() + ")";
    }
    if (is_float(a.elem)) {
      if (a.other_f != a.other_f) return "__builtin_nanf(\"\")";
      if (a.other_f == 1.0 / 0.0) return "__builtin_inff()";
      if (a.other_f == -1.0 / 0.0) return "(-__builtin_inff())";
      std::ostringstream c;
      c << std::hexfloat << (float)a.other_f << "f";
      return "(" + c.str() + ")";
    }
    return "(" + ctype(a.elem) + ")(" + std::to_string(a.other_i) + "LL)";
  }
  void mem_write(const Access &a, const std::string &addr, const std::string &pred, const std::string &value) {
    std::string v = value;
    if (a.elem == "f16") v = "down_f16_exact(" + v + ")";  // (a value of type f16 is held as the float it equals)
    if (a.elem == "bf16") v = "down_bf16(" + v + ")";
    os << pad() << (pred.empty() ? "" : "if (" + pred + ") ") << "((" << memtype(a.elem) << " *)p.ptr[" << a.base_arg << "])[" << addr
       << "] = " << v << ";\n";
  }

  // ---- bodies ------------------------------------------------------------
  // Values that a thread keeps for the elements it owns (element t + 256 n of the value's shape in slot n): the loads of
  // two-phase runs and loop-carried blocks.  They can be named only inside an element loop over the same shape;
  // elsewhere a load is read again in place and a carried block is refused.
  // A load that a run copied to LDS whole: loads of another shape than the run's, and loads read through a transpose
  // (coalesced into LDS where they stand, read back in any order).  pitch: elements between rows of a rank-2 block (one
  // more than its columns under a transpose, so that a column's elements fall into different banks).
  struct Staged { std::string name; int64_t pitch; };
  std::map<int, Staged> staged;
  std::string staged_at(int v, const std::string &i0, const std::string &i1) {
    const Staged &st = staged.at(v);
    const auto &sh = val(v).shape;
    if (sh.size() == 2 && st.pitch != sh.back()) return st.name + "[(" + i0 + " * " + std::to_string(st.pitch) + " + " + i1 + ")]";
    return st.name + "[" + linear(sh, i0, i1) + "]";
  }
  // loads of ops[k, end) that some tt.trans of the run reads, directly or through elementwise ops
  std::set<int> loads_behind_transposes(const std::vector<SOp> &ops, size_t k, size_t end) {
    std::set<int> found;
    std::function<void(int, int)> walk = [&](int v, int depth) {
      auto d = def.find(v);
      if (d == def.end() || depth > 16) return;
      const SOp &o = *d->second;
      if (o.kind == SK::Load) { found.insert(v); return; }
      if (o.kind == SK::Map || o.kind == SK::Broadcast || o.kind == SK::ExpandDims)
        for (int x : o.operands) walk(x, depth + 1);
    };
    for (size_t q = k; q < end; q++)
      if (ops[q].kind == SK::Map && ops[q].name.rfind("tt.trans", 0) == 0 && val(ops[q].result).shape.size() == 2)
        for (int x : ops[q].operands) walk(x, 0);
    return found;
  }
  // Costly vectors read through a broadcast: a value of one dimension (<= 4096 elements) that takes a transcendental
  // function or a division and that a loop over a larger block reads at [row] for every element of the row (the
  // exp(m_old - m_new) that rescales an attention accumulator) is computed once per element of its own, into LDS.
  // value id -> array.  `roots` are the values the next phase evaluates.
  std::map<int, std::string> lds_copy;
  void hoist_costly_vectors(const std::vector<int> &roots, std::vector<int> &copies) {
    std::vector<int> found;
    std::function<void(int, bool, int)> walk = [&](int v, bool through_broadcast, int depth) {
      auto d = def.find(v);
      if (v < 0 || d == def.end() || depth > 24 || lds_copy.count(v)) return;
      const SOp &o = *d->second;
      const Value &V = val(v);
      if (through_broadcast && o.kind == SK::Map && V.shape.size() == 1 && V.shape[0] > 1 && V.shape[0] <= 4096 && !held.count(v) && costly(v)) {
        if (std::find(found.begin(), found.end(), v) == found.end()) found.push_back(v);
        return;
      }
      if (o.kind == SK::Map) for (int x : o.operands) walk(x, through_broadcast, depth + 1);
      else if (o.kind == SK::Broadcast || o.kind == SK::ExpandDims) for (int x : o.operands) walk(x, true, depth + 1);
    };
    for (int r : roots) walk(r, false, 0);
    if (found.empty()) return;
    os << pad() << "__syncthreads();\n";
    for (int v : found) {
      const Value &V = val(v);
      const std::string name = "sv" + std::to_string(v);
      if (!declared_copies.count(v)) {
        decl << "  __shared__ " << ctype(V.dtype) << " " << name << "[" << V.shape[0] << "];\n";
        out_bytes += ((size_t)V.shape[0] * held_bytes(V.dtype) + 15) / 16 * 16;
        declared_copies.insert(v);
      }
      open_element_loop(V.shape);
      os << pad() << name << "[t] = " << at(v, idx0(V.shape), idx1(V.shape)) << ";\n";
      close_loop();
    }
    os << pad() << "__syncthreads();\n";
    for (int v : found) {
      lds_copy[v] = "sv" + std::to_string(v);
      copies.push_back(v);
    }
  }
  std::set<int> declared_copies;
  struct Held { std::string name; std::vector<int64_t> shape; std::string expr; };  // expr: what to write instead of name[n], if anything
  std::map<int, Held> held;
  // Loop-carried vectors that a loop also reads from blocks of another shape (the running maximum and sum of an online
  // softmax next to its [BM, BN] scores): besides the owning threads' registers they are kept in an LDS array, written
  // where the registers are, which any thread may read.  value id -> array
  std::map<int, std::string> mirror;
  void map_vars(const std::vector<int64_t> &shape) {
    for (auto &h : held) {
      if (h.second.shape == shape) var[h.first] = h.second.expr.empty() ? h.second.name + "[n]" : h.second.expr;
      else var.erase(h.first);
    }
  }
  // Which element a thread holds in slot n of a block.  Ordinarily t = threadIdx.x + 256 n: a wavefront's accesses are
  // contiguous, one element per lane.  For 16-bit data that is 2 bytes per lane and access; a program whose blocks of
  // 16-bit elements have whole groups of 2048 along the contiguous dimension is written "wide" instead: a thread owns
  // eight neighbouring elements, t = 8 threadIdx.x + (n & 7) + 2048 (n >> 3), and a group of eight that is valid as a
  // whole and 16-byte aligned moves in one access (two for 4-byte elements).  Only blocks of the one shape `wide_shape`
  // are laid out that way; every other shape of the program keeps the ordinary order.  Programs with scans, matrix
  // products or index shuffles (whose code relies on the ordinary order) are never wide.
  bool wide_mode = false;
  std::vector<int64_t> wide_shape;
  bool wide(const std::vector<int64_t> &shape) const { return wide_mode && shape == wide_shape; }
  bool vector_access(const Access &a) const {  // eight neighbouring elements are eight neighbouring addresses
    if (a.gather >= 0 || a.sizes.empty() || a.strides.size() != a.sizes.size() || a.offsets.size() != a.sizes.size()) return false;
    if (a.elem != "f16" && a.elem != "bf16" && a.elem != "f32" && a.elem != "i32" && a.elem != "i8") return false;
    for (int m : a.mods)
      if (m >= 0) return false;
    int64_t st = 0;
    return P.pool.is_const(a.strides.back(), &st) && st == 1;
  }
  void choose_wide_shape() {
    if (const char *e = getenv("TTS_TILE_WIDE"))
      if (e[0] == '0') return;
    bool refuse = false;
    std::vector<int64_t> best;
    std::function<void(const std::vector<SOp> &)> scan = [&](const std::vector<SOp> &ops) {
      for (const SOp &s : ops) {
        if (s.kind == SK::Scan || s.kind == SK::Dot) refuse = true;
        if (s.kind == SK::Map && (s.name.rfind("tt.trans", 0) == 0 || s.name == "tt.cat" || s.name == "tt.join" || s.name.rfind("tt.split", 0) == 0 ||
                                  s.name == "tt.reshape" || s.name == "tt.unsplat"))
          refuse = true;
        if ((s.kind == SK::Load || s.kind == SK::Store) && (s.acc.elem == "f16" || s.acc.elem == "bf16") && vector_access(s.acc)) {
          const auto &sz = s.acc.sizes;
          if (sz.size() <= 2 && sz.back() % 2048 == 0 && count(sz) <= TWO_PHASE_MAX && (best.empty() || count(sz) > count(best))) best = sz;
        }
        if (s.kind == SK::For || s.kind == SK::If) scan(s.body);
      }
    };
    scan(P.body);
    if (refuse || best.empty()) return;
    wide_mode = true;
    wide_shape = best;
  }
  // (i0, i1) moved by `delta` along the contiguous dimension: called once with i0 (use .first) and once with i1 (.second)
  static std::pair<std::string, std::string> along(const std::vector<int64_t> &shape, const std::string &i, const std::string &delta) {
    return {shape.size() < 2 ? "(" + i + delta + ")" : i, shape.size() < 2 ? i : "(" + i + delta + ")"};
  }
  // A wide program whose body loads a block that is the same for every program (a row of weights next to the row it
  // scales: its address and extent name no program id, loop variable or loaded value, and nothing stores to its argument)
  // is written "persistent": the launch has a few workgroups per CU, each walks the programs lin = blockIdx.x,
  // blockIdx.x + gridDim.x, ... and the shared blocks are loaded once per workgroup, before that loop (hoisted: their
  // code goes to hoist_os).  Read again by every program they stay in L2, but the L2 -> CU traffic is that of a second
  // row (RMSNorm fp16 [4096, 8192]: 27.5 -> 25.5 us).
  bool persistent = false;
  // In a persistent kernel every wide 16-bit load stays packed (two elements per register, widened where used): RMSNorm
  // on rows of 8192 then takes 75 registers instead of 111.  (With a workgroup per program the compiler keeps packed and
  // widened values side by side and takes more registers than without: 121 against 108; the launcher compiles that form,
  // unpacked, when the persistent one holds too few workgroups per CU.)
  bool pack_wide = false;
  std::set<int> hoisted;  // value ids of the loads emitted before the program loop
  std::ostringstream hoist_os;
  std::ostringstream loop_top;  // first statements of the program loop
  void choose_persistent() {
    if (!wide_mode) return;
    if (const char *e = getenv("TTS_TILE_PERSISTENT"))
      if (e[0] == '0') return;
    std::set<int> stored;
    std::function<void(const std::vector<SOp> &)> scan = [&](const std::vector<SOp> &ops) {
      for (const SOp &s : ops) {
        if (s.kind == SK::Store || s.kind == SK::ScalarStore) stored.insert(s.acc.base_arg);
        if (s.kind == SK::For || s.kind == SK::If) scan(s.body);
      }
    };
    scan(P.body);
    for (const SOp &s : P.body) {
      if (s.kind != SK::Load || !wide(s.acc.sizes) || !vector_access(s.acc) || stored.count(s.acc.base_arg) || s.acc.other_value >= 0) continue;
      std::vector<int> es = s.acc.offsets;
      es.insert(es.end(), s.acc.strides.begin(), s.acc.strides.end());
      es.insert(es.end(), s.acc.dims.begin(), s.acc.dims.end());
      bool fixed = true;
      for (int e : es)
        for (EK k : {EK::Pid, EK::NProg, EK::IV, EK::Iter, EK::Result, EK::Data}) fixed = fixed && (e < 0 || !P.pool.depends_on(e, k));  // (what the code before the program loop can name: arguments and constants)
      if (fixed) hoisted.insert(s.result);
    }
    persistent = !hoisted.empty();
    pack_wide = persistent;
  }
  std::string element_of_slot(const std::vector<int64_t> &shape) const {
    return wide(shape) ? "8 * (int)threadIdx.x + (n & 7) + 2048 * (n >> 3)" : "threadIdx.x + 256 * n";
  }
  // Row and column of element t of a block.  Every loop that names t names n as well (element_of_slot); with rows of a
  // multiple of 256 elements the row depends on n alone, which is a constant once the loop is unrolled (or the same in
  // every thread where it is not): written that way, the row's address arithmetic (row * pitch in 64 bits, per element
  // and access: quarter-rate multiplies) is the scalar unit's or the compiler's, not every lane's.
  std::string idx0(const std::vector<int64_t> &shape) const {
    if (shape.size() < 2) return "t";
    const int64_t C = shape.back();
    if (C % 256 == 0) return C == 256 ? "n" : "(n / " + std::to_string(C / 256) + ")";
    return "(t / " + std::to_string(C) + ")";
  }
  std::string idx1(const std::vector<int64_t> &shape) const {
    if (shape.size() < 2) return "0";
    const int64_t C = shape.back();
    if (wide(shape)) return "(8 * (int)threadIdx.x + (n & 7) + 2048 * ((n >> 3) % " + std::to_string(C / 2048) + "))";
    if (C % 256 == 0) return C == 256 ? "(int)threadIdx.x" : "((int)threadIdx.x + 256 * (n % " + std::to_string(C / 256) + "))";
    return "(t % " + std::to_string(C) + ")";
  }
  std::string cur_i0, cur_i1;  // the index expressions of the element loop being written
  void open_element_loop(const std::vector<int64_t> &shape) {
    const int64_t T = count(shape);
    cur_i0 = idx0(shape);
    cur_i1 = idx1(shape);
    os << pad() << "#pragma unroll\n" << pad() << "for (int n = 0; n < " << (T + 255) / 256 << "; n++) {\n";
    indent++;
    os << pad() << "const int t = " << element_of_slot(shape) << ";\n";
    if (T % 256) os << pad() << "if (t >= " << T << ") break;\n";  // (whole slots otherwise: 256 threads, launch bounds say so)
    map_vars(shape);
  }
  void close_loop() {
    indent--;
    os << pad() << "}\n";
  }

  // `defer`: the caller releases the values this body holds in registers (a loop does, after it has computed the
  // values it carries to the next iteration from them)
  void body(const std::vector<SOp> &ops, std::vector<int> *defer = nullptr) {
    for (auto &s : ops) {
      if (s.result >= 0) def[s.result] = &s;
      if (s.kind != SK::For)
        for (int r : s.results) def[r] = &s;
    }
    auto is_break = [](const SOp &s) {
      return s.kind == SK::For || s.kind == SK::If || s.kind == SK::ScalarLoad || s.kind == SK::ScalarStore || s.kind == SK::Reduce || s.kind == SK::Scan ||
             s.kind == SK::Dot;
    };
    std::vector<int> mine;  // loads this body holds in registers
    std::vector<int> copies;  // vectors this body keeps a copy of in LDS (hoist_costly_vectors)
    size_t k = 0;
    while (k < ops.size()) {
      const SOp &s = ops[k];
      if (s.kind == SK::For) { loop(s); k++; continue; }
      if (s.kind == SK::If && s.ival == 2) {  // a `while` leaves its loop: every thread does, the condition is a scalar
        if (!loop_depth) no("a loop exit outside a loop");
        map_vars({-1});
        os << pad() << "if (!(" << at(s.operands.at(0), "0", "0") << ")) break;\n";
        k++;
        continue;
      }
      if (s.kind == SK::If) {  // the condition is a scalar, the same for every thread: barriers inside are safe
        map_vars({-1});
        // results: a variable per scalar, a per-thread array per block, declared once (the `then` side comes first)
        // and assigned at the end of whichever side runs
        for (size_t j = 0; j < s.results.size(); j++) {
          const int r = s.results[j];
          const Value &R = val(r);
          const std::string name = "ifr" + std::to_string(r);
          if (R.shape.size() > 2) no("an if that yields a block of rank " + std::to_string(R.shape.size()));
          if (R.shape.empty()) {
            if (!var.count(r)) os << pad() << ctype(R.dtype) << " " << name << ";\n";
            var[r] = name;
          } else {
            if (count(R.shape) > TWO_PHASE_MAX) no("an if that yields a block of more than " + std::to_string(TWO_PHASE_MAX) + " elements");
            if (!held.count(r)) {
              os << pad() << ctype(R.dtype) << " " << name << "[" << (count(R.shape) + 255) / 256 << "];\n";
              mine.push_back(r);
            }
            held[r] = {name, R.shape};
          }
        }
        const std::string cond = at(s.operands.at(0), "0", "0");
        os << pad() << "if (" << (s.ival ? "!" : "") << "(" << cond << ")) {\n";
        indent++;
        std::vector<int> side_held;
        body(s.body, &side_held);
        for (size_t j = 0; j < s.results.size(); j++) {
          const Value &R = val(s.results[j]);
          const std::string name = "ifr" + std::to_string(s.results[j]);
          if (R.shape.empty()) {
            map_vars({-1});
            os << pad() << name << " = " << at(s.tile_yields.at(j), "0", "0") << ";\n";
          } else {
            open_element_loop(R.shape);
            var.erase(s.results[j]);  // the result itself is not readable while it is being written
            os << pad() << name << "[n] = " << at(s.tile_yields.at(j), idx0(R.shape), idx1(R.shape)) << ";\n";
            close_loop();
          }
        }
        for (int v : side_held) {
          held.erase(v);
          var.erase(v);
        }
        indent--;
        os << pad() << "}\n";
        k++;
        continue;
      }
      if (s.kind == SK::ScalarLoad) {
        map_vars({-1});
        // thread 0's scalar store to this argument (earlier in the program, or in the previous iteration) is visible
        if (scalar_store_bases_anywhere.count(s.acc.base_arg)) os << pad() << "__syncthreads();\n";
        std::string pred, addr = address(s.acc, "0", "0", pred);
        std::string name = "s" + std::to_string(s.result);
        os << pad() << "const " << ctype(val(s.result).dtype) << " " << name << " = "
           << (s.acc.mask_value >= 0 ? "(" + at(s.acc.mask_value, "0", "0") + ") ? " + mem_read(s.acc, addr) + " : " + other_of(s.acc) : mem_read(s.acc, addr)) << ";\n";
        var[s.result] = name;
        k++;
        continue;
      }
      if (s.kind == SK::ScalarStore) {
        map_vars({-1});
        // every thread has read what it reads from this argument before thread 0 overwrites it
        if (read_bases_anywhere.count(s.acc.base_arg)) os << pad() << "__syncthreads();\n";
        std::string pred, addr = address(s.acc, "0", "0", pred);
        os << pad() << "if (threadIdx.x == 0" << (s.acc.mask_value >= 0 ? " && (" + at(s.acc.mask_value, "0", "0") + ")" : "") << ") {\n";
        indent++;
        mem_write(s.acc, addr, "", at(s.operands.at(0), "0", "0"));
        indent--;
        os << pad() << "}\n";
        k++;
        continue;
      }
      if (s.kind == SK::Dot) {
        hoist_costly_vectors(s.operands, copies);
        dot(s, mine);
        k++;
        continue;
      }
      if (s.kind == SK::Reduce || s.kind == SK::Scan) {
        const std::vector<int64_t> shape = val(s.operands.at(0)).shape;
        if (shape.empty() || shape.size() > 4) no("a reduction over a block of rank " + std::to_string(shape.size()));
        if (s.kind == SK::Scan && shape.size() > 2) no("a scan over a block of rank " + std::to_string(shape.size()));
        if (s.kind == SK::Scan && count(shape) > TWO_PHASE_MAX) no("a scan over a block of more than " + std::to_string(TWO_PHASE_MAX) + " elements");
        // An operand that something else uses as well and that is costly to compute (the exponentials of a softmax: summed
        // here, divided and stored later) gets registers now; otherwise both uses write its expression out.
        hoist_costly_vectors(s.operands, copies);
        if (count(shape) <= TWO_PHASE_MAX && shape.size() <= 2)
          for (int o : s.operands) {
            auto d = def.find(o);
            if (d == def.end() || d->second->kind != SK::Map || val(o).shape != shape || held.count(o) || uses[o] < 2 || !costly(o)) continue;
            const std::string name = "mv" + std::to_string(o);
            os << pad() << ctype(val(o).dtype) << " " << name << "[" << (count(shape) + 255) / 256 << "];\n";
            open_element_loop(shape);
            os << pad() << name << "[n] = " << at(o, idx0(shape), idx1(shape)) << ";\n";
            close_loop();
            held[o] = {name, shape};
            mine.push_back(o);
          }
        reduce(s, shape);
        mine.insert(mine.end(), kept_by_scan.begin(), kept_by_scan.end());
        kept_by_scan.clear();
        k++;
        continue;
      }
      // a run of block ops up to the next loop, scalar access or reduction.  Its block shape is that of its stores (else
      // of its largest load); loads of other shapes are read where they are used.
      size_t end = k;
      {
        const std::vector<int64_t> *first_store = nullptr;  // stores of another block shape start a run of their own
        std::set<int> stored;  // a load from an argument that the run has stored to starts a run of its own as well: every
                               // load of a run is issued before the run's first store, and this one has to see that store
        for (; end < ops.size() && !is_break(ops[end]); end++) {
          if (ops[end].kind == SK::Load && stored.count(ops[end].acc.base_arg)) break;
          if (ops[end].kind == SK::Store) {
            if (first_store && ops[end].acc.sizes != *first_store) break;
            first_store = &ops[end].acc.sizes;
            stored.insert(ops[end].acc.base_arg);
          }
        }
      }
      for (size_t q = k; q < end; q++)
        if (ops[q].kind == SK::Load && scalar_store_bases_anywhere.count(ops[q].acc.base_arg)) {
          os << pad() << "__syncthreads();\n";  // thread 0's scalar store to an argument this run loads from is visible
          break;
        }
      std::vector<int64_t> shape;
      bool have = false, stores = false;
      for (size_t q = k; q < end; q++)
        if (ops[q].kind == SK::Store) {
          const auto &sz = ops[q].acc.sizes;
          if (sz.size() > 4 || sz.empty()) no("block accesses of rank " + std::to_string(sz.size()));
          if (!have) { shape = sz; have = stores = true; }
          if (sz != shape) no("block stores of different shapes next to each other");
        }
      for (size_t q = k; q < end; q++)
        if (ops[q].kind == SK::Load) {
          const auto &sz = ops[q].acc.sizes;
          if (sz.size() > 4 || sz.empty()) no("block accesses of rank " + std::to_string(sz.size()));
          if (!have || (!stores && count(sz) > count(shape))) { shape = sz; have = true; }
        }
      if (!have) { k = end; continue; }  // only elementwise ops: they are written out where their results are used
      auto own = [&](const SOp &o) { return o.kind == SK::Load && o.acc.sizes == shape; };
      // a larger block that is stored to an argument it is also loaded from still runs in two phases, whatever that
      // costs in registers (up to 256 values per thread, spilled if need be): the order of its memory effects is kept
      bool hazard = false;
      {
        std::set<int> load_bases;
        for (size_t q = k; q < end; q++)
          if (ops[q].kind == SK::Load) load_bases.insert(ops[q].acc.base_arg);
        for (size_t q = k; q < end; q++) hazard = hazard || (ops[q].kind == SK::Store && load_bases.count(ops[q].acc.base_arg));
      }
      const bool two_phase_run = count(shape) <= (hazard ? HAZARD_MAX : TWO_PHASE_MAX);
      auto big_other = [&](const SOp &o) {
        return two_phase_run && o.kind == SK::Load && o.acc.sizes != shape && count(o.acc.sizes) >= 2048 && count(o.acc.sizes) <= TWO_PHASE_MAX;
      };
      const int64_t T = count(shape);
      const bool two_phase = two_phase_run;
      const std::string i0 = idx0(shape), i1 = idx1(shape);
      auto emit_load = [&](const SOp &o, const std::string &target) {
        std::string pred, addr = address(o.acc, i0, i1, pred);
        os << pad() << target << " = " << (pred.empty() ? mem_read(o.acc, addr) : "(" + pred + ") ? " + mem_read(o.acc, addr) + " : " + other_of(o.acc, i0, i1))
           << ";\n";
      };
      // Loads of another shape are small blocks used through broadcasts (an index vector, a row of scales).  Read in
      // place they would sit in the address computation of the run's own loads, and every one of those would wait for
      // the one before it (loads complete in order): copy them to LDS first, at the place in the program where they stand.
      // A load that the run reads through a transpose is copied as well, whatever its shape: read where the transposed
      // element is used, a wavefront's addresses would be a row pitch apart (a [64, 64] fp32 tile transposed that way
      // moved 2.1 TB/s).
      const std::set<int> transposed = loads_behind_transposes(ops, k, end);
      for (size_t q = k; q < end; q++) {
        const SOp &o = ops[q];
        const bool behind_transpose = transposed.count(o.result) && o.acc.sizes.size() == 2;
        if (o.kind != SK::Load || ((own(o) || big_other(o)) && !behind_transpose) || staged.count(o.result)) continue;
        const int64_t pitch = behind_transpose ? o.acc.sizes.back() + 1 : (o.acc.sizes.empty() ? 1 : o.acc.sizes.back());
        const int64_t elems = behind_transpose ? o.acc.sizes[0] * pitch : count(o.acc.sizes);
        const size_t bytes = (size_t)elems * held_bytes(val(o.result).dtype);
        if (count(o.acc.sizes) > TWO_PHASE_MAX || pool_bytes + out_bytes + bytes > 48 * 1024) continue;
        const std::string name = "blk" + std::to_string(o.result);
        decl << "  __shared__ " << ctype(val(o.result).dtype) << " " << name << "[" << elems << "];\n";
        out_bytes += (bytes + 15) / 16 * 16;
        staged[o.result] = {name, pitch};
        // Inside a loop of the program: two loops, as for the run's own loads, so that every load is issued before the
        // first loaded value is looked at.  (In one loop, `lds[i] = valid ? *p : other` waits for each load before the
        // next goes out: the K block of a flash-attention step, 16 loads per thread, cost a fifth of the step.)  16-bit
        // floats travel as raw bits.  Outside loops the one-loop form stays: short programs overlap each other's waits,
        // and a tiled transpose measured 6 % slower in two loops.
        if (loop_depth == 0) {
          open_element_loop(o.acc.sizes);
          std::string pred, addr = address(o.acc, idx0(o.acc.sizes), idx1(o.acc.sizes), pred);
          os << pad() << staged_at(o.result, idx0(o.acc.sizes), idx1(o.acc.sizes)) << " = "
             << (pred.empty() ? mem_read(o.acc, addr) : "(" + pred + ") ? " + mem_read(o.acc, addr) + " : " + other_of(o.acc, idx0(o.acc.sizes), idx1(o.acc.sizes)))
             << ";\n";
          close_loop();
        } else {
          const std::string &el = o.acc.elem;
          const bool r16 = el == "f16" || el == "bf16";
          const std::string ct = ctype(val(o.result).dtype);
          const bool opaque = r16 || ct == "float" || ct == "int" || ct == "long long" || ct == "double";
          const std::string tmp = "stg" + std::to_string(o.result);
          const std::string i0s = idx0(o.acc.sizes), i1s = idx1(o.acc.sizes);
          os << pad() << "{\n";
          indent++;
          os << pad() << (r16 ? std::string("unsigned") : ct) << " " << tmp << "[" << (count(o.acc.sizes) + 255) / 256 << "];\n";
          open_element_loop(o.acc.sizes);
          {
            std::string pred, addr = address(o.acc, i0s, i1s, pred);
            const std::string raw = r16 ? "((const unsigned short *)p.ptr[" + std::to_string(o.acc.base_arg) + "])[" + addr + "]" : mem_read(o.acc, addr);
            os << pad() << (pred.empty() ? "" : "if (" + pred + ") ") << tmp << "[n] = " << raw << ";\n";
          }
          close_loop();
          open_element_loop(o.acc.sizes);
          {
            std::string pred, addr = address(o.acc, i0s, i1s, pred);
            if (opaque) os << pad() << "asm volatile(\"\" : \"+v\"(" << tmp << "[n]));\n";
            const std::string got = r16 ? std::string(el == "f16" ? "up_f16(" : "up_bf16(") + "(unsigned short)" + tmp + "[n])" : tmp + "[n]";
            os << pad() << staged_at(o.result, i0s, i1s) << " = " << (pred.empty() ? got : "(" + pred + ") ? " + got + " : " + other_of(o.acc, i0s, i1s)) << ";\n";
          }
          close_loop();
          indent--;
          os << pad() << "}\n";
        }
        os << pad() << "__syncthreads();\n";
      }
      if (two_phase) {
        // Registers for the run's own loads, and for large blocks of another shape (a [K, N] operand next to an [M, K]
        // one): those are held by the threads that own their elements and can be named in loops over their own shape.
        std::vector<std::vector<int64_t>> shapes = {shape};
        for (size_t q = k; q < end; q++)
          if (big_other(ops[q]) && std::find(shapes.begin(), shapes.end(), ops[q].acc.sizes) == shapes.end()) shapes.push_back(ops[q].acc.sizes);
        bool any_load = false;
        for (const auto &ls : shapes) {
          auto mine_here = [&](const SOp &o) { return o.kind == SK::Load && o.acc.sizes == ls && (own(o) || big_other(o)) && !staged.count(o.result); };
          bool any = false;
          for (size_t q = k; q < end; q++)
            if (mine_here(ops[q])) {
              if (pack_wide && !hoisted.count(ops[q].result) && wide(ls) && vector_access(ops[q].acc) && is16(ops[q].acc.elem))
                os << pad() << "u32x4_t rw" << ops[q].result << "[" << count(ls) / 2048 << "];\n";
              else if (hoisted.count(ops[q].result)) {
                // (16-bit blocks that stay in registers for the whole launch stay packed, two elements per register, and
                // are widened where they are used)
                if (is16(ops[q].acc.elem)) {
                  hoist_os << "  u32x4_t rw" << ops[q].result << "[" << count(ls) / 2048 << "];\n";
                  // (the empty asm says the words may have changed: the compiler would otherwise widen them once, before
                  // the loop, and keep twice the registers for the whole launch)
                  for (int64_t g = 0; g < count(ls) / 2048; g++) loop_top << "    asm volatile(\"\" : \"+v\"(rw" << ops[q].result << "[" << g << "]));\n";
                }
                else hoist_os << "  " << ctype(val(ops[q].result).dtype) << " ld" << ops[q].result << "[" << (count(ls) + 255) / 256 << "];\n";
              }
              else  // (inside a program loop a slot that a masked load leaves unwritten would otherwise hold, and carry, the last program's)
                os << pad() << ctype(val(ops[q].result).dtype) << " ld" << ops[q].result << "[" << (count(ls) + 255) / 256 << "]" << (persistent ? " = {}" : "") << ";\n";
              any = true;
            }
          if (!any) continue;
          any_load = true;
          const std::string l0 = idx0(ls), l1 = idx1(ls);
          // A masked load is written as `if (valid) x = *p;` here and gets its `other` in a second loop: selecting
          // between the loaded value and `other` on the spot would need the value, and with it a wait for every load
          // before the next one is issued.
          std::vector<std::pair<const SOp *, std::string>> fill;  // masked loads whose `other` is still to be filled in
          auto fill_others = [&]() {
            if (fill.empty()) return;
            open_element_loop(ls);
            for (auto &f : fill) {
              std::string pred, addr = address(f.first->acc, l0, l1, pred);
              if (raw16(*f.first)) {
                // The empty asm keeps the widening here: some compiler versions move it up into the `if (valid)` of the
                // load, where it waits for that load before the next one is issued (a row of 8192 fp16 values: 155 us
                // against 62).
                os << pad() << "asm volatile(\"\" : \"+v\"(" << f.second << "[n]));\n";
                os << pad() << f.second << "[n] = (" << pred << ") ? " << (f.first->acc.elem == "f16" ? "up_f16(" : "up_bf16(") << "(unsigned short)__float_as_uint("
                   << f.second << "[n])) : " << other_of(f.first->acc, l0, l1) << ";\n";
              }
              else
                os << pad() << "if (!(" << pred << ")) " << f.second << "[n] = " << other_of(f.first->acc, l0, l1) << ";\n";
            }
            close_loop();
            fill.clear();
          };
          // Wide blocks: when every group of eight of these loads starts on a 16-byte boundary (the same answer in every
          // thread of the program: the block's first element is aligned and, for blocks of rows, so is the row pitch), a
          // group moves in one 16-byte access (two for 4-byte elements), unconditionally: a group whose first element is
          // valid is read whole (what lies past the valid extent inside an aligned 16 bytes is on the same page), any
          // other from a dummy; a second loop unpacks, widens and fills in `other`.  No branch sits between the loads, so
          // none waits for another.  Otherwise the loads go element by element, as they would in the ordinary order.
          auto wide_load_any = [&](const SOp &o) { return wide(ls) && mine_here(o) && vector_access(o.acc); };
          for (int pass = 0; pass < 2; pass++) {  // pass 0: the loads hoisted out of the program loop, into hoist_os
            auto wide_load = [&](const SOp &o) { return wide_load_any(o) && (hoisted.count(o.result) != 0) == (pass == 0); };
            const int saved_indent = indent;
            if (pass == 0) {
              os.swap(hoist_os);
              indent = 1;
            }
            auto packed = [&](const SOp &o) { return (pass == 0 || pack_wide) && is16(o.acc.elem); };
            bool any_wide = false;
            for (size_t q = k; q < end; q++) any_wide = any_wide || wide_load(ops[q]);
            if (any_wide) {
              const int64_t G = count(ls) / 2048;
              uses_dummy = true;
              std::string aligned;
              for (size_t q = k; q < end; q++)
                if (wide_load(ops[q])) {
                  const SOp &o = ops[q];
                  std::string unused;
                  const int esz = mem_bytes(o.acc.elem);
                  const std::string mask = esz == 1 ? "7" : "15";  // a group of eight 1-byte elements is one 8-byte access
                  aligned += std::string(aligned.empty() ? "" : " && ") + "((unsigned long long)((const " + memtype(o.acc.elem) + " *)p.ptr[" + std::to_string(o.acc.base_arg) +
                             "] + (" + address(o.acc, "0", "0", unused) + ")) & " + mask + ") == 0";
                  if (ls.size() == 2) aligned += " && (((unsigned long long)(" + ex(o.acc.strides[0]) + ") * " + std::to_string(esz) + ") & " + mask + ") == 0";
                }
              os << pad() << "if (" << aligned << ") {\n";
              indent++;
              for (size_t q = k; q < end; q++)
                if (wide_load(ops[q]) && !packed(ops[q]))
                  os << pad() << (mem_bytes(ops[q].acc.elem) == 1 ? "u32x2_t rw" : "u32x4_t rw") << ops[q].result << "[" << G * (mem_bytes(ops[q].acc.elem) == 4 ? 2 : 1) << "];\n";
              os << pad() << "#pragma unroll\n" << pad() << "for (int g = 0; g < " << G << "; g++) {\n";
              indent++;
              os << pad() << "const int n = 8 * g;\n" << pad() << "const int t = " << element_of_slot(ls) << ";\n";
              for (size_t q = k; q < end; q++)
                if (wide_load(ops[q])) {
                  const SOp &o = ops[q];
                  const std::string id = std::to_string(o.result), mt = memtype(o.acc.elem);
                  std::string pred, addr = address(o.acc, l0, l1, pred);
                  os << pad() << "{\n";
                  indent++;
                  const std::string vt = mem_bytes(o.acc.elem) == 1 ? "u32x2_t" : "u32x4_t";
                  os << pad() << "const " << vt << " *const src = " << (pred.empty() ? "" : "!(" + pred + ") ? (const " + vt + " *)tts_dummy : ") << "(const " << vt << " *)((const " << mt
                     << " *)p.ptr[" << o.acc.base_arg << "] + (" << addr << "));\n";
                  if (mem_bytes(o.acc.elem) <= 2) os << pad() << "rw" << id << "[g] = src[0];\n";
                  else {  // the second 16 bytes may lie on another page than the first: read only if their first element is valid
                    std::string pred4;
                    address(o.acc, along(ls, l0, " + 4").first, along(ls, l1, " + 4").second, pred4);
                    os << pad() << "rw" << id << "[2 * g] = src[0];\n" << pad() << "rw" << id << "[2 * g + 1] = "
                       << (pred4.empty() ? "src[1]" : "*(!(" + pred4 + ") ? (const u32x4_t *)tts_dummy : src + 1)") << ";\n";
                  }
                  indent--;
                  os << pad() << "}\n";
                }
              indent--;
              os << pad() << "}\n";
              bool any_packed = false, any_unpacked = false;
              for (size_t q = k; q < end; q++) {
                any_packed = any_packed || (wide_load(ops[q]) && packed(ops[q]));
                any_unpacked = any_unpacked || (wide_load(ops[q]) && !packed(ops[q]));
              }
              if (any_unpacked) open_element_loop(ls);
              for (size_t q = k; q < end; q++)
                if (wide_load(ops[q]) && !packed(ops[q])) {
                  const SOp &o = ops[q];
                  const std::string id = std::to_string(o.result);
                  std::string pred, addr = address(o.acc, l0, l1, pred);
                  std::string got;
                  if (is16(o.acc.elem)) {
                    const std::string word = "rw" + id + "[n >> 3][(n & 7) >> 1]";
                    got = std::string(o.acc.elem == "f16" ? "up_f16(" : "up_bf16(") + "(unsigned short)((n & 1) ? " + word + " >> 16 : " + word + "))";
                  } else if (mem_bytes(o.acc.elem) == 1) {
                    got = "(signed char)(rw" + id + "[n >> 3][(n & 7) >> 2] >> (8 * (n & 3)))";
                  } else {
                    const std::string word = "rw" + id + "[n >> 2][n & 3]";
                    got = o.acc.elem == "f32" ? "__uint_as_float(" + word + ")" : "(int)" + word;
                  }
                  os << pad() << "ld" << id << "[n] = " << (pred.empty() ? got : "(" + pred + ") ? " + got + " : " + other_of(o.acc, l0, l1)) << ";\n";
                }
              if (any_unpacked) close_loop();
              indent--;
              os << pad() << "} else {\n";
              indent++;
              for (size_t q = k; q < end; q++)
                if (wide_load(ops[q]) && packed(ops[q])) os << pad() << "unsigned tm" << ops[q].result << "[" << count(ls) / 256 << "] = {};\n";
              if (any_packed) open_element_loop(ls);
              for (size_t q = k; q < end; q++)
                if (wide_load(ops[q]) && packed(ops[q])) {
                  std::string pred, addr = address(ops[q].acc, l0, l1, pred);
                  os << pad() << (pred.empty() ? "" : "if (" + pred + ") ") << "tm" << ops[q].result << "[n] = ((const unsigned short *)p.ptr[" << ops[q].acc.base_arg << "])[" << addr << "];\n";
                }
              if (any_packed) close_loop();
              for (size_t q = k; q < end; q++)
                if (wide_load(ops[q]) && packed(ops[q])) {
                  os << pad() << "#pragma unroll\n" << pad() << "for (int g = 0; g < " << G << "; g++)\n";
                  os << pad() << "  rw" << ops[q].result << "[g] = u32x4_t{";
                  for (int c = 0; c < 4; c++)
                    os << (c ? ", " : "") << "tm" << ops[q].result << "[8 * g + " << 2 * c << "] | tm" << ops[q].result << "[8 * g + " << 2 * c + 1 << "] << 16";
                  os << "};\n";
                }
              if (any_unpacked) open_element_loop(ls);
              for (size_t q = k; q < end; q++)
                if (wide_load(ops[q]) && !packed(ops[q])) {
                  const SOp &o = ops[q];
                  const std::string name = "ld" + std::to_string(o.result);
                  std::string pred, addr = address(o.acc, l0, l1, pred);
                  if (pred.empty()) os << pad() << name << "[n] = " << mem_read(o.acc, addr) << ";\n";
                  else if (is16(o.acc.elem))
                    os << pad() << "if (" << pred << ") " << name << "[n] = __uint_as_float(((const unsigned short *)p.ptr[" << o.acc.base_arg << "])[" << addr << "]);\n";
                  else os << pad() << "if (" << pred << ") " << name << "[n] = " << mem_read(o.acc, addr) << ";\n";
                }
              if (any_unpacked) close_loop();
              bool any_masked = false;
              for (size_t q = k; q < end; q++) any_masked = any_masked || (wide_load(ops[q]) && !packed(ops[q]) && !ops[q].acc.dims.empty());
              if (any_masked) {
                open_element_loop(ls);
                for (size_t q = k; q < end; q++)
                  if (wide_load(ops[q]) && !packed(ops[q]) && !ops[q].acc.dims.empty()) {
                    const SOp &o = ops[q];
                    const std::string name = "ld" + std::to_string(o.result);
                    std::string pred, addr = address(o.acc, l0, l1, pred);
                    if (is16(o.acc.elem)) {
                      os << pad() << "asm volatile(\"\" : \"+v\"(" << name << "[n]));\n";
                      os << pad() << name << "[n] = (" << pred << ") ? " << (o.acc.elem == "f16" ? "up_f16(" : "up_bf16(") << "(unsigned short)__float_as_uint(" << name
                         << "[n])) : " << other_of(o.acc, l0, l1) << ";\n";
                    } else
                      os << pad() << "if (!(" << pred << ")) " << name << "[n] = " << other_of(o.acc, l0, l1) << ";\n";
                  }
                close_loop();
              }
              indent--;
              os << pad() << "}\n";
              for (size_t q = k; q < end; q++)
                if (wide_load(ops[q])) {
                  const SOp &o = ops[q];
                  if (packed(o)) {
                    const std::string word = "rw" + std::to_string(o.result) + "[n >> 3][(n & 7) >> 1]";
                    std::string pred, addr = address(o.acc, l0, l1, pred);
                    const std::string got = std::string(o.acc.elem == "f16" ? "up_f16(" : "up_bf16(") + "(unsigned short)((n & 1) ? " + word + " >> 16 : " + word + "))";
                    held[o.result] = {"rw" + std::to_string(o.result), ls, "(" + (pred.empty() ? got : "(" + pred + ") ? " + got + " : " + other_of(o.acc, l0, l1)) + ")"};
                    var[o.result] = held[o.result].expr;
                  } else {
                    const std::string name = "ld" + std::to_string(o.result);
                    held[o.result] = {name, ls};
                    var[o.result] = name + "[n]";
                  }
                  mine.push_back(o.result);
                }
            }
            if (pass == 0) {
              os.swap(hoist_os);
              indent = saved_indent;
            }
          }
          auto wide_load = wide_load_any;
          bool any_classic = false;
          for (size_t q = k; q < end; q++) any_classic = any_classic || (mine_here(ops[q]) && !wide_load(ops[q]));
          if (!any_classic) continue;
          open_element_loop(ls);
          for (size_t q = k; q < end; q++)
            if (mine_here(ops[q]) && !wide_load(ops[q])) {
              const std::string name = "ld" + std::to_string(ops[q].result);
              std::string pred, addr = address(ops[q].acc, l0, l1, pred);
              bool needs_filled = false;  // indexed or masked by a load that still lacks its `other`
              for (auto &f : fill) needs_filled = needs_filled || addr.find(f.second + "[") != std::string::npos || pred.find(f.second + "[") != std::string::npos;
              if (needs_filled) {
                close_loop();
                fill_others();
                open_element_loop(ls);
              }
              if (pred.empty()) os << pad() << name << "[n] = " << mem_read(ops[q].acc, addr) << ";\n";
              else {
                if (raw16(ops[q]))  // the raw bits, in the register that will hold the value: widening them here would need the
                                    // loaded value, and with it a wait for every load before the next one is issued
                  os << pad() << "if (" << pred << ") " << name << "[n] = __uint_as_float(((const unsigned short *)p.ptr[" << ops[q].acc.base_arg << "])[" << addr
                     << "]);\n";
                else
                  os << pad() << "if (" << pred << ") " << name << "[n] = " << mem_read(ops[q].acc, addr) << ";\n";
                fill.push_back({&ops[q], name});
              }
              held[ops[q].result] = {name, ls};  // a later load of this run may be indexed by it
              var[ops[q].result] = name + "[n]";
              mine.push_back(ops[q].result);
            }
          close_loop();
          fill_others();
        }
        if (any_load) os << pad() << "__syncthreads();\n";
        if (stores && wide(shape))  // wide stores collect a group's eight values (see the Store case below)
          for (size_t q = k; q < end; q++)
            if (ops[q].kind == SK::Store && vector_access(ops[q].acc)) os << pad() << "unsigned sv" << q << "[8];\n";
        if (stores) open_element_loop(shape);
      } else {
        std::set<int> load_bases;
        for (size_t q = k; q < end; q++)
          if (ops[q].kind == SK::Load) load_bases.insert(ops[q].acc.base_arg);
        for (size_t q = k; q < end; q++)
          if (ops[q].kind == SK::Store && load_bases.count(ops[q].acc.base_arg))
            no("a block of more than " + std::to_string(HAZARD_MAX) + " elements is stored to an argument that is loaded next to the store");
        if (stores) {
          bool reads_held = false;  // a value of this shape that threads keep in registers (the result of a matrix product)
          for (auto &h : held) reads_held = reads_held || h.second.shape == shape;
          if (reads_held) {
            open_element_loop(shape);
          } else {
            os << pad() << "for (int n = 0, t = threadIdx.x; t < " << T << "; t += 256, n++) {\n";
            indent++;
            map_vars({-1});
            cur_i0 = i0;
            cur_i1 = i1;
          }
          for (size_t q = k; q < end; q++)
            if (own(ops[q]) && !staged.count(ops[q].result)) {
              std::string name = "v" + std::to_string(ops[q].result);
              emit_load(ops[q], "const " + ctype(val(ops[q].result).dtype) + " " + name);
              var[ops[q].result] = name;
            }
        }
      }
      if (stores) {
        for (size_t q = k; q < end; q++) {
          const SOp &o = ops[q];
          if (o.kind == SK::Map && val(o.result).shape == shape) {  // a whole-block op: name it, later ops reuse it
            std::string name = "v" + std::to_string(o.result);
            std::string e = at(o.result, i0, i1);
            os << pad() << "const " << ctype(val(o.result).dtype) << " " << name << " = " << e << ";\n";
            var[o.result] = name;
          } else if (o.kind == SK::Store) {
            all_store_bases.insert(o.acc.base_arg);
            const Value &sv = val(o.operands.at(0));
            if (sv.shape != shape) no("a stored value whose shape is not the block's");
            if (two_phase && wide(shape) && vector_access(o.acc)) {
              // the eighth element of a group writes the group: one 16-byte access (two for 4-byte elements) when all
              // eight are valid and the first is 16-byte aligned, element by element otherwise
              const bool half = is16(o.acc.elem), byte = mem_bytes(o.acc.elem) == 1;
              const std::string sv = "sv" + std::to_string(q), mt = memtype(o.acc.elem), value = at(o.operands[0], i0, i1);
              const std::string bits = o.acc.elem == "f16" ? "(unsigned)down_f16_exact(" + value + ")" : o.acc.elem == "bf16" ? "(unsigned)down_bf16(" + value + ")"
                                       : o.acc.elem == "f32" ? "__float_as_uint(" + value + ")" : byte ? "(unsigned)(unsigned char)(" + value + ")" : "(unsigned)(" + value + ")";
              os << pad() << sv << "[n & 7] = " << bits << ";\n";
              std::string pred_last, pred_e, addr0 = address(o.acc, along(shape, i0, " - 7").first, along(shape, i1, " - 7").second, pred_e);
              address(o.acc, i0, i1, pred_last);
              address(o.acc, along(shape, i0, " - 7 + e").first, along(shape, i1, " - 7 + e").second, pred_e);
              os << pad() << "if ((n & 7) == 7) {\n";
              indent++;
              os << pad() << mt << " *const dst = (" << mt << " *)p.ptr[" << o.acc.base_arg << "] + (" << addr0 << ");\n";
              os << pad() << "if (" << (pred_last.empty() ? "" : "(" + pred_last + ") && ") << "((unsigned long long)dst & " << (byte ? 7 : 15) << ") == 0) {\n";
              if (byte)
                os << pad() << "  __builtin_nontemporal_store(u32x2_t{" << sv << "[0] | " << sv << "[1] << 8 | " << sv << "[2] << 16 | " << sv << "[3] << 24, " << sv << "[4] | " << sv
                   << "[5] << 8 | " << sv << "[6] << 16 | " << sv << "[7] << 24}, (u32x2_t *)dst);\n";
              else if (half)
                os << pad() << "  __builtin_nontemporal_store(u32x4_t{" << sv << "[0] | " << sv << "[1] << 16, " << sv << "[2] | " << sv << "[3] << 16, " << sv << "[4] | " << sv
                   << "[5] << 16, " << sv << "[6] | " << sv << "[7] << 16}, (u32x4_t *)dst);\n";
              else
                os << pad() << "  __builtin_nontemporal_store(u32x4_t{" << sv << "[0], " << sv << "[1], " << sv << "[2], " << sv << "[3]}, (u32x4_t *)dst);\n"
                   << pad() << "  __builtin_nontemporal_store(u32x4_t{" << sv << "[4], " << sv << "[5], " << sv << "[6], " << sv << "[7]}, (u32x4_t *)dst + 1);\n";
              os << pad() << "} else {\n";
              os << pad() << "  #pragma unroll\n" << pad() << "  for (int e = 0; e < 8; e++)\n";
              os << pad() << "    if (" << (pred_e.empty() ? "true" : pred_e) << ") " << (byte ? "dst[e] = (signed char)" + sv + "[e]" : half ? "dst[e] = (unsigned short)" + sv + "[e]" : "((unsigned *)dst)[e] = " + sv + "[e]") << ";\n";
              os << pad() << "}\n";
              indent--;
              os << pad() << "}\n";
              continue;
            }
            std::string pred, addr = address(o.acc, i0, i1, pred);
            mem_write(o.acc, addr, pred, at(o.operands[0], i0, i1));
          }
        }
        close_loop();
        os << pad() << "__syncthreads();\n";
      }
      // values named inside the loop end with it (a load of a two-phase run stays in its registers)
      for (size_t q = k; q < end; q++)
        if (ops[q].result >= 0 && (ops[q].kind == SK::Map || (ops[q].kind == SK::Load && !held.count(ops[q].result)))) var.erase(ops[q].result);
      k = end;
    }
    for (int v : copies) lds_copy.erase(v);
    if (defer) {
      defer->insert(defer->end(), mine.begin(), mine.end());
      return;
    }
    for (int v : mine) {
      held.erase(v);
      var.erase(v);
    }
  }

  int loop_depth = 0;  // how many loops of the program enclose what is being written
  void loop(const SOp &s) {
    const std::string L = std::to_string(s.loop);
    // loop-carried block values live in per-thread arrays (element-wise programs never move a value between
    // elements, so each thread carries the elements it owns), each of <= 16384 elements; values of one shape are
    // initialised and stepped together
    // A carried scalar that is not an index expression (a running maximum or sum, as in a softmax over a row read in
    // pieces) is one variable per thread: every thread holds the same value, as it does for a reduction's result.
    std::vector<std::vector<int64_t>> cshapes;
    auto scalar = [&](size_t q) { return val(s.tile_args[q]).shape.empty(); };
    for (size_t q = 0; q < s.tile_args.size(); q++)
      if (scalar(q)) os << pad() << ctype(val(s.tile_args[q]).dtype) << " car" << L << "_" << q << " = " << at(s.tile_inits[q], "0", "0") << ";\n";
    for (size_t q = 0; q < s.tile_args.size(); q++) {
      const Value &V = val(s.tile_args[q]);
      if (scalar(q)) continue;
      if (V.shape.size() > 4) no("a loop-carried value of rank " + std::to_string(V.shape.size()));
      if (count(V.shape) > 2 * TWO_PHASE_MAX) no("a loop-carried block value of more than " + std::to_string(2 * TWO_PHASE_MAX) + " elements");
      if (std::find(cshapes.begin(), cshapes.end(), V.shape) == cshapes.end()) cshapes.push_back(V.shape);
      os << pad() << ctype(V.dtype) << " car" << L << "_" << q << "[" << (count(V.shape) + 255) / 256 << "];\n";
    }
    // carried vectors of a loop that also works on blocks of another shape get an LDS copy (see `mirror`)
    std::vector<std::string> mirrored(s.tile_args.size());
    {
      std::function<bool(const std::vector<SOp> &, const std::vector<int64_t> &)> other_shape = [&](const std::vector<SOp> &ops, const std::vector<int64_t> &sh) {
        for (const SOp &o : ops) {
          if (o.result >= 0 && !val(o.result).shape.empty() && val(o.result).shape != sh) return true;
          if (other_shape(o.body, sh)) return true;
        }
        return false;
      };
      for (size_t q = 0; q < s.tile_args.size(); q++) {
        const Value &V = val(s.tile_args[q]);
        const size_t bytes = (size_t)count(V.shape) * held_bytes(V.dtype);
        if (V.shape.size() != 1 || count(V.shape) > 4096 || !other_shape(s.body, V.shape) || pool_bytes + out_bytes + bytes > 56 * 1024) continue;
        mirrored[q] = "carm" + L + "_" + std::to_string(q);
        decl << "  __shared__ " << ctype(V.dtype) << " " << mirrored[q] << "[" << count(V.shape) << "];\n";
        out_bytes += (bytes + 15) / 16 * 16;
      }
    }
    bool any_mirror = false;
    for (const auto &m : mirrored) any_mirror = any_mirror || !m.empty();
    for (const auto &cshape : cshapes) {
      open_element_loop(cshape);
      for (size_t q = 0; q < s.tile_args.size(); q++)
        if (val(s.tile_args[q]).shape == cshape) {
          os << pad() << "car" << L << "_" << q << "[n] = " << at(s.tile_inits[q], idx0(cshape), idx1(cshape)) << ";\n";
          if (!mirrored[q].empty()) os << pad() << mirrored[q] << "[t] = car" << L << "_" << q << "[n];\n";
        }
      close_loop();
    }
    if (any_mirror) os << pad() << "__syncthreads();\n";
    for (size_t q = 0; q < s.tile_args.size(); q++) {
      if (scalar(q)) {
        var[s.tile_args[q]] = "car" + L + "_" + std::to_string(q);
        continue;
      }
      held[s.tile_args[q]] = {"car" + L + "_" + std::to_string(q), val(s.tile_args[q]).shape};
      if (!mirrored[q].empty()) mirror[s.tile_args[q]] = mirrored[q];
    }
    for (size_t q = 0; q < s.int_iters.size(); q++)
      os << pad() << "long long it" << L << "_" << q << " = " << ex(s.int_iters[q].init) << ";\n";
    // the induction variable wraps at the width of the loop's bounds
    os << pad() << "for (long long iv" << L << " = " << ex(s.lb) << "; iv" << L << " < " << ex(s.ub) << "; iv" << L << " = "
       << (P.pool.at(s.lb).bits == 32 ? "(long long)(int)" : "") << "(iv" << L << " + " << ex(s.step) << ")) {\n";
    indent++;
    std::vector<int> body_held;
    loop_depth++;
    body(s.body, &body_held);
    loop_depth--;
    // the scalars' new values first, their assignment last: the blocks' new values may be written in terms of the old scalars
    for (size_t q = 0; q < s.tile_args.size(); q++)
      if (scalar(q)) os << pad() << "const " << ctype(val(s.tile_args[q]).dtype) << " nys" << L << "_" << q << " = " << at(s.tile_yields[q], "0", "0") << ";\n";
    // With LDS copies: every new value is computed (and every reader of the old copies is done) before a copy changes, and
    // the new copies are complete before the next iteration reads them.
    if (any_mirror) {
      for (size_t q = 0; q < s.tile_args.size(); q++) if (!scalar(q)) os << pad() << ctype(val(s.tile_args[q]).dtype) << " nyv" << L << "_" << q << "[" << (count(val(s.tile_args[q]).shape) + 255) / 256 << "];\n";
      for (const auto &cshape : cshapes) {
        open_element_loop(cshape);
        for (size_t q = 0; q < s.tile_args.size(); q++)
          if (val(s.tile_args[q]).shape == cshape) os << pad() << "nyv" << L << "_" << q << "[n] = " << at(s.tile_yields[q], idx0(cshape), idx1(cshape)) << ";\n";
        close_loop();
      }
      os << pad() << "__syncthreads();\n";
      for (const auto &cshape : cshapes) {
        open_element_loop(cshape);
        for (size_t q = 0; q < s.tile_args.size(); q++)
          if (val(s.tile_args[q]).shape == cshape) {
            os << pad() << "car" << L << "_" << q << "[n] = nyv" << L << "_" << q << "[n];\n";
            if (!mirrored[q].empty()) os << pad() << mirrored[q] << "[t] = nyv" << L << "_" << q << "[n];\n";
          }
        close_loop();
      }
      os << pad() << "__syncthreads();\n";
    } else
    for (const auto &cshape : cshapes) {  // all new values of a shape first, then the assignments: a yield may read another carried value
      open_element_loop(cshape);
      for (size_t q = 0; q < s.tile_args.size(); q++)
        if (val(s.tile_args[q]).shape == cshape)
          os << pad() << "const " << ctype(val(s.tile_args[q]).dtype) << " ny" << q << " = " << at(s.tile_yields[q], idx0(cshape), idx1(cshape)) << ";\n";
      for (size_t q = 0; q < s.tile_args.size(); q++)
        if (val(s.tile_args[q]).shape == cshape) os << pad() << "car" << L << "_" << q << "[n] = ny" << q << ";\n";
      close_loop();
    }
    for (size_t q = 0; q < s.tile_args.size(); q++)
      if (scalar(q)) os << pad() << "car" << L << "_" << q << " = nys" << L << "_" << q << ";\n";
    for (int v : body_held) {
      held.erase(v);
      var.erase(v);
    }
    for (size_t q = 0; q < s.int_iters.size(); q++)
      os << pad() << "const long long nx" << L << "_" << q << " = " << ex(s.int_iters[q].next) << ";\n";
    for (size_t q = 0; q < s.int_iters.size(); q++) os << pad() << "it" << L << "_" << q << " = nx" << L << "_" << q << ";\n";
    indent--;
    os << pad() << "}\n";
    for (size_t q = 0; q < s.int_iters.size(); q++)
      os << pad() << "const long long res" << L << "_" << q << " = it" << L << "_" << q << ";\n";
    // after the loop the carried arrays hold the results
    for (size_t q = 0; q < s.tile_args.size(); q++) {
      held.erase(s.tile_args[q]);
      var.erase(s.tile_args[q]);
      mirror.erase(s.tile_args[q]);
      if (scalar(q)) {
        if (s.results[q] >= 0) var[s.results[q]] = "car" + L + "_" + std::to_string(q);
        continue;
      }
      if (s.results[q] >= 0) {
        held[s.results[q]] = {"car" + L + "_" + std::to_string(q), val(s.tile_args[q]).shape};
        if (!mirrored[q].empty()) mirror[s.results[q]] = mirrored[q];  // (a result read from another shape after the loop)
      }
    }
  }

  // ---- small matrix products ----------------------------------------------
  // result = a x b + c (ConversionPatterns.hpp:1128-1201: linalg.matmul into zeros, then + c), for products that are not
  // shaped like the tiled kernels of the GEMM families: a and b are staged in LDS as fp32, every thread folds k in
  // index order for the outputs it owns (the reference's loop order) and keeps them in registers.
  void dot(const SOp &s, std::vector<int> &mine) {
    const Value &A = val(s.operands.at(0)), &B = val(s.operands.at(1)), &R = val(s.result);
    if (A.shape.size() != 2 || B.shape.size() != 2 || R.shape.size() != 2 || A.shape[1] != B.shape[0] || R.shape[0] != A.shape[0] ||
        R.shape[1] != B.shape[1])
      no("a matrix product whose operands are not [M, K] x [K, N]");
    const int64_t M = A.shape[0], K = A.shape[1], N = B.shape[1];
    if (M * N > 2 * TWO_PHASE_MAX) no("a matrix product with more than " + std::to_string(2 * TWO_PHASE_MAX) + " outputs outside the tiled matmul kernels");
    // operands of a 16-bit type are staged in that type (their values are exactly representable), others as fp32
    auto narrow = [](const std::string &t) { return t == "f16" || t == "bf16"; };
    const size_t a_size = narrow(A.dtype) ? 2 : 4, b_size = narrow(B.dtype) ? 2 : 4;
    if (((size_t)(M * K) * a_size + 15) / 16 * 16 + (size_t)(K * N) * b_size > 96 * 1024)
      no("a matrix product whose operands need " + std::to_string(((size_t)(M * K) * a_size + 15) / 16 * 16 + (size_t)(K * N) * b_size) +
         " bytes of LDS (limit 98304)");
    // The 16-bit matrix-core path reads 16-byte fragments of 32 consecutive rows at once: rows K elements apart would
    // fall into the same few banks (measured: more cycles of bank conflict than of anything else), so its rows are K + 8
    // elements apart when that still fits.
    const bool both16 = A.dtype == B.dtype && narrow(A.dtype);
    const bool both32 = A.dtype == "f32" && B.dtype == "f32";
    const size_t band_bytes = (size_t)32 * N * 4;
    const bool shaped = !(!is_float(A.dtype) && !is_float(B.dtype)) && M % 32 == 0 && N % 32 == 0 && ((both16 && K % 16 == 0) || (both32 && K % 2 == 0)) &&
                        band_bytes <= 32 * 1024;
    const int64_t KP = (shaped && both16 && (size_t)(M + N) * (K + 8) * 2 + band_bytes <= 112 * 1024) ? K + 8 : K;  // row pitch of the staged operands
    const size_t a_bytes = ((size_t)(M * KP) * a_size + 15) / 16 * 16, bytes = a_bytes + (size_t)(KP * N) * b_size;
    // integers (i8 x i8 -> i32 and the like): staged as 32-bit integers, multiplied and added with wrap-around
    const bool integer = !is_float(A.dtype) && !is_float(B.dtype) && !is_float(R.dtype);
    if (!integer && (!is_float(A.dtype) || !is_float(B.dtype) || !is_float(R.dtype))) no("a matrix product that mixes integers and floats");
    if (A.dtype == "f64" || B.dtype == "f64" || R.dtype == "f64" || A.dtype == "i64" || B.dtype == "i64" || R.dtype == "i64")
      no("a matrix product of 64-bit elements");
    pool_bytes = std::max(pool_bytes, bytes);
    const std::string id = std::to_string(s.result);
    auto staged_type = [&](const std::string &t) { return integer ? std::string("int") : narrow(t) ? std::string("unsigned short") : std::string("float"); };
    auto put = [&](const std::string &t, const std::string &e) { return t == "f16" ? "down_f16_exact(" + e + ")" : t == "bf16" ? "down_bf16(" + e + ")" : e; };
    auto get = [&](const std::string &t, const std::string &e) { return t == "f16" ? "up_f16(" + e + ")" : t == "bf16" ? "up_bf16(" + e + ")" : e; };
    os << pad() << "__syncthreads();\n";
    os << pad() << staged_type(A.dtype) << " *const da" << id << " = (" << staged_type(A.dtype) << " *)pool;\n";
    os << pad() << staged_type(B.dtype) << " *const db" << id << " = (" << staged_type(B.dtype) << " *)(pool + " << a_bytes << ");\n";
    open_element_loop(A.shape);
    os << pad() << "da" << id << "[" << (KP == K ? std::string("t") : idx0(A.shape) + " * " + std::to_string(KP) + " + " + idx1(A.shape)) << "] = "
       << put(A.dtype, at(s.operands[0], idx0(A.shape), idx1(A.shape))) << ";\n";
    close_loop();
    // for the 16-bit matrix-core path B is staged transposed ([N][K], K contiguous), so that a lane's eight consecutive k
    // of a column are one 16-byte LDS read, as they are for A
    const bool mfma = !integer && shaped && bytes + band_bytes <= 112 * 1024;
    open_element_loop(B.shape);
    if (mfma && both16)
      os << pad() << "db" << id << "[" << idx1(B.shape) << " * " << KP << " + " << idx0(B.shape) << "] = " << put(B.dtype, at(s.operands[1], idx0(B.shape), idx1(B.shape))) << ";\n";
    else
      os << pad() << "db" << id << "[t] = " << put(B.dtype, at(s.operands[1], idx0(B.shape), idx1(B.shape))) << ";\n";
    close_loop();
    os << pad() << "__syncthreads();\n";
    const std::string name = "dot" + id;
    os << pad() << (integer ? "int " : "float ") << name << "[" << (M * N + 255) / 256 << "];\n";
    // Matrix cores when the shapes allow: 32 x 32 output blocks, one 32-row band of the result at a time.  The four
    // wavefronts take the band's column blocks in turn, accumulate over K with v_mfma_f32_32x32x16 (16-bit operands) or
    // 32x32x2 (fp32), and leave the band in LDS, from where every thread picks up the elements it owns.
    if (mfma) {
      const size_t band_off = (bytes + 15) / 16 * 16;
      uses_mfma = true;
      os << pad() << "float *const dc" << id << " = (float *)(pool + " << band_off << ");\n";
      // When the whole result fits next to the operands, the wavefronts take its 32 x 32 blocks in turn and meet once:
      // two barriers instead of two per band, and no wavefront idles because a band has fewer than four column blocks
      // (a [128, 64] x [64, 64] product of a flash-attention step: 4 bands of 2 blocks).
      if (band_off + (size_t)M * N * 4 <= 112 * 1024) {
        pool_bytes = std::max(pool_bytes, band_off + (size_t)M * N * 4);
        os << pad() << "for (int blk = threadIdx.x >> 6; blk < " << (M / 32) * (N / 32) << "; blk += 4) {\n";
        indent++;
        os << pad() << "const int br = blk / " << N / 32 << ", bc = blk % " << N / 32 << ";\n";
        os << pad() << "const int ln = threadIdx.x & 63, row = br * 32 + (ln & 31), col = bc * 32 + (ln & 31), kg = ln >> 5;\n";
        os << pad() << "f32x16_t acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};\n";
        if (both16) {
          os << pad() << "for (int k0 = 0; k0 < " << K << "; k0 += 16) {\n";
          indent++;
          os << pad() << "const u16x8_t fa = *(const u16x8_t *)&da" << id << "[row * " << KP << " + k0 + 8 * kg], fb = *(const u16x8_t *)&db" << id << "[col * " << KP
             << " + k0 + 8 * kg];\n";
          os << pad() << "acc = " << (A.dtype == "bf16" ? "__builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, fa), __builtin_bit_cast(bf16x8_t, fb)"
                                                        : "__builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, fa), __builtin_bit_cast(f16x8_t, fb)")
             << ", acc, 0, 0, 0);\n";
          indent--;
          os << pad() << "}\n";
        } else {
          os << pad() << "for (int k0 = 0; k0 < " << K << "; k0 += 2) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(da" << id << "[row * " << K << " + k0 + kg], db" << id
             << "[(k0 + kg) * " << N << " + col], acc, 0, 0, 0);\n";
        }
        os << pad() << "#pragma unroll\n" << pad() << "for (int v = 0; v < 16; v++) dc" << id << "[(br * 32 + 8 * (v >> 2) + 4 * kg + (v & 3)) * " << N
           << " + col] = acc[v];\n";
        indent--;
        os << pad() << "}\n" << pad() << "__syncthreads();\n";
        open_element_loop(R.shape);
        os << pad() << name << "[n] = " << rounded(R.dtype, "dc" + id + "[t] + " + at(s.operands.at(2), idx0(R.shape), idx1(R.shape))) << ";\n";
        close_loop();
        os << pad() << "__syncthreads();\n";
        held[s.result] = {name, R.shape};
        mine.push_back(s.result);
        return;
      }
      pool_bytes = std::max(pool_bytes, band_off + band_bytes);
      // With few bands the band loop is unrolled, so that the slots of the result a thread fills from a band (N / 8 of
      // them, consecutive) are known at compile time and the result stays in registers.
      const bool unrolled_bands = M / 32 <= 8;
      if (unrolled_bands) os << pad() << "#pragma unroll\n";
      os << pad() << "for (int br = 0; br < " << M / 32 << "; br++) {\n";
      indent++;
      os << pad() << "for (int bc = threadIdx.x >> 6; bc < " << N / 32 << "; bc += 4) {\n";
      indent++;
      os << pad() << "const int ln = threadIdx.x & 63, row = br * 32 + (ln & 31), col = bc * 32 + (ln & 31), kg = ln >> 5;\n";
      os << pad() << "f32x16_t acc = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};\n";
      if (both16) {
        os << pad() << "for (int k0 = 0; k0 < " << K << "; k0 += 16) {\n";
        indent++;
        os << pad() << "const u16x8_t fa = *(const u16x8_t *)&da" << id << "[row * " << KP << " + k0 + 8 * kg], fb = *(const u16x8_t *)&db" << id << "[col * " << KP
           << " + k0 + 8 * kg];\n";
        os << pad() << "acc = " << (A.dtype == "bf16" ? "__builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, fa), __builtin_bit_cast(bf16x8_t, fb)"
                                                      : "__builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, fa), __builtin_bit_cast(f16x8_t, fb)")
           << ", acc, 0, 0, 0);\n";
        indent--;
        os << pad() << "}\n";
      } else {
        os << pad() << "for (int k0 = 0; k0 < " << K << "; k0 += 2) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(da" << id << "[row * " << K << " + k0 + kg], db" << id
           << "[(k0 + kg) * " << N << " + col], acc, 0, 0, 0);\n";
      }
      os << pad() << "#pragma unroll\n" << pad() << "for (int v = 0; v < 16; v++) dc" << id << "[(8 * (v >> 2) + 4 * kg + (v & 3)) * " << N << " + col] = acc[v];\n";
      indent--;
      os << pad() << "}\n" << pad() << "__syncthreads();\n";
      if (unrolled_bands) {
        os << pad() << "#pragma unroll\n" << pad() << "for (int q = 0; q < " << N / 8 << "; q++) {\n";
        indent++;
        os << pad() << "const int n = br * " << N / 8 << " + q;\n" << pad() << "const int t = threadIdx.x + 256 * n;\n";
        cur_i0 = idx0(R.shape);
        cur_i1 = idx1(R.shape);
        map_vars(R.shape);
        os << pad() << name << "[n] = "
           << rounded(R.dtype, "dc" + id + "[(" + idx0(R.shape) + " % 32) * " + std::to_string(N) + " + " + idx1(R.shape) + "] + " +
                                   at(s.operands.at(2), idx0(R.shape), idx1(R.shape)))
           << ";\n";
        close_loop();
      } else {
        open_element_loop(R.shape);
        os << pad() << "if (" << idx0(R.shape) << " / 32 == br) " << name << "[n] = "
           << rounded(R.dtype, "dc" + id + "[(" + idx0(R.shape) + " % 32) * " + std::to_string(N) + " + " + idx1(R.shape) + "] + " +
                                   at(s.operands.at(2), idx0(R.shape), idx1(R.shape)))
           << ";\n";
        close_loop();
      }
      os << pad() << "__syncthreads();\n";
      indent--;
      os << pad() << "}\n";
      held[s.result] = {name, R.shape};
      mine.push_back(s.result);
      return;
    }
    if (integer) {
      open_element_loop(R.shape);
      os << pad() << "unsigned sum = 0u;\n";
      os << pad() << "for (int k = 0; k < " << K << "; k++) sum += (unsigned)da" << id << "[" << idx0(R.shape) << " * " << K << " + k] * (unsigned)db" << id << "[k * "
         << N << " + " << idx1(R.shape) << "];\n";
      os << pad() << name << "[n] = (int)(sum + (unsigned)" << at(s.operands.at(2), idx0(R.shape), idx1(R.shape)) << ");\n";
      close_loop();
      os << pad() << "__syncthreads();\n";
      held[s.result] = {name, R.shape};
      mine.push_back(s.result);
      return;
    }
    open_element_loop(R.shape);
    os << pad() << "float sum = 0.f;\n";
    os << pad() << "for (int k = 0; k < " << K << "; k++) sum += " << get(A.dtype, "da" + id + "[" + idx0(R.shape) + " * " + std::to_string(K) + " + k]") << " * "
       << get(B.dtype, "db" + id + "[k * " + std::to_string(N) + " + " + idx1(R.shape) + "]") << ";\n";
    os << pad() << name << "[n] = " << rounded(R.dtype, "sum + " + at(s.operands.at(2), idx0(R.shape), idx1(R.shape))) << ";\n";
    close_loop();
    os << pad() << "__syncthreads();\n";
    held[s.result] = {name, R.shape};
    mine.push_back(s.result);
  }

  // ---- reductions and scans ----------------------------------------------
  static size_t held_bytes(const std::string &t) { return (t == "i64" || t == "f64") ? 8 : (t == "i1" || t == "i8") ? 1 : t == "i16" ? 2 : 4; }

  // `void <fname>(a0.., b0.., &r0..)`: r = combine(a, b)
  void combiner(const SOp &s, const std::string &fname) {
    const size_t k = s.operands.size();
    std::ostringstream f;
    f << "__device__ inline void " << fname << "(";
    for (size_t j = 0; j < k; j++) f << "const " << ctype(val(s.operands[j]).dtype) << " a" << j << ", ";
    for (size_t j = 0; j < k; j++) f << "const " << ctype(val(s.operands[j]).dtype) << " b" << j << ", ";
    for (size_t j = 0; j < k; j++) f << (j ? ", " : "") << ctype(val(s.operands[j]).dtype) << " &r" << j;
    f << ") {\n";
    if (s.body.empty()) {
      const std::string &dt = val(s.operands[0]).dtype;
      if (s.name == "arith.addf" && (dt == "f16" || dt == "bf16")) {
        f << "  r0 = a0 + b0;\n";  // 16-bit sums accumulate in f32 and round once (ConversionPatterns.hpp:1280-1286)
      } else {
        SOp m;
        m.kind = SK::Map;
        m.name = s.name;
        m.result = s.operands[0];  // the element type of the result is the operand's
        m.operands = {s.operands[0], s.operands[0]};
        f << "  r0 = " << map_expr(m, {"a0", "b0"}) << ";\n";
      }
    } else {
      std::map<int, std::string> saved = var;
      for (size_t j = 0; j < k; j++) {
        var[s.tile_args.at(j)] = "a" + std::to_string(j);
        var[s.tile_args.at(k + j)] = "b" + std::to_string(j);
      }
      for (auto &o : s.body) {
        if (o.kind != SK::Map && o.kind != SK::Const) no("a combiner with an op that is not scalar arithmetic");
        def[o.result] = &o;
      }
      for (auto &o : s.body) {
        const std::string name = "c" + std::to_string(o.result);
        f << "  const " << ctype(val(o.result).dtype) << " " << name << " = " << at(o.result, "0", "0") << ";\n";
        var[o.result] = name;
      }
      for (size_t j = 0; j < k; j++) f << "  r" << j << " = " << at(s.tile_yields.at(j), "0", "0") << ";\n";
      var = saved;
    }
    f << "}\n";
    fns << f.str();
  }

  // The operand blocks are staged in LDS; each output line is cut into SEG pieces combined by SEG threads and then in
  // piece order by one (lines of >= 256 outputs: one thread per line, in element order, as the reference's loop does).
  void reduce(const SOp &s, const std::vector<int64_t> &shape) {
    const std::string i0 = idx0(shape), i1 = idx1(shape);
    const size_t k = s.operands.size();
    const bool scan = s.kind == SK::Scan;
    const std::string id = std::to_string(s.result);
    for (int o : s.operands)
      if (val(o).shape != shape) no("a reduction or scan over a block whose shape is not the body's");
    const int rank = (int)shape.size();
    if (s.axis < 0 || s.axis >= rank) no("a reduction axis outside the block's rank");
    const int64_t T = count(shape), L = shape[s.axis], O = T / L;
    const bool big = T > TWO_PHASE_MAX;  // nothing of this shape is held in registers: loops need not be unrolled
    const std::string unroll = big ? std::string() : "#pragma unroll\n" + pad();
    const bool lines_of_256 = !scan && L % 256 == 0 && (rank == 1 || (rank == 2 && s.axis == 1));
    // Blocks too large to stage, and blocks of rank above 2: one thread per line.  It walks its line in index order (the
    // order of the reference's sequential loop) and reads every element from its definition, so the operands must be
    // computable in place (loads read where they are used); neighbouring threads read neighbouring lines.
    if (!scan && !lines_of_256 && (big || rank > 2)) {
      const std::string fname = "comb" + id;
      combiner(s, fname);
      std::vector<int64_t> rshape = shape;
      rshape.erase(rshape.begin() + s.axis);
      Idx full = split_index(rshape, rshape.size() >= 2 ? "(o / " + std::to_string(rshape.back()) + ")" : "o",
                             rshape.size() >= 2 ? "(o % " + std::to_string(rshape.back()) + ")" : "0");
      full.insert(full.begin() + s.axis, "l");
      const auto ij = join_index(shape, full);
      std::vector<std::string> Tn(k);
      for (size_t j = 0; j < k; j++) {
        Tn[j] = ctype(val(s.operands[j]).dtype);
        const size_t sz = held_bytes(val(s.operands[j]).dtype);
        decl << "  __shared__ " << Tn[j] << " out" << id << "_" << j << "[" << O << "];\n";
        out_bytes += (O * sz + 15) / 16 * 16;
      }
      if (out_bytes + pool_bytes > 60 * 1024) no("a reduction whose results need more than 60 KB of LDS");
      auto list = [&](const std::string &pre) {
        std::string r;
        for (size_t j = 0; j < k; j++) r += (j ? ", " : "") + pre + std::to_string(j);
        return r;
      };
      map_vars({-1});
      cur_i0.clear();
      cur_i1.clear();
      os << pad() << "__syncthreads();\n";
      os << pad() << "for (int o = threadIdx.x; o < " << O << "; o += 256) {\n";
      indent++;
      for (size_t j = 0; j < k; j++) os << pad() << Tn[j] << " acc" << j << ";\n";
      os << pad() << "for (int l = 0; l < " << L << "; l++) {\n";
      indent++;
      for (size_t j = 0; j < k; j++) os << pad() << "const " << Tn[j] << " el" << j << " = " << at(s.operands[j], ij.first, ij.second) << ";\n";
      os << pad() << "if (l == 0) { ";
      for (size_t j = 0; j < k; j++) os << "acc" << j << " = el" << j << "; ";
      os << "} else " << fname << "(" << list("acc") << ", " << list("el") << ", " << list("acc") << ");\n";
      indent--;
      os << pad() << "}\n";
      for (size_t j = 0; j < k; j++) {
        const std::string &dt = val(s.operands[j]).dtype;
        os << pad() << "out" << id << "_" << j << "[o] = " << (s.body.empty() && s.name == "arith.addf" ? rounded(dt, "acc" + std::to_string(j)) : "acc" + std::to_string(j)) << ";\n";
      }
      indent--;
      os << pad() << "}\n" << pad() << "__syncthreads();\n";
      return;
    }
    if (big && !lines_of_256) no("a scan over a block of more than " + std::to_string(TWO_PHASE_MAX) + " elements");
    const int64_t OS = rank == 1 ? 0 : s.axis == 1 ? shape[1] : 1, LS = rank == 1 ? 1 : s.axis == 1 ? 1 : shape[1];
    int64_t SEG = 1;
    while (SEG * 2 * O <= 256 && (SEG * 2) * (SEG * 2) <= 2 * L) SEG *= 2;  // about sqrt(L) pieces: L / SEG + SEG steps
    const int64_t CH = (L + SEG - 1) / SEG, NSEG = scan ? (L + CH - 1) / CH : SEG, PS = O * NSEG;
    const std::string fname = "comb" + id;
    combiner(s, fname);
    // Lines along the contiguous dimension whose length is a multiple of the workgroup size: every thread owns
    // L / 256 elements of each line.  It folds those in registers, the wavefront folds its 64 partials with a butterfly
    // of lane exchanges, and one LDS round trip folds the four wavefronts: no staging of the block.
    if (lines_of_256) {
      std::vector<std::string> Tn(k);
      size_t off = 0;
      os << pad() << "__syncthreads();\n";
      for (size_t j = 0; j < k; j++) {
        Tn[j] = ctype(val(s.operands[j]).dtype);
        const size_t sz = held_bytes(val(s.operands[j]).dtype);
        os << pad() << Tn[j] << " *const wp" << id << "_" << j << " = (" << Tn[j] << " *)(pool + " << off << ");\n";
        off = (off + O * 4 * sz + 15) / 16 * 16;
        // (a single result: every thread folds the four wavefronts' partials itself and keeps the result in a register,
        // which saves the round through LDS and a barrier)
        if (O == 1) decl << "  " << Tn[j] << " out" << id << "_" << j << "[1];\n";
        else {
          decl << "  __shared__ " << Tn[j] << " out" << id << "_" << j << "[" << O << "];\n";
          out_bytes += (O * sz + 15) / 16 * 16;
        }
      }
      pool_bytes = std::max(pool_bytes, off);
      auto list = [&](const std::string &pre, const std::string &post) {
        std::string r;
        for (size_t j = 0; j < k; j++) r += (j ? ", " : "") + pre + std::to_string(j) + post;
        return r;
      };
      auto final_value = [&](size_t j, const std::string &e) {
        const std::string &dt = val(s.operands[j]).dtype;
        return s.body.empty() && s.name == "arith.addf" ? rounded(dt, e) : e;
      };
      const int64_t LQ = L / 256;
      map_vars(shape);
      cur_i0 = i0;
      cur_i1 = i1;
      os << pad() << unroll << "for (int o = 0; o < " << O << "; o++) {\n";
      indent++;
      for (size_t j = 0; j < k; j++) os << pad() << Tn[j] << " acc" << j << ";\n";
      os << pad() << unroll << "for (int q = 0; q < " << LQ << "; q++) {\n";
      indent++;
      os << pad() << "const int n = o * " << LQ << " + q;\n" << pad() << "const int t = " << element_of_slot(shape) << ";\n";
      for (size_t j = 0; j < k; j++) os << pad() << "const " << Tn[j] << " el" << j << " = " << at(s.operands[j], i0, i1) << ";\n";
      os << pad() << "if (q == 0) { ";
      for (size_t j = 0; j < k; j++) os << "acc" << j << " = el" << j << "; ";
      os << "} else " << fname << "(" << list("acc", "") << ", " << list("el", "") << ", " << list("acc", "") << ");\n";
      indent--;
      os << pad() << "}\n";
      os << pad() << "#pragma unroll\n" << pad() << "for (int m = 32; m >= 1; m >>= 1) {\n";
      indent++;
      for (size_t j = 0; j < k; j++) {
        const std::string &dt = val(s.operands[j]).dtype;
        const bool narrow = dt == "i1" || dt == "i8" || dt == "i16";
        os << pad() << "const " << Tn[j] << " ot" << j << " = " << (narrow ? "(" + Tn[j] + ")__shfl_xor((int)acc" + std::to_string(j) + ", m)"
                                                                          : "__shfl_xor(acc" + std::to_string(j) + ", m)") << ";\n";
      }
      os << pad() << fname << "(" << list("acc", "") << ", " << list("ot", "") << ", " << list("acc", "") << ");\n";
      indent--;
      os << pad() << "}\n";
      os << pad() << "if ((threadIdx.x & 63) == 0) { ";
      for (size_t j = 0; j < k; j++) os << "wp" << id << "_" << j << "[o * 4 + (threadIdx.x >> 6)] = acc" << j << "; ";
      os << "}\n";
      indent--;
      os << pad() << "}\n" << pad() << "__syncthreads();\n";
      if (O == 1) os << pad() << "{\n" << pad() << "  const int o = 0;\n";
      else os << pad() << "for (int o = threadIdx.x; o < " << O << "; o += 256) {\n";
      indent++;
      for (size_t j = 0; j < k; j++) os << pad() << Tn[j] << " acc" << j << " = wp" << id << "_" << j << "[o * 4];\n";
      os << pad() << "#pragma unroll\n" << pad() << "for (int w = 1; w < 4; w++) " << fname << "(" << list("acc", "") << ", " << list("wp" + id + "_", "[o * 4 + w]") << ", " << list("acc", "") << ");\n";
      for (size_t j = 0; j < k; j++) os << pad() << "out" << id << "_" << j << "[o] = " << final_value(j, "acc" + std::to_string(j)) << ";\n";
      indent--;
      os << pad() << "}\n";
      if (O != 1) os << pad() << "__syncthreads();\n";
      cur_i0.clear();
      cur_i1.clear();
      return;
    }
    // The same lines, scanned: the 64 elements a wavefront owns in one slot are consecutive, so it scans them with lane
    // exchanges (Hillis-Steele, earlier elements always on the left of the combiner); the totals of the 4 L / 256
    // pieces of a line meet in LDS, and every piece folds the totals before it into its elements.
    if (scan && !s.ival && L % 256 == 0 && (rank == 1 || s.axis == 1)) {
      std::vector<std::string> Tn(k);
      const int64_t LQ = L / 256, slots = O * LQ;
      size_t off = 0;
      // Results that are only read element by element, in blocks of this shape, stay in the registers of the threads that
      // own them: no copy in LDS, and no barrier after the last step.
      bool in_registers = true;
      for (size_t j = 0; j < k; j++) in_registers = in_registers && read_in_place_only(s.results.empty() ? s.result : s.results[j], shape);
      os << pad() << "__syncthreads();\n";
      for (size_t j = 0; j < k; j++) {
        Tn[j] = ctype(val(s.operands[j]).dtype);
        const size_t sz = held_bytes(val(s.operands[j]).dtype);
        os << pad() << Tn[j] << " *const wp" << id << "_" << j << " = (" << Tn[j] << " *)(pool + " << off << ");\n";
        off = (off + slots * 4 * sz + 15) / 16 * 16;
        os << pad() << Tn[j] << " *const wq" << id << "_" << j << " = (" << Tn[j] << " *)(pool + " << off << ");\n";  // what precedes each piece in its line
        off = (off + slots * 4 * sz + 15) / 16 * 16;
        if (!in_registers) {
          decl << "  __shared__ " << Tn[j] << " out" << id << "_" << j << "[" << T << "];\n";
          out_bytes += (T * sz + 15) / 16 * 16;
        }
      }
      pool_bytes = std::max(pool_bytes, off);
      auto list = [&](const std::string &pre, const std::string &post) {
        std::string r;
        for (size_t j = 0; j < k; j++) r += (j ? ", " : "") + pre + std::to_string(j) + post;
        return r;
      };
      auto shfl = [&](size_t j, const std::string &what) {
        const std::string &dt = val(s.operands[j]).dtype;
        const bool narrow = dt == "i1" || dt == "i8" || dt == "i16";
        return narrow ? "(" + Tn[j] + ")__shfl_up((int)" + what + ", d)" : "__shfl_up(" + what + ", d)";
      };
      map_vars(shape);
      cur_i0 = i0;
      cur_i1 = i1;
      for (size_t j = 0; j < k; j++) os << pad() << Tn[j] << " sc" << id << "_" << j << "[" << slots << "];\n";
      os << pad() << "#pragma unroll\n" << pad() << "for (int n = 0; n < " << slots << "; n++) {\n";
      indent++;
      os << pad() << "const int t = threadIdx.x + 256 * n;\n";
      for (size_t j = 0; j < k; j++) os << pad() << Tn[j] << " acc" << j << " = " << at(s.operands[j], i0, i1) << ";\n";
      bool all32 = true;  // 32-bit values move between lanes inside the ALU (DPP); others go through the LDS crossbar
      for (size_t j = 0; j < k; j++) all32 = all32 && (Tn[j] == "float" || Tn[j] == "int");
      if (all32) {
        // rows of 16 lanes: shifts by 1, 2, 4, 8 inside a row; then lane 15 of a row to the next row (rows 1 and 3), then
        // lane 31 to the upper half -- the wavefront's inclusive scan in six steps, the earlier element always on the left
        static const struct { const char *ctrl, *rows, *cond; } steps[6] = {
            {"0x111", "0xF", "(threadIdx.x & 15) >= 1"}, {"0x112", "0xF", "(threadIdx.x & 15) >= 2"}, {"0x114", "0xF", "(threadIdx.x & 15) >= 4"},
            {"0x118", "0xF", "(threadIdx.x & 15) >= 8"}, {"0x142", "0xA", "(threadIdx.x & 16) != 0"},   {"0x143", "0xC", "(threadIdx.x & 32) != 0"}};
        for (const auto &st : steps) {
          os << pad() << "{\n";
          indent++;
          for (size_t j = 0; j < k; j++)
            os << pad() << "const " << Tn[j] << " ot" << j << " = " << (Tn[j] == "float" ? "TTS_DPP_F(acc" : "TTS_DPP_I(acc") << j << ", " << st.ctrl << ", " << st.rows << ");\n";
          os << pad() << "if (" << st.cond << ") " << fname << "(" << list("ot", "") << ", " << list("acc", "") << ", " << list("acc", "") << ");\n";
          indent--;
          os << pad() << "}\n";
        }
      } else {
        os << pad() << "#pragma unroll\n" << pad() << "for (int d = 1; d < 64; d <<= 1) {\n";
        indent++;
        for (size_t j = 0; j < k; j++) os << pad() << "const " << Tn[j] << " ot" << j << " = " << shfl(j, "acc" + std::to_string(j)) << ";\n";
        os << pad() << "if ((threadIdx.x & 63) >= d) " << fname << "(" << list("ot", "") << ", " << list("acc", "") << ", " << list("acc", "") << ");\n";
        indent--;
        os << pad() << "}\n";
      }
      for (size_t j = 0; j < k; j++) os << pad() << "sc" << id << "_" << j << "[n] = acc" << j << ";\n";
      os << pad() << "if ((threadIdx.x & 63) == 63) { ";
      for (size_t j = 0; j < k; j++) os << "wp" << id << "_" << j << "[n * 4 + (threadIdx.x >> 6)] = acc" << j << "; ";
      os << "}\n";
      indent--;
      os << pad() << "}\n" << pad() << "__syncthreads();\n";
      // one thread per piece folds the totals of the pieces before it in its line (in piece order), once for the workgroup
      os << pad() << "for (int q = threadIdx.x; q < " << slots * 4 << "; q += 256) {\n";
      indent++;
      os << pad() << "const int first = (q / " << LQ * 4 << ") * " << LQ * 4 << ";\n";
      os << pad() << "if (q > first) {\n";
      indent++;
      for (size_t j = 0; j < k; j++) os << pad() << Tn[j] << " carry" << j << " = wp" << id << "_" << j << "[first];\n";
      os << pad() << "for (int i = first + 1; i < q; i++) " << fname << "(" << list("carry", "") << ", " << list("wp" + id + "_", "[i]") << ", " << list("carry", "") << ");\n";
      for (size_t j = 0; j < k; j++) os << pad() << "wq" << id << "_" << j << "[q] = carry" << j << ";\n";
      indent--;
      os << pad() << "}\n";
      indent--;
      os << pad() << "}\n" << pad() << "__syncthreads();\n";
      os << pad() << "#pragma unroll\n" << pad() << "for (int n = 0; n < " << slots << "; n++) {\n";
      indent++;
      os << pad() << "const int t = threadIdx.x + 256 * n;\n";
      os << pad() << "const int first = (n / " << LQ << ") * " << LQ * 4 << ", pieces = (n % " << LQ << ") * 4 + (threadIdx.x >> 6);\n";
      for (size_t j = 0; j < k; j++) os << pad() << Tn[j] << " res" << j << " = sc" << id << "_" << j << "[n];\n";
      os << pad() << "if (pieces > 0) " << fname << "(" << list("wq" + id + "_", "[first + pieces]") << ", " << list("sc" + id + "_", "[n]") << ", " << list("res", "") << ");\n";
      for (size_t j = 0; j < k; j++) {
        if (in_registers) os << pad() << "sc" << id << "_" << j << "[n] = res" << j << ";\n";
        else os << pad() << "out" << id << "_" << j << "[t] = res" << j << ";\n";
      }
      indent--;
      os << pad() << "}\n";
      if (in_registers) {
        for (size_t j = 0; j < k; j++) {
          const int r = s.results.empty() ? s.result : s.results[j];
          held[r] = {"sc" + id + "_" + std::to_string(j), shape};
          kept_by_scan.push_back(r);
        }
      } else {
        os << pad() << "__syncthreads();\n";
      }
      cur_i0.clear();
      cur_i1.clear();
      return;
    }
    // LDS: staging and partials in the shared pool, results in arrays of their own.  Rows that are reduced along their
    // length are staged one element apart from a multiple of the bank count: the threads of a wavefront walk different
    // rows at the same position, which would otherwise meet in one or two banks (rows of 64 floats: 32 threads per bank).
    const int64_t PAD = (!scan && rank == 2 && s.axis == 1 && shape[1] % 2 == 0) ? 1 : 0;
    const int64_t SOS = OS + PAD;  // staged pitch between lines
    std::vector<std::string> Tn(k);
    size_t off = 0;
    os << pad() << "__syncthreads();\n";
    for (size_t j = 0; j < k; j++) {
      Tn[j] = ctype(val(s.operands[j]).dtype);
      const size_t sz = held_bytes(val(s.operands[j]).dtype);
      os << pad() << Tn[j] << " *const st" << id << "_" << j << " = (" << Tn[j] << " *)(pool + " << off << ");\n";
      off = (off + (T + O * PAD) * sz + 15) / 16 * 16;
      os << pad() << Tn[j] << " *const pt" << id << "_" << j << " = (" << Tn[j] << " *)(pool + " << off << ");\n";
      off = (off + PS * sz + 15) / 16 * 16;
      const int64_t n_out = scan ? T : O;
      decl << "  __shared__ " << Tn[j] << " out" << id << "_" << j << "[" << n_out << "];\n";
      out_bytes += (n_out * sz + 15) / 16 * 16;
    }
    pool_bytes = std::max(pool_bytes, off);
    auto list = [&](const std::string &pre, const std::string &post) {
      std::string r;
      for (size_t j = 0; j < k; j++) r += (j ? ", " : "") + pre + std::to_string(j) + post;
      return r;
    };
    const std::string S = "st" + id + "_", Pt = "pt" + id + "_", Out = "out" + id + "_";
    // stage
    open_element_loop(shape);
    for (size_t j = 0; j < k; j++)
      os << pad() << S << j << "[" << (PAD ? i0 + " * " + std::to_string(SOS) + " + " + i1 : std::string("t")) << "] = " << at(s.operands[j], i0, i1) << ";\n";
    close_loop();
    os << pad() << "__syncthreads();\n";
    auto final_value = [&](size_t j, const std::string &e) {  // a 16-bit sum is rounded once, here
      const std::string &dt = val(s.operands[j]).dtype;
      return s.body.empty() && s.name == "arith.addf" ? rounded(dt, e) : e;
    };
    if (!scan) {
      os << pad() << "for (int q = threadIdx.x; q < " << PS << "; q += 256) {\n";
      indent++;
      os << pad() << "const int o = q / " << SEG << ", sg = q % " << SEG << ";\n";
      for (size_t j = 0; j < k; j++) os << pad() << Tn[j] << " acc" << j << " = " << S << j << "[o * " << SOS << " + sg * " << LS << "];\n";
      os << pad() << "for (int l = sg + " << SEG << "; l < " << L << "; l += " << SEG << ") " << fname << "(" << list("acc", "") << ", "
         << list(S, "[o * " + std::to_string(SOS) + " + l * " + std::to_string(LS) + "]") << ", " << list("acc", "") << ");\n";
      for (size_t j = 0; j < k; j++) {
        if (SEG == 1) os << pad() << Out << j << "[o] = " << final_value(j, "acc" + std::to_string(j)) << ";\n";
        else os << pad() << Pt << j << "[q] = acc" << j << ";\n";
      }
      indent--;
      os << pad() << "}\n" << pad() << "__syncthreads();\n";
      if (SEG > 1) {
        os << pad() << "for (int o = threadIdx.x; o < " << O << "; o += 256) {\n";
        indent++;
        for (size_t j = 0; j < k; j++) os << pad() << Tn[j] << " acc" << j << " = " << Pt << j << "[o * " << SEG << "];\n";
        os << pad() << "for (int sg = 1; sg < " << SEG << "; sg++) " << fname << "(" << list("acc", "") << ", "
           << list(Pt, "[o * " + std::to_string(SEG) + " + sg]") << ", " << list("acc", "") << ");\n";
        for (size_t j = 0; j < k; j++) os << pad() << Out << j << "[o] = " << final_value(j, "acc" + std::to_string(j)) << ";\n";
        indent--;
        os << pad() << "}\n" << pad() << "__syncthreads();\n";
      }
      return;
    }
    // scan: each piece on its own, then the pieces' totals in order, then the carry into every later piece
    const std::string at_l = "[o * " + std::to_string(OS) + " + " + (s.ival ? "(" + std::to_string(L - 1) + " - l)" : std::string("l")) + " * " +
                             std::to_string(LS) + "]";
    os << pad() << "for (int q = threadIdx.x; q < " << PS << "; q += 256) {\n";
    indent++;
    os << pad() << "const int o = q / " << NSEG << ", sg = q % " << NSEG << ";\n";
    os << pad() << "int l = sg * " << CH << ";\n" << pad() << "const int l1 = l + " << CH << " < " << L << " ? l + " << CH << " : " << L << ";\n";
    for (size_t j = 0; j < k; j++) os << pad() << Tn[j] << " acc" << j << " = " << S << j << at_l << ";\n";
    for (size_t j = 0; j < k; j++) os << pad() << Out << j << at_l << " = acc" << j << ";\n";
    os << pad() << "for (l++; l < l1; l++) {\n";
    indent++;
    os << pad() << fname << "(" << list("acc", "") << ", " << list(S, at_l) << ", " << list("acc", "") << ");\n";
    for (size_t j = 0; j < k; j++) os << pad() << Out << j << at_l << " = acc" << j << ";\n";
    indent--;
    os << pad() << "}\n";
    for (size_t j = 0; j < k; j++) os << pad() << Pt << j << "[q] = acc" << j << ";\n";
    indent--;
    os << pad() << "}\n" << pad() << "__syncthreads();\n";
    if (NSEG > 1) {
      os << pad() << "for (int o = threadIdx.x; o < " << O << "; o += 256) {\n";
      indent++;
      for (size_t j = 0; j < k; j++) os << pad() << Tn[j] << " acc" << j << " = " << Pt << j << "[o * " << NSEG << "];\n";
      os << pad() << "for (int sg = 1; sg < " << NSEG << "; sg++) {\n";
      indent++;
      for (size_t j = 0; j < k; j++) os << pad() << "const " << Tn[j] << " tot" << j << " = " << Pt << j << "[o * " << NSEG << " + sg];\n";
      for (size_t j = 0; j < k; j++) os << pad() << Pt << j << "[o * " << NSEG << " + sg] = acc" << j << ";\n";
      os << pad() << fname << "(" << list("acc", "") << ", " << list("tot", "") << ", " << list("acc", "") << ");\n";
      indent--;
      os << pad() << "}\n";
      indent--;
      os << pad() << "}\n" << pad() << "__syncthreads();\n";
      os << pad() << "for (int q = threadIdx.x; q < " << PS << "; q += 256) {\n";
      indent++;
      os << pad() << "const int o = q / " << NSEG << ", sg = q % " << NSEG << ";\n" << pad() << "if (sg == 0) continue;\n";
      os << pad() << "const int l1 = (sg + 1) * " << CH << " < " << L << " ? (sg + 1) * " << CH << " : " << L << ";\n";
      for (size_t j = 0; j < k; j++) os << pad() << "const " << Tn[j] << " carry" << j << " = " << Pt << j << "[q];\n";
      os << pad() << "for (int l = sg * " << CH << "; l < l1; l++) {\n";
      indent++;
      for (size_t j = 0; j < k; j++) os << pad() << Tn[j] << " upd" << j << ";\n";
      os << pad() << fname << "(" << list("carry", "") << ", " << list(Out, at_l) << ", " << list("upd", "") << ");\n";
      for (size_t j = 0; j < k; j++) os << pad() << Out << j << at_l << " = upd" << j << ";\n";
      indent--;
      os << pad() << "}\n";
      indent--;
      os << pad() << "}\n" << pad() << "__syncthreads();\n";
    }
  }

};

const char *TILE_PRELUDE = R"SRC(
struct Args { void *ptr[%N%]; long long ival[%N%]; double fval[%N%]; };
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
#define TTS_DPP_I(v, ctrl, rows) __builtin_amdgcn_update_dpp((int)(v), (int)(v), ctrl, rows, 0xF, false)
#define TTS_DPP_F(v, ctrl, rows) __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), ctrl, rows, 0xF, false))
__device__ inline double maximum_d(double a, double b) { return (a != a || b != b) ? __builtin_nan("") : fmax(a, b); }
__device__ inline double minimum_d(double a, double b) { return (a != a || b != b) ? __builtin_nan("") : fmin(a, b); }
__device__ inline long long smin(long long a, long long b) { return a < b ? a : b; }
__device__ inline long long smax(long long a, long long b) { return a > b ? a : b; }
__device__ inline long long sdiv(long long a, long long b) { return b == 0 ? 0 : a / b; }
__device__ inline long long srem(long long a, long long b) { return b == 0 ? 0 : a % b; }
// The same on 32-bit values (what the index arithmetic of a Triton program almost always is): one unsigned 32-bit division,
// a tenth of the 64-bit one's instructions, and no branch, so that equal divisions of neighbouring code merge.  Truncates
// toward zero, 0 for a zero divisor, and the most negative value over -1 wraps, as the 64-bit form does after narrowing.
__device__ inline long long sdiv32(long long a, long long b) {
  const int x = (int)a, y = (int)b;
  const unsigned ux = x < 0 ? 0u - (unsigned)x : (unsigned)x, uy = y < 0 ? 0u - (unsigned)y : (unsigned)y;
  const unsigned uq = ux / (uy == 0u ? 1u : uy);
  return y == 0 ? 0LL : (long long)(int)((x ^ y) < 0 ? 0u - uq : uq);
}
__device__ inline long long srem32(long long a, long long b) {
  const int x = (int)a, y = (int)b;
  const unsigned ux = x < 0 ? 0u - (unsigned)x : (unsigned)x, uy = y < 0 ? 0u - (unsigned)y : (unsigned)y;
  const unsigned ur = ux % (uy == 0u ? 1u : uy);
  return y == 0 ? 0LL : (long long)(int)(x < 0 ? 0u - ur : ur);
}
__device__ inline long long wrap(long long x, long long m) { return m > 0 ? ((x % m) + m) % m : x; }
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned u32x2_t __attribute__((ext_vector_type(2)));
typedef unsigned short u16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
)SRC";

}  // namespace

namespace {
// Programs are independent, so the launcher may hand them to the hardware in any order, and the hardware starts workgroups
// in the order of blockIdx.x first.  When what a program stores is contiguous along a dimension that program_id(1) walks
// (and not program_id(0)), neighbouring workgroups should be neighbours along program_id(1): the source then starts with
// the line below, and the launcher swaps the grid's x and y (x + bias[None, :] on [32, 256] tiles of an 8192 x 8192 matrix,
// row blocks on program_id(0): 119 us; with column blocks there: 100).
const char *const SWAP_MARK = "// tts: swap_xy\n";
const char *const PERSISTENT_MARK = "// tts: persistent\n";  // the launcher starts a few workgroups per CU, which walk the programs
bool stores_walk_columns_with_pid1(const Program &p) {
  int votes_for = 0, votes_against = 0;
  std::function<void(const std::vector<SOp> &)> scan = [&](const std::vector<SOp> &ops) {
    for (const SOp &s : ops) {
      if (s.kind == SK::For || s.kind == SK::If) scan(s.body);
      if (s.kind != SK::Store || s.acc.gather >= 0 || s.acc.sizes.size() < 2 || s.acc.offsets.size() != s.acc.sizes.size() ||
          s.acc.strides.size() != s.acc.sizes.size())
        continue;
      const size_t d = s.acc.sizes.size() - 1;
      int64_t st = 0;
      const bool unit = p.pool.is_const(s.acc.strides[d], &st) && st == 1;
      const int off = s.acc.offsets[d];
      bool other_on_x = false;
      for (size_t e = 0; e < d; e++) other_on_x = other_on_x || p.pool.depends_on(s.acc.offsets[e], EK::Pid, 0);
      if (unit && !p.pool.depends_on(off, EK::Pid, 0) && p.pool.depends_on(off, EK::Pid, 1) && !p.pool.depends_on(off, EK::Pid, 2) && other_on_x)
        votes_for++;
      else
        votes_against++;
    }
  };
  scan(p.body);
  return votes_for > 0 && votes_against == 0;
}
}  // namespace

namespace {
// Two barriers with nothing between them are one.
std::string without_double_barriers(std::string src) {
  const std::string bar = "__syncthreads();\n";
  for (size_t pos = src.find(bar); pos != std::string::npos; pos = src.find(bar, pos + bar.size())) {
    for (;;) {
      size_t next = pos + bar.size(), q = next;
      while (q < src.size() && src[q] == ' ') q++;
      if (src.compare(q, bar.size(), bar) != 0) break;
      src.erase(next, q + bar.size() - next);
    }
  }
  return src;
}
// The body of a persistent kernel's program loop with the thread's index read from a variable that an empty asm renews in
// every iteration: what depends on it alone -- 32 element masks, 32 64-bit element offsets -- is otherwise computed once,
// before the loop, and held in registers for the whole launch (LayerNorm's input gradient: 211 registers instead of 149).
std::string per_program_thread_index(std::string body) {
  const std::string from = "threadIdx.x", to = "tidx";
  for (size_t pos = 0; (pos = body.find(from, pos)) != std::string::npos; pos += to.size()) body.replace(pos, from.size(), to);
  return "    unsigned tidx = threadIdx.x;\n    asm volatile(\"\" : \"+v\"(tidx));\n" + body;
}
}  // namespace

bool tile_program_swaps_grid(const std::string &source) { return source.compare(0, strlen(SWAP_MARK), SWAP_MARK) == 0; }
bool tile_program_is_persistent(const std::string &source) { return source.compare(0, strlen(PERSISTENT_MARK), PERSISTENT_MARK) == 0; }

std::string tile_program_source(const Program &p, bool allow_persistent) {
  if ((int)p.arg_names.size() > TILE_MAX_ARGS) throw Unsupported("tile_program: more than " + std::to_string(TILE_MAX_ARGS) + " kernel arguments");
  Gen g(p);
  std::string pre = TILE_PRELUDE;
  const std::string n = std::to_string(TILE_MAX_ARGS);
  for (size_t pos = 0; (pos = pre.find("%N%", pos)) != std::string::npos;) pre.replace(pos, 3, n);
  g.collect_bases(p.body);
  g.choose_wide_shape();
  if (allow_persistent) g.choose_persistent();
  if (g.persistent) g.indent = 2;
  g.body(p.body);
  // (a CU has 160 KB of LDS and the compiler lets one workgroup declare all of it; 128 KB leaves room for a second, small one)
  if (g.pool_bytes + g.out_bytes > 128 * 1024)
    throw Unsupported("tile_program: the reductions of this program need " + std::to_string(g.pool_bytes + g.out_bytes) + " bytes of LDS (limit 131072)");
  std::ostringstream all;
  if (g.persistent) all << PERSISTENT_MARK;
  else if (stores_walk_columns_with_pid1(p)) all << SWAP_MARK;
  all << pre << g.fns.str();
  if (g.uses_dummy) all << "__device__ __attribute__((aligned(16))) unsigned tts_dummy[8];\n";
  // swap_xy: the launcher has exchanged the grid's x and y (see SWAP_MARK)
  // lgx != 0: the launch is one-dimensional and numbers the programs of an lgx x lgy x lgz grid itself, x fastest (the
  // device's grid holds 65535 along y and z; the reference's launcher loops over any extents, backend/driver.py:116-133)
  all << "extern \"C\" __global__ __launch_bounds__(256) void tile_program(const Args p, const int swap_xy, const int lgx, const int lgy, const int lgz) {\n";
  if (g.pool_bytes) all << "  __shared__ __attribute__((aligned(16))) unsigned char pool[" << g.pool_bytes << "];\n";
  all << g.decl.str();
  if (g.persistent) {
    // a one-dimensional launch of any number of workgroups (lgx, lgy, lgz always hold the grid); what the programs share
    // is loaded first; the barrier at the end keeps a program's LDS arrays from the next program's writes
    all << g.hoist_os.str()
        << "  for (unsigned lin = blockIdx.x; lin < (unsigned)lgx * (unsigned)lgy * (unsigned)lgz; lin += gridDim.x) {  // (fewer than 2^31 programs: the launcher sees to it)\n"
        << "    const long long pidx = lin % (unsigned)lgx, pidy = (lin / (unsigned)lgx) % (unsigned)lgy, pidz = lin / ((unsigned)lgx * (unsigned)lgy);\n"
        << "    const long long npx = lgx, npy = lgy, npz = lgz;\n"
        << "    (void)pidx; (void)pidy; (void)pidz; (void)npx; (void)npy; (void)npz; (void)swap_xy;\n"
        << g.loop_top.str() << per_program_thread_index(g.os.str()) << "    __syncthreads();\n  }\n}\n";
  } else {
    all << "  const long long lin = blockIdx.x;\n"
        << "  const long long pidx = lgx ? lin % lgx : swap_xy ? blockIdx.y : blockIdx.x, pidy = lgx ? (lin / lgx) % lgy : swap_xy ? blockIdx.x : blockIdx.y,\n"
        << "                  pidz = lgx ? lin / ((long long)lgx * lgy) : blockIdx.z;\n"
        << "  const long long npx = lgx ? lgx : swap_xy ? gridDim.y : gridDim.x, npy = lgx ? lgy : swap_xy ? gridDim.x : gridDim.y, npz = lgx ? lgz : gridDim.z;\n"
        << "  (void)pidx; (void)pidy; (void)pidz; (void)npx; (void)npy; (void)npz;\n"
        << g.os.str() << "}\n";
  }
  for (int b : g.all_inline_bases)
    if (g.all_store_bases.count(b))
      throw Unsupported("tile_program: an argument is both stored to and read by a load that is not of its body's block shape");
  return without_double_barriers(all.str());
}

// What a matmul kernel does to its accumulator between the K loop and the store (an activation, a bias, a residual, the
// narrowing cast), as the functor the matrix-product kernels of gemm_device.h call on every accumulator value: `ops` are
// the program's top-level ops outside the loop, `acc` the loop's result, `out` the value that is stored, BM x BN the
// Triton kernel's block.  Those kernels use a tiling of their own, so the functor finds the program that owns the element
// (its ids through a table the launcher fills) and the element's indices inside that program's block, and evaluates the
// stored value for that one element: whatever can be written out per element goes (loads of a bias row or a residual
// block included); anything that needs other elements of the accumulator throws Unsupported.
std::string gemm_epilogue_source(const Program &p, const std::vector<const SOp *> &ops, int acc, int out, int64_t BM, int64_t BN) {
  if ((int)p.arg_names.size() > TILE_MAX_ARGS) throw Unsupported("more than " + std::to_string(TILE_MAX_ARGS) + " kernel arguments");
  Gen g(p);
  for (const SOp *s : ops) {
    if (s->result >= 0) g.def[s->result] = s;
    std::vector<int> es = s->acc.offsets;
    es.insert(es.end(), s->acc.strides.begin(), s->acc.strides.end());
    es.insert(es.end(), s->acc.dims.begin(), s->acc.dims.end());
    es.insert(es.end(), s->acc.mods.begin(), s->acc.mods.end());
    if (s->expr >= 0) es.push_back(s->expr);
    for (EK k : {EK::IV, EK::Iter, EK::Result, EK::Data})
      for (int e : es)
        if (e >= 0 && p.pool.depends_on(e, k)) throw Unsupported("an epilogue value that depends on the K loop or on data");
  }
  g.var[acc] = "acc";
  g.cur_i0 = "i0";
  g.cur_i1 = "i1";
  // The stored value is usually the narrowing cast of an fp32 value: the matrix-product kernels narrow what the functor
  // returns themselves (round to nearest even, two values per instruction), so the functor hands over the cast's operand;
  // rounding it here as well, in integer arithmetic, cost 11 us of the 4096^3 product's 120.
  int shown = out;
  {
    auto d = g.def.find(out);
    if (d != g.def.end() && d->second->kind == SK::Map && d->second->name == "arith.truncf" && d->second->operands.size() == 1 &&
        p.values.at(d->second->operands[0]).dtype == "f32")
      shown = d->second->operands[0];
  }
  g.name_index_exprs = true;
  const std::string expr = g.at(shown, "i0", "i1");
  if (!g.fns.str().empty() || g.pool_bytes || g.out_bytes) throw Unsupported("an epilogue that needs more than one element at a time");
  std::string pre = TILE_PRELUDE;
  const std::string n = std::to_string(TILE_MAX_ARGS);
  for (size_t pos = 0; (pos = pre.find("%N%", pos)) != std::string::npos;) pre.replace(pos, 3, n);
  std::ostringstream all;
  // `at`: the stored value of element (i0, i1) of the block of program q (its linear id); the call operator looks the owner
  // of (row, col) up.  A kernel that knows which of its elements share an owner (BM, BN say how far one owner reaches)
  // looks it up once for all of them and calls `at`, so that what depends on the program alone is computed once.
  all << pre << "struct TtsEp {\n  Args p;\n  const int *tile_pid;\n  int tiles_n, gx, gy, gz;\n"
      << "  static constexpr int BM = " << BM << ", BN = " << BN << ";\n"
      << "  __device__ __forceinline__ float at(int q, float acc, int i0, int i1) const {\n"
      << "    const long long pidx = q % gx, pidy = (q / gx) % gy, pidz = q / (gx * gy), npx = gx, npy = gy, npz = gz;\n"
      << "    (void)i0; (void)i1; (void)pidx; (void)pidy; (void)pidz; (void)npx; (void)npy; (void)npz;\n"
      << g.index_locals.str()
      << "    return " << expr << ";\n  }\n"
      << "  __device__ __forceinline__ float operator()(float acc, long long row, long long col) const {\n"
      << "    return at(tile_pid[(row / BM) * tiles_n + col / BN], acc, (int)(row % BM), (int)(col % BN));\n  }\n};\n";
  return all.str();
}

}  // namespace tts
