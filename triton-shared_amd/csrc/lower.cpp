// TTIR -> structured program.
//
// Restates, for structured (non-gather, non-wraparound) accesses:
//   * tts::PtrAnalysis / PtrState  lib/AnalysisStructured/PtrAnalysis.cpp:276-503
//     (addState), :539-625 (mulState), :901-1100 (make_range, expand_dims,
//     broadcast, splat, addptr, const splat), :1200-1303 (visitOperand dispatch),
//     :1480-1602 (loop-carried pointer state becomes loop-carried offsets/strides),
//     :1672-1733 / :1813-1862 (load / store rewriting);
//   * triton::MaskState  lib/Analysis/MaskAnalysis.cpp:32-59 (dispatch), :181-222
//     (add), :269-286 (min), :288-338 (constants, scalars), :461-603 (cmp; the
//     max(min(end, n), start) - start rule at :568-585), :696-846 (make_range,
//     broadcast, splat, expand_dims);
//   * the op lowering table of include/triton-shared/Conversion/
//     TritonArithToLinalg/ConversionPatterns.hpp: splat :629-650, broadcast
//     :674-719, expand_dims :721-749, make_range :764-805, matmul :1128-1201,
//     reduce :1203-1440, dense constant :1919-1939; elementwise arith/math ops
//     become one whole-tile map each (TritonArithToLinalg.cpp:104).
// Ops whose results feed only address or mask computations are dropped at the
// end, as the reference's final remove-dead-values/CSE/canonicalize does
// (TritonToLinalgExperimentalPass.cpp:80-86).
#include <cmath>
#include <cstring>
#include <functional>
#include <set>

#include "structured.h"

namespace tts {

namespace {

struct PtrState {   // PtrAnalysis.h:52-129, structured fields only
  int source = -1;  // kernel argument index
  int scalar = -1;  // index expr
  std::vector<int> offsets, strides;
  std::vector<int64_t> sizes;
  // per-dim wraparound period in elements of the pointee, already multiplied by the stride
  // (PtrState::shape, PtrAnalysis.h:52-129); -1 = the dimension does not wrap.  The address
  // contribution of dim d at index j is (offsets[d] + j * strides[d]) mod mods[d].
  std::vector<int> mods;
  // block pointers (tt.make_tensor_ptr) only: the extent of the parent tensor and the block's current position in
  // it, per dimension, in elements; a load or store with boundaryCheck on a dimension keeps indices below the extent
  std::vector<int> bshape, boff;
  size_t rank() const { return sizes.size(); }
  bool has_mod() const {
    for (int m : mods)
      if (m >= 0) return true;
    return false;
  }
  void pad_mods() { mods.resize(sizes.size(), -1); }
};

struct MaskState {  // MaskAnalysis.h:63-180
  int start = -1, end = -1, scalar = -1;
  std::vector<int> dims;
  size_t rank() const { return dims.size(); }
};

struct Def {
  const Op *op = nullptr;  // defining op, null for function / region arguments
  int index = 0;           // result number
  Type type;
  int func_arg = -1;       // >= 0 for kernel arguments
};

static double parse_float_literal(const std::string &lit, const std::string &elem) {
  // MLIR prints non-finite and some exact values as hex bit patterns.
  if (lit.rfind("0x", 0) == 0 || lit.rfind("0X", 0) == 0) {
    uint64_t bits = std::stoull(lit, nullptr, 16);
    if (elem == "f32") {
      uint32_t b = (uint32_t)bits;
      float f;
      memcpy(&f, &b, 4);
      return f;
    }
    if (elem == "f64") {
      double d;
      memcpy(&d, &bits, 8);
      return d;
    }
    if (elem == "f16") {
      uint32_t h = (uint32_t)bits, s = (h >> 15) & 1, e = (h >> 10) & 31, m = h & 1023;
      double v = e == 31 ? (m ? NAN : INFINITY) : e == 0 ? std::ldexp((double)m, -24) : std::ldexp(1024.0 + m, (int)e - 25);
      return s ? -v : v;
    }
    if (elem == "bf16") {
      uint32_t b = (uint32_t)bits << 16;
      float f;
      memcpy(&f, &b, 4);
      return f;
    }
    throw Unsupported("hex float literal of type " + elem);
  }
  return std::stod(lit);
}

class Lowerer {
 public:
  explicit Lowerer(const Func &f) : f_(f) {}

  Program run() {
    P.name = f_.name;
    P.arg_names = f_.arg_names;
    P.arg_types = f_.arg_types;
    for (size_t i = 0; i < f_.arg_names.size(); i++) {
      Def d;
      d.type = f_.arg_types[i];
      d.func_arg = (int)i;
      if (d.type.is_tensor) throw Unsupported("tensor-typed kernel argument");
      defs_[f_.arg_names[i]] = d;
    }
    cur_ = &P.body;
    lower_block(f_.body);
    dce();
    return std::move(P);
  }

 private:
  const Func &f_;
  Program P;
  std::map<std::string, Def> defs_;
  std::map<std::string, int> int_memo_;       // scalar integer SSA name -> expr
  int in_region_ = 0;                         // inside a combiner region: scalar integers are data, not index expressions
  std::map<std::string, PtrState> known_ptr_; // loop-carried / loop-result pointer states
  // an unstructured address: base pointer + scalar offset + a block of per-element integer offsets
  struct Scattered { int base = -1, scalar = -1, value = -1; };
  std::map<std::string, Scattered> carried_scatter_;  // loop-carried / loop-result blocks of pointers that are gathers
  std::map<std::string, int> data_;           // SSA name -> value id
  std::vector<SOp> *cur_ = nullptr;

  // ---------------------------------------------------------------- helpers
  const Def &def(const std::string &name) const {
    auto it = defs_.find(name);
    if (it == defs_.end()) throw Unsupported("use of unknown SSA value " + name);
    return it->second;
  }
  int c64(int64_t v) { return P.pool.constant(v, 64); }

  int new_value(const Type &t) {
    Value v;
    v.shape = t.shape;
    v.dtype = t.elem;
    P.values.push_back(v);
    return (int)P.values.size() - 1;
  }

  static Type result_type(const Op &op) {
    if (!op.result_types.empty()) return op.result_types[0];
    if (op.types.empty()) throw Unsupported("cannot infer the result type of " + op.name);
    if (op.name == "tt.load") {
      Type t = op.types[0];
      t.ptr = false;
      return t;
    }
    if (op.name == "arith.cmpi" || op.name == "arith.cmpf") {
      Type t = op.types[0];
      t.elem = "i1";
      return t;
    }
    if (op.name == "tt.addptr") return op.types[0];
    return op.types.back();
  }

  // ------------------------------------------------- scalar integer values
  int int_of(const std::string &name) {
    auto it = int_memo_.find(name);
    if (it != int_memo_.end()) return it->second;
    const Def &d = def(name);
    if (d.type.is_tensor || !d.type.is_int()) throw Unsupported(name + " is not a scalar integer");
    int bits = (d.type.elem == "i64" || d.type.elem == "index") ? 64 : 32;
    int e = -1;
    if (d.func_arg >= 0) {
      e = P.pool.arg(d.func_arg, bits);
    } else if (!d.op) {
      throw Unsupported("integer region argument " + name + " has no known value");
    } else {
      const Op &op = *d.op;
      auto opnd = [&](int i) { return int_of(op.operands.at(i)); };
      static const std::map<std::string, EK> bins = {
          {"arith.addi", EK::Add}, {"arith.subi", EK::Sub},   {"arith.muli", EK::Mul}, {"arith.divsi", EK::DivS},
          {"arith.remsi", EK::RemS}, {"arith.minsi", EK::MinS}, {"arith.maxsi", EK::MaxS}};
      if (op.name == "arith.constant") {
        if (op.literal == "true") e = P.pool.constant(1, 32);
        else if (op.literal == "false") e = P.pool.constant(0, 32);
        else e = P.pool.constant(std::stoll(op.literal), bits);
      } else if (op.name == "tt.get_program_id" || op.name == "tt.get_num_programs") {
        int axis = op.words.empty() ? 0 : (op.words[0] == "x" ? 0 : op.words[0] == "y" ? 1 : 2);
        e = op.name == "tt.get_program_id" ? P.pool.pid(axis) : P.pool.nprog(axis);
      } else if (bins.count(op.name)) {
        e = P.pool.bin(bins.at(op.name), opnd(0), opnd(1));
      } else if (op.name == "arith.extsi" || op.name == "arith.index_cast") {
        int a = opnd(0);
        e = bits == 64 ? P.pool.sext(a) : P.pool.trunc(a);
      } else if (op.name == "arith.trunci") {
        e = P.pool.trunc(opnd(0));
      } else if (op.name == "arith.select") {
        const Def &c = def(op.operands[0]);
        if (!c.op || c.op->name != "arith.cmpi") throw Unsupported("scalar select on a non-cmpi condition");
        static const std::map<std::string, int> preds = {{"slt", 0}, {"sle", 1}, {"sgt", 2}, {"sge", 3}, {"eq", 4}, {"ne", 5}};
        auto pit = preds.find(c.op->words.at(0));
        if (pit == preds.end()) throw Unsupported("scalar cmpi predicate " + c.op->words[0]);
        e = P.pool.cmpsel(pit->second, int_of(c.op->operands[0]), int_of(c.op->operands[1]), opnd(1), opnd(2));
      } else if (op.name == "arith.cmpi") {  // a scalar condition: 1 or 0
        static const std::map<std::string, int> preds = {{"slt", 0}, {"sle", 1}, {"sgt", 2}, {"sge", 3}, {"eq", 4}, {"ne", 5}};
        auto pit = preds.find(op.words.at(0));
        if (pit == preds.end()) throw Unsupported("scalar cmpi predicate " + op.words[0]);
        e = P.pool.cmpsel(pit->second, opnd(0), opnd(1), P.pool.constant(1, 32), P.pool.constant(0, 32));
      } else if (op.name == "arith.andi" && d.type.elem == "i1") {
        e = P.pool.bin(EK::Mul, opnd(0), opnd(1));
      } else {
        // a value read from memory, reduced, yielded by a branch, or computed from one by an op the expressions do not
        // know: a leaf that names the data value (the device knows it, the host does not)
        int v = -1;
        auto dit = data_.find(name);
        if (dit != data_.end()) {
          v = dit->second;
        } else if (is_elementwise(op.name) && !in_region_) {
          SOp s;
          s.kind = SK::Map;
          s.name = map_name(op);
          for (auto &o : op.operands) s.operands.push_back(data_of(o));
          s.result = new_value(d.type);
          cur_->push_back(s);
          data_[name] = v = s.result;
        } else {
          throw Unsupported("scalar integer op " + op.name + " (line " + std::to_string(op.line) + ")");
        }
        e = P.pool.data(v, bits);
      }
    }
    int_memo_[name] = e;
    return e;
  }

  // ------------------------------------------------------------ PtrAnalysis
  PtrState add_state(const PtrState &l, const PtrState &r, const Op &op) {  // PtrAnalysis.cpp:276-503
    if (l.rank() != r.rank()) throw Unsupported("PtrAnalysis: rank mismatch at line " + std::to_string(op.line));
    if (l.source >= 0 && r.source >= 0) throw Unsupported("PtrAnalysis: adding two states that both have a base pointer");
    PtrState s;
    s.source = l.source >= 0 ? l.source : r.source;
    if (l.scalar >= 0 && r.scalar >= 0) s.scalar = P.pool.bin(EK::Add, l.scalar, r.scalar);
    else if (l.rank() == 0) s.scalar = l.scalar >= 0 ? l.scalar : r.scalar;
    for (size_t i = 0; i < l.rank(); i++) {
      s.offsets.push_back(P.pool.bin(EK::Add, l.offsets[i], r.offsets[i]));
      s.strides.push_back(P.pool.bin(EK::Add, l.strides[i], r.strides[i]));
      s.sizes.push_back(l.sizes[i]);
    }
    // wraparound (PtrAnalysis.cpp:440-500): a dimension that wraps keeps its period when the other
    // side adds nothing to it.  A scalar added to every lane (a splat, whose value sits in dim 0)
    // is added after the wrap, so it moves to a dimension that does not wrap.
    s.pad_mods();
    const PtrState *a = &l, *b = &r;
    if (b->has_mod()) std::swap(a, b);
    if (b->has_mod()) throw Unsupported("PtrAnalysis: adding two wraparound index expressions");
    if (a->has_mod()) {
      for (size_t i = 0; i < a->rank(); i++) {
        if (a->mods[i] < 0) continue;
        s.mods[i] = a->mods[i];
        if (is_zero(b->offsets[i]) && is_zero(b->strides[i])) continue;
        size_t other = a->rank();
        for (size_t j = 0; j < a->rank(); j++)
          if (j != i && a->mods[j] < 0) { other = j; break; }
        if (!is_zero(b->strides[i]) || other == a->rank())
          throw Unsupported("PtrAnalysis: adding an index tensor to a dimension that wraps around (line " + std::to_string(op.line) + ")");
        s.offsets[i] = a->offsets[i];
        s.offsets[other] = P.pool.bin(EK::Add, s.offsets[other], b->offsets[i]);
      }
    }
    return s;
  }

  bool is_zero(int e) {
    const Expr x = P.pool.at(e);
    return x.k == EK::Const && x.val == 0;
  }

  PtrState mul_state(const PtrState &lhs, const PtrState &rhs, const Op &op) {  // PtrAnalysis.cpp:539-625
    if (lhs.source >= 0 || rhs.source >= 0) throw Unsupported("PtrAnalysis: multiplying a base pointer");
    if (lhs.scalar < 0 && rhs.scalar < 0)
      throw Unsupported("PtrAnalysis: product of two non-scalar index tensors (line " + std::to_string(op.line) + ")");
    const PtrState *l = &lhs, *r = &rhs;
    if (r->scalar < 0 && l->scalar >= 0) std::swap(l, r);
    PtrState s;
    if (lhs.scalar >= 0 && rhs.scalar >= 0) s.scalar = P.pool.bin(EK::Mul, lhs.scalar, rhs.scalar);
    if (r->has_mod()) throw Unsupported("PtrAnalysis: multiplying by a wraparound index expression");
    for (size_t i = 0; i < l->rank(); i++) {
      s.offsets.push_back(P.pool.bin(EK::Mul, l->offsets[i], r->scalar));
      s.strides.push_back(P.pool.bin(EK::Mul, l->strides[i], r->scalar));
      s.sizes.push_back(l->sizes[i]);
      s.mods.push_back(i < l->mods.size() && l->mods[i] >= 0 ? P.pool.bin(EK::Mul, l->mods[i], r->scalar) : -1);
    }
    return s;
  }

  PtrState visit(const std::string &name) {  // PtrAnalysis.cpp:1200-1303
    auto kp = known_ptr_.find(name);
    if (kp != known_ptr_.end()) return kp->second;
    const Def &d = def(name);
    PtrState s;
    if (!d.type.is_tensor && d.type.is_int()) {
      s.scalar = P.pool.to_index(int_of(name));
      return s;
    }
    if (!d.type.is_tensor && d.type.ptr) {
      if (d.func_arg >= 0) {
        s.source = d.func_arg;
        return s;
      }
      if (d.op && d.op->name == "tt.addptr") return visit_addptr(*d.op);
      if (d.op && d.op->name == "tt.bitcast") {
        // the same memory read as another type of the same width (float bits as integers): offsets count elements, so
        // they stay what they are; a cast that changes the element width would rescale every offset and is refused
        static const std::map<std::string, int> width = {{"i1", 1}, {"i8", 1}, {"i16", 2}, {"f16", 2}, {"bf16", 2}, {"i32", 4}, {"f32", 4}, {"i64", 8}, {"f64", 8}};
        auto from = width.find(def(d.op->operands.at(0)).type.elem), to = width.find(d.type.elem);
        if (from == width.end() || to == width.end() || from->second != to->second)
          throw Unsupported("pointer cast that changes the element width (line " + std::to_string(d.op->line) + ")");
        return visit(d.op->operands[0]);
      }
      throw Unsupported("scalar pointer produced by " + (d.op ? d.op->name : std::string("a region argument")));
    }
    if (!d.op) throw Unsupported("PtrAnalysis: tensor region argument " + name + " without a known state");
    const Op &op = *d.op;
    if (op.name == "arith.addi") return add_state(visit(op.operands[0]), visit(op.operands[1]), op);
    if (op.name == "arith.muli") return mul_state(visit(op.operands[0]), visit(op.operands[1]), op);
    if (op.name == "tt.addptr") return visit_addptr(op);
    if (op.name == "arith.extsi") return visit(op.operands[0]);
    if (op.name == "tt.make_range") {  // :901-919
      int64_t start = std::stoll(op.attrs.at("start")), end = std::stoll(op.attrs.at("end"));
      int64_t n = d.type.shape.at(0);
      if ((end - start + n - 1) / n != 1) throw Unsupported("make_range with stride != 1");
      s.offsets.push_back(c64(start));
      s.sizes.push_back(n);
      s.strides.push_back(c64(1));
      return s;
    }
    if (op.name == "tt.expand_dims") {  // :921-952
      s = visit(op.operands[0]);
      int axis = std::stoi(op.attrs.at("axis"));
      s.offsets.insert(s.offsets.begin() + axis, c64(0));
      s.sizes.insert(s.sizes.begin() + axis, 1);
      s.strides.insert(s.strides.begin() + axis, c64(0));
      s.pad_mods();
      s.mods.insert(s.mods.begin() + axis, -1);
      s.mods.resize(s.sizes.size());
      return s;
    }
    if (op.name == "tt.broadcast") {  // :954-989
      s = visit(op.operands[0]);
      const Type &src = def(op.operands[0]).type;
      for (size_t i = 0; i < d.type.shape.size(); i++)
        if (src.shape[i] < d.type.shape[i]) s.sizes[i] = d.type.shape[i];
      return s;
    }
    if (op.name == "tt.splat") {  // :991-1030
      s = visit(op.operands[0]);
      if (s.rank() != 0) throw Unsupported("splat of a non-scalar");
      for (auto n : d.type.shape) {
        s.offsets.push_back(c64(0));
        s.sizes.push_back(n);
        s.strides.push_back(c64(0));
      }
      if (s.scalar >= 0) s.offsets[0] = s.scalar;
      return s;
    }
    if (op.name == "arith.constant") {  // :1068-1100
      int64_t v = dense_int(op);
      s.scalar = c64(v);
      for (size_t i = 0; i < d.type.shape.size(); i++) {
        s.offsets.push_back(i == 0 ? s.scalar : c64(0));
        s.sizes.push_back(d.type.shape[i]);
        s.strides.push_back(c64(0));
      }
      return s;
    }
    if (op.name == "tt.make_tensor_ptr") {  // :1105-1160 (base, shape, strides, offsets; the order attribute is a layout hint)
      size_t r = d.type.shape.size();
      if (!d.type.block || op.operands.size() != 1 + 3 * r)
        throw Unsupported("tt.make_tensor_ptr with " + std::to_string(op.operands.size()) + " operands for rank " + std::to_string(r));
      PtrState b = visit(op.operands[0]);
      if (b.source < 0 || b.rank() != 0) throw Unsupported("tt.make_tensor_ptr whose base is not a scalar pointer");
      s.source = b.source;
      for (size_t i = 0; i < r; i++) {
        int shape = P.pool.to_index(int_of(op.operands[1 + i]));
        int stride = P.pool.to_index(int_of(op.operands[1 + r + i]));
        int off = P.pool.to_index(int_of(op.operands[1 + 2 * r + i]));
        s.sizes.push_back(d.type.shape[i]);
        s.strides.push_back(stride);
        s.offsets.push_back(P.pool.bin(EK::Mul, off, stride));
        s.bshape.push_back(shape);
        s.boff.push_back(off);
      }
      if (b.scalar >= 0) s.offsets[0] = P.pool.bin(EK::Add, s.offsets[0], P.pool.to_index(b.scalar));
      s.pad_mods();
      return s;
    }
    if (op.name == "tt.advance") {  // :1162-1198
      s = visit(op.operands[0]);
      if (s.boff.size() != s.rank() || op.operands.size() != 1 + s.rank()) throw Unsupported("tt.advance on something that is not a block pointer");
      for (size_t i = 0; i < s.rank(); i++) {
        int delta = P.pool.to_index(int_of(op.operands[1 + i]));
        s.boff[i] = P.pool.bin(EK::Add, s.boff[i], delta);
        s.offsets[i] = P.pool.bin(EK::Add, s.offsets[i], P.pool.bin(EK::Mul, delta, s.strides[i]));
      }
      return s;
    }
    if (op.name == "arith.remsi") {  // :810-891
      PtrState rhs = visit(op.operands[1]);
      if (rhs.scalar < 0) throw Unsupported("PtrAnalysis: remainder by something that is not a scalar");
      s = visit(op.operands[0]);
      s.pad_mods();
      if (s.has_mod()) throw Unsupported("PtrAnalysis: several modulo operations in one index expression");
      if (s.rank() == 1) s.mods[0] = rhs.scalar;
      else if (s.rank() == 2 && d.type.shape[0] == 1) s.mods[1] = rhs.scalar;
      else if (s.rank() == 2 && d.type.shape[1] == 1) s.mods[0] = rhs.scalar;
      else throw Unsupported("PtrAnalysis: modulo on a tensor of this shape");
      return s;
    }
    throw Unsupported("PtrAnalysis: address computed by " + op.name + " (line " + std::to_string(op.line) +
                      ") is not a structured access");
  }

  PtrState visit_addptr(const Op &op) {  // :1032-1066
    PtrState p = visit(op.operands[0]);
    PtrState o = visit(op.operands[1]);
    if (p.source < 0) throw Unsupported("tt.addptr whose pointer operand has no base");
    return add_state(p, o, op);
  }

  static int64_t dense_int(const Op &op) {
    const std::string &lit = op.literal;
    if (lit.rfind("dense<", 0) != 0) throw Unsupported("non-splat constant " + lit);
    std::string in = lit.substr(6, lit.size() - 7);
    if (in == "true") return 1;
    if (in == "false") return 0;
    if (in.find('[') != std::string::npos) throw Unsupported("non-splat dense constant");
    return std::stoll(in);
  }

  // ----------------------------------------------------------- MaskAnalysis
  MaskState mask_parse(const std::string &name) {  // MaskAnalysis.cpp:32-59
    const Def &d = def(name);
    MaskState m;
    if (d.op && d.op->name == "arith.constant") {  // :288-310
      m.scalar = d.type.is_tensor ? c64(dense_int(*d.op)) : P.pool.to_index(int_of(name));
      return m;
    }
    if (!d.type.is_tensor && d.type.is_int()) {  // :312-324
      m.scalar = P.pool.to_index(int_of(name));  // an i1 scalar is 1 or 0: see the conjunction below
      return m;
    }
    if (!d.op) throw Unsupported("MaskAnalysis: loop-carried mask operand");
    const Op &op = *d.op;
    if (op.name == "arith.addi") {  // :181-222, :340-353
      MaskState l = mask_parse(op.operands[0]), r = mask_parse(op.operands[1]);
      if ((l.scalar >= 0) == (r.scalar >= 0)) throw Unsupported("MaskAnalysis: add needs exactly one scalar side");
      const MaskState &t = l.scalar >= 0 ? r : l;
      int sc = l.scalar >= 0 ? l.scalar : r.scalar;
      if (t.start < 0) throw Unsupported("MaskAnalysis: add on a state without a range");
      m.start = P.pool.bin(EK::Add, t.start, sc);
      m.end = P.pool.bin(EK::Add, t.end, sc);
      m.dims = t.dims;
      return m;
    }
    if (op.name == "arith.andi") {  // :355-453, :269-286
      MaskState l = mask_parse(op.operands[0]), r = mask_parse(op.operands[1]);
      if (l.scalar >= 0 && r.scalar >= 0) throw Unsupported("MaskAnalysis: conjunction of two scalar conditions");
      if (l.scalar >= 0 || r.scalar >= 0) {
        // a splatted scalar condition keeps the other side's extents when it holds and empties them otherwise
        // (MaskAnalysis.cpp:269-286, exercised by test_mask.py's scalar-conjunction cases)
        const MaskState &t = l.scalar >= 0 ? r : l;
        const int c = l.scalar >= 0 ? l.scalar : r.scalar;
        for (size_t i = 0; i < t.rank(); i++) m.dims.push_back(P.pool.cmpsel(5, c, c64(0), t.dims[i], c64(0)));
        return m;
      }
      if (l.rank() != r.rank()) throw Unsupported("MaskAnalysis: conjunction of different ranks");
      for (size_t i = 0; i < l.rank(); i++) m.dims.push_back(P.pool.bin(EK::MinS, l.dims[i], r.dims[i]));
      return m;
    }
    if (op.name == "arith.cmpi") return mask_cmp(op);
    if (op.name == "arith.extsi") return mask_parse(op.operands[0]);
    if (op.name == "tt.make_range") {  // :696-720
      int64_t start = std::stoll(op.attrs.at("start")), end = std::stoll(op.attrs.at("end"));
      int64_t n = d.type.shape.at(0);
      if ((end - start + n - 1) / n != 1) throw Unsupported("MaskAnalysis: make_range with stride != 1");
      m.start = c64(start);
      m.end = c64(end);
      m.dims.push_back(c64(n));
      return m;
    }
    if (op.name == "tt.broadcast") {  // :722-750
      m = mask_parse(op.operands[0]);
      const Type &src = def(op.operands[0]).type;
      for (size_t i = 0; i < d.type.shape.size(); i++)
        if (src.shape[i] < d.type.shape[i]) m.dims[i] = c64(d.type.shape[i]);
      return m;
    }
    if (op.name == "tt.splat") {  // :752-783
      const Def &src = def(op.operands[0]);
      if (src.type.is_tensor || !src.type.is_int()) throw Unsupported("MaskAnalysis: splat of a non-integer");
      m = mask_parse(op.operands[0]);
      for (auto n : d.type.shape) m.dims.push_back(c64(n));
      return m;
    }
    if (op.name == "tt.expand_dims") {  // :785-846
      m = mask_parse(op.operands[0]);
      int axis = std::stoi(op.attrs.at("axis"));
      m.dims.insert(m.dims.begin() + axis, c64(1));
      return m;
    }
    throw Unsupported("MaskAnalysis: mask computed by " + op.name + " (line " + std::to_string(op.line) + ")");
  }

  MaskState mask_cmp(const Op &op) {  // MaskAnalysis.cpp:461-603
    const std::string &pred = op.words.at(0);
    if (pred != "slt" && pred != "ult" && pred != "sge") throw Unsupported("MaskAnalysis: cmpi " + pred);
    MaskState l = mask_parse(op.operands[0]), r = mask_parse(op.operands[1]);
    int64_t zero;
    if (pred == "sge" && !(r.scalar >= 0 && P.pool.is_const(r.scalar, &zero) && zero == 0))
      throw Unsupported("MaskAnalysis: sge against a non-zero bound");
    if (l.scalar >= 0) throw Unsupported("MaskAnalysis: comparison of two scalars");
    if (r.scalar < 0) throw Unsupported("MaskAnalysis: comparison against a non-scalar");
    int cmp_dim = -1;
    for (size_t i = 0; i < l.rank(); i++) {
      int64_t v;
      if (!(P.pool.is_const(l.dims[i], &v) && v == 1)) {
        if (cmp_dim != -1) throw Unsupported("MaskAnalysis: cmpi over more than one non-unit dimension");
        cmp_dim = (int)i;
      }
    }
    if (cmp_dim < 0) throw Unsupported("MaskAnalysis: cmpi over a unit tensor");
    int new_dim;
    if (pred == "sge") {
      new_dim = l.dims[cmp_dim];
    } else {
      if (l.start < 0) throw Unsupported("MaskAnalysis: cmpi lhs without a range");
      // :568-585  an entirely masked-off block must give 0, hence the max with start
      int new_end = P.pool.bin(EK::MinS, l.end, r.scalar);
      new_end = P.pool.bin(EK::MaxS, new_end, l.start);
      new_dim = P.pool.bin(EK::Sub, new_end, l.start);
    }
    MaskState m;
    m.dims = l.dims;
    m.dims[cmp_dim] = new_dim;
    return m;
  }

  // --------------------------------------------------------- data lowering
  int data_of(const std::string &name) {
    auto it = data_.find(name);
    if (it != data_.end()) return it->second;
    const Def &d = def(name);
    if (!d.type.is_tensor && d.type.is_int()) {  // integer scalar used as data
      int expr = -1;
      try {
        expr = int_of(name);
      } catch (const Unsupported &) {
        // not an index expression (it depends on a value read from memory): computed as data, op by op
        if (!d.op || !is_elementwise(d.op->name)) throw;
        const Op &op = *d.op;
        SOp s;
        s.kind = SK::Map;
        s.name = map_name(op);
        for (auto &o : op.operands) s.operands.push_back(data_of(o));
        s.result = new_value(d.type);
        cur_->push_back(s);
        return s.result;
      }
      SOp s;
      s.kind = SK::FromIndex;
      s.expr = expr;
      s.result = new_value(d.type);
      cur_->push_back(s);
      // not memoised across scopes: an expression may depend on a loop's state
      return s.result;
    }
    if (!d.type.is_tensor && d.type.is_float() && d.func_arg >= 0) {
      SOp s;
      s.kind = SK::ScalarArg;
      s.ival = d.func_arg;
      s.result = new_value(d.type);
      cur_->push_back(s);
      data_[name] = s.result;
      return s.result;
    }
    throw Unsupported("value " + name + " (" + d.type.str() + ") is not available as data");
  }

  Access make_access(const PtrState &st, const Type &elem_type) {
    if (st.source < 0) throw Unsupported("memory access without a base pointer");
    Access a;
    a.base_arg = st.source;
    a.elem = elem_type.elem;
    a.sizes = st.sizes;
    a.offsets = st.offsets;
    a.strides = st.strides;
    if (st.has_mod()) {
      a.mods = st.mods;
      a.mods.resize(st.rank(), -1);
    }
    if (st.rank() == 0) a.offsets.push_back(st.scalar >= 0 ? st.scalar : c64(0));
    return a;
  }

  void scalar_other(const std::string &name, SOp &s) {  // TritonStructuredOps.cpp:38-98
    Access &a = s.acc;
    const Def &d = def(name);
    const Op *op = d.op;
    if (op && op->name == "tt.splat") op = def(op->operands[0]).op;
    if (!op || op->name != "arith.constant") {  // a value computed by the program: read as data where the mask is false
      a.has_other = true;
      a.other_value = data_of(name);
      s.operands.push_back(a.other_value);
      return;
    }
    std::string lit = op->literal;
    if (lit.rfind("dense<", 0) == 0) lit = lit.substr(6, lit.size() - 7);
    a.has_other = true;
    if (d.type.is_float()) a.other_f = parse_float_literal(lit, d.type.elem);
    else a.other_i = lit == "true" ? 1 : lit == "false" ? 0 : std::stoll(lit);
  }

  // ---- unstructured addresses: base pointer + scalar offset + a tile of per-element integer offsets
  int widen_to_i64(int v) {
    if (P.values[v].dtype == "i64") return v;
    SOp s;
    s.kind = SK::Map;
    s.name = "arith.extsi";
    s.operands = {v};
    Type t;
    t.is_tensor = true;
    t.shape = P.values[v].shape;
    t.elem = "i64";
    s.result = new_value(t);
    cur_->push_back(s);
    return s.result;
  }
  Scattered scattered(const std::string &name) {
    const Def &d = def(name);
    Scattered u;
    if (!d.type.is_tensor) {
      PtrState st = visit(name);
      if (st.source < 0) throw Unsupported("pointer without a base argument");
      u.base = st.source;
      u.scalar = st.scalar >= 0 ? st.scalar : c64(0);
      return u;
    }
    {
      auto it = carried_scatter_.find(name);
      if (it != carried_scatter_.end()) return it->second;
    }
    if (!d.op || d.op->name == "scf.for") throw Unsupported("a tensor of pointers carried around a loop is not a structured access");
    const Op &op = *d.op;
    if (op.name == "tt.splat") return scattered(op.operands[0]);
    if (op.name == "tt.broadcast" || op.name == "tt.expand_dims") {
      u = scattered(op.operands[0]);
      if (u.value >= 0) {
        SOp s;
        s.kind = op.name == "tt.broadcast" ? SK::Broadcast : SK::ExpandDims;
        if (s.kind == SK::ExpandDims) s.axis = std::stoi(op.attrs.at("axis"));
        s.operands = {u.value};
        Type t;
        t.is_tensor = true;
        t.shape = d.type.shape;
        t.elem = P.values[u.value].dtype;
        s.result = new_value(t);
        cur_->push_back(s);
        u.value = s.result;
      }
      return u;
    }
    if (op.name == "tt.addptr") {
      u = scattered(op.operands[0]);
      const Def &o = def(op.operands[1]);
      if (!o.type.is_tensor) {
        u.scalar = P.pool.add_index(u.scalar, int_of(op.operands[1]));
        return u;
      }
      int v = widen_to_i64(data_of(op.operands[1]));
      if (u.value < 0) {
        u.value = v;
      } else {
        SOp s;
        s.kind = SK::Map;
        s.name = "arith.addi";
        s.operands = {widen_to_i64(u.value), v};
        Type t;
        t.is_tensor = true;
        t.shape = d.type.shape;
        t.elem = "i64";
        s.result = new_value(t);
        cur_->push_back(s);
        u.value = s.result;
      }
      return u;
    }
    if (op.name == "arith.select") {  // tl.where between two blocks of pointers into one argument: a choice of offsets
      Scattered a = scattered(op.operands[1]), b = scattered(op.operands[2]);
      if (a.base != b.base) throw Unsupported("select between pointers into different arguments (line " + std::to_string(op.line) + ")");
      const Def &c = def(op.operands[0]);
      if (!c.type.is_tensor) throw Unsupported("select between blocks of pointers on a scalar condition (line " + std::to_string(op.line) + ")");
      SOp s;
      s.kind = SK::Map;
      s.name = "arith.select";
      s.operands = {data_of(op.operands[0]), offsets_block(a, d.type.shape), offsets_block(b, d.type.shape)};
      Type t;
      t.is_tensor = true;
      t.shape = d.type.shape;
      t.elem = "i64";
      s.result = new_value(t);
      cur_->push_back(s);
      u.base = a.base;
      u.scalar = c64(0);
      u.value = s.result;
      return u;
    }
    throw Unsupported("address computed by " + op.name + " (line " + std::to_string(op.line) + ")");
  }
  // the per-element offsets of an unstructured address as one block of 64-bit integers, its scalar part added in
  int offsets_block(const Scattered &u, const std::vector<int64_t> &shape) {
    int v = u.value >= 0 ? widen_to_i64(u.value) : -1;
    int64_t c = 0;
    if (v >= 0 && P.pool.is_const(u.scalar, &c) && c == 0) return v;
    Type st;
    st.elem = "i64";
    SOp f;
    f.kind = SK::FromIndex;
    f.expr = P.pool.to_index(u.scalar);
    f.result = new_value(st);
    cur_->push_back(f);
    Type bt = st;
    bt.is_tensor = true;
    bt.shape = shape;
    SOp sp;
    sp.kind = SK::Splat;
    sp.operands = {f.result};
    sp.result = new_value(bt);
    cur_->push_back(sp);
    if (v < 0) return sp.result;
    SOp a;
    a.kind = SK::Map;
    a.name = "arith.addi";
    a.operands = {v, sp.result};
    a.result = new_value(bt);
    cur_->push_back(a);
    return a.result;
  }
  // the access of a load / store whose pointer PtrAnalysis or whose mask MaskAnalysis cannot describe
  void scattered_access(const Op &op, size_t mask_operand, const Type &elem_type, SOp &s) {
    Scattered u = scattered(op.operands[0]);
    if (u.value < 0) throw Unsupported("unstructured access without per-element offsets");
    s.acc = Access();
    s.acc.base_arg = u.base;
    s.acc.elem = elem_type.elem;
    s.acc.sizes = def(op.operands[0]).type.shape;
    s.acc.offsets = {u.scalar};
    s.acc.gather = u.value;
    s.operands.push_back(u.value);
    if (op.operands.size() > mask_operand) {
      s.acc.mask_value = data_of(op.operands[mask_operand]);
      s.operands.push_back(s.acc.mask_value);
    }
  }

  // boundaryCheck = array<i32: d, ...> of a block-pointer access: per checked dimension, the count of indices that stay
  // below the parent tensor's extent (the upper bound only, a count from the block's first index as for every mask)
  void boundary_dims(const Op &op, const PtrState &st, Access &a) {
    auto it = op.attrs.find("boundaryCheck");
    if (it == op.attrs.end()) return;
    std::string in = it->second;
    size_t colon = in.find(':');
    if (colon == std::string::npos) return;  // array<i32>: nothing checked
    std::vector<bool> checked(st.rank(), false);
    bool any = false;
    for (size_t p = colon + 1; p < in.size();) {
      if (!isdigit((unsigned char)in[p])) { p++; continue; }
      size_t q = p;
      while (q < in.size() && isdigit((unsigned char)in[q])) q++;
      size_t dim = std::stoul(in.substr(p, q - p));
      if (dim >= st.rank()) throw Unsupported("boundaryCheck names dimension " + std::to_string(dim));
      checked[dim] = any = true;
      p = q;
    }
    if (!any) return;
    for (size_t i = 0; i < st.rank(); i++) {
      int n = c64(st.sizes[i]);
      if (checked[i]) {
        int left = P.pool.bin(EK::MaxS, P.pool.bin(EK::Sub, st.bshape[i], st.boff[i]), c64(0));
        n = P.pool.bin(EK::MinS, left, n);
      }
      a.dims.push_back(n);
    }
  }
  void lower_block_load(const Op &op) {  // tt.load of a !tt.ptr<tensor<...>>: no mask operands, boundaryCheck + padding
    Type rt = def(op.operands[0]).type;
    rt.ptr = rt.block = false;
    PtrState st = visit(op.operands[0]);
    if (st.boff.size() != st.rank()) throw Unsupported("block-pointer load without a block position");
    SOp s;
    s.kind = SK::Load;
    s.acc = make_access(st, rt);
    boundary_dims(op, st, s.acc);
    auto pad = op.attrs.find("padding");
    if (!s.acc.dims.empty() && pad != op.attrs.end()) {  // 1 = zero, 2 = NaN (PaddingOption)
      int kind = std::stoi(pad->second);
      s.acc.has_other = true;
      if (kind == 2) {
        if (!rt.is_float()) throw Unsupported("NaN padding of an integer block");
        s.acc.other_f = std::numeric_limits<double>::quiet_NaN();
      } else if (kind != 1) {
        throw Unsupported("padding option " + pad->second);
      }
    }
    s.result = new_value(rt);
    data_[op.results[0]] = s.result;
    cur_->push_back(s);
  }
  void lower_block_store(const Op &op) {
    Type vt = def(op.operands[1]).type;
    PtrState st = visit(op.operands[0]);
    if (st.boff.size() != st.rank()) throw Unsupported("block-pointer store without a block position");
    SOp s;
    s.kind = SK::Store;
    s.acc = make_access(st, vt);
    s.operands.push_back(data_of(op.operands[1]));
    boundary_dims(op, st, s.acc);
    cur_->push_back(s);
  }

  void lower_load(const Op &op) {
    const Def &p = def(op.operands[0]);
    if (p.type.block) return lower_block_load(op);
    Type rt = result_type(op);
    SOp s;
    if (p.type.is_tensor) {
      // structured when PtrAnalysis and MaskAnalysis succeed, otherwise a gather (PtrAnalysis.cpp:200-275 marks
      // such dimensions unstructured and TritonToStructured falls back to make_gather_scatter_tptr)
      bool structured = true;
      try {
        PtrState st = visit(op.operands[0]);
        s.acc = make_access(st, rt);
        if (op.operands.size() >= 2) {
          MaskState m = mask_parse(op.operands[1]);
          if (m.rank() != st.rank()) throw Unsupported("mask rank differs from pointer rank");
          s.acc.dims = m.dims;
        }
      } catch (const Unsupported &) {
        structured = false;
      }
      if (!structured) {
        s.kind = SK::Load;
        scattered_access(op, 1, rt, s);
        if (op.operands.size() >= 3) scalar_other(op.operands[2], s);
        s.result = new_value(rt);
        data_[op.results[0]] = s.result;
        cur_->push_back(s);
        return;
      }
      s = SOp();
    }
    PtrState st = visit(op.operands[0]);
    s.acc = make_access(st, rt);
    if (!p.type.is_tensor) {
      s.kind = SK::ScalarLoad;
      if (op.operands.size() > 1) {  // a scalar condition: the value is `other` (or zero) when it is false
        s.acc.mask_value = data_of(op.operands[1]);
        s.operands.push_back(s.acc.mask_value);
        if (op.operands.size() >= 3) scalar_other(op.operands[2], s);
      }
    } else {
      s.kind = SK::Load;
      if (op.operands.size() >= 2) {
        MaskState m = mask_parse(op.operands[1]);
        if (m.rank() != st.rank()) throw Unsupported("mask rank differs from pointer rank");
        s.acc.dims = m.dims;
      }
      if (op.operands.size() >= 3) scalar_other(op.operands[2], s);
    }
    s.result = new_value(rt);
    data_[op.results[0]] = s.result;
    cur_->push_back(s);
  }

  void lower_store(const Op &op) {
    const Def &p = def(op.operands[0]);
    if (p.type.block) return lower_block_store(op);
    SOp s;
    Type vt = def(op.operands[1]).type;
    if (p.type.is_tensor) {
      bool structured = true;
      try {
        PtrState st = visit(op.operands[0]);
        if (op.operands.size() >= 3 && mask_parse(op.operands[2]).rank() != st.rank()) throw Unsupported("mask rank differs from pointer rank");
      } catch (const Unsupported &) {
        structured = false;
      }
      if (!structured) {  // a scatter
        s.kind = SK::Store;
        s.operands.push_back(data_of(op.operands[1]));
        scattered_access(op, 2, vt, s);
        cur_->push_back(s);
        return;
      }
    }
    PtrState st = visit(op.operands[0]);
    s.acc = make_access(st, vt);
    s.operands.push_back(data_of(op.operands[1]));
    if (!p.type.is_tensor) {
      s.kind = SK::ScalarStore;
      if (op.operands.size() > 2) {
        s.acc.mask_value = data_of(op.operands[2]);
        s.operands.push_back(s.acc.mask_value);
      }
    } else {
      s.kind = SK::Store;
      if (op.operands.size() >= 3) {
        MaskState m = mask_parse(op.operands[2]);
        if (m.rank() != st.rank()) throw Unsupported("mask rank differs from pointer rank");
        s.acc.dims = m.dims;
      }
    }
    cur_->push_back(s);
  }

  // Elementwise ops (one result element per operand element) and the name their Map op carries.
  static bool is_elementwise(const std::string &n) {
    static const std::set<std::string> tt_ops = {"tt.bitcast", "tt.clampf", "tt.mulhiui", "tt.precise_sqrt", "tt.precise_divf"};
    return n.rfind("arith.", 0) == 0 || n.rfind("math.", 0) == 0 || tt_ops.count(n) > 0;
  }
  static std::string map_name(const Op &op) {
    std::string name = op.name;
    if (op.name == "arith.cmpi" || op.name == "arith.cmpf") name += "." + op.words.at(0);
    if (op.name == "tt.clampf") {  // propagateNan = none | all
      bool all = false;
      for (auto &w : op.words) all = all || w == "all";
      auto it = op.attrs.find("propagateNan");
      if (it != op.attrs.end() && it->second.find("all") != std::string::npos) all = true;
      name += all ? ".all" : ".none";
    }
    return name;
  }

  void emit_simple(const Op &op, SK kind, const std::string &name, std::vector<std::string> operand_names) {
    SOp s;
    s.kind = kind;
    s.name = name;
    for (auto &n : operand_names) s.operands.push_back(data_of(n));
    s.result = new_value(result_type(op));
    data_[op.results[0]] = s.result;
    cur_->push_back(s);
  }

  void lower_for(const Op &op) {  // PtrAnalysis.cpp:1480-1602 + TritonToStructuredPass.cpp:72-171
    SOp s;
    s.kind = SK::For;
    s.loop = P.num_loops++;
    s.lb = int_of(op.operands[0]);
    s.ub = int_of(op.operands[1]);
    s.step = int_of(op.operands[2]);
    const Def &lbd = def(op.operands[0]);
    int iv_bits = (lbd.type.elem == "i64" || lbd.type.elem == "index") ? 64 : 32;
    {
      Def d;
      d.type = lbd.type;
      defs_[op.iv] = d;
      int_memo_[op.iv] = P.pool.iv(s.loop, iv_bits);
    }
    struct Carried { int kind; PtrState st; size_t first_slot; int tile_index; int base; };  // 0 ptr, 1 int, 2 tile, 3 gathered ptrs
    std::vector<Carried> carried;
    for (size_t j = 0; j < op.iter_names.size(); j++) {
      const Type &t = op.result_types[j];
      Def d;
      d.type = t;
      defs_[op.iter_names[j]] = d;
      Carried c{};
      bool gathered = false;
      PtrState init;
      if (t.ptr) {
        try {
          init = visit(op.iter_inits[j]);
        } catch (const Unsupported &) {
          if (!t.is_tensor) throw;
          gathered = true;
        }
      }
      if (gathered) {
        // a block of pointers that PtrAnalysis cannot describe (rows picked by loaded indices, walked along K): carried
        // as its base argument and a block of 64-bit element offsets
        Scattered u = scattered(op.iter_inits[j]);
        c.kind = 3;
        c.base = u.base;
        c.tile_index = (int)s.tile_args.size();
        s.tile_inits.push_back(offsets_block(u, t.shape));
        Type ot;
        ot.is_tensor = true;
        ot.shape = t.shape;
        ot.elem = "i64";
        int v = new_value(ot);
        s.tile_args.push_back(v);
        Scattered inside;
        inside.base = u.base;
        inside.scalar = c64(0);
        inside.value = v;
        carried_scatter_[op.iter_names[j]] = inside;
      } else if (t.ptr) {
        c.kind = 0;
        c.first_slot = s.int_iters.size();
        PtrState inside = init;
        auto carry = [&](int init_expr) {
          IntIter it;
          int slot = (int)s.int_iters.size();
          it.init = init_expr;
          it.iter_expr = P.pool.iter(s.loop, slot, 64);
          it.result_expr = P.pool.result(s.loop, slot, 64);
          s.int_iters.push_back(it);
          return it.iter_expr;
        };
        if (init.rank() == 0) {
          inside.scalar = carry(init.scalar >= 0 ? init.scalar : c64(0));
        } else {
          for (auto &o : inside.offsets) o = carry(o);
          for (auto &st : inside.strides) st = carry(st);
          for (auto &o : inside.boff) o = carry(o);
        }
        c.st = inside;
        known_ptr_[op.iter_names[j]] = inside;
      } else if (!t.is_tensor && t.is_int()) {
        c.kind = 1;
        c.first_slot = s.int_iters.size();
        int bits = (t.elem == "i64" || t.elem == "index") ? 64 : 32;
        IntIter it;
        it.init = int_of(op.iter_inits[j]);
        it.iter_expr = P.pool.iter(s.loop, (int)c.first_slot, bits);
        it.result_expr = P.pool.result(s.loop, (int)c.first_slot, bits);
        s.int_iters.push_back(it);
        int_memo_[op.iter_names[j]] = it.iter_expr;
      } else {
        // block values, integer ones included: an address built from a carried integer block is then not a
        // structured access and is lowered as a gather / scatter

        c.kind = 2;
        c.tile_index = (int)s.tile_args.size();
        s.tile_inits.push_back(data_of(op.iter_inits[j]));
        int v = new_value(t);
        s.tile_args.push_back(v);
        data_[op.iter_names[j]] = v;
      }
      carried.push_back(c);
    }
    // body
    std::vector<SOp> *saved = cur_;
    cur_ = &s.body;
    const Block &body = op.regions.at(0);
    const Op *yield = nullptr;
    for (auto &bop : body.ops) {
      if (bop->name == "scf.yield") {
        yield = bop.get();
        break;
      }
      lower_op(*bop);
    }
    if (!op.iter_names.empty()) {
      if (!yield || yield->operands.size() != op.iter_names.size()) throw Unsupported("scf.for without a matching scf.yield");
      s.tile_yields.resize(s.tile_args.size());
      for (size_t j = 0; j < carried.size(); j++) {
        const Carried &c = carried[j];
        const std::string &y = yield->operands[j];
        if (c.kind == 0) {
          PtrState ns = visit(y);
          ns.pad_mods();
          if (ns.source != c.st.source || ns.sizes != c.st.sizes || ns.mods != c.st.mods || ns.bshape != c.st.bshape)
            throw Unsupported("loop-carried pointer changes its base, block shape, parent extent or wraparound");
          size_t slot = c.first_slot;
          if (ns.rank() == 0) {
            s.int_iters[slot].next = ns.scalar;
          } else {
            for (auto o : ns.offsets) s.int_iters[slot++].next = o;
            for (auto st : ns.strides) s.int_iters[slot++].next = st;
            for (auto o : ns.boff) s.int_iters[slot++].next = o;
          }
        } else if (c.kind == 1) {
          s.int_iters[c.first_slot].next = int_of(y);
        } else if (c.kind == 3) {
          Scattered ny = scattered(y);
          if (ny.base != c.base) throw Unsupported("loop-carried pointer changes its base");
          s.tile_yields[c.tile_index] = offsets_block(ny, op.result_types[j].shape);
        } else {
          s.tile_yields[c.tile_index] = data_of(y);
        }
      }
    }
    cur_ = saved;
    // results
    s.results.resize(s.tile_args.size());
    for (size_t j = 0; j < carried.size(); j++) {
      const Carried &c = carried[j];
      const std::string &rname = op.results.at(j);
      Def d;
      d.type = op.result_types[j];
      d.op = &op;
      d.index = (int)j;
      defs_[rname] = d;
      if (c.kind == 0) {
        PtrState after = c.st;
        size_t slot = c.first_slot;
        if (after.rank() == 0) {
          after.scalar = s.int_iters[slot].result_expr;
        } else {
          for (auto &o : after.offsets) o = s.int_iters[slot++].result_expr;
          for (auto &st : after.strides) st = s.int_iters[slot++].result_expr;
          for (auto &o : after.boff) o = s.int_iters[slot++].result_expr;
        }
        known_ptr_[rname] = after;
      } else if (c.kind == 1) {
        int_memo_[rname] = s.int_iters[c.first_slot].result_expr;
      } else if (c.kind == 3) {
        Type ot = d.type;
        ot.ptr = false;
        ot.elem = "i64";
        int v = new_value(ot);
        s.results[c.tile_index] = v;
        Scattered after;
        after.base = c.base;
        after.scalar = c64(0);
        after.value = v;
        carried_scatter_[rname] = after;
      } else {
        int v = new_value(d.type);
        s.results[c.tile_index] = v;
        data_[rname] = v;
      }
    }
    cur_->push_back(std::move(s));
  }

  void lower_reduce(const Op &op) {  // ConversionPatterns.hpp:1203-1440 (one combiner op), :1443-1769 (argmin / argmax)
    const bool scan = op.name == "tt.scan";
    const size_t k = op.operands.size();
    if (op.regions.size() != 1 || k == 0) throw Unsupported(op.name + " without operands or combiner");
    const Block &rb = op.regions[0];
    if (rb.arg_names.size() != 2 * k || op.result_types.size() != k) throw Unsupported(op.name + " whose combiner does not take two values per operand");
    if (rb.ops.empty() || rb.ops.back()->name != (scan ? "tt.scan.return" : "tt.reduce.return") || rb.ops.back()->operands.size() != k)
      throw Unsupported(op.name + " whose combiner does not end in a return of one value per operand");
    SOp s;
    s.kind = scan ? SK::Scan : SK::Reduce;
    s.axis = std::stoi(op.attrs.at("axis"));
    if (scan) s.ival = op.attrs.count("reverse") && op.attrs.at("reverse") == "true";
    for (auto &o : op.operands) s.operands.push_back(data_of(o));
    // the common case: one op that combines the two block arguments
    static const std::set<std::string> ok = {"arith.addf", "arith.addi", "arith.maxnumf", "arith.maximumf",
                                             "arith.minnumf", "arith.minimumf", "arith.mulf", "arith.maxsi",
                                             "arith.minsi", "arith.maxui", "arith.minui", "arith.ori",
                                             "arith.andi", "arith.xori", "arith.muli"};
    if (k == 1 && rb.ops.size() == 2) {
      const Op &comb = *rb.ops[0];
      std::set<std::string> ins(comb.operands.begin(), comb.operands.end());
      if (ok.count(comb.name) && comb.operands.size() == 2 && ins.count(rb.arg_names[0]) && ins.count(rb.arg_names[1]) &&
          rb.ops[1]->operands[0] == comb.results.at(0))
        s.name = comb.name;
    }
    if (!s.name.empty() && !scan) {
      s.result = new_value(result_type(op));
      data_[op.results[0]] = s.result;
      cur_->push_back(s);
      return;
    }
    // the combiner as a region of scalar ops
    if (s.name.empty()) s.name = "region";
    std::vector<SOp> *saved = cur_;
    cur_ = &s.body;
    in_region_++;
    for (size_t i = 0; i < rb.arg_names.size(); i++) {
      Def d;
      d.type = rb.arg_types.at(i);
      defs_[rb.arg_names[i]] = d;
      int v = new_value(d.type);
      data_[rb.arg_names[i]] = v;
      s.tile_args.push_back(v);
    }
    for (size_t i = 0; i + 1 < rb.ops.size(); i++) lower_op(*rb.ops[i]);
    for (auto &r : rb.ops.back()->operands) s.tile_yields.push_back(data_of(r));
    in_region_--;
    cur_ = saved;
    for (size_t j = 0; j < k; j++) {
      int v = new_value(op.result_types[j]);
      data_[op.results.at(j)] = v;
      s.results.push_back(v);
    }
    s.result = s.results[0];
    cur_->push_back(std::move(s));
  }

  void lower_constant(const Op &op) {
    Type t = result_type(op);
    if (!t.is_tensor && t.is_int() && !in_region_) return;  // reached through int_of on demand
    SOp s;
    s.kind = SK::Const;
    std::string lit = op.literal;
    if (t.is_tensor) {
      if (lit.rfind("dense<", 0) != 0) throw Unsupported("non-dense tensor constant");
      lit = lit.substr(6, lit.size() - 7);
      if (lit.find('[') != std::string::npos) throw Unsupported("non-splat tensor constant");
    }
    if (t.is_float()) s.fval = parse_float_literal(lit, t.elem);
    else s.ival = lit == "true" ? 1 : lit == "false" ? 0 : std::stoll(lit);
    s.result = new_value(t);
    data_[op.results[0]] = s.result;
    cur_->push_back(s);
  }

  void lower_op(const Op &op) {
    // record definitions first so later uses can find types
    if (op.name != "scf.for")
      for (size_t i = 0; i < op.results.size(); i++) {
        Def d;
        d.op = &op;
        d.index = (int)i;
        d.type = i < op.result_types.size() ? op.result_types[i] : result_type(op);
        defs_[op.results[i]] = d;
        // sibling regions may use one SSA name for different values: nothing remembered under it survives a new definition
        int_memo_.erase(op.results[i]);
        data_.erase(op.results[i]);
      }
    const std::string &n = op.name;
    if (n == "tt.return" || n == "tt.assert") return;  // assertions are dropped, as the reference does (triton_assert.mlir)
    if (n == "scf.for") return lower_for(op);
    if (n == "cf.if" || n == "scf.if") return lower_if(op);
    if (n == "tts.break_unless") {  // where a `while` leaves its loop (ttir.cpp: parse_while): an If without a body, ival = 2
      SOp s;
      s.kind = SK::If;
      s.operands.push_back(data_of(op.operands.at(0)));
      s.ival = 2;
      cur_->push_back(s);
      return;
    }
    if (n == "tt.load") return lower_load(op);
    if (n == "tt.store") return lower_store(op);
    if (n == "tt.reduce" || n == "tt.scan") return lower_reduce(op);
    if (n == "arith.constant") return lower_constant(op);
    if (n == "tt.split") {  // [.., 2] -> two blocks: one Map per half, "tt.split.0" and "tt.split.1"
      if (op.results.size() != 2) throw Unsupported("tt.split without two results (line " + std::to_string(op.line) + ")");
      const int x = data_of(op.operands.at(0));
      if (P.values[x].shape.size() != 2 || P.values[x].shape[1] != 2) throw Unsupported("tt.split of a block that is not [N, 2]");
      Type t = result_type(op);
      for (int half = 0; half < 2; half++) {
        SOp s;
        s.kind = SK::Map;
        s.name = "tt.split." + std::to_string(half);
        s.operands.push_back(x);
        s.result = new_value(t);
        data_[op.results[half]] = s.result;
        cur_->push_back(s);
      }
      return;
    }
    if (op.results.size() != 1) throw Unsupported("operation " + n + " (line " + std::to_string(op.line) + ")");
    Type rt = result_type(op);
    if (rt.ptr) {  // address computation: PtrAnalysis reads it on demand
      static const std::set<std::string> ptr_ops = {"tt.addptr", "tt.splat", "tt.broadcast", "tt.expand_dims", "tt.make_tensor_ptr", "tt.advance", "arith.select"};
      if (!ptr_ops.count(n) && !(n == "tt.bitcast" && !rt.is_tensor))
        throw Unsupported("pointer-valued operation " + n + " (line " + std::to_string(op.line) + ")");
      return;
    }
    if (!rt.is_tensor && rt.is_int() && !in_region_) {  // scalar integer: int_of reads it on demand
      static const std::set<std::string> int_ops = {
          "tt.get_program_id", "tt.get_num_programs", "arith.addi", "arith.subi", "arith.muli", "arith.divsi",
          "arith.remsi", "arith.minsi", "arith.maxsi", "arith.extsi", "arith.index_cast", "arith.trunci",
          "arith.select", "arith.cmpi"};
      // the index expressions know the ops above; any other elementwise op on scalars is computed as data when used
      if (!int_ops.count(n) && !is_elementwise(n)) throw Unsupported("scalar integer operation " + n + " (line " + std::to_string(op.line) + ")");
      return;
    }
    if (n == "tt.make_range") {
      SOp s;
      s.kind = SK::Iota;
      s.ival = std::stoll(op.attrs.at("start"));
      s.result = new_value(rt);
      data_[op.results[0]] = s.result;
      cur_->push_back(s);
      return;
    }
    if (n == "tt.splat") return emit_simple(op, SK::Splat, "", {op.operands[0]});
    if (n == "tt.broadcast") return emit_simple(op, SK::Broadcast, "", {op.operands[0]});
    if (n == "tt.expand_dims") {
      emit_simple(op, SK::ExpandDims, "", {op.operands[0]});
      cur_->back().axis = std::stoi(op.attrs.at("axis"));
      return;
    }
    if (n == "tt.dot") {  // ConversionPatterns.hpp:1128-1201
      if (op.operands.size() != 3) throw Unsupported("tt.dot without an accumulator operand");
      return emit_simple(op, SK::Dot, "", op.operands);
    }
    if (n == "tt.extern_elementwise") {  // a libdevice-style function by name (convert_extern_elementwise.mlir)
      auto it = op.attrs.find("symbol");
      if (it == op.attrs.end()) throw Unsupported("tt.extern_elementwise without a symbol (line " + std::to_string(op.line) + ")");
      std::string sym;
      for (char ch : it->second)
        if (isalnum((unsigned char)ch) || ch == '_') sym += ch;
      return emit_simple(op, SK::Map, "extern." + sym, op.operands);
    }
    if (n == "tt.cat" || n == "tt.join" || n == "tt.unsplat") {  // index shuffles of rank-1 blocks
      for (auto &o : op.operands)
        if (def(o).type.shape.size() > 1) throw Unsupported(n + " of blocks of rank > 1 (line " + std::to_string(op.line) + ")");
      return emit_simple(op, SK::Map, n, op.operands);
    }
    if (n == "tt.trans") {  // an index shuffle: a Map whose element reads another element of its operand; result dim d is operand dim order[d]
      // {order = array<i32: 1, 0>}: the numbers after the element type
      auto it = op.attrs.find("order");
      std::string order = it == op.attrs.end() ? "" : it->second, name = "tt.trans";
      const size_t colon = order.find(':');
      size_t dims = 0;
      for (char ch : order.substr(colon == std::string::npos ? 0 : colon))
        if (isdigit((unsigned char)ch)) {
          name += std::string(".") + ch;
          dims++;
        }
      if (dims != rt.shape.size() || dims > 4) throw Unsupported("tt.trans whose order does not fit its block (line " + std::to_string(op.line) + ")");
      return emit_simple(op, SK::Map, name == "tt.trans.1.0" ? "tt.trans" : name, {op.operands.at(0)});
    }
    if (n == "tt.reshape") return emit_simple(op, SK::Map, n, {op.operands.at(0)});  // row-major element order is kept
    if (is_elementwise(n)) return emit_simple(op, SK::Map, map_name(op), op.operands);
    throw Unsupported("operation " + n + " (line " + std::to_string(op.line) + ") has no structured lowering");
  }

  // A branch on a scalar condition: an early `return` (cf.cond_br to a block that only returns), an `if` around memory
  // effects, or an `if` / `else` that yields values.  Each side becomes one If op on the same condition value; with
  // results, both sides name the same result values and give their own yields.
  void lower_if(const Op &op) {
    const int cond = data_of(op.operands.at(0));
    const size_t nres = op.results.size();
    if (nres && op.regions.size() != 2) throw Unsupported("scf.if with results but without an else region");
    std::vector<int> results;
    // A scalar pointer that both sides derive from one argument is yielded as its offset from that argument, a 64-bit
    // integer like any other result; after the branch the pointer is the argument plus that value.  A block of pointers
    // is yielded the same way, as a block of 64-bit offsets, and is an unstructured address from there on.
    std::vector<int> ptr_base(nres, -1);
    for (size_t j = 0; j < nres; j++) {
      Type t = op.result_types.at(j);
      if (t.ptr) {
        if (t.block) throw Unsupported("scf.if that yields a block pointer (line " + std::to_string(op.line) + ")");
        ptr_base[j] = -2;  // the sides fill it in
        t.ptr = false;
        t.elem = "i64";
      }
      results.push_back(new_value(t));
    }
    for (int side = 0; side < 2 && side < (int)op.regions.size(); side++) {
      const Block &region = op.regions[side];
      if (region.ops.empty() && !nres) continue;
      SOp s;
      s.kind = SK::If;
      s.operands.push_back(cond);
      s.ival = side;
      s.results = results;
      std::vector<SOp> *saved = cur_;
      cur_ = &s.body;
      size_t count = region.ops.size();
      if (nres) {
        if (region.ops.empty() || region.ops.back()->name != "scf.yield" || region.ops.back()->operands.size() != nres)
          throw Unsupported("scf.if region that does not end in a yield of its results (line " + std::to_string(op.line) + ")");
        count--;
      }
      for (size_t i = 0; i < count; i++) lower_op(*region.ops[i]);
      if (nres)
        for (size_t j = 0; j < nres; j++) {
          const std::string &y = region.ops.back()->operands[j];
          if (ptr_base[j] == -1) {
            s.tile_yields.push_back(data_of(y));
            continue;
          }
          if (op.result_types[j].is_tensor) {
            Scattered u = scattered(y);
            if (ptr_base[j] >= 0 && ptr_base[j] != u.base)
              throw Unsupported("scf.if whose sides yield pointers into different arguments (line " + std::to_string(op.line) + ")");
            ptr_base[j] = u.base;
            s.tile_yields.push_back(offsets_block(u, op.result_types[j].shape));
            continue;
          }
          PtrState st = visit(y);
          if (st.rank() != 0 || st.source < 0) throw Unsupported("scf.if that yields a pointer without a base argument (line " + std::to_string(op.line) + ")");
          if (ptr_base[j] >= 0 && ptr_base[j] != st.source)
            throw Unsupported("scf.if whose sides yield pointers into different arguments (line " + std::to_string(op.line) + ")");
          ptr_base[j] = st.source;
          SOp f;
          f.kind = SK::FromIndex;
          f.expr = P.pool.to_index(st.scalar >= 0 ? st.scalar : c64(0));
          Type it;
          it.elem = "i64";
          f.result = new_value(it);
          cur_->push_back(f);
          s.tile_yields.push_back(f.result);
        }
      cur_ = saved;
      if (!s.body.empty() || nres) cur_->push_back(std::move(s));
    }
    // the results are data from here on (an integer result is not an index expression: what is computed from it is data too)
    for (size_t j = 0; j < nres; j++) {
      if (ptr_base[j] == -1) {
        data_[op.results[j]] = results[j];
        continue;
      }
      if (op.result_types[j].is_tensor) {
        Scattered after;
        after.base = ptr_base[j];
        after.scalar = c64(0);
        after.value = results[j];
        carried_scatter_[op.results[j]] = after;
        continue;
      }
      PtrState after;
      after.source = ptr_base[j];
      after.scalar = P.pool.data(results[j], 64);
      known_ptr_[op.results[j]] = after;
    }
  }

  void lower_block(const Block &b) {
    for (auto &op : b.ops) lower_op(*op);
  }

  // ------------------------------------------------------------------ DCE
  void dce() {
    std::vector<char> live(P.values.size(), 0);
    for (int e = 0; e < P.pool.size(); e++)  // what an index expression reads stays
      if (P.pool.at(e).k == EK::Data) live[P.pool.at(e).a] = 1;
    bool changed = true;
    std::function<bool(std::vector<SOp> &)> mark = [&](std::vector<SOp> &ops) {
      bool any_effect = false;
      for (auto it = ops.rbegin(); it != ops.rend(); ++it) {
        SOp &s = *it;
        auto use = [&](int v) {
          if (v >= 0 && !live[v]) {
            live[v] = 1;
            changed = true;
          }
        };
        if (s.kind == SK::Store || s.kind == SK::ScalarStore) {
          any_effect = true;
          for (int v : s.operands) use(v);
        } else if (s.kind == SK::For) {
          bool eff = mark(s.body);
          bool res_live = false;
          for (int r : s.results) res_live |= (r >= 0 && live[r]);
          if (eff || res_live) {
            any_effect |= eff;
            for (size_t j = 0; j < s.tile_args.size(); j++) {
              // a carried tile matters if its result or its region value is read
              if ((s.results[j] >= 0 && live[s.results[j]]) || live[s.tile_args[j]]) {
                use(s.tile_yields[j]);
                use(s.tile_inits[j]);
                use(s.tile_args[j]);
              }
            }
            mark(s.body);
          }
        } else if (s.kind == SK::If) {
          bool res_live = false;
          for (int r : s.results) res_live |= live[r];
          const bool eff = mark(s.body) || s.ival == 2;  // (a loop's exit is an effect: what the loop does depends on it)
          if (eff || res_live) {
            any_effect |= eff;
            for (int v : s.operands) use(v);
            if (res_live) {
              for (int r : s.results) use(r);          // both sides of the branch keep all of them
              for (int y : s.tile_yields) use(y);
              mark(s.body);
            }
          }
        } else if (!s.results.empty()) {  // a reduction or scan with a combiner region: all of it or nothing
          bool res_live = false;
          for (int r : s.results) res_live |= live[r];
          if (res_live) {
            for (int v : s.operands) use(v);
            for (int r : s.results) use(r);
          }
        } else if (s.result >= 0 && live[s.result]) {
          for (int v : s.operands) use(v);
        }
      }
      return any_effect;
    };
    while (changed) {
      changed = false;
      mark(P.body);
    }
    // Loops whose carried integers are read after them (EK::Result nodes in the index expressions of what is kept) stay
    // too, even with no block result and no effect inside: found as a fixed point over the expressions of the kept ops.
    std::set<int> need_loop;
    {
      std::vector<char> seen(P.pool.size(), 0);
      bool grew = true;
      std::function<void(int)> note = [&](int e) {
        if (e < 0 || seen[e]) return;
        seen[e] = 1;
        const Expr &x = P.pool.at(e);
        switch (x.k) {
          case EK::Const: case EK::Arg: case EK::Pid: case EK::NProg: case EK::IV: case EK::Iter: case EK::Data: return;
          case EK::Result:
            if (need_loop.insert(x.a).second) grew = true;
            return;
          default:
            note(x.a); note(x.b); note(x.c); note(x.d);
        }
      };
      std::function<bool(const std::vector<SOp> &)> scan = [&](const std::vector<SOp> &ops) {
        bool keep_any = false;
        for (auto &s : ops) {
          bool keep;
          if (s.kind == SK::Store || s.kind == SK::ScalarStore) keep = true;
          else if (s.kind == SK::For) {
            keep = scan(s.body) || need_loop.count(s.loop);
            for (int r : s.results) keep = keep || (r >= 0 && live[r]);
          } else if (s.kind == SK::If) {
            keep = scan(s.body) || s.ival == 2;
            for (int r : s.results) keep = keep || live[r];
          } else if (!s.results.empty()) keep = live[s.results[0]];
          else keep = s.result >= 0 && live[s.result];
          if (!keep) continue;
          keep_any = true;
          for (auto *list : {&s.acc.offsets, &s.acc.strides, &s.acc.dims, &s.acc.mods})
            for (int e : *list) note(e);
          note(s.expr); note(s.lb); note(s.ub); note(s.step);
          for (auto &it : s.int_iters) { note(it.init); note(it.next); }
        }
        return keep_any;
      };
      while (grew) {
        grew = false;
        scan(P.body);
      }
    }
    std::function<bool(std::vector<SOp> &)> sweep = [&](std::vector<SOp> &ops) {
      bool keep_any = false;
      std::vector<SOp> out;
      for (auto &s : ops) {
        bool keep;
        if (s.kind == SK::Store || s.kind == SK::ScalarStore) keep = true;
        else if (s.kind == SK::For) {
          bool eff = sweep(s.body);
          bool res_live = need_loop.count(s.loop) > 0;
          for (int r : s.results) res_live |= (r >= 0 && live[r]);
          keep = eff || res_live;
          if (keep) {
            // drop carried tiles nobody reads
            std::vector<int> a, i, y, r;
            for (size_t j = 0; j < s.tile_args.size(); j++)
              if (live[s.tile_args[j]] || (s.results[j] >= 0 && live[s.results[j]])) {
                a.push_back(s.tile_args[j]);
                i.push_back(s.tile_inits[j]);
                y.push_back(s.tile_yields[j]);
                r.push_back(s.results[j]);
              }
            s.tile_args = a;
            s.tile_inits = i;
            s.tile_yields = y;
            s.results = r;
          }
        } else if (s.kind == SK::If) {
          bool res_live = false;
          for (int r : s.results) res_live = res_live || live[r];
          if (!res_live) {  // nobody reads what the branch yields
            s.results.clear();
            s.tile_yields.clear();
          }
          keep = sweep(s.body) || res_live || s.ival == 2;
        }
        else if (!s.results.empty()) keep = live[s.results[0]];
        else keep = s.result >= 0 && live[s.result];
        if (keep) {
          out.push_back(std::move(s));
          keep_any = true;
        }
      }
      ops = std::move(out);
      return keep_any;
    };
    sweep(P.body);
  }
};

}  // namespace

Program lower_ttir(const Func &f) { return Lowerer(f).run(); }

}  // namespace tts
