// Integer expression pool: construction with the folding shortcuts of
// lib/Analysis/OpFoldResultUtils.cpp:178-350 (x+0, x-0, x*0, x*1, constant
// folding, signed min/max), evaluation and printing.
#include "iexpr.h"

#include <stdexcept>

namespace tts {

static int64_t wrap(int64_t v, int bits) {
  if (bits == 32) return (int64_t)(int32_t)(uint32_t)(uint64_t)v;
  return v;
}

int ExprPool::intern(const Expr &e) {
  std::string key;
  key.reserve(48);
  key += std::to_string((int)e.k) + ":" + std::to_string((int)e.bits) + ":" + std::to_string(e.val) + ":" +
         std::to_string(e.a) + ":" + std::to_string(e.b) + ":" + std::to_string(e.c) + ":" + std::to_string(e.d);
  auto it = index_.find(key);
  if (it != index_.end()) return it->second;
  nodes_.push_back(e);
  int id = (int)nodes_.size() - 1;
  index_[key] = id;
  return id;
}

int ExprPool::push_raw(const Expr &e) { return intern(e); }

int ExprPool::constant(int64_t v, int bits) {
  Expr e{EK::Const, (uint8_t)bits};
  e.val = wrap(v, bits);
  return intern(e);
}
int ExprPool::arg(int index, int bits) {
  Expr e{EK::Arg, (uint8_t)bits};
  e.a = index;
  return intern(e);
}
int ExprPool::pid(int axis) {
  Expr e{EK::Pid, 32};
  e.a = axis;
  return intern(e);
}
int ExprPool::nprog(int axis) {
  Expr e{EK::NProg, 32};
  e.a = axis;
  return intern(e);
}
int ExprPool::iv(int loop, int bits) {
  Expr e{EK::IV, (uint8_t)bits};
  e.a = loop;
  return intern(e);
}
int ExprPool::iter(int loop, int slot, int bits) {
  Expr e{EK::Iter, (uint8_t)bits};
  e.a = loop;
  e.b = slot;
  return intern(e);
}
int ExprPool::result(int loop, int slot, int bits) {
  Expr e{EK::Result, (uint8_t)bits};
  e.a = loop;
  e.b = slot;
  return intern(e);
}

static int64_t apply(EK k, int64_t x, int64_t y, int bits) {
  switch (k) {
    case EK::Add: return wrap((int64_t)((uint64_t)x + (uint64_t)y), bits);
    case EK::Sub: return wrap((int64_t)((uint64_t)x - (uint64_t)y), bits);
    case EK::Mul: return wrap((int64_t)((uint64_t)x * (uint64_t)y), bits);
    case EK::DivS:
      if (y == 0) throw std::runtime_error("integer division by zero in a kernel scalar expression");
      if (y == -1) return wrap((int64_t)(0 - (uint64_t)x), bits);
      return x / y;  // C++ truncates toward zero, as arith.divsi does
    case EK::RemS:
      if (y == 0) throw std::runtime_error("integer remainder by zero in a kernel scalar expression");
      if (y == -1) return 0;
      return x % y;
    case EK::MinS: return x < y ? x : y;
    case EK::MaxS: return x > y ? x : y;
    default: throw std::logic_error("apply: not a binary kind");
  }
}

int ExprPool::bin(EK k, int a, int b) {
  const Expr ea = at(a), eb = at(b);
  if (ea.bits != eb.bits) throw std::logic_error("iexpr: width mismatch in binary op");
  int bits = ea.bits;
  bool ca = ea.k == EK::Const, cb = eb.k == EK::Const;
  if (ca && cb && !((k == EK::DivS || k == EK::RemS) && eb.val == 0))
    return constant(apply(k, ea.val, eb.val, bits), bits);
  if (k == EK::Add) {
    if (cb && eb.val == 0) return a;
    if (ca && ea.val == 0) return b;
  } else if (k == EK::Sub) {
    if (cb && eb.val == 0) return a;
    if (a == b) return constant(0, bits);
  } else if (k == EK::Mul) {
    if (ca && ea.val == 0) return a;
    if (ca && ea.val == 1) return b;
    if (cb && eb.val == 0) return b;
    if (cb && eb.val == 1) return a;
  } else if (k == EK::MinS || k == EK::MaxS) {
    if (a == b) return a;
  }
  // commutative kinds get a canonical operand order so that a+b and b+a share an id
  if ((k == EK::Add || k == EK::Mul || k == EK::MinS || k == EK::MaxS) && a > b) std::swap(a, b);
  Expr e{k, (uint8_t)bits};
  e.a = a;
  e.b = b;
  return intern(e);
}

int ExprPool::sext(int a) {
  const Expr ea = at(a);
  if (ea.bits == 64) return a;
  if (ea.k == EK::Const) return constant(ea.val, 64);
  Expr e{EK::Sext, 64};
  e.a = a;
  return intern(e);
}

int ExprPool::trunc(int a) {
  const Expr ea = at(a);
  if (ea.bits == 32) return a;
  if (ea.k == EK::Const) return constant(ea.val, 32);
  if (ea.k == EK::Sext) return ea.a;
  Expr e{EK::Trunc, 32};
  e.a = a;
  return intern(e);
}

static bool cmp(int pred, int64_t x, int64_t y) {
  switch (pred) {
    case 0: return x < y;
    case 1: return x <= y;
    case 2: return x > y;
    case 3: return x >= y;
    case 4: return x == y;
    case 5: return x != y;
  }
  throw std::logic_error("bad predicate");
}

int ExprPool::cmpsel(int pred, int a, int b, int c, int d) {
  const Expr ea = at(a), eb = at(b);
  if (ea.bits != eb.bits || at(c).bits != at(d).bits) throw std::logic_error("iexpr: width mismatch in select");
  if (ea.k == EK::Const && eb.k == EK::Const) return cmp(pred, ea.val, eb.val) ? c : d;
  if (c == d) return c;
  Expr e{EK::CmpSel, at(c).bits};
  e.val = pred;
  e.a = a;
  e.b = b;
  e.c = c;
  e.d = d;
  return intern(e);
}

int ExprPool::data(int value, int bits) {
  Expr e{EK::Data, (uint8_t)bits};
  e.a = value;
  return intern(e);
}

bool ExprPool::has_data() const {
  for (auto &e : nodes_)
    if (e.k == EK::Data) return true;
  return false;
}

int64_t ExprPool::eval(int id, const EvalEnv &env) const {
  const Expr &e = nodes_[id];
  switch (e.k) {
    case EK::Data: throw std::runtime_error("an index expression that depends on data has no value on the host");
    case EK::Const: return e.val;
    case EK::Arg: return wrap(env.args[e.a], e.bits);
    case EK::Pid: return env.pid[e.a];
    case EK::NProg: return env.nprog[e.a];
    case EK::IV: return env.iv.at(e.a);
    case EK::Iter: return env.iter.at(e.a).at(e.b);
    case EK::Result: return env.result.at(e.a).at(e.b);
    case EK::Sext: return eval(e.a, env);
    case EK::Trunc: return wrap(eval(e.a, env), 32);
    case EK::CmpSel: return cmp((int)e.val, eval(e.a, env), eval(e.b, env)) ? eval(e.c, env) : eval(e.d, env);
    default: return apply(e.k, eval(e.a, env), eval(e.b, env), e.bits);
  }
}

bool ExprPool::depends_on(int id, EK kind, int a) const {
  const Expr &e = nodes_[id];
  if (e.k == kind && (a < 0 || e.a == a)) return true;
  switch (e.k) {
    case EK::Const: case EK::Arg: case EK::Pid: case EK::NProg: case EK::IV: case EK::Iter: case EK::Result: case EK::Data:
      return false;
    case EK::Sext: case EK::Trunc: return depends_on(e.a, kind, a);
    case EK::CmpSel:
      return depends_on(e.a, kind, a) || depends_on(e.b, kind, a) || depends_on(e.c, kind, a) ||
             depends_on(e.d, kind, a);
    default: return depends_on(e.a, kind, a) || depends_on(e.b, kind, a);
  }
}

std::string ExprPool::str(int id) const {
  const Expr &e = nodes_[id];
  auto two = [&](const char *op) { return "(" + str(e.a) + " " + op + " " + str(e.b) + ")"; };
  static const char *axes = "xyz";
  switch (e.k) {
    case EK::Const: return std::to_string(e.val);
    case EK::Arg: return "arg" + std::to_string(e.a);
    case EK::Pid: return std::string("pid.") + axes[e.a];
    case EK::NProg: return std::string("nprog.") + axes[e.a];
    case EK::IV: return "iv" + std::to_string(e.a);
    case EK::Iter: return "it" + std::to_string(e.a) + "." + std::to_string(e.b);
    case EK::Result: return "res" + std::to_string(e.a) + "." + std::to_string(e.b);
    case EK::Data: return "value" + std::to_string(e.a);
    case EK::Add: return two("+");
    case EK::Sub: return two("-");
    case EK::Mul: return two("*");
    case EK::DivS: return two("/");
    case EK::RemS: return two("%");
    case EK::MinS: return "min(" + str(e.a) + ", " + str(e.b) + ")";
    case EK::MaxS: return "max(" + str(e.a) + ", " + str(e.b) + ")";
    case EK::Sext: return str(e.a);
    case EK::Trunc: return "i32(" + str(e.a) + ")";
    case EK::CmpSel: {
      static const char *ps[] = {"<", "<=", ">", ">=", "==", "!="};
      return "(" + str(e.a) + " " + ps[e.val] + " " + str(e.b) + " ? " + str(e.c) + " : " + str(e.d) + ")";
    }
  }
  return "?";
}

}  // namespace tts
