// Symbolic integer expressions over kernel scalars, program ids and loop state.
//
// The reference keeps such values as OpFoldResult (an attribute or an SSA value)
// and folds them with the helpers of lib/Analysis/OpFoldResultUtils.cpp:178-403.
// Here they are nodes of a hash-consed DAG: two structurally equal expressions
// share one id, which lets the pattern matcher compare addresses and mask
// extents by id.  Every node has a width: 32 for i32 arithmetic (wrapping, as
// arith.* on i32 does) and 64 for `index`, the type PtrAnalysis/MaskAnalysis
// compute in after arith.index_cast.
#pragma once
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

namespace tts {

enum class EK : uint8_t {
  Const,   // val
  Arg,     // a = kernel argument index (non-constexpr scalars)
  Pid,     // a = axis
  NProg,   // a = axis
  IV,      // a = loop id (induction variable)
  Iter,    // a = loop id, b = slot (loop-carried integer, value at iteration start)
  Result,  // a = loop id, b = slot (loop-carried integer after the loop)
  Add, Sub, Mul, DivS, RemS, MinS, MaxS,
  Sext,    // i32 -> index
  Trunc,   // index/i64 -> i32
  CmpSel,  // (a pred b) ? c : d ; pred in val: 0 slt, 1 sle, 2 sgt, 3 sge, 4 eq, 5 ne
  Data,    // a = id of a scalar integer value the program computes from memory (a loaded offset, a reduced count):
           // known only on the device, so no host-side evaluation of an expression that holds one
};

struct Expr {
  EK k;
  uint8_t bits;  // 32 or 64
  int64_t val = 0;
  int a = -1, b = -1, c = -1, d = -1;
};

struct EvalEnv {
  const int64_t *args = nullptr;  // indexed by kernel argument index
  int64_t pid[3] = {0, 0, 0};
  int64_t nprog[3] = {1, 1, 1};
  std::vector<int64_t> iv;                    // by loop id
  std::vector<std::vector<int64_t>> iter;     // [loop][slot], value at iteration start
  std::vector<std::vector<int64_t>> result;   // [loop][slot], value after the loop
};

class ExprPool {
 public:
  int constant(int64_t v, int bits);
  int arg(int index, int bits);
  int pid(int axis);
  int nprog(int axis);
  int iv(int loop, int bits);
  int iter(int loop, int slot, int bits);
  int result(int loop, int slot, int bits);
  int bin(EK k, int a, int b);
  int sext(int a);
  int trunc(int a);
  int cmpsel(int pred, int a, int b, int c, int d);
  int data(int value, int bits);
  bool has_data() const;  // any Data leaf in the pool
  // index-typed helpers (operands are widened when needed)
  int to_index(int a) { return at(a).bits == 64 ? a : sext(a); }
  int add_index(int a, int b) { return bin(EK::Add, to_index(a), to_index(b)); }
  int mul_index(int a, int b) { return bin(EK::Mul, to_index(a), to_index(b)); }

  const Expr &at(int id) const { return nodes_[id]; }
  int size() const { return (int)nodes_.size(); }
  bool is_const(int id, int64_t *v = nullptr) const {
    if (nodes_[id].k != EK::Const) return false;
    if (v) *v = nodes_[id].val;
    return true;
  }
  int64_t eval(int id, const EvalEnv &env) const;
  // true if the expression reads pid/iv/iter of the given kind anywhere below it
  bool depends_on(int id, EK kind, int a = -1) const;
  std::string str(int id) const;     // readable, for diagnostics and goldens
  // raw (re)construction used by the text reader: no folding, no dedup lookup
  int push_raw(const Expr &e);

 private:
  int intern(const Expr &e);
  std::vector<Expr> nodes_;
  std::unordered_map<std::string, int> index_;
};

}  // namespace tts
