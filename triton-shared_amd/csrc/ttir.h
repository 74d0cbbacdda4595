// TTIR text reader.
//
// The reference hands the Triton IR to its middle layer as text
// (backend/compiler.py:48-67: str(mod) -> tt.mlir -> subprocess).  This backend
// consumes the same text.  What is understood: the MLIR custom assembly that the
// TTIR pass list of backend/compiler.py:244-260 prints, and the hand-written forms
// of the reference's conversion tests (signatures over several lines, generic-form
// tt.reduce, loops without a type suffix); anything else raises tts::Unsupported so
// the caller can refuse the kernel instead of guessing.
#pragma once
#include <cstdint>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace tts {

struct Unsupported : std::runtime_error {
  using std::runtime_error::runtime_error;
};

// A TTIR type: scalar (shape empty, is_tensor false) or ranked tensor.
// elem is "i1","i8","i16","i32","i64","f16","bf16","f32","f64","index";
// ptr is true for !tt.ptr<elem> (scalar) or tensor<...x!tt.ptr<elem>>.
struct Type {
  std::vector<int64_t> shape;
  bool is_tensor = false;
  bool ptr = false;
  bool block = false;  // !tt.ptr<tensor<...>>: one pointer to a block (tt.make_tensor_ptr), not a block of pointers
  std::string elem;
  bool is_int() const { return !ptr && (elem[0] == 'i'); }
  bool is_float() const { return !ptr && (elem[0] == 'f' || elem[0] == 'b'); }
  int64_t numel() const {
    int64_t n = 1;
    for (auto s : shape) n *= s;
    return n;
  }
  std::string str() const;
};

Type parse_type(const std::string &s);

struct Op;
struct Block {
  std::vector<std::string> arg_names;  // region block arguments (%x)
  std::vector<Type> arg_types;
  std::vector<std::unique_ptr<Op>> ops;
};

struct Op {
  std::string name;                      // e.g. "arith.addi", "tt.load", "scf.for"
  std::vector<std::string> results;      // SSA names, "%a" or "%a#1" for packs
  std::vector<Type> result_types;
  std::vector<std::string> operands;     // SSA names in textual order
  std::vector<std::string> words;        // bare identifiers (cmpi predicate, pid axis)
  std::map<std::string, std::string> attrs;  // {key = value : type} dictionaries
  std::vector<Type> types;               // everything after the type colon
  std::string literal;                   // arith.constant payload
  // scf.for
  std::string iv;
  std::vector<std::string> iter_names;   // region iter-arg names
  std::vector<std::string> iter_inits;
  std::vector<Block> regions;
  int line = 0;
};

struct Func {
  std::string name;
  std::vector<std::string> arg_names;
  std::vector<Type> arg_types;
  std::vector<Type> result_types;  // of a callee; a kernel has none
  Block body;
};

// Parses one module: exactly one public tt.func (the kernel) and any number of private ones, whose calls (tt.call, from
// functions the front end kept out of line) are inlined into the kernel.  A function body that is a graph of basic
// blocks (early returns) comes back as a tree of "cf.if" ops.
Func parse_ttir(const std::string &text);

}  // namespace tts
