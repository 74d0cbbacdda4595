// Structured program: what this backend's "ttsharedir" stage holds.
//
// It carries the same information as the reference's ttshared.mlir after
// --triton-to-linalg-experimental (TritonToLinalgExperimentalPass.cpp:52-88):
//   * every block load/store as a structured access
//     {base argument, per-dim offsets/strides/sizes, per-dim valid extent, other}
//     = tts.make_tptr + tts.load / tts.store (TritonStructuredDialect.td:33-121,
//     232-298), which StructuredToMemref.cpp:528-551,794-853,1163-1196 turns into
//     reinterpret_cast + subview + copy;
//   * every compute op as a whole-tile op: elementwise map (linalg.generic),
//     fill/splat, reduce, matmul (ConversionPatterns.hpp:629-805,1128-1440);
//   * scf.for with loop-carried tiles, and loop-carried pointer state turned into
//     loop-carried index values (PtrAnalysis.cpp:1480-1602);
//   * program ids / grid sizes as free integer symbols (they are the six trailing
//     i32 arguments in the reference, TritonArithToLinalgPass.cpp:51-76).
// Integer index arithmetic lives in an ExprPool; data values are numbered tiles
// (rank 0 = scalar).
#pragma once
#include <string>
#include <vector>

#include "iexpr.h"
#include "ttir.h"

namespace tts {

struct Value {           // a data value: tile or scalar
  std::vector<int64_t> shape;
  std::string dtype;     // f32, f16, bf16, i1, i8, i32, i64 ...
};

enum class SK {
  Load,        // structured block load
  Store,       // structured block store; operands[0] = value
  ScalarLoad,  // base[offset] -> scalar (UnstructuredToMemrefPass.cpp:71-113)
  ScalarStore, // base[offset] = operands[0] (UnstructuredToMemrefPass.cpp:115-158)
  Map,         // elementwise op `name` over operands (linalg.generic, parallel)
  Splat,       // scalar operand -> tile (linalg.fill)
  Const,       // dense splat constant (linalg.fill of a constant)
  Iota,        // tt.make_range as data: start + i (linalg.generic with linalg.index)
  FromIndex,   // integer expression -> i32/i64 scalar data value
  ScalarArg,   // floating-point kernel argument as a scalar data value; ival = argument index
  Reduce,      // linalg.reduce over `axis` with combiner `name`
  Scan,        // inclusive scan along `axis` (tt.scan, ttx.cumsum for addf); ival = 1 when reversed
  Dot,         // linalg.matmul(a,b) then + c
  ExpandDims,  // tensor.expand_shape
  Broadcast,   // linalg.generic broadcast
  For,         // scf.for
  If,          // body runs iff the scalar i1 operand is true (false when ival = 1); no results (cf.cond_br trees, scf.if).
               // ival = 2, no body: the enclosing loop ends here unless the operand is true (scf.while's scf.condition)
};

struct Access {          // the tts.make_tptr + mask part of a load/store
  int base_arg = -1;                 // kernel argument index of the base pointer
  std::string elem;                  // pointee type
  std::vector<int64_t> sizes;        // block shape
  std::vector<int> offsets;          // per-dim, already multiplied by the stride (index exprs)
  std::vector<int> strides;          // per-dim (index exprs)
  std::vector<int> dims;             // per-dim valid extent (index exprs); empty = unmasked
  std::vector<int> mods;             // per-dim wraparound period (index exprs, in elements, -1 = none); empty = no wraparound:
                                     // dim d at index j contributes (offsets[d] + j * strides[d]) mod mods[d] to the address
                                     // (tts.make_tptr `shape`, TritonStructuredDialect.td:33-121; StructuredToMemref.cpp:263-487)
  // Unstructured (gather / scatter) access, used when the address is not an affine block: element e is at
  // base[offsets[0] + value(gather)[e]] and is valid iff value(mask_value)[e] (tts.make_gather_scatter_tptr,
  // StructuredToMemref.cpp:855-993,1034-1157, restated per element).  sizes is the block shape; strides/dims unused.
  int gather = -1;                   // value id of the integer offset tile, or -1 for a structured access
  int mask_value = -1;               // value id of the i1 mask tile, or -1
  bool has_other = false;
  double other_f = 0;                // value of `other` when the element type is a float
  int64_t other_i = 0;               // ... when it is an integer
  int other_value = -1;              // value id (a scalar, or a block of the access's shape) when `other` is not a constant
};

struct IntIter {         // loop-carried integer (offset or stride of a carried pointer, or an i32)
  int iter_expr = -1;    // the EK::Iter node
  int init = -1;
  int next = -1;         // value yielded, in terms of iter_expr / iv
  int result_expr = -1;  // the EK::Result node
};

struct SOp {
  SK kind;
  std::string name;              // Map: arith/math op (+predicate), Reduce: combiner, Const: literal
  int result = -1;               // value id; For uses results[]
  std::vector<int> operands;     // value ids
  Access acc;                    // Load/Store/ScalarLoad/ScalarStore
  int axis = 0;                  // Reduce / ExpandDims
  int64_t ival = 0;              // Iota start; Const integer payload
  double fval = 0;               // Const float payload
  int expr = -1;                 // FromIndex
  // For
  int loop = -1;
  int lb = -1, ub = -1, step = -1;   // i32 exprs
  std::vector<IntIter> int_iters;
  std::vector<int> tile_args;        // region values standing for carried tiles
  std::vector<int> tile_inits;       // value ids
  std::vector<int> tile_yields;      // value ids (inside body)
  std::vector<int> results;          // value ids after the loop (parallel to tile_args)
  std::vector<SOp> body;
  // Reduce / Scan whose combiner is more than one op of the two block arguments (argmin / argmax, ConversionPatterns.hpp:
  // 1443-1769), or that take several operands: name = "region"; operands = the k input blocks; results = the k results
  // (result = results[0]); tile_args = the 2k scalar region arguments (k left, then k right); body = the combiner's
  // scalar ops; tile_yields = the k values it returns.  Every Scan has this form.
};

struct Program {
  std::string name;
  std::vector<std::string> arg_names;
  std::vector<Type> arg_types;       // pointers and scalars, in kernel-argument order
  ExprPool pool;
  std::vector<Value> values;
  std::vector<SOp> body;
  int num_loops = 0;
};

// TTIR -> structured program (PtrAnalysis + MaskAnalysis + op lowering restated).
Program lower_ttir(const Func &f);

// Text form (the ttsharedir artefact) and its reader.
std::string print_program(const Program &p);
Program read_program(const std::string &text);

}  // namespace tts
