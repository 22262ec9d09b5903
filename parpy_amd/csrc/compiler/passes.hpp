// Entry points of the compiler passes, in pipeline order.
#pragma once
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "ast.hpp"
#include "sexpr.hpp"

namespace parpy {

// ---- decoration time (front.cpp)
std::unique_ptr<ParsedFun> parse_function(const std::string& sexpr,
                                          const std::map<std::string, const ParsedFun*>& tops);

// ---- call time: argument / option descriptors (specialize.cpp)
struct ArgDesc {
  enum Kind { Int, Float, Scalar, Tensor, Dict } k = Int;
  int64_t iv = 0;
  double fv = 0;
  ElemSize sz = ElemSize::F32;
  std::vector<int64_t> shape;
  std::vector<std::pair<std::string, ArgDesc>> fields;  // sorted by key
};
std::vector<ArgDesc> parse_args(const std::string& sexpr);
Options parse_options(const std::string& sexpr);

// ---- shared helpers
E fold_expr(const E& e);                 // constant folding (constfold.cpp)
Stmts fold_stmts(const Stmts& ss);       // folds expressions, prunes constant ifs, flattens scopes
E neutral_element(BinOp op, ElemSize sz, const Info& i);  // src/utils/reduce.rs:75-88

// integer interval of an expression given intervals of its free variables
struct Interval { bool known = false; int64_t lo = 0, hi = 0; };
using RangeEnv = std::map<Name, Interval>;
Interval expr_range(const E& e, const RangeEnv& env);

// Iterations per thread of a loop of `extent` iterations spread over `n` threads when the loop is printed in
// counted form (`for (k = 0; k < trips; ++k) v = tid + k*n`), -1 when it is printed as a strided loop instead.
// Counted form gives every thread the same compile-time trip count, which is what lets the memory passes keep
// per-iteration values in register arrays.  An extent that n does not divide is counted too as long as the trip
// count stays small (the last iteration is guarded by `v < hi`); long ragged loops stay strided, where the
// compiler can keep several unguarded loads in flight.
inline int64_t counted_trips(int64_t extent, int64_t n) {
  if (extent <= 0 || n <= 0) return -1;
  if (extent % n == 0) return extent / n;
  int64_t t = (extent + n - 1) / n;
  return t <= 32 ? t : -1;
}

// ---- call time pipeline
// specialise on the arguments, expand slices, type-check (specialize.cpp)
FunDef specialize(const ParsedFun& pf, const std::vector<ArgDesc>& args, const Options& opts, NameGen& gen);
// N-d indexing -> flat indexing, labels -> LoopPar, GPU contexts (lower.cpp)
FunDef lower(const FunDef& f, const Options& opts, NameGen& gen);
// synchronisation structure, kernel split, grid mapping, kernel extraction (gpu.cpp)
Program gpu_codegen(const FunDef& f, const Options& opts, NameGen& gen);
// gfx950 memory codegen: vectorised access, LDS rows, register caching, hoisting (hipopt.cpp)
void hip_optimize(Program& p, const Options& opts, NameGen& gen);
// device source text and host launch plan (hipprint.cpp)
std::string hip_print_device(const Program& p, const Options& opts);
std::string hip_print_plan(const Program& p);
// one human-readable listing (device source + host plan as pseudo launches)
std::string hip_print_listing(const Program& p, const Options& opts);

using DebugHook = std::function<void(const std::string& stage, const std::string& text)>;

}  // namespace parpy
