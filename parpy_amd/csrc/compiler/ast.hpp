// AST shared by every pass of the compiler core.
//
// One expression / statement family is used from the parsed Python-like tree
// down to the per-kernel device code; passes refine it in place of the four
// separate ASTs (py -> ir -> gpu -> target) of the reference
// (src/py/ast.rs, src/ir/ast.rs, src/gpu/ast.rs, src/cuda/ast.rs).  Nodes are
// immutable once built and shared through shared_ptr; passes rebuild what
// they change.
#pragma once
#include <cmath>
#include <cstdint>
#include <map>
#include <memory>
#include <set>
#include <stdexcept>
#include <string>
#include <vector>

namespace parpy {

constexpr int64_t WAVE_SIZE = 64;      // CDNA wavefront width (reference: WARP_SIZE = 32, src/gpu/par.rs:18)
constexpr int64_t DEFAULT_TPB = 1024;  // src/par.rs:7
constexpr int64_t MAX_GRID_YZ = 65535; // src/gpu/par.rs:284-305
constexpr const char* REDUCE_PAR_LABEL = "_reduce";

// ---------------------------------------------------------------- errors
enum class ErrKind { Runtime = 0, Type = 1, Name = 2 };  // src/utils/err.rs:79-87

struct Info {
  int l0 = 0, c0 = 0, l1 = 0, c1 = 0;
  bool valid() const { return l0 > 0; }
  static Info merge(const Info& a, const Info& b) {
    if (!a.valid()) return b;
    if (!b.valid()) return a;
    Info r = a;
    if (b.l0 < r.l0 || (b.l0 == r.l0 && b.c0 < r.c0)) { r.l0 = b.l0; r.c0 = b.c0; }
    if (b.l1 > r.l1 || (b.l1 == r.l1 && b.c1 > r.c1)) { r.l1 = b.l1; r.c1 = b.c1; }
    return r;
  }
};

struct CompileError : std::runtime_error {
  ErrKind kind;
  Info info;
  CompileError(ErrKind k, const Info& i, const std::string& msg)
      : std::runtime_error(msg), kind(k), info(i) {}
};

[[noreturn]] inline void fail(ErrKind k, const Info& i, const std::string& msg) {
  throw CompileError(k, i, msg);
}
[[noreturn]] inline void fail_rt(const Info& i, const std::string& m) { fail(ErrKind::Runtime, i, m); }
[[noreturn]] inline void fail_ty(const Info& i, const std::string& m) { fail(ErrKind::Type, i, m); }
[[noreturn]] inline void fail_name(const Info& i, const std::string& m) { fail(ErrKind::Name, i, m); }

// ---------------------------------------------------------------- types
enum class ElemSize { Bool, I8, I16, I32, I64, U8, U16, U32, U64, F16, F32, F64 };

inline bool is_signed(ElemSize s) { return s >= ElemSize::I8 && s <= ElemSize::I64; }
inline bool is_unsigned(ElemSize s) { return s >= ElemSize::U8 && s <= ElemSize::U64; }
inline bool is_int(ElemSize s) { return is_signed(s) || is_unsigned(s); }
inline bool is_float(ElemSize s) { return s >= ElemSize::F16; }
inline int elem_bytes(ElemSize s) {
  switch (s) {
    case ElemSize::Bool: case ElemSize::I8: case ElemSize::U8: return 1;
    case ElemSize::I16: case ElemSize::U16: case ElemSize::F16: return 2;
    case ElemSize::I32: case ElemSize::U32: case ElemSize::F32: return 4;
    default: return 8;
  }
}
const char* elem_tag(ElemSize s);             // "f32", "i64", ...
const char* elem_pyname(ElemSize s);          // "float32", ...
const char* elem_ctype(ElemSize s);           // "float", "int64_t", ...
bool parse_elem_tag(const std::string& t, ElemSize* out);

enum class Mem { Global = 0, LDS = 1 };

struct Type {
  enum Kind { Unknown, Void, Tensor, Pointer, Dict, Str, Tuple } k = Unknown;
  ElemSize sz = ElemSize::F32;
  std::vector<int64_t> shape;                        // Tensor; empty = scalar
  Mem mem = Mem::Global;                             // Pointer
  std::vector<std::pair<std::string, Type>> fields;  // Dict, sorted by key
  std::vector<Type> elems;                           // Tuple

  static Type scalar(ElemSize s) { Type t; t.k = Tensor; t.sz = s; return t; }
  static Type tensor(ElemSize s, std::vector<int64_t> sh) { Type t; t.k = Tensor; t.sz = s; t.shape = std::move(sh); return t; }
  static Type pointer(ElemSize s, Mem m = Mem::Global) { Type t; t.k = Pointer; t.sz = s; t.mem = m; return t; }
  static Type vvoid() { Type t; t.k = Void; return t; }
  bool is_scalar() const { return k == Tensor && shape.empty(); }
  bool is_array() const { return k == Tensor && !shape.empty(); }
  bool is_pointer() const { return k == Pointer; }
  int64_t numel() const { int64_t n = 1; for (auto d : shape) n *= d; return n; }
  bool operator==(const Type& o) const;
  bool operator!=(const Type& o) const { return !(*this == o); }
  std::string str() const;
};

// ---------------------------------------------------------------- operators
enum class UnOp { Sub, Not, BitNeg, Exp, Log, Cos, Sin, Sqrt, Tanh, Abs };
enum class BinOp {
  Add, Sub, Mul, Div, FloorDiv, Rem, Pow, And, Or, BitAnd, BitOr, BitXor, BitShl, BitShr,
  Eq, Neq, Leq, Geq, Lt, Gt, Max, Min, Atan2
};
enum class Builtin {
  Exp, Inf, Log, Min, Max, Abs, Cos, Sin, Sqrt, Tanh, Atan2, Sum, Prod, Convert, Label, Gpu
};
const char* unop_name(UnOp);
const char* binop_name(BinOp);
bool is_compare(BinOp op);

// ---------------------------------------------------------------- names
struct Name {
  std::string s;
  int64_t id = 0;  // 0 = not yet symbolised
  bool operator==(const Name& o) const { return id == o.id && s == o.s; }
  bool operator!=(const Name& o) const { return !(*this == o); }
  bool operator<(const Name& o) const { return id != o.id ? id < o.id : s < o.s; }
  std::string str() const { return id ? s + "_" + std::to_string(id) : s; }
};

struct NameGen {
  int64_t next = 1;
  Name fresh(const std::string& s) { return Name{s, next++}; }
};

// ---------------------------------------------------------------- expressions
struct Expr;
using E = std::shared_ptr<const Expr>;
struct FunDef;

// Signature of an externally defined device function (parpy.external): what a call site needs to
// type its arguments and what the printer needs to emit the call and the include.
struct ExtSig {
  std::string py_name, name, header;
  std::vector<Type> params;
  Type ret;
  int backend = 3;          // Backend the declaration was made for (as the enum's integer value)
  int64_t par_threads = 0;  // > 0: the function is executed by that many threads of a workgroup together
};

struct Expr {
  enum Kind {
    Var, Int, Float, Bool, Str, UnOpE, BinOpE, IfExpr, Subscript, Slice, Tuple, BuiltinE, Call,
    Convert, NeutralElement,
    // after lowering
    Index,      // args[0] = base (pointer/array var expression), args[1] = flat index
    AddrOf,     // &args[0][args[1]]
    ThreadIdx, BlockIdx,  // dim in iv (0=x,1=y,2=z)
    RegElem,    // register-array element: name = array var, args[0] = constant index expr
    Raw         // verbatim target text in sval (used by target-specific lowering)
  } k = Var;
  Type ty;
  Info i;
  Name name;              // Var / RegElem
  std::string sval;       // Str value / Call function / Raw text
  int64_t iv = 0;         // Int value / axis / dim
  double fv = 0;          // Float value
  bool bv = false;        // Bool value; Slice: unused
  bool has_axis = false;  // BuiltinE
  UnOp uop = UnOp::Sub;
  BinOp bop = BinOp::Add;
  Builtin fn = Builtin::Exp;
  std::vector<E> args;    // children; Slice: args[0]=lo or null, args[1]=hi or null
  // Index/AddrOf only: the per-dimension indices the flat index was built from
  // and the shape of the indexed array (kept for the row-structure analyses of
  // the HIP memory passes).
  std::vector<E> dim_idx;
  std::vector<int64_t> dim_shape;
  std::shared_ptr<const ExtSig> ext;  // Call only: the external the call refers to
  // Call only, when calls of jitted functions inside expressions are kept (device_functions option): before type
  // checking the callee as parsed, afterwards its instance for the argument types of this call
  std::shared_ptr<const FunDef> callee;
};

E mk_var(const Name& n, const Type& ty, const Info& i = Info());
E mk_int(int64_t v, ElemSize sz = ElemSize::I64, const Info& i = Info());
E mk_float(double v, ElemSize sz = ElemSize::F64, const Info& i = Info());
E mk_bool(bool v, const Info& i = Info());
E mk_unop(UnOp op, E a, const Type& ty, const Info& i = Info());
E mk_binop(BinOp op, E a, E b, const Type& ty, const Info& i = Info());
E mk_convert(E a, ElemSize sz);
E mk_index(E base, E idx, const Type& elem_ty, const Info& i = Info());
E mk_raw(const std::string& text, const Type& ty);
E mk_ifexpr(E c, E a, E b, const Type& ty, const Info& i = Info());
E with_type(const E& e, const Type& ty);
// structural equality ignoring Info
bool expr_eq(const E& a, const E& b);
// rebuild with children mapped through f
template <class F> E map_children(const E& e, F f) {
  bool changed = false;
  std::vector<E> na;
  na.reserve(e->args.size());
  for (auto& a : e->args) {
    E n = a ? f(a) : a;
    if (n != a) changed = true;
    na.push_back(n);
  }
  std::vector<E> nd;
  nd.reserve(e->dim_idx.size());
  for (auto& a : e->dim_idx) {
    E n = f(a);
    if (n != a) changed = true;
    nd.push_back(n);
  }
  if (!changed) return e;
  auto r = std::make_shared<Expr>(*e);
  r->args = std::move(na);
  r->dim_idx = std::move(nd);
  return r;
}

// ---------------------------------------------------------------- loop parallelism
struct LoopPar {  // src/par.rs:11-91
  int64_t nthreads = 0;
  bool reduction = false;
  int64_t tpb = DEFAULT_TPB;
  bool is_parallel() const { return nthreads > 0; }
  bool operator==(const LoopPar& o) const { return nthreads == o.nthreads && reduction == o.reduction && tpb == o.tpb; }
  // src/par.rs:83-91; returns false when the two specs conflict
  bool try_merge(const LoopPar& o);
  std::string str() const;
};

// ---------------------------------------------------------------- statements
struct Stmt;
using S = std::shared_ptr<const Stmt>;
using Stmts = std::vector<S>;

enum class SyncKind { BlockLocal, InterBlock };

struct Dim3 { int64_t x = 1, y = 1, z = 1; };

// How a parallel loop's iterations are laid onto the grid (filled by the grid mapper).
struct GpuMap {
  enum Kind { None, Thread, Block, ThreadBlock } k = None;
  int dim = 0;            // 0=x 1=y 2=z
  int64_t n = 0;          // Thread: #threads; Block: #blocks; ThreadBlock: #threads total
  int64_t tpb = 0;        // ThreadBlock: threads per block
  int64_t mult = 1;       // Block: divisor when several loops share one grid dimension
};

struct Stmt {
  enum Kind {
    Def,        // id : ty = expr
    Assign,     // dst = expr
    For,        // for id in lo..hi step: body  (labels / par)
    While,      // while expr: body
    If,         // if expr: body else els
    WithGpu,    // with gpu: body
    CallStmt,   // fname(args)
    Label,      // fname = label text
    Return,     // return expr
    // GPU structure
    SyncPoint,  // marks the end of a parallel loop; sync = kind
    Sync,       // __syncthreads()
    Alloc,      // id = device allocation of iv elements of type ty.sz
    Free,       // free id
    Launch,     // kernel launch: fname, grid/block, args
    PersistentLaunch,  // one launch of kernel fname that runs a whole host loop of launches (kept in body) with barriers between workgroups (iv = counters they need)
    Scope,      // { body }; with args: the pointer variables in args do not alias each other inside
    WaveReduce, // id = wave_reduce<bop>(id)
    LdsDecl,    // __shared__ ty.sz id[iv]
    RegDecl,    // ty.sz id[iv] (per-thread register array)
    RawStmt     // verbatim text in fname
  } k = Def;
  Info i;
  Name id;
  Type ty;
  E dst, expr, lo, hi;
  int64_t step = 1;
  int64_t iv = 0;
  Stmts body, els;
  std::vector<std::string> labels;
  LoopPar par;
  GpuMap map;
  SyncKind sync = SyncKind::InterBlock;
  BinOp bop = BinOp::Add;
  std::string fname;
  std::vector<E> args;
  Dim3 grid, block;
  bool unroll = false;    // For: emit an unroll pragma
};

S mk_def(const Name& id, const Type& ty, E expr, const Info& i = Info());
S mk_assign(E dst, E expr, const Info& i = Info());
S mk_for(const Name& id, E lo, E hi, int64_t step, Stmts body, const LoopPar& par, const Info& i = Info());
S mk_if(E cond, Stmts thn, Stmts els, const Info& i = Info());
S mk_sync();
S mk_scope(Stmts body);
S mk_rawstmt(const std::string& text);

template <class F> S map_body(const S& s, F f) {  // f : Stmts -> Stmts
  if (s->body.empty() && s->els.empty()) return s;
  auto r = std::make_shared<Stmt>(*s);
  r->body = f(s->body);
  r->els = f(s->els);
  return r;
}
// map every expression directly held by the statement (not those of nested statements)
template <class F> S map_exprs(const S& s, F f) {
  auto r = std::make_shared<Stmt>(*s);
  if (r->dst) r->dst = f(r->dst);
  if (r->expr) r->expr = f(r->expr);
  if (r->lo) r->lo = f(r->lo);
  if (r->hi) r->hi = f(r->hi);
  for (auto& a : r->args) a = f(a);
  return r;
}
// apply f to all expressions in the statement tree (deep)
template <class F> S map_exprs_deep(const S& s, F f) {
  auto r = std::const_pointer_cast<Stmt>(std::static_pointer_cast<const Stmt>(map_exprs(s, f)));
  for (auto& b : r->body) b = map_exprs_deep(b, f);
  for (auto& b : r->els) b = map_exprs_deep(b, f);
  return r;
}
template <class F> void visit_exprs(const E& e, F f) {
  if (!e) return;
  f(e);
  for (auto& a : e->args) visit_exprs(a, f);
}
template <class F> void visit_stmt_exprs(const S& s, F f) {  // deep, pre-order
  visit_exprs(s->dst, f);
  visit_exprs(s->expr, f);
  visit_exprs(s->lo, f);
  visit_exprs(s->hi, f);
  for (auto& a : s->args) visit_exprs(a, f);
  for (auto& b : s->body) visit_stmt_exprs(b, f);
  for (auto& b : s->els) visit_stmt_exprs(b, f);
}
template <class F> void visit_stmts(const Stmts& ss, F f) {  // deep, pre-order
  for (auto& s : ss) {
    f(s);
    visit_stmts(s->body, f);
    visit_stmts(s->els, f);
  }
}

// ---------------------------------------------------------------- functions / program
struct Param {
  Name id;
  Type ty;
  Info i;
};

struct FunDef {
  Name id;
  std::vector<Param> params;
  Stmts body;
  Type res_ty;
  Info i;
  // functions called inside expressions that stay functions on the device (device_functions option): one typed
  // instance per callee and argument types, callees before their callers
  std::vector<std::shared_ptr<const FunDef>> device_funs;
};

// Function as parsed at decoration time: untyped, labels attached, callees inlined.
struct ParsedFun {
  std::shared_ptr<const ExtSig> ext;  // set for an external declaration (fun then only carries the name)
  FunDef fun;
  NameGen gen;
  // the same function with the calls of jitted functions inside expressions kept as calls (statement calls are
  // inlined in both): what the device_functions option compiles
  FunDef fun_calls;
  NameGen gen_calls;
  // set when the function can only be compiled with its callees as functions (a callee returns from inside a loop):
  // reported when it is compiled without the device_functions option
  std::shared_ptr<const CompileError> inline_error;
  std::string source_text;  // printable form, used for cache keys
};

// ---------------------------------------------------------------- options
enum class Backend { Auto, Cuda, Metal, Hip };

struct Options {  // src/option.rs:14-108
  std::map<std::string, LoopPar> parallelize;
  bool debug_print = false;
  Backend backend = Backend::Hip;
  bool use_graphs = false;
  bool device_functions = false;  // jitted functions called inside expressions become device functions instead of being inlined
  bool persistent_loops = false;  // host loops of launches run inside one kernel, steps separated by a barrier over all workgroups
  bool has_force_int = false, has_force_float = false;
  ElemSize force_int = ElemSize::I64, force_float = ElemSize::F64;
  std::vector<std::string> includes;
  // HIP memory-codegen switches (all on by default; tests and benchmarks turn
  // them off individually to measure what each one buys)
  bool opt_vectorize = true;
  bool opt_lds_rows = true;
  bool opt_reg_cache = true;
  bool opt_hoist_invariant = true;
  bool opt_narrow_index = true;
  bool opt_mfma_sddmm = false;  // per-thread dot products on the matrix cores (4x4x1 tiles): measured slower, opt-in
  bool opt_unswitch = false;   // measured slower on the HMM kernels (higher register pressure): opt-in
  bool opt_gather_transpose = true;
  bool opt_noalias_scopes = false; // aliases that always name different arrays are declared not to alias; measured slower on the HMM kernels: opt-in
  bool opt_unswitch_uniform = true; // `for x: if (uniform) A else B` -> `if (uniform) for x: A else for x: B`
  bool opt_offset32 = true;         // global elements at base + 32-bit byte offset when the offset provably fits
  bool opt_if_convert = true;       // branches that only assign cheap scalar values become selects
  bool opt_drop_barriers = true;   // barriers between regions that share no written array are removed
  bool opt_lane_split = true;      // eight lanes share each long per-thread dot product
  bool opt_nontemporal = true;   // non-temporal stores to arrays a kernel only writes
  bool opt_guard_bounds = true;       // `for t: if t < X: work` with X fixed and uniform runs to min(hi, X) without the test
  bool opt_prefetch_steps = true;     // loads indexed by the counter of a barrier-stepped loop are issued one step ahead
  bool opt_pack_accesses = true;      // four adjacent 4-byte accesses of one iteration become one 16-byte access
  bool opt_share_iterations = true;   // what all iterations of one thread have in common is evaluated once per thread
  bool opt_keep_own = false;     // ... and across steps when source and destination swap every step (own elements never re-read from LDS)
  bool opt_keep_stored = true;   // values a thread stores and reads back itself later in the same step stay in registers
  bool opt_fence_iterations = true;   // the unrolled iterations of a thread that read and write LDS are scheduled one after the other
  bool opt_expand_short_loops = true; // counted loops of <= 8 iterations inside a parallel iteration are expanded in place
  int64_t reg_budget = 0;     // 32-bit registers per thread the caching passes may claim (0 = by block size)
  int64_t reg_budget_scale = 100;   // percent of the by-block-size budget (the driver lowers it when a code object spills)
  bool assume_aligned = true;  // array arguments are at least 16-byte aligned
  ElemSize int_size() const { return has_force_int ? force_int : ElemSize::I64; }
  ElemSize float_size() const { return has_force_float ? force_float : ElemSize::F64; }
};

// ---------------------------------------------------------------- kernels / output
struct KernelParam {
  Name id;
  Type ty;       // Pointer or scalar
  bool read_only = false;
};

struct Kernel {
  std::string name;
  std::vector<KernelParam> params;
  Stmts body;
  Dim3 grid, block;
  int64_t lds_bytes = 0;
  bool aligned_params = false;  // every pointer argument is 16-byte aligned (checked by the caller)
  bool cached_stores = false;   // what this kernel writes is read by the next one: no non-temporal stores
  bool opaque_body = false;     // the body is a call of a device helper: parameters are described by the creator
  bool no_restrict = false;     // workgroups exchange data through the parameters during the kernel: no no-alias promise
  bool fence_lds_iterations = false;  // keep a thread's LDS load / compute / store groups apart when the code is scheduled
  std::vector<std::vector<Name>> distinct_pointers;  // local pointer variables that never name the same array while both are in scope
};

struct Program {
  std::string name;
  std::vector<Param> entry_params;   // flattened entry parameters in call order
  std::vector<Kernel> kernels;
  Stmts host;                        // host statements (loops, allocs, launches)
  std::vector<std::string> includes;
  std::vector<std::string> preamble; // device helper definitions needed by the kernels
  std::vector<FunDef> device_funs;   // typed and lowered functions the kernels call, callees before their callers
};

// pretty printers (debug / cache key)
std::string print_expr(const E& e);
std::string print_stmts(const Stmts& ss, int indent = 0);
std::string print_fun(const FunDef& f);

}  // namespace parpy
