// ParPy HIP runtime for MI355X: buffers, hiprtc compilation, code-object
// loading and the launch-plan interpreter (include/parpy_hip.h).
//
// The reference's runtime is 39 lines of CUDA runtime calls
// (python/parpy/native/parpy_cuda.cpp:3-39) because its generated host code is
// compiled by nvcc.  Here the host side of a compiled function is a launch
// plan: a small tree of host loops, scalar / pointer assignments, temporary
// allocations and kernel launches that this file interprets, calling
// hipModuleLaunchKernel for each launch.
#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <atomic>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <set>
#include <string>
#include <vector>

#include "../../../include/parpy_hip.h"
#include "../compiler/sexpr.hpp"

using parpy::SXP;

namespace {

thread_local std::string g_error = "no error";

int32_t fail(const std::string& msg) {
  g_error = msg;
  return 1;
}

int32_t check(hipError_t e, const char* what) {
  if (e == hipSuccess) return 0;
  g_error = std::string(what) + ": " + hipGetErrorString(e);
  (void)hipGetLastError();
  return (int32_t)e;
}

// ---------------------------------------------------------------- plan data
enum class Kind : uint8_t { Ptr, Bool, I8, I16, I32, I64, U8, U16, U32, U64, F16, F32, F64 };

bool parse_kind(const std::string& s, Kind* k) {
  static const std::map<std::string, Kind> m = {
      {"ptr", Kind::Ptr}, {"bool", Kind::Bool}, {"i8", Kind::I8}, {"i16", Kind::I16}, {"i32", Kind::I32},
      {"i64", Kind::I64}, {"u8", Kind::U8}, {"u16", Kind::U16}, {"u32", Kind::U32}, {"u64", Kind::U64},
      {"f16", Kind::F16}, {"f32", Kind::F32}, {"f64", Kind::F64}};
  auto it = m.find(s);
  if (it == m.end()) return false;
  *k = it->second;
  return true;
}

bool kind_is_float(Kind k) { return k == Kind::F16 || k == Kind::F32 || k == Kind::F64; }

struct Val {
  enum T : uint8_t { I, F, P } t = I;
  int64_t i = 0;
  double f = 0;
  void* p = nullptr;
  double as_f() const { return t == F ? f : (double)i; }
  int64_t as_i() const { return t == I ? i : t == F ? (int64_t)f : (int64_t)(intptr_t)p; }
};

struct HExpr {
  enum Op : uint8_t { Var, Lit, Neg, Not, BitNeg, Bin, Ite, Cvt, Addr } op = Lit;
  int slot = -1;
  Val lit;
  std::string bin;
  int binop = 0;
  bool flt = false;
  Kind kind = Kind::I64;
  int64_t elem_bytes = 1;
  std::vector<HExpr> args;
};

enum BinCode { ADD, SUB, MUL, DIV, FLOORDIV, REM, AND, OR, BITAND, BITOR, BITXOR, SHL, SHR, EQ, NEQ, LEQ, GEQ, LT, GT, MAX, MIN };

struct HStmt {
  enum Op : uint8_t { Launch, For, While, If, Def, Set, Alloc, Free, Persist } op = Launch;
  int kernel = -1;
  unsigned grid[3] = {1, 1, 1}, block[3] = {1, 1, 1};
  std::vector<HExpr> args;
  int slot = -1;
  HExpr a, b;       // For: lo, hi; While/If: cond in a; Def/Set: value in a
  int64_t step = 1;
  int64_t nbytes = 0;
  std::vector<HStmt> body, els;   // Persist: body = the loop of launches that the kernel stands for
  bool fits = false;              // Persist: every workgroup of the launch can be resident at once (checked at creation)
  int64_t groups = 1;            // Persist: groups of workgroups that meet among themselves at the barrier (one counter each)
};

constexpr int64_t KEEP_LIMIT = int64_t(1) << 30;         // per plan
constexpr int64_t KEEP_LIMIT_ALL = int64_t(8) << 30;     // over all live plans of the process
std::atomic<int64_t> g_kept_all{0};
thread_local bool g_div_by_zero = false;                  // set by eval, checked after every statement

}  // namespace

// Device memory for the temporaries of parpy_hip_plan_run_noalloc: part of the library's code
// object, so every GPU the library runs on holds one copy from the first use until the process
// ends.  The name below is only a host-side handle; the device address is looked up once per
// device with hipGetSymbolAddress and that address is what plans receive.
static __device__ __align__(256) unsigned char scratch[PARPY_HIP_SCRATCH_BYTES];

namespace {

constexpr int MAX_DEVICES = 64;
std::mutex g_scratch_mu;
unsigned char* g_scratch_ptr[MAX_DEVICES] = {};

// Device address of the scratch array on the current device (nullptr + message on failure).
unsigned char* scratch_on_current_device() {
  int dev = -1;
  if (check(hipGetDevice(&dev), "hipGetDevice")) return nullptr;
  if (dev < 0 || dev >= MAX_DEVICES) { fail("device ordinal out of range for the scratch table"); return nullptr; }
  std::lock_guard<std::mutex> g(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    if (check(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return nullptr;
    g_scratch_ptr[dev] = (unsigned char*)ptr;
  }
  return g_scratch_ptr[dev];
}

struct Plan {
  hipModule_t module = nullptr;
  std::vector<hipFunction_t> fns;
  std::vector<std::vector<Kind>> kparams;
  std::vector<std::string> knames;
  std::map<std::string, int> slots;
  int nparams = 0;
  std::vector<HStmt> body;
  std::vector<Val> env;
  int64_t launches = 0;
  // Device temporaries stay allocated between runs of the plan (up to KEEP_LIMIT bytes per plan):
  // a run then costs no allocator call.  Indexed by variable slot.
  struct Kept { void* ptr = nullptr; int64_t nbytes = 0; bool in_use = false; };
  std::vector<Kept> kept;
  int64_t kept_bytes = 0;
  std::vector<void*> unkept;   // temporaries of the current run that are freed when it ends, also when it fails half way
  hipEvent_t ev_start = nullptr, ev_stop = nullptr;  // created on the first timed run
  // Graph replay (the analogue of the reference's use_cuda_graphs, src/cuda/graphs.rs): the
  // launches of one run are captured into a HIP graph and later runs with the same pointer
  // arguments replay it with a single hipGraphLaunch.
  bool use_graph = false;
  int graph_state = 0;                 // 0 = first run still to come (eager, allocates the temporaries), 1 = usable, -1 = given up
  hipStream_t cap_stream = nullptr;    // capture needs a stream of its own; replays go to the null stream
  hipStream_t launch_stream = nullptr; // where run_stmt enqueues: null stream, or cap_stream while capturing
  bool capturing = false;
  hipGraph_t graph = nullptr;
  hipGraphExec_t graph_exec = nullptr;
  std::vector<void*> graph_args;
  int64_t graph_launches = 0;
  int64_t graph_replays = 0;           // runs served by hipGraphLaunch so far
  // A run writes the plan's variable slots and temporaries, and callers reach this library through
  // foreign-function calls that release the interpreter lock: two threads calling one compiled
  // function must take turns (the device work they enqueue is ordered by the stream anyway).
  std::mutex mu;
  // Set for the duration of a run through parpy_hip_plan_run_noalloc: temporaries are carved out of
  // the scratch array (stack discipline) instead of being allocated.
  unsigned char* scratch_base = nullptr;
  int64_t scratch_top = 0;
  struct Carved { int slot; int64_t off; };
  std::vector<Carved> carved;
  // Loops that run inside one kernel (persist statements): status word and counters of the barrier between
  // workgroups (device memory allocated when the plan is created: the status word in the first 128 bytes, then
  // one counter every 128 bytes, as many as the statement with the most groups of workgroups needs), whether a
  // launch since the last check may have set the status, and how many runs used such a kernel.
  unsigned* barrier_words = nullptr;
  int64_t barrier_counters = 0;
  bool barrier_pending = false;
  int64_t persistent_launches = 0;
};

// plans that own barrier words: parpy_sync looks at their status after the device has finished
std::mutex g_plans_mu;
std::set<Plan*> g_barrier_plans;

int32_t check_barrier_status(Plan& p) {
  if (!p.barrier_pending || !p.barrier_words) return 0;
  p.barrier_pending = false;
  unsigned status = 0;
  if (int32_t rc = check(hipMemcpy(&status, p.barrier_words, sizeof status, hipMemcpyDeviceToHost), "reading the barrier status")) return rc;
  if (status != 0) {
    // the status word is only ever cleared here, after it has been reported: a later launch of the same plan
    // finds it set, leaves at its first barrier, and cannot hide that an earlier one was cut short
    (void)hipMemset(p.barrier_words, 0, sizeof status);
    return fail("a barrier over all workgroups of a kernel that runs a whole loop of steps timed out: the workgroups "
                "left the kernel early and its results are incomplete (PARPY_HIP_BARRIER_POLLS sets the limit)");
  }
  return 0;
}

struct PlanBuilder {
  Plan& p;
  explicit PlanBuilder(Plan& plan) : p(plan) {}

  int slot(const std::string& name, bool create) {
    auto it = p.slots.find(name);
    if (it != p.slots.end()) return it->second;
    if (!create) throw std::runtime_error("launch plan refers to unknown variable " + name);
    int s = (int)p.slots.size();
    p.slots[name] = s;
    return s;
  }

  HExpr expr(const SXP& x) {
    HExpr e;
    const std::string& h = x->head();
    if (h == "v") { e.op = HExpr::Var; e.slot = slot(x->at(1)->atom, false); }
    else if (h == "i") { e.op = HExpr::Lit; e.lit.t = Val::I; e.lit.i = x->at(1)->as_int(); }
    else if (h == "f") { e.op = HExpr::Lit; e.lit.t = Val::F; e.lit.f = x->at(1)->as_double(); }
    else if (h == "un") {
      const std::string& o = x->at(1)->atom;
      e.op = o == "neg" ? HExpr::Neg : o == "not" ? HExpr::Not : HExpr::BitNeg;
      e.args.push_back(expr(x->at(2)));
    } else if (h == "bin") {
      static const std::map<std::string, int> codes = {
          {"add", ADD}, {"sub", SUB}, {"mul", MUL}, {"div", DIV}, {"floordiv", FLOORDIV}, {"rem", REM}, {"and", AND},
          {"or", OR}, {"bitand", BITAND}, {"bitor", BITOR}, {"bitxor", BITXOR}, {"shl", SHL}, {"shr", SHR}, {"eq", EQ},
          {"neq", NEQ}, {"leq", LEQ}, {"geq", GEQ}, {"lt", LT}, {"gt", GT}, {"max", MAX}, {"min", MIN}};
      e.op = HExpr::Bin;
      auto it = codes.find(x->at(1)->atom);
      if (it == codes.end()) throw std::runtime_error("unknown host operator " + x->at(1)->atom);
      e.binop = it->second;
      e.flt = x->at(2)->atom == "f";
      e.args.push_back(expr(x->at(3)));
      e.args.push_back(expr(x->at(4)));
    } else if (h == "ite") {
      e.op = HExpr::Ite;
      for (int k = 1; k <= 3; ++k) e.args.push_back(expr(x->at(k)));
    } else if (h == "cvt") {
      e.op = HExpr::Cvt;
      if (!parse_kind(x->at(1)->atom, &e.kind)) throw std::runtime_error("bad conversion in launch plan");
      e.args.push_back(expr(x->at(2)));
    } else if (h == "addr") {
      e.op = HExpr::Addr;
      e.args.push_back(expr(x->at(1)));
      e.args.push_back(expr(x->at(2)));
      e.elem_bytes = x->at(3)->as_int();
    } else {
      throw std::runtime_error("unknown host expression '" + h + "' in launch plan");
    }
    return e;
  }

  std::vector<HStmt> stmts(const SXP& lst, size_t from) {
    std::vector<HStmt> out;
    for (size_t k = from; k < lst->size(); ++k) out.push_back(stmt(lst->at(k)));
    return out;
  }

  HStmt stmt(const SXP& x) {
    HStmt s;
    const std::string& h = x->head();
    if (h == "launch") {
      s.op = HStmt::Launch;
      s.kernel = (int)x->at(1)->as_int();
      if (s.kernel < 0 || s.kernel >= (int)p.fns.size()) throw std::runtime_error("launch of unknown kernel index");
      for (int d = 0; d < 3; ++d) {
        s.grid[d] = (unsigned)x->at(2 + d)->as_int();
        s.block[d] = (unsigned)x->at(5 + d)->as_int();
      }
      const SXP& a = x->at(8);
      for (size_t k = 1; k < a->size(); ++k) s.args.push_back(expr(a->at(k)));
      if (s.args.size() != p.kparams[s.kernel].size())
        throw std::runtime_error("argument count mismatch for kernel " + p.knames[s.kernel]);
    } else if (h == "persist") {
      s.op = HStmt::Persist;
      s.kernel = (int)x->at(1)->as_int();
      if (s.kernel < 0 || s.kernel >= (int)p.fns.size()) throw std::runtime_error("launch of unknown kernel index");
      for (int d = 0; d < 3; ++d) {
        s.grid[d] = (unsigned)x->at(2 + d)->as_int();
        s.block[d] = (unsigned)x->at(5 + d)->as_int();
      }
      const SXP& a = x->at(8);
      for (size_t k = 1; k < a->size(); ++k) s.args.push_back(expr(a->at(k)));
      // the kernel takes the barrier's counter, its status word and the poll limit after the plan's arguments
      if (s.args.size() + 3 != p.kparams[s.kernel].size())
        throw std::runtime_error("argument count mismatch for kernel " + p.knames[s.kernel]);
      s.body = stmts(x->at(9), 1);
      // groups of workgroups that meet among themselves, one counter each
      s.groups = x->size() > 10 ? x->at(10)->as_int() : 1;
      if (s.groups < 1 || s.groups > (int64_t)s.grid[0] * s.grid[1] * s.grid[2]) throw std::runtime_error("bad number of barrier groups in launch plan");
      if (p.fns[s.kernel]) {
        int per_cu = 0, cus = 0, dev = 0;
        unsigned threads = s.block[0] * s.block[1] * s.block[2];
        bool ok = hipGetDevice(&dev) == hipSuccess &&
                  hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
                  hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, p.fns[s.kernel], (int)threads, 0) == hipSuccess;
        if (!ok) (void)hipGetLastError();
        s.fits = ok && (int64_t)per_cu * cus >= (int64_t)s.grid[0] * s.grid[1] * s.grid[2];
        if (s.fits && p.barrier_counters < s.groups) {
          // nothing of this plan has run yet: a smaller block made for an earlier statement can go
          if (p.barrier_words) (void)hipFree(p.barrier_words);
          p.barrier_words = nullptr;
          p.barrier_counters = 0;
          void* w = nullptr;
          size_t bytes = (size_t)(s.groups + 1) * 32 * sizeof(unsigned);
          if (hipMalloc(&w, bytes) != hipSuccess) { (void)hipGetLastError(); w = nullptr; }
          else if (hipMemset(w, 0, bytes) != hipSuccess) { (void)hipGetLastError(); (void)hipFree(w); w = nullptr; }
          p.barrier_words = (unsigned*)w;
          if (w) p.barrier_counters = s.groups;
        }
      }
    } else if (h == "for") {
      s.op = HStmt::For;
      s.a = expr(x->at(2));
      s.b = expr(x->at(3));
      s.slot = slot(x->at(1)->atom, true);
      s.step = x->at(4)->as_int();
      s.body = stmts(x->at(5), 1);
    } else if (h == "while") {
      s.op = HStmt::While;
      s.a = expr(x->at(1));
      s.body = stmts(x->at(2), 1);
    } else if (h == "if") {
      s.op = HStmt::If;
      s.a = expr(x->at(1));
      s.body = stmts(x->at(2), 1);
      s.els = stmts(x->at(3), 1);
    } else if (h == "def") {
      s.op = HStmt::Def;
      s.a = expr(x->at(3));
      s.slot = slot(x->at(1)->atom, true);
    } else if (h == "set") {
      s.op = HStmt::Set;
      s.slot = slot(x->at(1)->atom, false);
      s.a = expr(x->at(2));
    } else if (h == "alloc") {
      s.op = HStmt::Alloc;
      s.slot = slot(x->at(1)->atom, true);
      s.nbytes = x->at(2)->as_int();
    } else if (h == "free") {
      s.op = HStmt::Free;
      s.slot = slot(x->at(1)->atom, false);
    } else {
      throw std::runtime_error("unknown statement '" + h + "' in launch plan");
    }
    return s;
  }
};

// ---------------------------------------------------------------- interpreter
Val eval(const Plan& p, const HExpr& e) {
  switch (e.op) {
    case HExpr::Var: return p.env[e.slot];
    case HExpr::Lit: return e.lit;
    case HExpr::Neg: {
      Val a = eval(p, e.args[0]);
      if (a.t == Val::F) a.f = -a.f; else a.i = -a.i;
      return a;
    }
    case HExpr::Not: { Val a = eval(p, e.args[0]); Val r; r.i = a.as_i() == 0; return r; }
    case HExpr::BitNeg: { Val a = eval(p, e.args[0]); Val r; r.i = ~a.as_i(); return r; }
    case HExpr::Ite: return eval(p, e.args[0]).as_i() != 0 ? eval(p, e.args[1]) : eval(p, e.args[2]);
    case HExpr::Cvt: {
      Val a = eval(p, e.args[0]);
      Val r;
      if (kind_is_float(e.kind)) { r.t = Val::F; r.f = e.kind == Kind::F32 ? (double)(float)a.as_f() : a.as_f(); return r; }
      int64_t v = a.as_i();
      switch (e.kind) {
        case Kind::Bool: v = v != 0; break;
        case Kind::I8: v = (int8_t)v; break;
        case Kind::I16: v = (int16_t)v; break;
        case Kind::I32: v = (int32_t)v; break;
        case Kind::U8: v = (uint8_t)v; break;
        case Kind::U16: v = (uint16_t)v; break;
        case Kind::U32: v = (uint32_t)v; break;
        default: break;
      }
      r.i = v;
      return r;
    }
    case HExpr::Addr: {
      Val b = eval(p, e.args[0]);
      Val r;
      r.t = Val::P;
      r.p = (char*)b.p + eval(p, e.args[1]).as_i() * e.elem_bytes;
      return r;
    }
    case HExpr::Bin: {
      Val a = eval(p, e.args[0]), b = eval(p, e.args[1]);
      Val r;
      if (e.flt) {
        double x = a.as_f(), y = b.as_f();
        switch (e.binop) {
          case ADD: r.t = Val::F; r.f = x + y; break;
          case SUB: r.t = Val::F; r.f = x - y; break;
          case MUL: r.t = Val::F; r.f = x * y; break;
          case DIV: r.t = Val::F; r.f = x / y; break;
          case MAX: r.t = Val::F; r.f = std::fmax(x, y); break;
          case MIN: r.t = Val::F; r.f = std::fmin(x, y); break;
          case EQ: r.i = x == y; break;
          case NEQ: r.i = x != y; break;
          case LEQ: r.i = x <= y; break;
          case GEQ: r.i = x >= y; break;
          case LT: r.i = x < y; break;
          case GT: r.i = x > y; break;
          default: break;
        }
        return r;
      }
      int64_t x = a.as_i(), y = b.as_i();
      switch (e.binop) {
        case ADD: r.i = x + y; break;
        case SUB: r.i = x - y; break;
        case MUL: r.i = x * y; break;
        case DIV: case FLOORDIV: if (y == 0) g_div_by_zero = true; r.i = y ? x / y : 0; break;
        case REM: if (y == 0) g_div_by_zero = true; r.i = y ? x % y : 0; break;
        case AND: r.i = (x != 0) && (y != 0); break;
        case OR: r.i = (x != 0) || (y != 0); break;
        case BITAND: r.i = x & y; break;
        case BITOR: r.i = x | y; break;
        case BITXOR: r.i = x ^ y; break;
        case SHL: r.i = x << y; break;
        case SHR: r.i = x >> y; break;
        case EQ: r.i = x == y; break;
        case NEQ: r.i = x != y; break;
        case LEQ: r.i = x <= y; break;
        case GEQ: r.i = x >= y; break;
        case LT: r.i = x < y; break;
        case GT: r.i = x > y; break;
        case MAX: r.i = x > y ? x : y; break;
        case MIN: r.i = x < y ? x : y; break;
      }
      return r;
    }
  }
  return Val();
}

union Packed {
  void* p;
  int64_t i64;
  int32_t i32;
  int16_t i16;
  int8_t i8;
  uint64_t u64;
  uint32_t u32;
  uint16_t u16;
  uint8_t u8;
  float f32;
  double f64;
  _Float16 f16;
  bool b;
};

int32_t run_stmts(Plan& p, const std::vector<HStmt>& ss);

int32_t run_stmt(Plan& p, const HStmt& s) {
  switch (s.op) {
    case HStmt::Launch: case HStmt::Persist: {
      const bool persist = s.op == HStmt::Persist;
      // a loop inside one kernel needs its whole grid resident, memory for the barrier and a stream that is
      // not being captured (the barrier words are cleared with a memset); otherwise the loop of launches runs
      if (persist && !(s.fits && p.barrier_words && p.barrier_counters >= s.groups && !p.capturing)) return run_stmts(p, s.body);
      const auto& kinds = p.kparams[s.kernel];
      Packed storage[64];
      void* ptrs[64];
      size_t n = s.args.size();
      if (n + (persist ? 3 : 0) > 64) return fail("kernel " + p.knames[s.kernel] + " has more than 64 parameters");
      for (size_t k = 0; k < n; ++k) {
        Val v = eval(p, s.args[k]);
        Packed& q = storage[k];
        switch (kinds[k]) {
          case Kind::Ptr: q.p = v.p; break;
          case Kind::Bool: q.b = v.as_i() != 0; break;
          case Kind::I8: q.i8 = (int8_t)v.as_i(); break;
          case Kind::I16: q.i16 = (int16_t)v.as_i(); break;
          case Kind::I32: q.i32 = (int32_t)v.as_i(); break;
          case Kind::I64: q.i64 = v.as_i(); break;
          case Kind::U8: q.u8 = (uint8_t)v.as_i(); break;
          case Kind::U16: q.u16 = (uint16_t)v.as_i(); break;
          case Kind::U32: q.u32 = (uint32_t)v.as_i(); break;
          case Kind::U64: q.u64 = (uint64_t)v.as_i(); break;
          case Kind::F16: q.f16 = (_Float16)v.as_f(); break;
          case Kind::F32: q.f32 = (float)v.as_f(); break;
          case Kind::F64: q.f64 = v.as_f(); break;
        }
        ptrs[k] = &storage[k];
      }
      if (persist) {
        // the counters (from 128 bytes on) start from zero in every launch; the status word in front of them stays as it
        // is until the host has read it
        if (int32_t rc = check(hipMemsetAsync(p.barrier_words + 32, 0, (size_t)s.groups * 32 * sizeof(unsigned), p.launch_stream), "clearing the barrier counters")) return rc;
        // polls of the counter before a workgroup gives up: about a microsecond each, two seconds by default
        unsigned limit = 1u << 21;
        if (const char* e = getenv("PARPY_HIP_BARRIER_POLLS")) limit = (unsigned)strtoul(e, nullptr, 10);
        storage[n].p = p.barrier_words + 32;
        storage[n + 1].p = p.barrier_words;
        storage[n + 2].u32 = limit;
        for (size_t k = n; k < n + 3; ++k) ptrs[k] = &storage[k];
        p.barrier_pending = true;
        ++p.persistent_launches;
      }
      ++p.launches;
      return check(hipModuleLaunchKernel(p.fns[s.kernel], s.grid[0], s.grid[1], s.grid[2], s.block[0], s.block[1],
                                         s.block[2], 0, p.launch_stream, ptrs, nullptr),
                   p.knames[s.kernel].c_str());
    }
    case HStmt::For: {
      int64_t lo = eval(p, s.a).as_i(), hi = eval(p, s.b).as_i();
      for (int64_t v = lo; s.step > 0 ? v < hi : v > hi; v += s.step) {
        p.env[s.slot].t = Val::I;
        p.env[s.slot].i = v;
        if (int32_t rc = run_stmts(p, s.body)) return rc;
      }
      return 0;
    }
    case HStmt::While:
      while (eval(p, s.a).as_i() != 0)
        if (int32_t rc = run_stmts(p, s.body)) return rc;
      return 0;
    case HStmt::If:
      return run_stmts(p, eval(p, s.a).as_i() != 0 ? s.body : s.els);
    case HStmt::Def: case HStmt::Set:
      p.env[s.slot] = eval(p, s.a);
      return 0;
    case HStmt::Alloc: {
      if (p.scratch_base) {
        int64_t off = (p.scratch_top + 255) & ~int64_t(255);
        if (s.nbytes < 0 || off + s.nbytes > (int64_t)PARPY_HIP_SCRATCH_BYTES)
          return fail("the device temporaries of this plan need " + std::to_string(off + s.nbytes) +
                      " bytes, more than the " + std::to_string((int64_t)PARPY_HIP_SCRATCH_BYTES) +
                      " bytes of scratch memory that parpy_hip_plan_run_noalloc has; use parpy_hip_plan_run");
        p.carved.push_back({s.slot, off});
        p.scratch_top = off + s.nbytes;
        p.env[s.slot].t = Val::P;
        p.env[s.slot].p = p.scratch_base + off;
        return 0;
      }
      if (p.kept.size() < p.env.size()) p.kept.resize(p.env.size());
      Plan::Kept& kp = p.kept[s.slot];
      if (kp.ptr && kp.nbytes == s.nbytes && !kp.in_use) {
        kp.in_use = true;
        p.env[s.slot].t = Val::P;
        p.env[s.slot].p = kp.ptr;
        return 0;
      }
      if (p.capturing) return fail("a device temporary would have to be allocated inside a graph capture");
      void* ptr = nullptr;
      hipError_t e = hipMallocAsync(&ptr, (size_t)s.nbytes, nullptr);
      if (e != hipSuccess) {
        (void)hipGetLastError();
        e = hipMalloc(&ptr, (size_t)s.nbytes);
      }
      if (int32_t rc = check(e, "allocation of a device temporary")) return rc;
      p.env[s.slot].t = Val::P;
      p.env[s.slot].p = ptr;
      if (!kp.ptr && p.kept_bytes + s.nbytes <= KEEP_LIMIT && g_kept_all.load() + s.nbytes <= KEEP_LIMIT_ALL) {
        kp.ptr = ptr;
        kp.nbytes = s.nbytes;
        kp.in_use = true;
        p.kept_bytes += s.nbytes;
        g_kept_all += s.nbytes;
      } else {
        p.unkept.push_back(ptr);
      }
      return 0;
    }
    case HStmt::Free: {
      if (p.scratch_base) {
        // the most recent temporary gives its space back; others stay carved until the run ends
        if (!p.carved.empty() && p.carved.back().slot == s.slot) {
          p.scratch_top = p.carved.back().off;
          p.carved.pop_back();
        }
        p.env[s.slot].p = nullptr;
        return 0;
      }
      void* ptr = p.env[s.slot].p;
      p.env[s.slot].p = nullptr;
      if ((size_t)s.slot < p.kept.size() && p.kept[s.slot].ptr == ptr && ptr) {
        p.kept[s.slot].in_use = false;  // stays allocated for the next run
        return 0;
      }
      for (size_t k = 0; k < p.unkept.size(); ++k)
        if (p.unkept[k] == ptr) { p.unkept.erase(p.unkept.begin() + k); break; }
      hipError_t e = hipFreeAsync(ptr, nullptr);
      if (e != hipSuccess) {
        (void)hipGetLastError();
        e = hipFree(ptr);
      }
      return check(e, "release of a device temporary");
    }
  }
  return 0;
}

int32_t run_stmts(Plan& p, const std::vector<HStmt>& ss) {
  for (auto& s : ss) {
    if (int32_t rc = run_stmt(p, s)) return rc;
    if (g_div_by_zero) return fail("division by zero in the host part of the launch plan");
  }
  return 0;
}

// what a run that stopped half way still holds
void release_unkept(Plan& p) {
  for (void* ptr : p.unkept)
    if (hipFreeAsync(ptr, nullptr) != hipSuccess) {
      (void)hipGetLastError();
      (void)hipFree(ptr);
    }
  p.unkept.clear();
}

}  // namespace

extern "C" {

void parpy_init(int64_t) {
  // look up this device's scratch array now when a device is there; a later call retries
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess || n == 0) { (void)hipGetLastError(); return; }
  if (!scratch_on_current_device()) g_error = "no error";
}

int32_t parpy_sync(void) {
  if (int32_t rc = check(hipDeviceSynchronize(), "hipDeviceSynchronize")) return rc;
  // kernels that run a loop of steps report a barrier that timed out through a status word
  std::lock_guard<std::mutex> g(g_plans_mu);
  for (Plan* p : g_barrier_plans) {
    std::lock_guard<std::mutex> turn(p->mu);
    if (int32_t rc = check_barrier_status(*p)) return rc;
  }
  return 0;
}

void* parpy_alloc_buffer(int64_t nbytes) {
  void* ptr = nullptr;
  if (nbytes < 0) { fail("negative allocation size"); return nullptr; }
  if (hipMallocAsync(&ptr, (size_t)nbytes, nullptr) != hipSuccess) {
    (void)hipGetLastError();
    if (check(hipMalloc(&ptr, (size_t)nbytes), "hipMalloc")) return nullptr;
  }
  return ptr;
}

int32_t parpy_memcpy(void* dst, void* src, int64_t nbytes, int64_t kind) {
  hipMemcpyKind k = kind == 0 ? hipMemcpyHostToHost : kind == 1 ? hipMemcpyHostToDevice
                  : kind == 2 ? hipMemcpyDeviceToHost : hipMemcpyDeviceToDevice;
  return check(hipMemcpyAsync(dst, src, (size_t)nbytes, k, nullptr), "hipMemcpyAsync");
}

int32_t parpy_memset(void* ptr, int64_t nbytes, int8_t value) {
  return check(hipMemset(ptr, value, (size_t)nbytes), "hipMemset");
}

int32_t parpy_free_buffer(void* ptr) {
  hipError_t e = hipFreeAsync(ptr, nullptr);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    e = hipFree(ptr);
  }
  return check(e, "hipFree");
}

const char* parpy_get_error_message(void) { return g_error.c_str(); }

int32_t parpy_hip_compile(const char* source, const char* const* options, int32_t noptions, void** code, size_t* size) {
  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, source, "parpy_kernels.hip", 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) return fail(std::string("hiprtcCreateProgram: ") + hiprtcGetErrorString(r));
  std::vector<const char*> opts;
  bool has_arch = false;
  for (int32_t k = 0; k < noptions; ++k) {
    opts.push_back(options[k]);
    if (std::strstr(options[k], "--offload-arch") || std::strstr(options[k], "--gpu-architecture")) has_arch = true;
  }
  if (!has_arch) opts.push_back("--offload-arch=gfx950");
  r = hiprtcCompileProgram(prog, (int)opts.size(), opts.data());
  if (r != HIPRTC_SUCCESS) {
    size_t n = 0;
    hiprtcGetProgramLogSize(prog, &n);
    std::string log(n, '\0');
    if (n) hiprtcGetProgramLog(prog, &log[0]);
    hiprtcDestroyProgram(&prog);
    return fail(std::string("Compilation of generated HIP code failed (") + hiprtcGetErrorString(r) + "):\n" + log);
  }
  size_t n = 0;
  r = hiprtcGetCodeSize(prog, &n);
  if (r != HIPRTC_SUCCESS || n == 0) {
    hiprtcDestroyProgram(&prog);
    return fail("hiprtcGetCodeSize failed");
  }
  void* buf = malloc(n);
  r = hiprtcGetCode(prog, (char*)buf);
  hiprtcDestroyProgram(&prog);
  if (r != HIPRTC_SUCCESS) {
    free(buf);
    return fail(std::string("hiprtcGetCode: ") + hiprtcGetErrorString(r));
  }
  *code = buf;
  *size = n;
  return 0;
}

void parpy_hip_free_code(void* code) { free(code); }

int32_t parpy_hip_module_load(const void* code, size_t, void** module) {
  hipModule_t m;
  if (int32_t rc = check(hipModuleLoadData(&m, code), "hipModuleLoadData")) return rc;
  *module = m;
  return 0;
}

int32_t parpy_hip_module_unload(void* module) { return check(hipModuleUnload((hipModule_t)module), "hipModuleUnload"); }

int32_t parpy_hip_launch(void* module, const char* kernel, const int64_t grid[3], const int64_t block[3],
                         int64_t lds_bytes, void** args) {
  hipFunction_t f;
  if (int32_t rc = check(hipModuleGetFunction(&f, (hipModule_t)module, kernel), kernel)) return rc;
  return check(hipModuleLaunchKernel(f, (unsigned)grid[0], (unsigned)grid[1], (unsigned)grid[2], (unsigned)block[0],
                                     (unsigned)block[1], (unsigned)block[2], (unsigned)lds_bytes, nullptr, args, nullptr),
               kernel);
}

int32_t parpy_hip_plan_create(void* module, const char* plan_text, void** plan) {
  auto p = new Plan();
  p->module = (hipModule_t)module;
  try {
    SXP x = parpy::parse_sexpr(plan_text);
    if (x->head() != "plan") throw std::runtime_error("not a launch plan");
    PlanBuilder b(*p);
    const SXP& params = x->at(2);
    for (size_t k = 1; k < params->size(); ++k) b.slot(params->at(k)->at(0)->atom, true);
    p->nparams = (int)params->size() - 1;
    const SXP& kernels = x->at(3);
    for (size_t k = 1; k < kernels->size(); ++k) {
      const SXP& kd = kernels->at(k);
      p->knames.push_back(kd->at(0)->atom);
      std::vector<Kind> kinds;
      const SXP& kp = kd->at(1);
      for (size_t j = 1; j < kp->size(); ++j) {
        Kind kk;
        if (!parse_kind(kp->at(j)->atom, &kk)) throw std::runtime_error("bad kernel parameter kind " + kp->at(j)->atom);
        kinds.push_back(kk);
      }
      p->kparams.push_back(kinds);
      hipFunction_t f = nullptr;
      if (module) {
        hipError_t e = hipModuleGetFunction(&f, p->module, p->knames.back().c_str());
        if (e != hipSuccess) {
          (void)hipGetLastError();
          throw std::runtime_error("kernel " + p->knames.back() + " not found in module: " + hipGetErrorString(e));
        }
      }
      p->fns.push_back(f);
    }
    p->body = b.stmts(x->at(4), 1);
    p->env.resize(p->slots.size());
    if (p->barrier_words) {
      std::lock_guard<std::mutex> g(g_plans_mu);
      g_barrier_plans.insert(p);
    }
  } catch (const std::exception& e) {
    if (p->barrier_words) (void)hipFree(p->barrier_words);   // (a statement after a persist statement was malformed)
    delete p;
    return fail(std::string("invalid launch plan: ") + e.what());
  }
  *plan = p;
  return 0;
}

}  // extern "C"

namespace {

void drop_graph(Plan& p) {
  if (p.graph_exec) (void)hipGraphExecDestroy(p.graph_exec);
  if (p.graph) (void)hipGraphDestroy(p.graph);
  p.graph_exec = nullptr;
  p.graph = nullptr;
}

// Capture one run of the plan.  Returns false (and leaves graph_state = -1) when the plan cannot
// be captured; the caller then runs it eagerly.
bool capture_graph(Plan& p, void* const* args, int32_t nargs) {
  drop_graph(p);
  if (!p.cap_stream && hipStreamCreate(&p.cap_stream) != hipSuccess) {
    (void)hipGetLastError();
    p.graph_state = -1;
    return false;
  }
  if (hipStreamBeginCapture(p.cap_stream, hipStreamCaptureModeThreadLocal) != hipSuccess) {
    (void)hipGetLastError();
    p.graph_state = -1;
    return false;
  }
  p.launch_stream = p.cap_stream;
  p.capturing = true;
  p.launches = 0;
  int32_t rc = run_stmts(p, p.body);
  p.capturing = false;
  p.launch_stream = nullptr;
  hipError_t e = hipStreamEndCapture(p.cap_stream, &p.graph);
  if (rc == 0 && e == hipSuccess) e = hipGraphInstantiate(&p.graph_exec, p.graph, nullptr, nullptr, 0);
  if (rc != 0 || e != hipSuccess) {
    (void)hipGetLastError();
    drop_graph(p);
    p.graph_state = -1;
    return false;
  }
  p.graph_args.assign(args, args + nargs);
  p.graph_launches = p.launches;
  return true;
}

}  // namespace

extern "C" {

int32_t parpy_hip_plan_set_graph(void* plan, int32_t enable) {
  Plan& p = *(Plan*)plan;
  std::lock_guard<std::mutex> turn(p.mu);
  p.use_graph = enable != 0;
  if (!p.use_graph) drop_graph(p);
  p.graph_state = 0;
  return 0;
}

}  // extern "C"

namespace {

int32_t plan_run_locked(Plan& p, void* const* args, int32_t nargs) {
  if (nargs != p.nparams)
    return fail("launch plan expects " + std::to_string(p.nparams) + " pointer arguments, received " + std::to_string(nargs));
  if (!p.module) return fail("launch plan was created without a loaded module");
  for (int k = 0; k < nargs; ++k) {
    p.env[k].t = Val::P;
    p.env[k].p = args[k];
  }
  for (auto& kp : p.kept) kp.in_use = false;  // a run that failed half way may have left a temporary marked
  if (p.use_graph && p.graph_state == 1) {
    bool same = p.graph_exec && p.graph_args.size() == (size_t)nargs && std::equal(args, args + nargs, p.graph_args.begin());
    if (same || capture_graph(p, args, nargs)) {
      p.launches = p.graph_launches;
      ++p.graph_replays;
      return check(hipGraphLaunch(p.graph_exec, nullptr), "hipGraphLaunch");
    }
    for (auto& kp : p.kept) kp.in_use = false;
  }
  p.launches = 0;
  g_div_by_zero = false;
  int32_t rc = run_stmts(p, p.body);
  if (rc != 0) {
    std::string msg = g_error;
    release_unkept(p);
    g_error = msg;
  }
  if (p.use_graph && p.graph_state == 0) p.graph_state = rc == 0 ? 1 : -1;  // temporaries exist now: capture from the next run on
  return rc;
}

}  // namespace

extern "C" {

int32_t parpy_hip_plan_run(void* plan, void* const* args, int32_t nargs) {
  Plan& p = *(Plan*)plan;
  std::lock_guard<std::mutex> turn(p.mu);
  return plan_run_locked(p, args, nargs);
}

int32_t parpy_hip_plan_run_timed(void* plan, void* const* args, int32_t nargs, float* elapsed_ms) {
  Plan& p = *(Plan*)plan;
  std::lock_guard<std::mutex> turn(p.mu);
  if (!p.ev_start) {
    if (int32_t rc = check(hipEventCreate(&p.ev_start), "hipEventCreate")) return rc;
    if (int32_t rc = check(hipEventCreate(&p.ev_stop), "hipEventCreate")) return rc;
  }
  if (int32_t rc = check(hipEventRecord(p.ev_start, nullptr), "hipEventRecord")) return rc;
  if (int32_t rc = plan_run_locked(p, args, nargs)) return rc;
  if (int32_t rc = check(hipEventRecord(p.ev_stop, nullptr), "hipEventRecord")) return rc;
  if (int32_t rc = check(hipEventSynchronize(p.ev_stop), "hipEventSynchronize")) return rc;
  if (int32_t rc = check_barrier_status(p)) return rc;
  return check(hipEventElapsedTime(elapsed_ms, p.ev_start, p.ev_stop), "hipEventElapsedTime");
}

int32_t parpy_hip_plan_run_noalloc(void* plan, void* const* args, int32_t nargs) {
  Plan& p = *(Plan*)plan;
  std::lock_guard<std::mutex> turn(p.mu);
  unsigned char* base = scratch_on_current_device();
  if (!base) return 1;
  if (nargs != p.nparams)
    return fail("launch plan expects " + std::to_string(p.nparams) + " pointer arguments, received " + std::to_string(nargs));
  if (!p.module) return fail("launch plan was created without a loaded module");
  for (int k = 0; k < nargs; ++k) {
    p.env[k].t = Val::P;
    p.env[k].p = args[k];
  }
  p.scratch_base = base;
  p.scratch_top = 0;
  p.carved.clear();
  p.launches = 0;
  g_div_by_zero = false;
  int32_t rc = run_stmts(p, p.body);   // eager launches on the null stream; no graph, no kept temporaries
  p.scratch_base = nullptr;
  return rc;
}

int64_t parpy_hip_plan_launch_count(void* plan) { return ((Plan*)plan)->launches; }

int64_t parpy_hip_plan_graph_replays(void* plan) { return ((Plan*)plan)->graph_replays; }

int64_t parpy_hip_plan_persistent_launches(void* plan) { return ((Plan*)plan)->persistent_launches; }

int32_t parpy_hip_plan_destroy(void* plan) {
  Plan* p = (Plan*)plan;
  {
    std::lock_guard<std::mutex> g(g_plans_mu);
    g_barrier_plans.erase(p);
  }
  if (p->barrier_words) (void)hipFree(p->barrier_words);
  if (p->ev_start) (void)hipEventDestroy(p->ev_start);
  if (p->ev_stop) (void)hipEventDestroy(p->ev_stop);
  drop_graph(*p);
  if (p->cap_stream) (void)hipStreamDestroy(p->cap_stream);
  for (auto& kp : p->kept)
    if (kp.ptr) (void)hipFree(kp.ptr);
  g_kept_all -= p->kept_bytes;
  delete p;
  return 0;
}

}  // extern "C"
