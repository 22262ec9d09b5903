// HIP C++ (gfx950) pretty-printer: device source for hiprtc, the host launch
// plan for the runtime, and a combined human-readable listing.
//
// Takes the place of the reference's src/cuda/pprint.rs:40-570 and
// src/cuda/codegen.rs:120-358.  There is no generated host translation unit:
// host loops, temporaries and launches are emitted as a launch plan that the
// runtime library interprets (hipModuleLaunchKernel), so nothing but device
// code goes through a compiler at call time.
#include <cinttypes>
#include <sstream>

#include "passes.hpp"

namespace parpy {

namespace {

std::string fmt_f32(double v) {
  if (std::isinf(v)) return v > 0 ? "__builtin_huge_valf()" : "(-__builtin_huge_valf())";
  if (std::isnan(v)) return "__builtin_nanf(\"\")";
  char buf[64];
  snprintf(buf, sizeof buf, "%.9g", v);
  std::string s = buf;
  if (s.find('.') == std::string::npos && s.find('e') == std::string::npos) s += ".0";
  return s + "f";
}

std::string fmt_f64(double v) {
  if (std::isinf(v)) return v > 0 ? "__builtin_huge_val()" : "(-__builtin_huge_val())";
  if (std::isnan(v)) return "__builtin_nan(\"\")";
  char buf[64];
  snprintf(buf, sizeof buf, "%.17g", v);
  std::string s = buf;
  if (s.find('.') == std::string::npos && s.find('e') == std::string::npos) s += ".0";
  return s;
}

const char* red_suffix(BinOp op) {
  switch (op) {
    case BinOp::Add: return "add";
    case BinOp::Mul: return "mul";
    case BinOp::Max: return "max";
    case BinOp::Min: return "min";
    case BinOp::BitAnd: case BinOp::And: return "and";
    case BinOp::BitOr: case BinOp::Or: return "or";
    case BinOp::BitXor: return "xor";
    default: return "add";
  }
}

// Device helpers shared by all generated kernels.  Cross-lane reductions use
// DPP row operations inside each row of 16 lanes, row broadcasts across the
// four rows of a 64-lane wavefront, and a readlane broadcast so that every
// lane ends up holding the result.
const char* PREAMBLE = R"(#if defined(__HIPCC_RTC__)
typedef signed char int8_t;
typedef short int16_t;
typedef int int32_t;
typedef long long int64_t;
typedef unsigned char uint8_t;
typedef unsigned short uint16_t;
typedef unsigned int uint32_t;
typedef unsigned long long uint64_t;
#else
#include <hip/hip_runtime.h>
#include <stdint.h>
#endif

template <int CTRL, class T> __device__ __forceinline__ T parpy_dpp(T v) {
  if constexpr (sizeof(T) == 8) {
    unsigned long long x = __builtin_bit_cast(unsigned long long, v);
    int lo = (int)(unsigned)x, hi = (int)(unsigned)(x >> 32);
    lo = __builtin_amdgcn_update_dpp(lo, lo, CTRL, 0xF, 0xF, false);
    hi = __builtin_amdgcn_update_dpp(hi, hi, CTRL, 0xF, 0xF, false);
    x = ((unsigned long long)(unsigned)hi << 32) | (unsigned)lo;
    return __builtin_bit_cast(T, x);
  } else if constexpr (sizeof(T) == 4) {
    int x = __builtin_bit_cast(int, v);
    x = __builtin_amdgcn_update_dpp(x, x, CTRL, 0xF, 0xF, false);
    return __builtin_bit_cast(T, x);
  } else if constexpr (sizeof(T) == 2) {   // the bits travel, not the value: a half must not be rounded to an integer
    int x = (int)__builtin_bit_cast(unsigned short, v);
    x = __builtin_amdgcn_update_dpp(x, x, CTRL, 0xF, 0xF, false);
    return __builtin_bit_cast(T, (unsigned short)x);
  } else {
    int x = (int)__builtin_bit_cast(unsigned char, v);
    x = __builtin_amdgcn_update_dpp(x, x, CTRL, 0xF, 0xF, false);
    return __builtin_bit_cast(T, (unsigned char)x);
  }
}
template <class T> __device__ __forceinline__ T parpy_readlane(T v, int lane) {
  if constexpr (sizeof(T) == 8) {
    unsigned long long x = __builtin_bit_cast(unsigned long long, v);
    unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)x, lane);
    unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(x >> 32), lane);
    x = ((unsigned long long)hi << 32) | lo;
    return __builtin_bit_cast(T, x);
  } else if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(T, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
  } else if constexpr (sizeof(T) == 2) {
    return __builtin_bit_cast(T, (unsigned short)__builtin_amdgcn_readlane((int)__builtin_bit_cast(unsigned short, v), lane));
  } else {
    return __builtin_bit_cast(T, (unsigned char)__builtin_amdgcn_readlane((int)__builtin_bit_cast(unsigned char, v), lane));
  }
}
struct parpy_op_add { template <class T> __device__ __forceinline__ T operator()(T a, T b) const { return a + b; } };
struct parpy_op_mul { template <class T> __device__ __forceinline__ T operator()(T a, T b) const { return a * b; } };
struct parpy_op_and { template <class T> __device__ __forceinline__ T operator()(T a, T b) const { return a & b; } };
struct parpy_op_or { template <class T> __device__ __forceinline__ T operator()(T a, T b) const { return a | b; } };
struct parpy_op_xor { template <class T> __device__ __forceinline__ T operator()(T a, T b) const { return a ^ b; } };
struct parpy_op_max {
  __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
  __device__ __forceinline__ double operator()(double a, double b) const { return fmax(a, b); }
  template <class T> __device__ __forceinline__ T operator()(T a, T b) const { return a > b ? a : b; }
};
struct parpy_op_min {
  __device__ __forceinline__ float operator()(float a, float b) const { return fminf(a, b); }
  __device__ __forceinline__ double operator()(double a, double b) const { return fmin(a, b); }
  template <class T> __device__ __forceinline__ T operator()(T a, T b) const { return a < b ? a : b; }
};
template <class T> __device__ __forceinline__ T parpy_max(T a, T b) { return parpy_op_max()(a, b); }
template <class T> __device__ __forceinline__ T parpy_min(T a, T b) { return parpy_op_min()(a, b); }
// fp32 max / min of a statement as the one machine instruction (three operands: v_max3 / v_min3).  Through
// fmaxf() every operand that comes from memory is first passed through a quieting `v_max_f32 x, x`, because a
// signalling NaN must not reach the instruction under the C rules.  The instruction returns the other operand
// when one is a quiet NaN -- the behaviour that log-space kernels rely on -- and no arithmetic produces a
// signalling NaN.  The `c` forms take a compile-time constant as last operand (kept in a scalar register).
__device__ __forceinline__ float parpy_fmax(float a, float b) { float r; asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b)); return r; }
__device__ __forceinline__ float parpy_fmin(float a, float b) { float r; asm("v_min_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b)); return r; }
__device__ __forceinline__ float parpy_fmaxc(float a, float c) { float r; asm("v_max_f32 %0, %1, %2" : "=v"(r) : "s"(c), "v"(a)); return r; }
__device__ __forceinline__ float parpy_fminc(float a, float c) { float r; asm("v_min_f32 %0, %1, %2" : "=v"(r) : "s"(c), "v"(a)); return r; }
__device__ __forceinline__ float parpy_fmax3(float a, float b, float c) { float r; asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c)); return r; }
__device__ __forceinline__ float parpy_fmin3(float a, float b, float c) { float r; asm("v_min3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c)); return r; }
__device__ __forceinline__ float parpy_fmax3c(float a, float b, float c) { float r; asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "s"(c)); return r; }
__device__ __forceinline__ float parpy_fmin3c(float a, float b, float c) { float r; asm("v_min3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "s"(c)); return r; }
// reduce over each row of 16 lanes; afterwards every lane of a row holds the row's result
template <class Op, class T> __device__ __forceinline__ T parpy_row_reduce(T v) {
  Op op;
  v = op(v, parpy_dpp<0xB1>(v));   // quad_perm [1,0,3,2]
  v = op(v, parpy_dpp<0x4E>(v));   // quad_perm [2,3,0,1]
  v = op(v, parpy_dpp<0x141>(v));  // row_half_mirror
  v = op(v, parpy_dpp<0x140>(v));  // row_mirror
  return v;
}
// reduce over the 64 lanes of a wavefront; every lane receives the result
template <class Op, class T> __device__ __forceinline__ T parpy_wave_reduce(T v) {
  Op op;
  v = parpy_row_reduce<Op>(v);
  v = op(v, parpy_dpp<0x142>(v));  // row_bcast:15 (lane 15 of each row into the next row)
  v = op(v, parpy_dpp<0x143>(v));  // row_bcast:31 (lane 31 into rows 2 and 3)
  return parpy_readlane(v, 63);
}
// block reduction: one LDS slot per wavefront, then every wavefront reduces the partials
template <class Op, int NWAVES, class T>
__device__ __forceinline__ T parpy_block_reduce(T v, T neutral, T* slots, bool sync_after) {
  v = parpy_wave_reduce<Op>(v);
  if constexpr (NWAVES > 1) {
    const int lane = threadIdx.x & 63;
    if (lane == 0) slots[threadIdx.x >> 6] = v;
    __syncthreads();
    v = lane < NWAVES ? slots[lane] : neutral;
    v = parpy_row_reduce<Op>(v);
    v = parpy_readlane(v, 0);
    if (sync_after) __syncthreads();
  }
  return v;
}
// element i of p, for an i whose byte offset is known to fit 32 bits
template <class T> __device__ __forceinline__ T& parpy_at(T* p, unsigned i) { return *(T*)((char*)p + i * (unsigned)sizeof(T)); }
template <class T> __device__ __forceinline__ const T& parpy_at(const T* p, unsigned i) { return *(const T*)((const char*)p + i * (unsigned)sizeof(T)); }
// sum over each aligned group of 8 lanes; every lane of the group receives it
template <class T> __device__ __forceinline__ T parpy_sum8(T v) {
  v = v + parpy_dpp<0xB1>(v);   // lane ^ 1
  v = v + parpy_dpp<0x4E>(v);   // lane ^ 2
  v = v + parpy_dpp<0x141>(v);  // the other quad of the 8-lane half row
  return v;
}
// Barrier over all workgroups of a launch whose whole grid is resident on the device.  The kernels that use it
// load and store what they exchange at device scope, so no cache has to be written back or emptied here: every
// wave waits until its own memory operations have completed, the workgroup's first thread counts the workgroup in
// and waits until the counter shows that all have arrived (the counter is never reset: call number e waits for
// e * nblocks).  The wait is bounded: after `limit` polls, or when another workgroup has given up, the status word
// is set and false is returned to the whole workgroup, which leaves the kernel.
__device__ __forceinline__ bool parpy_grid_barrier(unsigned* counter, unsigned* status, unsigned nblocks, unsigned& epoch, unsigned limit) {
  __shared__ unsigned parpy_bar_ok;
  __builtin_amdgcn_s_waitcnt(0x0070);   // vmcnt(0) lgkmcnt(0): this wave's loads and stores are done
  __syncthreads();
  epoch += 1;
  if (threadIdx.x == 0 && threadIdx.y == 0 && threadIdx.z == 0) {
    const unsigned target = epoch * nblocks;
    __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    unsigned ok = 1, polls = 0;
    while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
      if (polls++ >= limit || __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) { ok = 0; break; }
      __builtin_amdgcn_s_sleep(1);
    }
    if (!ok) __hip_atomic_store(status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    parpy_bar_ok = ok;
  }
  __syncthreads();
  return parpy_bar_ok != 0;
}
typedef float parpy_f32x4 __attribute__((ext_vector_type(4)));
template <class T> using parpy_vec4 = T __attribute__((ext_vector_type(4)));
__device__ __forceinline__ int parpy_lane_id() { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }
// dst[c][r] = src[r][c] for a ROWS x COLS matrix in 64 x 64 tiles: a 256-thread workgroup reads
// 64-word row segments of its tile, turns the tile round in LDS and writes 64-word row segments
// of the result, so both sides move whole 256-byte lines.  Launched on a (ceil(COLS/64), ceil(ROWS/64))
// grid; the bounds tests of the edge tiles are compile-time false when 64 divides the extents.
template <class T, int ROWS, int COLS> __device__ __forceinline__ void parpy_transpose_tile(const T* __restrict__ src, T* __restrict__ dst) {
  __shared__ T tile[64][65];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int c0 = (int)blockIdx.x * 64, r0 = (int)blockIdx.y * 64;
  #pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int r = r0 + j * 4 + ty, c = c0 + tx;
    if ((ROWS % 64 == 0 || r < ROWS) && (COLS % 64 == 0 || c < COLS)) tile[j * 4 + ty][tx] = src[(long long)r * COLS + c];
  }
  __syncthreads();
  #pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int c = c0 + j * 4 + ty, r = r0 + tx;
    if ((COLS % 64 == 0 || c < COLS) && (ROWS % 64 == 0 || r < ROWS)) dst[(long long)c * ROWS + r] = tile[tx][j * 4 + ty];
  }
}
)";

struct PE {  // printed integer expression: text + whether it was computed in 32-bit arithmetic
  std::string s;
  bool narrow = false;
};

bool fits32(const Interval& r) { return r.known && r.lo >= INT32_MIN && r.hi <= INT32_MAX; }

struct DevicePrinter {
  const Options& opts;
  const Kernel* kernel = nullptr;
  RangeEnv ranges;
  std::set<Name> narrow_vars;     // 64-bit integer variables declared as 32-bit because their range allows it
  std::set<Name> reassigned;      // variables assigned after their definition (their range is not tracked)
  std::set<Name> stream_out;      // global arrays the kernel only stores to: written with non-temporal stores
  std::ostringstream os;
  int red_sites = 0;
  std::vector<std::string> lds_decls;
  std::set<Name> lds_arrays;   // names of the arrays the kernel declares in LDS

  explicit DevicePrinter(const Options& o) : opts(o) {}

  std::string ind(int n) { return std::string(n, ' '); }

  // ---------------------------------------------------------------- expressions
  std::string ctype(const Type& t) {
    if (t.k == Type::Pointer && t.mem == Mem::LDS)
      return "__attribute__((address_space(3))) " + std::string(elem_ctype(t.sz)) + "*";
    if (t.k == Type::Pointer) return std::string(elem_ctype(t.sz)) + "*";
    if (t.k == Type::Tensor && !t.shape.empty()) return std::string(elem_ctype(t.sz)) + "*";
    if (t.k == Type::Tensor) return elem_ctype(t.sz);
    return "void";
  }

  std::string idx_name(Expr::Kind k, int dim) {
    return std::string(k == Expr::ThreadIdx ? "threadIdx." : "blockIdx.") + "xyz"[dim];
  }

  bool is_i64(const E& e) { return e->ty.is_scalar() && (e->ty.sz == ElemSize::I64); }

  // integer expressions whose semantic type is int64 are computed in 32 bits
  // when interval analysis proves that neither the result nor any intermediate
  // value leaves the int32 range
  PE pint(const E& e) {
    PE r;
    if (!opts.opt_narrow_index || !is_i64(e)) { r.s = pexpr_plain(e); return r; }
    switch (e->k) {
      case Expr::Int:
        if (e->iv >= INT32_MIN && e->iv <= INT32_MAX) { r.s = e->iv < 0 ? "(" + std::to_string(e->iv) + ")" : std::to_string(e->iv); r.narrow = true; }
        else r.s = "((int64_t)" + std::to_string(e->iv) + "LL)";
        return r;
      case Expr::Var: {
        r.s = e->name.str();
        r.narrow = narrow_vars.count(e->name) > 0;
        if (!r.narrow) {
          // a 64-bit variable whose value is known to fit (for instance because it indexes a dimension)
          auto it = ranges.find(e->name);
          if (it != ranges.end() && fits32(it->second)) { r.s = "(int)" + r.s; r.narrow = true; }
        }
        return r;
      }
      case Expr::ThreadIdx: case Expr::BlockIdx:
        r.s = "(int)" + idx_name(e->k, (int)e->iv);
        r.narrow = true;
        return r;
      case Expr::Convert: {
        const E& a = e->args[0];
        if (a->ty.is_scalar() && is_int(a->ty.sz) && elem_bytes(a->ty.sz) <= 4 && !(a->ty.sz == ElemSize::U32)) {
          r.s = "(int)" + paren(pexpr(a));
          r.narrow = true;
          return r;
        }
        r.s = pexpr_plain(e);
        return r;
      }
      case Expr::BinOpE: {
        BinOp op = e->bop;
        bool arith = op == BinOp::Add || op == BinOp::Sub || op == BinOp::Mul || op == BinOp::FloorDiv ||
                     op == BinOp::Div || op == BinOp::Rem || op == BinOp::BitAnd || op == BinOp::BitOr ||
                     op == BinOp::BitXor || op == BinOp::BitShl || op == BinOp::BitShr || op == BinOp::Max || op == BinOp::Min;
        if (!arith) { r.s = pexpr_plain(e); return r; }
        PE a = pint(e->args[0]), b = pint(e->args[1]);
        bool ok = a.narrow && b.narrow && fits32(expr_range(e, ranges));
        std::string as = a.s, bs = b.s;
        if (!ok) {
          if (a.narrow) as = "(int64_t)" + paren(as);
          if (b.narrow) bs = "(int64_t)" + paren(bs);
        }
        r.narrow = ok;
        if (op == BinOp::Max || op == BinOp::Min)
          r.s = std::string(op == BinOp::Max ? "parpy_max" : "parpy_min") + (ok ? "<int>(" : "<int64_t>(") + as + ", " + bs + ")";
        else
          r.s = "(" + as + " " + cop(op) + " " + bs + ")";
        return r;
      }
      default:
        r.s = pexpr_plain(e);
        return r;
    }
  }

  static std::string paren(const std::string& s) {
    if (!s.empty() && s.front() == '(' && s.back() == ')') {
      int depth = 0;
      bool wraps = true;
      for (size_t k = 0; k < s.size(); ++k) {
        if (s[k] == '(') ++depth;
        else if (s[k] == ')') { --depth; if (depth == 0 && k + 1 != s.size()) { wraps = false; break; } }
      }
      if (wraps) return s;
    }
    return "(" + s + ")";
  }

  static const char* cop(BinOp op) {
    switch (op) {
      case BinOp::FloorDiv: return "/";
      case BinOp::Pow: return "**";
      default: return binop_name(op);
    }
  }

  std::string math_fn(const char* base, ElemSize sz, bool fast) {
    // single precision uses the hardware approximations (v_exp_f32, v_log_f32, ...)
    // like the reference's CUDA backend does (src/cuda/pprint.rs:70-92)
    if (sz == ElemSize::F64) return base;
    if (fast) return std::string("__") + base + "f";
    return std::string(base) + "f";
  }

  // accesses that must be coherent across the device: global elements of arrays that a kernel with
  // device-wide barriers may write (everything that is not a read-only parameter)
  bool as_lvalue = false;
  bool wide_division = false;   // set while printing an expression that contains a 64-bit quotient or remainder
  bool exchanged(const E& e) const {
    if (!kernel || !kernel->no_restrict || e->k != Expr::Index) return false;
    const E& base = e->args[0];
    if (base->ty.mem == Mem::LDS || elem_bytes(e->ty.sz) < 4) return false;
    return !read_only_param(base);
  }

  // fp32 values that come straight from memory (a load, or a variable that only names one): what the compiler
  // would have to quiet before a max / min; maxima and minima of such values count as well, since they are
  // printed as opaque instructions
  std::set<Name> loaded_f32;
  static bool float_literal(const E& x) {
    return x->k == Expr::Float || (x->k == Expr::UnOpE && x->uop == UnOp::Sub && x->args[0]->k == Expr::Float) ||
           (x->k == Expr::Convert && float_literal(x->args[0]));
  }
  bool straight_from_memory(const E& x) const {
    if (x->k == Expr::Index || x->k == Expr::RegElem) return true;
    if (x->k == Expr::Var) return loaded_f32.count(x->name) > 0;
    if (x->k == Expr::BinOpE && (x->bop == BinOp::Max || x->bop == BinOp::Min) && x->args[0]->ty.sz == ElemSize::F32)
      return straight_from_memory(x->args[0]) || straight_from_memory(x->args[1]);
    return false;
  }

  std::string pexpr(const E& e) {
    if (is_i64(e)) return pint(e).s;
    return pexpr_plain(e);
  }

  std::string pexpr_plain(const E& e) {
    switch (e->k) {
      case Expr::Var: return e->name.str();
      case Expr::Int: {
        if (e->ty.is_scalar() && elem_bytes(e->ty.sz) == 8) {
          if (e->ty.sz == ElemSize::U64) return "((uint64_t)" + std::to_string((uint64_t)e->iv) + "ULL)";
          if (e->iv == INT64_MIN) return "((int64_t)(-9223372036854775807LL - 1))";
          return "((int64_t)" + std::to_string(e->iv) + "LL)";
        }
        if (e->ty.is_scalar() && e->ty.sz != ElemSize::I32) return "((" + std::string(elem_ctype(e->ty.sz)) + ")" + std::to_string(e->iv) + ")";
        return e->iv < 0 ? "(" + std::to_string(e->iv) + ")" : std::to_string(e->iv);
      }
      case Expr::Float: {
        // negative literals are parenthesised: `-` in front of one must not read as a decrement
        bool neg = std::signbit(e->fv) && !std::isnan(e->fv) && !std::isinf(e->fv);
        if (e->ty.sz == ElemSize::F64) return neg ? "(" + fmt_f64(e->fv) + ")" : fmt_f64(e->fv);
        if (e->ty.sz == ElemSize::F16) return "((_Float16)" + fmt_f32(e->fv) + ")";
        return neg ? "(" + fmt_f32(e->fv) + ")" : fmt_f32(e->fv);
      }
      case Expr::Bool: return e->bv ? "true" : "false";
      case Expr::UnOpE: {
        std::string a = pexpr(e->args[0]);
        ElemSize sz = e->ty.sz;
        bool f16 = sz == ElemSize::F16;
        auto call = [&](const std::string& fn) {
          if (f16) return "((_Float16)" + fn + "((float)" + paren(a) + "))";
          return fn + paren(a);
        };
        switch (e->uop) {
          case UnOp::Sub: return "(-" + paren(a) + ")";
          case UnOp::Not: return "(!" + a + ")";
          case UnOp::BitNeg: return "(~" + a + ")";
          // single precision: the hardware base-2 instructions with the scale folded in
          // (v_exp_f32 / v_log_f32, about 1 ulp, no denormal fix-up)
          case UnOp::Exp:
            if (sz == ElemSize::F32) return "__builtin_amdgcn_exp2f(1.44269504088896341f * " + paren(a) + ")";
            return call(math_fn("exp", f16 ? ElemSize::F32 : sz, true));
          case UnOp::Log:
            if (sz == ElemSize::F32) return "(0.693147180559945309f * __builtin_amdgcn_logf" + paren(a) + ")";
            return call(math_fn("log", f16 ? ElemSize::F32 : sz, true));
          case UnOp::Cos: return call(math_fn("cos", f16 ? ElemSize::F32 : sz, true));
          case UnOp::Sin: return call(math_fn("sin", f16 ? ElemSize::F32 : sz, true));
          case UnOp::Sqrt: return call(math_fn("sqrt", f16 ? ElemSize::F32 : sz, false));
          case UnOp::Tanh: return call(math_fn("tanh", f16 ? ElemSize::F32 : sz, false));
          case UnOp::Abs:
            if (is_float(sz)) return call(math_fn("fabs", f16 ? ElemSize::F32 : sz, false));
            return "(" + a + " < 0 ? -" + a + " : " + a + ")";
        }
        return a;
      }
      case Expr::BinOpE: {
        std::string a = pexpr(e->args[0]), b = pexpr(e->args[1]);
        ElemSize sz = e->args[0]->ty.sz;
        switch (e->bop) {
          case BinOp::Max: case BinOp::Min: {
            const char* base = e->bop == BinOp::Max ? "max" : "min";
            if (sz == ElemSize::F32 && straight_from_memory(e)) {
              // one v_max / v_min, or v_max3 / v_min3 for a nested pair (see the preamble for why not fmaxf)
              auto same = [&](const E& x) { return x->k == Expr::BinOpE && x->bop == e->bop && x->args[0]->ty.sz == ElemSize::F32; };
              std::string f = std::string("parpy_f") + base;
              if (float_literal(e->args[1])) {
                if (same(e->args[0]) && !float_literal(e->args[0]->args[0]) && !float_literal(e->args[0]->args[1]))
                  return f + "3c(" + pexpr(e->args[0]->args[0]) + ", " + pexpr(e->args[0]->args[1]) + ", " + b + ")";
                return f + "c(" + a + ", " + b + ")";
              }
              if (float_literal(e->args[0])) return f + "c(" + b + ", " + a + ")";
              if (same(e->args[0]) && !float_literal(e->args[0]->args[0]) && !float_literal(e->args[0]->args[1]))
                return f + "3(" + pexpr(e->args[0]->args[0]) + ", " + pexpr(e->args[0]->args[1]) + ", " + b + ")";
              if (same(e->args[1]) && !float_literal(e->args[1]->args[0]) && !float_literal(e->args[1]->args[1]))
                return f + "3(" + a + ", " + pexpr(e->args[1]->args[0]) + ", " + pexpr(e->args[1]->args[1]) + ")";
              return f + "(" + a + ", " + b + ")";
            }
            if (sz == ElemSize::F32) return std::string("f") + base + "f(" + a + ", " + b + ")";
            if (sz == ElemSize::F64) return std::string("f") + base + "(" + a + ", " + b + ")";
            if (sz == ElemSize::F16) return std::string("((_Float16)f") + base + "f((float)" + paren(a) + ", (float)" + paren(b) + "))";
            return std::string("parpy_") + base + "<" + elem_ctype(sz) + ">(" + a + ", " + b + ")";
          }
          case BinOp::FloorDiv: case BinOp::Div: case BinOp::Rem: {
            // A quotient or remainder of 64-bit integers whose operands provably fit 31 bits is computed in 32
            // bits (one multiply-high for a constant divisor instead of a 64-bit sequence).  The wide form is also
            // kept out of 32-bit offsets (see `parpy_at`): a 64-bit division by a constant whose result was only
            // used truncated to 32 bits has produced wrong element offsets on gfx950 (the same source with the
            // 32-bit division is correct), so such an index stays a plain 64-bit one.
            bool wide = e->ty.is_scalar() && (e->ty.sz == ElemSize::I64 || e->ty.sz == ElemSize::U64) && e->args[0]->ty.is_scalar() &&
                        is_int(e->args[0]->ty.sz) && e->args[1]->ty.is_scalar() && is_int(e->args[1]->ty.sz);
            if (wide) {
              Interval ra = expr_range(e->args[0], ranges), rb = expr_range(e->args[1], ranges);
              if (ra.known && rb.known && ra.lo >= 0 && ra.hi <= INT32_MAX && rb.lo > 0 && rb.hi <= INT32_MAX)
                return "((" + std::string(elem_ctype(e->ty.sz)) + ")((int)" + paren(a) + " " + cop(e->bop) + " (int)" + paren(b) + "))";
              wide_division = true;
            }
            return "(" + a + " " + cop(e->bop) + " " + b + ")";
          }
          case BinOp::Atan2: return std::string(sz == ElemSize::F64 ? "atan2" : "atan2f") + "(" + a + ", " + b + ")";
          case BinOp::Pow: return std::string(sz == ElemSize::F64 ? "pow" : "__powf") + "(" + a + ", " + b + ")";
          default: return "(" + a + " " + cop(e->bop) + " " + b + ")";
        }
      }
      case Expr::IfExpr: return "(" + pexpr(e->args[0]) + " ? " + pexpr(e->args[1]) + " : " + pexpr(e->args[2]) + ")";
      case Expr::Convert: return "((" + std::string(elem_ctype(e->ty.sz)) + ")" + paren(pexpr(e->args[0])) + ")";
      case Expr::Index: {
        if (!as_lvalue) {
          if (cur_pack_loads) {
            auto pk = cur_pack_loads->find(e.get());
            if (pk != cur_pack_loads->end()) return pk->second;
          }
        }
        // Indexing is in bounds by contract: a variable used as the index of one dimension lies in
        // [0, extent) while this address is computed, which lets gathered indices (loaded from memory,
        // so of unknown range) take part in 32-bit address arithmetic.
        std::vector<Name> assumed;
        std::vector<std::pair<Name, Interval>> narrowed;
        for (size_t d = 0; d < e->dim_idx.size() && d < e->dim_shape.size(); ++d) {
          E x = e->dim_idx[d];
          while (x->k == Expr::Convert && x->ty.is_scalar() && is_int(x->ty.sz) && x->args[0]->ty.is_scalar() && is_int(x->args[0]->ty.sz) &&
                 elem_bytes(x->ty.sz) >= elem_bytes(x->args[0]->ty.sz))
            x = x->args[0];  // (a narrow index widened: same value)
          if (!(x->k == Expr::Var && x->ty.is_scalar() && is_int(x->ty.sz))) continue;
          Interval r;
          r.known = true;
          r.lo = 0;
          r.hi = e->dim_shape[d] - 1;
          auto it = ranges.find(x->name);
          if (it == ranges.end()) {
            assumed.push_back(x->name);
          } else {
            // a range that is only the variable's type (an int8 observation: -128..127) is cut to the extent
            if (!it->second.known || (it->second.lo >= 0 && it->second.hi <= r.hi)) continue;
            narrowed.push_back({x->name, it->second});
            r.lo = std::max(r.lo, it->second.lo);
            r.hi = std::min(r.hi, it->second.hi);
            if (r.lo > r.hi) { narrowed.pop_back(); continue; }
          }
          ranges[x->name] = r;
        }
        std::string out = pexpr(e->args[0]) + "[" + pexpr(e->args[1]) + "]";
        if (opts.opt_offset32 && e->args[0]->ty.mem != Mem::LDS && read_only_param(e->args[0]) && !walks_sequentially(e->args[1])) {
          // An element whose byte offset provably fits 32 bits is addressed as base + 32-bit offset, the
          // form the global memory instructions take (64-bit scalar base, 32-bit per-lane offset): no
          // sign extension and no 64-bit add per access.  Matters where address arithmetic competes with
          // the computation for the vector ALU (a 262144-state HMM step in global memory: 61 -> 55 us).
          // Only arrays the kernel never writes: with offsets that wrap modulo 2^32 the device compiler can no
          // longer tell that a store to a[i] leaves a[i + 4] alone, and loops that update an array in place
          // were serialised (softmax over rows of 10^6 floats on 64 threads: 2.8 -> 3.6 ms).  For the same
          // reason an index that advances with a sequential loop keeps its plain form: there the device
          // compiler's own strength reduction and wide loads are worth more (one thread summing a row of
          // 10^5 floats: 0.7 ms against 1.1 ms).
          Interval r = expr_range(e->args[1], ranges);
          int64_t eb = elem_bytes(e->ty.sz);
          if (r.known && r.lo >= 0 && r.hi * eb + eb <= (int64_t)UINT32_MAX) {
            bool outer = wide_division;
            wide_division = false;
            std::string idx = pexpr(e->args[1]);
            if (!wide_division) out = "parpy_at(" + pexpr(e->args[0]) + ", (unsigned)(" + idx + "))";
            wide_division = wide_division || outer;
          }
        }
        for (auto& n : assumed) ranges.erase(n);
        for (auto& kv : narrowed) ranges[kv.first] = kv.second;
        // Workgroups of this kernel exchange data through global memory between device-wide barriers: what is
        // not read-only is loaded and stored at device scope (past the caches that are private to a compute
        // unit or a die), so the barrier itself needs no cache write-back or invalidation.
        if (exchanged(e) && !as_lvalue)
          return "__hip_atomic_load(&" + out + ", __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)";
        return out;
      }
      case Expr::AddrOf: return "(&" + pexpr(e->args[0]) + "[" + pexpr(e->args[1]) + "])";
      case Expr::ThreadIdx: case Expr::BlockIdx: return "((int64_t)" + idx_name(e->k, (int)e->iv) + ")";
      case Expr::RegElem: return e->name.str() + "[" + pexpr(e->args[0]) + "]";
      case Expr::Raw: return e->sval;
      case Expr::Call: {
        std::string out = (e->ext ? e->ext->name : e->sval) + "(";
        for (size_t a = 0; a < e->args.size(); ++a) out += (a ? ", " : "") + pexpr(e->args[a]);
        return out + ")";
      }
      default: fail_rt(e->i, "Cannot print expression " + print_expr(e) + " (internal error)");
    }
  }

  // ---------------------------------------------------------------- statements
  static void find_reassigned(const Stmts& ss, std::set<Name>& out) {
    for (auto& s : ss) {
      if (s->k == Stmt::Assign && s->dst->k == Expr::Var) out.insert(s->dst->name);
      if (s->k == Stmt::WaveReduce) out.insert(s->id);
      find_reassigned(s->body, out);
      find_reassigned(s->els, out);
    }
  }

  std::set<Name> seq_loop_vars;   // variables of the enclosing sequential loops that are kept as loops

  bool walks_sequentially(const E& idx) const {
    bool hit = false;
    visit_exprs(idx, [&](const E& x) { if (x->k == Expr::Var && seq_loop_vars.count(x->name)) hit = true; });
    return hit;
  }

  bool read_only_param(const E& base) const {
    if (base->k != Expr::Var) return false;
    for (auto& p : kernel->params)
      if (p.id == base->name) return p.read_only;
    return false;
  }

  std::string map_index(const GpuMap& m) {
    switch (m.k) {
      case GpuMap::Thread: return "(int)threadIdx." + std::string(1, "xyz"[m.dim]);
      case GpuMap::Block: {
        int64_t tot = m.dim == 0 ? kernel->grid.x : m.dim == 1 ? kernel->grid.y : kernel->grid.z;
        std::string b = "(int)blockIdx." + std::string(1, "xyz"[m.dim]);
        if (tot > m.n) return "((" + b + " / " + std::to_string(m.mult) + ") % " + std::to_string(m.n) + ")";
        return b;
      }
      case GpuMap::ThreadBlock:
        return "((int)blockIdx.x * " + std::to_string(m.tpb) + " + (int)threadIdx.x)";
      default: return "0";
    }
  }

  Interval map_index_range(const GpuMap& m) {
    Interval r;
    r.known = true;
    r.lo = 0;
    r.hi = m.k == GpuMap::ThreadBlock ? (m.n + m.tpb - 1) / m.tpb * m.tpb - 1 : m.n - 1;
    return r;
  }

  static bool reads_and_writes_lds(const Stmts& body) {
    bool rd = false, wr = false;
    visit_stmts(body, [&](const S& c) {
      if (c->k == Stmt::Assign && c->dst->k == Expr::Index && c->dst->args[0]->ty.mem == Mem::LDS) wr = true;
      auto scan = [&](const E& root, bool skip_root) {
        visit_exprs(root, [&](const E& x) {
          if (x->k == Expr::Index && x->args[0]->ty.mem == Mem::LDS && !(skip_root && x.get() == root.get())) rd = true;
        });
      };
      if (c->expr) scan(c->expr, false);
      if (c->dst) scan(c->dst, c->k == Stmt::Assign);
    });
    return rd && wr;
  }

  void pfor(const S& s, int n) {
    Interval lo = expr_range(s->lo, ranges), hi = expr_range(s->hi, ranges);
    bool is64 = s->lo->ty.is_scalar() && s->lo->ty.sz == ElemSize::I64;
    Interval vr;
    if (lo.known && hi.known) {
      vr.known = true;
      vr.lo = s->step > 0 ? lo.lo : hi.lo + 1;
      vr.hi = s->step > 0 ? std::max(hi.hi - 1, lo.lo) : lo.hi;
    }
    bool narrow = opts.opt_narrow_index && is64 && fits32(vr) && !reassigned.count(s->id);
    // the strided increment may step past hi by up to step * N before the loop test fails
    int64_t stride = s->step * (s->map.k == GpuMap::None ? 1 : s->map.n);
    if (narrow && !(vr.hi + std::abs(stride) <= INT32_MAX && vr.lo - std::abs(stride) >= INT32_MIN)) narrow = false;
    std::string vty = narrow ? "int" : elem_ctype(s->lo->ty.sz);
    std::string v = s->id.str();
    if (vr.known && !reassigned.count(s->id)) ranges[s->id] = vr;
    if (narrow) narrow_vars.insert(s->id);
    const char* cmp = s->step > 0 ? " < " : " > ";
    std::string los = pexpr(s->lo), his = pexpr(s->hi);

    if (s->map.k == GpuMap::None) {
      if (s->unroll) os << ind(n) << "#pragma unroll\n";
      os << ind(n) << "for (" << vty << " " << v << " = " << los << "; " << v << cmp << his << "; " << v << " += " << s->step << ") {\n";
      bool fresh = !s->unroll && seq_loop_vars.insert(s->id).second;
      pstmts(s->body, n + 2);
      if (fresh) seq_loop_vars.erase(s->id);
      os << ind(n) << "}\n";
      return;
    }
    const GpuMap& m = s->map;
    std::string idx = map_index(m);
    int64_t N = m.n;
    bool const_bounds = s->lo->k == Expr::Int && s->hi->k == Expr::Int;
    int64_t extent = 0;
    if (const_bounds)
      extent = s->step > 0 ? (s->hi->iv - s->lo->iv + s->step - 1) / s->step : (s->lo->iv - s->hi->iv - s->step - 1) / (-s->step);
    int64_t launched = m.k == GpuMap::ThreadBlock ? (m.n + m.tpb - 1) / m.tpb * m.tpb : m.n;
    std::string guard;
    if (m.k == GpuMap::ThreadBlock && launched != m.n) guard = idx + " < " + std::to_string(m.n);
    std::string stepmul = s->step == 1 ? "" : std::to_string(s->step) + " * ";
    auto init = [&](const std::string& i) {
      if (s->lo->k == Expr::Int && s->lo->iv == 0) return stepmul + i;
      return los + " + " + stepmul + i;
    };
    if (const_bounds && extent <= N) {
      // every thread (block) runs at most one iteration: no loop
      os << ind(n) << "{\n";
      os << ind(n + 2) << vty << " " << v << " = " << init(idx) << ";\n";
      std::string cond;
      if (extent < launched) cond = v + cmp + his;
      if (!guard.empty() && cond.empty()) cond = guard;  // v < hi already implies the launch guard (extent <= N)
      if (!cond.empty()) {
        os << ind(n + 2) << "if (" << cond << ") {\n";
        pstmts(s->body, n + 4);
        os << ind(n + 2) << "}\n";
      } else {
        pstmts(s->body, n + 2);
      }
      os << ind(n) << "}\n";
      return;
    }
    if (const_bounds && guard.empty() && counted_trips(extent, N) > 0) {
      // every thread runs the same, compile-time known number of iterations (the last one guarded when N does
      // not divide the extent)
      int64_t per = counted_trips(extent, N);
      bool ragged = extent % N != 0;
      std::string k = v + "_k";
      {
        // the iteration counter can be named by the memory passes (register array slots)
        Interval kr;
        kr.known = true;
        kr.lo = 0;
        kr.hi = per - 1;
        ranges[Name{k, 0}] = kr;
        narrow_vars.insert(Name{k, 0});
      }
      // what the thread's iterations have in common (kept in `els` by the pass that finds it) comes first, in
      // terms of the thread's first iteration `<v>_g`
      bool shared_first = !s->els.empty();
      if (shared_first) {
        os << ind(n) << "{\n";
        n += 2;
        Interval gr;
        gr.known = true;
        gr.lo = 0;
        gr.hi = N - 1;
        ranges[Name{v + "_g", 0}] = gr;
        if (narrow) narrow_vars.insert(Name{v + "_g", 0});
        os << ind(n) << vty << " " << v << "_g = " << idx << ";\n";
        pstmts(s->els, n);
      }
      if (s->unroll) {
        os << ind(n) << "#pragma unroll\n";
      } else {
        // Left alone, the device compiler unrolls a loop of 16 iterations completely: 16 vector loads in flight
        // per thread need more than 64 registers, and a 1024-thread workgroup then has its CU to itself, with
        // nothing to overlap its load, reduce and store phases.  A few iterations in flight are enough (row sums
        // of 65536 floats on 1024 threads per row: 47.8 -> 40.3 us; smaller workgroups are unrolled four times
        // by default anyway).
        int64_t threads = kernel->block.x * kernel->block.y * kernel->block.z;
        os << ind(n) << "#pragma unroll " << (threads >= 1024 ? 2 : 4) << "\n";
      }
      os << ind(n) << "for (int " << k << " = 0; " << k << " < " << per << "; ++" << k << ") {\n";
      os << ind(n + 2) << vty << " " << v << " = " << init("(" + (shared_first ? v + "_g" : idx) + " + " + k + " * " + std::to_string(N) + ")") << ";\n";
      if (ragged) {
        os << ind(n + 2) << "if (" << v << cmp << his << ") {\n";
        pstmts(s->body, n + 4);
        os << ind(n + 2) << "}\n";
      } else {
        pstmts(s->body, n + 2);
      }
      if (kernel->fence_lds_iterations && s->unroll && per > 1 && reads_and_writes_lds(s->body)) {
        // Left to itself the device compiler issues the LDS loads of all unrolled iterations first.  Every wave of
        // the workgroup then queues at the LDS at the same moment (they have just left the same barrier) with the
        // vector ALU idle, and computes afterwards with the LDS idle.  With the iterations kept apart the waves
        // drift out of step and one wave's arithmetic covers another's LDS traffic (scaled 7-mer HMM step: 19.0 ->
        // 17.8 ms per batch).  Only for steps without exponentials or logarithms: those are bound by the vector
        // ALU and lose a little (reference form 56.8 -> 58.2 ms), the grouped form neither gains nor loses.
        os << ind(n + 2) << "__builtin_amdgcn_sched_barrier(0);\n";
      }
      os << ind(n) << "}\n";
      if (shared_first) {
        n -= 2;
        os << ind(n) << "}\n";
      }
      return;
    }
    std::string cond = v + cmp + his;
    if (!guard.empty()) cond += " && " + guard;
    {
      // a strided loop whose trip count differs per thread is not unrolled by the compiler on its own; with one
      // iteration at a time every thread has a single load in flight.  Four iterations per round trip let the
      // loads of the next three issue before the first is used (arithmetic stays in program order).  Measured on a
      // 10 x 1e8 row sum: 2.6 -> 4.8 TB/s with 32 blocks per row, 320 -> 580 GB/s with one; 8 and 16 are no better.
      bool plain = true;
      visit_stmts(s->body, [&](const S& c) {
        if (c->k == Stmt::Sync || c->k == Stmt::While || c->k == Stmt::RawStmt || (c->k == Stmt::For && !c->unroll)) plain = false;
      });
      if (plain) os << ind(n) << "#pragma unroll 4\n";
    }
    os << ind(n) << "for (" << vty << " " << v << " = " << init(idx) << "; " << cond << "; " << v << " += "
       << (s->step * N) << ") {\n";
    pstmts(s->body, n + 2);
    os << ind(n) << "}\n";
  }

  void pstmt(const S& s, int n) {
    switch (s->k) {
      case Stmt::Def: {
        Interval r = expr_range(s->expr, ranges);
        bool is64 = s->ty.is_scalar() && s->ty.sz == ElemSize::I64;
        bool fixed = !reassigned.count(s->id);
        if (fixed && r.known) ranges[s->id] = r;
        if (fixed && s->ty.is_scalar() && s->ty.sz == ElemSize::F32 && s->expr && straight_from_memory(s->expr)) loaded_f32.insert(s->id);
        bool narrow = opts.opt_narrow_index && is64 && fixed && fits32(r);
        if (narrow) narrow_vars.insert(s->id);
        std::string rhs = pexpr(s->expr);
        // aliases may point at read-only parameters: the qualifier is dropped, stores never go through them
        if (!s->ty.is_scalar()) rhs = "(" + ctype(s->ty) + ")" + rhs;
        os << ind(n) << (narrow ? std::string("int") : ctype(s->ty)) << " " << s->id.str() << " = " << rhs << ";\n";
        break;
      }
      case Stmt::Assign: {
        std::string rhs = pexpr(s->expr);
        if (s->dst->k == Expr::Var && !s->dst->ty.is_scalar()) rhs = "(" + ctype(s->dst->ty) + ")" + rhs;
        {
          if (cur_pack_store.first >= 0) {
            os << ind(n) << packs[cur_pack_store.first].var << "." << "xyzw"[cur_pack_store.second] << " = " << rhs << ";\n";
            break;
          }
        }
        if (s->dst->k == Expr::Index && s->dst->args[0]->k == Expr::Var && stream_out.count(s->dst->args[0]->name) &&
            elem_bytes(s->dst->ty.sz) >= 4) {
          // write-once data bypasses the caches on its way to HBM (measured: 7.1 instead of 5.8 TB/s on a plain copy)
          os << ind(n) << "__builtin_nontemporal_store((" << elem_ctype(s->dst->ty.sz) << ")" << paren(rhs) << ", &" << pexpr(s->dst) << ");\n";
          break;
        }
        if (s->dst->k == Expr::Index && exchanged(s->dst)) {
          as_lvalue = true;
          std::string lhs = pexpr(s->dst);
          as_lvalue = false;
          os << ind(n) << "__hip_atomic_store(&" << lhs << ", (" << elem_ctype(s->dst->ty.sz) << ")" << paren(rhs)
             << ", __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n";
          break;
        }
        os << ind(n) << pexpr(s->dst) << " = " << rhs << ";\n";
        break;
      }
      case Stmt::For: pfor(s, n); break;
      case Stmt::While:
        os << ind(n) << "while (" << pexpr(s->expr) << ") {\n";
        pstmts(s->body, n + 2);
        os << ind(n) << "}\n";
        break;
      case Stmt::If:
        os << ind(n) << "if " << paren(pexpr(s->expr)) << " {\n";
        pstmts(s->body, n + 2);
        if (!s->els.empty()) {
          os << ind(n) << "} else {\n";
          pstmts(s->els, n + 2);
        }
        os << ind(n) << "}\n";
        break;
      case Stmt::Sync: os << ind(n) << "__syncthreads();\n"; break;
      case Stmt::Return: os << ind(n) << "return " << pexpr(s->expr) << ";\n"; break;   // (device functions only)
      case Stmt::Scope:
        if (!s->args.empty()) {
          // an immediately invoked, always inlined lambda: its restrict-qualified parameters shadow
          // the pointer variables of the same names, which is how the no-alias fact reaches the optimiser
          std::string params, actuals;
          for (size_t a = 0; a < s->args.size(); ++a) {
            params += (a ? ", " : "") + ctype(s->args[a]->ty) + " __restrict__ " + s->args[a]->name.str();
            actuals += (a ? ", " : "") + s->args[a]->name.str();
          }
          os << ind(n) << "[&](" << params << ") __attribute__((always_inline)) {\n";
          pstmts(s->body, n + 2);
          os << ind(n) << "}(" << actuals << ");\n";
          break;
        }
        os << ind(n) << "{\n";
        pstmts(s->body, n + 2);
        os << ind(n) << "}\n";
        break;
      case Stmt::WaveReduce: {
        int64_t nwaves = std::max<int64_t>(1, s->iv / WAVE_SIZE);
        std::string ty = elem_ctype(s->ty.sz);
        std::string op = std::string("parpy_op_") + red_suffix(s->bop);
        std::string v = s->id.str();
        if (nwaves == 1) {
          os << ind(n) << v << " = parpy_wave_reduce<" << op << ">(" << v << ");\n";
        } else {
          std::string slots = "parpy_red_" + std::to_string(red_sites++);
          lds_decls.push_back("__shared__ " + ty + " " + slots + "[" + std::to_string(nwaves) + "];");
          E ne = neutral_element(s->bop == BinOp::And ? BinOp::BitAnd : s->bop == BinOp::Or ? BinOp::BitOr : s->bop, s->ty.sz, s->i);
          os << ind(n) << v << " = parpy_block_reduce<" << op << ", " << nwaves << ">(" << v << ", (" << ty << ")" << pexpr(ne)
             << ", " << slots << ", " << (s->unroll ? "true" : "false") << ");\n";
        }
        break;
      }
      case Stmt::LdsDecl:
        lds_decls.push_back("__shared__ __attribute__((aligned(16))) " + std::string(elem_ctype(s->ty.sz)) + " " + s->id.str() + "[" +
                            std::to_string(s->iv) + "];");
        break;
      case Stmt::RegDecl:
        os << ind(n) << elem_ctype(s->ty.sz) << " " << s->id.str() << "[" << s->iv << "];\n";
        break;
      case Stmt::RawStmt: os << ind(n) << s->fname << "\n"; break;
      default:
        fail_rt(s->i, "Statement kind not supported in device code (internal error)");
    }
  }

  // ---- four adjacent 4-byte accesses of one iteration as one 16-byte access
  // `x0 = a[4q]; ...; b[4q] = r0; x1 = a[4q + 1]; ...; b[4q + 1] = r1; ...` (what a loop over the four
  // elements of a group becomes once it is expanded): the four loads are issued as one vector load where the
  // first of them stands, the four stores as one vector store where the last of them stands.  The device
  // compiler does not do this by itself when `a` and `b` are pointers that may name the same array; it is safe
  // here because an access that changes places only passes accesses to other elements: a store to y[f + c1] and a
  // load of x[f + c2] with c1 != c2 never touch the same element, whether or not x and y are the same array, and
  // accesses to LDS and to global memory never do.  On LDS this is the difference between four partial-bank
  // accesses and one full-rate one per lane.
  struct Pack { std::string var, decl_ty, addr; bool is_store = false, streamed = false; size_t first = 0, last = 0; const Stmts* owner = nullptr; };
  // Plans are kept per place (block and position in it), not per node: expression and statement nodes are
  // shared between the copies that loop expansion and unswitching make.
  using Place = std::pair<const Stmts*, size_t>;
  std::map<Place, std::map<const Expr*, std::string>> pack_loads;  // statement -> its load expressions -> "pk.x"
  std::map<Place, std::pair<int, int>> pack_stores;                // store statement -> (pack index, component)
  const std::map<const Expr*, std::string>* cur_pack_loads = nullptr;   // of the statement being printed
  std::pair<int, int> cur_pack_store{-1, -1};
  std::vector<Pack> packs;
  int pack_counter = 0;

  static bool multiple_of_four(const E& e) {
    if (e->k == Expr::Int) return e->iv % 4 == 0;
    if (e->k == Expr::Convert) return multiple_of_four(e->args[0]);
    if (e->k != Expr::BinOpE) return false;
    if (e->bop == BinOp::Mul) return (e->args[0]->k == Expr::Int && e->args[0]->iv % 4 == 0) || (e->args[1]->k == Expr::Int && e->args[1]->iv % 4 == 0);
    if (e->bop == BinOp::Add || e->bop == BinOp::Sub) return multiple_of_four(e->args[0]) && multiple_of_four(e->args[1]);
    return false;
  }
  // idx == f + c with f a multiple of four and 0 <= c < 4; the constant may sit anywhere in a sum
  static void sum_terms(const E& e, std::vector<E>& terms, int64_t& c) {
    if (e->k == Expr::BinOpE && e->bop == BinOp::Add) { sum_terms(e->args[0], terms, c); sum_terms(e->args[1], terms, c); return; }
    if (e->k == Expr::Int) { c += e->iv; return; }
    terms.push_back(e);
  }
  static bool split_offset(const E& idx, E* f, int64_t* c) {
    std::vector<E> terms;
    int64_t k = 0;
    sum_terms(idx, terms, k);
    if (terms.empty()) return false;
    for (auto& t : terms) if (!multiple_of_four(t)) return false;
    int64_t base = k - (((k % 4) + 4) % 4);
    E sum = terms[0];
    for (size_t i = 1; i < terms.size(); ++i) sum = mk_binop(BinOp::Add, sum, terms[i], idx->ty);
    if (base != 0) sum = mk_binop(BinOp::Add, sum, mk_int(base, idx->ty.sz), idx->ty);
    *f = sum;
    *c = k - base;
    return true;
  }
  bool packable(const E& x) const {
    if (x->k != Expr::Index || x->args[0]->k != Expr::Var || elem_bytes(x->ty.sz) != 4 || !x->ty.is_scalar()) return false;
    const E& base = x->args[0];
    if (exchanged(x)) return false;
    if (base->ty.mem == Mem::LDS) return true;
    // global: a parameter of a kernel whose pointer arguments are 16-byte aligned
    if (!kernel->aligned_params) return false;
    for (auto& p : kernel->params)
      if (p.id == base->name) return p.ty.k == Type::Pointer;
    return false;
  }

  // two different names that cannot stand for the same memory: arrays declared in LDS, pointer parameters that
  // carry the no-alias promise, local pointers that the alias analysis found never to coincide
  bool distinct_arrays(const Name& a, const Name& b) const {
    if (lds_arrays.count(a) && lds_arrays.count(b)) return true;
    if (!kernel->no_restrict) {
      bool pa = false, pb = false;
      for (auto& p : kernel->params) {
        if (p.ty.k != Type::Pointer) continue;
        pa = pa || p.id == a;
        pb = pb || p.id == b;
      }
      if (pa && pb) return true;
    }
    for (auto& g : kernel->distinct_pointers)
      if (std::find(g.begin(), g.end(), a) != g.end() && std::find(g.begin(), g.end(), b) != g.end()) return true;
    return false;
  }

  struct Access { size_t pos; const Expr* e; const Stmt* st; bool store; Name base; Mem mem; E f; int64_t c; bool tracked; };

  void plan_packs(const Stmts& ss, size_t lo, size_t hi) {
    // every element access of the run in program order (an assignment evaluates its right-hand side first)
    std::vector<Access> acc;
    for (size_t i = lo; i < hi; ++i) {
      const S& st = ss[i];
      auto scan = [&](const E& root) {
        visit_exprs(root, [&](const E& x) {
          if (x->k != Expr::Index) return;
          Access a{i, x.get(), st.get(), false, x->args[0]->k == Expr::Var ? x->args[0]->name : Name(), x->args[0]->ty.mem, E(), 0, false};
          a.tracked = x->args[0]->k == Expr::Var && split_offset(x->args[1], &a.f, &a.c);
          acc.push_back(a);
        });
      };
      if (st->expr) scan(st->expr);
      if (st->k == Stmt::Assign && st->dst->k == Expr::Index) {
        scan(st->dst->args[1]);
        Access a{i, st->dst.get(), st.get(), true, st->dst->args[0]->k == Expr::Var ? st->dst->args[0]->name : Name(), st->dst->args[0]->ty.mem, E(), 0, false};
        a.tracked = st->dst->args[0]->k == Expr::Var && split_offset(st->dst->args[1], &a.f, &a.c);
        acc.push_back(a);
      } else if (st->dst) {
        scan(st->dst);
      }
    }
    auto independent = [&](const Access& a, const Access& b) {
      if (a.mem != b.mem) return true;                                   // LDS and global memory are disjoint
      if (!(a.base == b.base) && distinct_arrays(a.base, b.base)) return true;
      if (a.tracked && b.tracked && expr_eq(a.f, b.f) && a.c != b.c) return true;   // other elements of the same group
      return false;
    };
    auto lookup = [&](const Access& a) -> E {
      for (size_t i = lo; i < hi; ++i) {
        E found;
        auto scan = [&](const E& root) { visit_exprs(root, [&](const E& x) { if (x.get() == a.e) found = x; }); };
        if (ss[i]->expr) scan(ss[i]->expr);
        if (ss[i]->dst) scan(ss[i]->dst);
        if (found) return found;
      }
      return E();
    };
    std::set<size_t> used;
    for (size_t i = 0; i < acc.size(); ++i) {
      const Access& a0 = acc[i];
      if (used.count(i) || !a0.tracked || a0.c != 0) continue;
      E e0 = lookup(a0);
      if (!e0 || !packable(e0)) continue;
      // the other three elements, same direction, same array, same f
      size_t member[4] = {i, 0, 0, 0};
      bool ok = true;
      for (int64_t c = 1; c < 4 && ok; ++c) {
        bool found = false;
        for (size_t j = 0; j < acc.size(); ++j)
          if (!used.count(j) && acc[j].tracked && acc[j].store == a0.store && acc[j].base == a0.base && acc[j].c == c && expr_eq(acc[j].f, a0.f)) {
            member[c] = j;
            found = true;
            break;
          }
        ok = found;
      }
      if (!ok) continue;
      // each element of the array may appear once in the group's direction (a second load of a[4q] keeps its place)
      size_t first = i, last = i;
      for (int c = 0; c < 4; ++c) { first = std::min(first, member[c]); last = std::max(last, member[c]); }
      // loads move up to the first member, stores down to the last: everything passed on the way must be independent
      for (int c = 0; c < 4 && ok; ++c) {
        size_t from = a0.store ? member[c] + 1 : first, to = a0.store ? last + 1 : member[c];
        for (size_t j = from; j < to && ok; ++j) {
          bool is_member = false;
          for (int d = 0; d < 4; ++d) is_member = is_member || member[d] == j;
          if (is_member) continue;
          // a load passes stores, a store passes loads and stores
          if (!a0.store && !acc[j].store) continue;
          if (!independent(acc[member[c]], acc[j])) ok = false;
        }
      }
      // the index of the group must not use anything defined or assigned inside the span it moves across
      if (ok) {
        std::set<Name> defined;
        for (size_t s2 = acc[first].pos; s2 <= acc[last].pos && s2 < hi; ++s2)
          if (ss[s2]->k == Stmt::Def) defined.insert(ss[s2]->id);
          else if (ss[s2]->k == Stmt::Assign && ss[s2]->dst->k == Expr::Var) defined.insert(ss[s2]->dst->name);   // `q = q + 1` between two members: same text, other element
        visit_exprs(a0.f, [&](const E& x) { if (x->k == Expr::Var && defined.count(x->name)) ok = false; });
      }
      if (!ok) continue;
      Pack pk;
      pk.var = "pk_" + std::to_string(pack_counter++);
      pk.is_store = a0.store;
      pk.first = acc[first].pos;
      pk.last = acc[last].pos;
      pk.owner = &ss;
      pk.streamed = a0.store && stream_out.count(a0.base) > 0;   // write-once data keeps bypassing the caches
      pk.decl_ty = std::string("parpy_vec4<") + elem_ctype(e0->ty.sz) + ">";
      as_lvalue = true;
      std::string elem = pexpr(e0);
      as_lvalue = false;
      bool lds_ptr = e0->args[0]->ty.mem == Mem::LDS;
      pk.addr = std::string("(") + (lds_ptr ? "__attribute__((address_space(3))) " : "") + (a0.store ? "" : "const ") + pk.decl_ty + "*)&" + elem;
      int pi = (int)packs.size();
      packs.push_back(pk);
      static const char* comp = "xyzw";
      for (int c = 0; c < 4; ++c) {
        used.insert(member[c]);
        if (a0.store) pack_stores[{&ss, acc[member[c]].pos}] = {pi, c};
        else pack_loads[{&ss, acc[member[c]].pos}][acc[member[c]].e] = pk.var + "." + comp[c];
      }
    }
  }

  void pstmts(const Stmts& ss, int n) {
    size_t first_pack = packs.size();
    if (opts.opt_pack_accesses && kernel) {
      // straight-line runs of definitions and assignments
      for (size_t i = 0; i < ss.size();) {
        if (!(ss[i]->k == Stmt::Def || ss[i]->k == Stmt::Assign)) { ++i; continue; }
        size_t j = i;
        while (j < ss.size() && (ss[j]->k == Stmt::Def || ss[j]->k == Stmt::Assign)) ++j;
        if (j - i >= 4) plan_packs(ss, i, j);
        i = j;
      }
    }
    for (size_t i = 0; i < ss.size(); ++i) {
      for (size_t p = first_pack; p < packs.size(); ++p)
        if (packs[p].owner == &ss && packs[p].first == i) {
          if (packs[p].is_store) os << ind(n) << packs[p].decl_ty << " " << packs[p].var << ";\n";
          else os << ind(n) << "const " << packs[p].decl_ty << " " << packs[p].var << " = *" << packs[p].addr << ";\n";
        }
      {
        auto saved_loads = cur_pack_loads;
        auto saved_store = cur_pack_store;
        auto pl = pack_loads.find({&ss, i});
        cur_pack_loads = pl == pack_loads.end() ? nullptr : &pl->second;
        auto ps = pack_stores.find({&ss, i});
        cur_pack_store = ps == pack_stores.end() ? std::pair<int, int>{-1, -1} : ps->second;
        pstmt(ss[i], n);
        cur_pack_loads = saved_loads;
        cur_pack_store = saved_store;
      }
      for (size_t p = first_pack; p < packs.size(); ++p)
        if (packs[p].owner == &ss && packs[p].is_store && packs[p].last == i) {
          if (packs[p].streamed) os << ind(n) << "__builtin_nontemporal_store(" << packs[p].var << ", " << packs[p].addr << ");\n";
          else os << ind(n) << "*" << packs[p].addr << " = " << packs[p].var << ";\n";

        }
    }
  }

  // A jitted function that the kernels call (device_functions option): scalars in, a scalar out, printed through
  // the statement printer of the kernels with the function's parameters in the place of a kernel's.
  std::string device_function_text(const FunDef& f) {
    Kernel k;
    k.name = f.id.str();
    for (auto& q : f.params) {
      KernelParam kp;
      kp.id = q.id;
      kp.ty = q.ty;
      k.params.push_back(kp);
    }
    k.body = f.body;
    k.block = {1, 1, 1};
    k.grid = {1, 1, 1};
    k.cached_stores = true;
    kernel = &k;
    ranges.clear();
    narrow_vars.clear();
    reassigned.clear();
    lds_decls.clear();
    lds_arrays.clear();
    pack_loads.clear();
    pack_stores.clear();
    packs.clear();
    stream_out.clear();
    os.str("");
    find_reassigned(k.body, reassigned);
    // parameters are plain local variables of the function: an assignment to one must not be mistaken for a constant
    pstmts(k.body, 2);
    std::ostringstream out;
    out << "__device__ __forceinline__ " << elem_ctype(f.res_ty.sz) << " " << k.name << "(";
    for (size_t i = 0; i < f.params.size(); ++i) out << (i ? ", " : "") << elem_ctype(f.params[i].ty.sz) << " " << f.params[i].id.str();
    out << ") {\n" << os.str() << "}\n";
    kernel = nullptr;
    return out.str();
  }

  std::string kernel_text(const Kernel& k) {
    kernel = &k;
    ranges.clear();
    narrow_vars.clear();
    reassigned.clear();
    lds_decls.clear();
    lds_arrays.clear();
    visit_stmts(k.body, [&](const S& st) { if (st->k == Stmt::LdsDecl) lds_arrays.insert(st->id); });
    pack_loads.clear();
    pack_stores.clear();
    packs.clear();
    os.str("");
    find_reassigned(k.body, reassigned);
    stream_out.clear();
    if (opts.opt_nontemporal && !k.cached_stores) {
      // parameters that are stored to (directly, never through an alias) and never read in this kernel
      std::set<Name> read, aliased;
      visit_stmts(k.body, [&](const S& st) {
        auto scan = [&](const E& root, bool is_dst) {
          visit_exprs(root, [&](const E& x) {
            if (x->k == Expr::Index && x->args[0]->k == Expr::Var && !(is_dst && x == root)) read.insert(x->args[0]->name);
            if (x->k == Expr::AddrOf) visit_exprs(x->args[0], [&](const E& y) { if (y->k == Expr::Var) aliased.insert(y->name); });
          });
        };
        if (st->dst) scan(st->dst, st->k == Stmt::Assign);
        if (st->expr) scan(st->expr, false);
        if (st->lo) scan(st->lo, false);
        if (st->hi) scan(st->hi, false);
        bool alias_def = (st->k == Stmt::Def && !st->ty.is_scalar()) ||
                         (st->k == Stmt::Assign && st->dst->k == Expr::Var && !st->dst->ty.is_scalar());
        if (alias_def) visit_exprs(st->expr, [&](const E& y) { if (y->k == Expr::Var) aliased.insert(y->name); });
      });
      for (auto& q : k.params)
        if (q.ty.k == Type::Pointer && !q.read_only && !read.count(q.id) && !aliased.count(q.id)) stream_out.insert(q.id);
    }
    pstmts(k.body, 2);
    std::string body = os.str();
    std::ostringstream out;
    int64_t threads = k.block.x * k.block.y * k.block.z;
    out << "extern \"C\" __global__ void __launch_bounds__(" << threads << ") " << k.name << "(";
    for (size_t i = 0; i < k.params.size(); ++i) {
      const auto& p = k.params[i];
      out << (i ? ", " : "");
      if (p.ty.k == Type::Pointer)
        out << (p.read_only ? "const " : "") << elem_ctype(p.ty.sz) << (k.no_restrict && !p.read_only ? "* " : "* __restrict__ ") << p.id.str();
      else out << elem_ctype(p.ty.sz) << " " << p.id.str();
    }
    out << ") {\n";
    for (auto& d : lds_decls) out << "  " << d << "\n";
    if (k.aligned_params)
      for (auto& p : k.params)
        if (p.ty.k == Type::Pointer)
          out << "  " << p.id.str() << " = (" << (p.read_only ? "const " : "") << elem_ctype(p.ty.sz) << "*)__builtin_assume_aligned("
              << p.id.str() << ", 16);\n";
    out << body << "}\n";
    return out.str();
  }
};

// ---------------------------------------------------------------- host plan
struct PlanPrinter {
  const Program& p;
  std::ostringstream os;

  explicit PlanPrinter(const Program& prog) : p(prog) {}

  std::string hexpr(const E& e) {
    switch (e->k) {
      case Expr::Var: return "(v " + sx_quote(e->name.str()) + ")";
      case Expr::Int: return "(i " + std::to_string(e->iv) + ")";
      case Expr::Float: {
        char buf[64];
        if (std::isinf(e->fv)) return e->fv > 0 ? "(f inf)" : "(f -inf)";
        if (std::isnan(e->fv)) return "(f nan)";
        snprintf(buf, sizeof buf, "%.17g", e->fv);
        return std::string("(f ") + buf + ")";
      }
      case Expr::Bool: return e->bv ? "(i 1)" : "(i 0)";
      case Expr::UnOpE: {
        const char* n = e->uop == UnOp::Sub ? "neg" : e->uop == UnOp::Not ? "not" : e->uop == UnOp::BitNeg ? "bitneg" : nullptr;
        if (!n) fail_rt(e->i, "Operator not supported in host code");
        return std::string("(un ") + n + " " + hexpr(e->args[0]) + ")";
      }
      case Expr::BinOpE: {
        static const std::map<BinOp, const char*> names = {
            {BinOp::Add, "add"}, {BinOp::Sub, "sub"}, {BinOp::Mul, "mul"}, {BinOp::Div, "div"}, {BinOp::FloorDiv, "floordiv"},
            {BinOp::Rem, "rem"}, {BinOp::And, "and"}, {BinOp::Or, "or"}, {BinOp::BitAnd, "bitand"}, {BinOp::BitOr, "bitor"},
            {BinOp::BitXor, "bitxor"}, {BinOp::BitShl, "shl"}, {BinOp::BitShr, "shr"}, {BinOp::Eq, "eq"}, {BinOp::Neq, "neq"},
            {BinOp::Leq, "leq"}, {BinOp::Geq, "geq"}, {BinOp::Lt, "lt"}, {BinOp::Gt, "gt"}, {BinOp::Max, "max"}, {BinOp::Min, "min"}};
        auto it = names.find(e->bop);
        if (it == names.end()) fail_rt(e->i, "Operator not supported in host code");
        bool flt = e->args[0]->ty.is_scalar() && is_float(e->args[0]->ty.sz);
        return std::string("(bin ") + it->second + (flt ? " f " : " i ") + hexpr(e->args[0]) + " " + hexpr(e->args[1]) + ")";
      }
      case Expr::IfExpr: return "(ite " + hexpr(e->args[0]) + " " + hexpr(e->args[1]) + " " + hexpr(e->args[2]) + ")";
      case Expr::Convert: return std::string("(cvt ") + elem_tag(e->ty.sz) + " " + hexpr(e->args[0]) + ")";
      case Expr::AddrOf: return "(addr " + hexpr(e->args[0]) + " " + hexpr(e->args[1]) + " " + std::to_string(elem_bytes(e->ty.sz)) + ")";
      default: fail_rt(e->i, "Expression " + print_expr(e) + " is not supported in host code");
    }
  }

  std::string kind_of(const Type& t) {
    if (t.k == Type::Pointer || (t.k == Type::Tensor && !t.shape.empty())) return "ptr";
    return elem_tag(t.sz);
  }

  void stmts(const Stmts& ss) {
    for (auto& s : ss) {
      switch (s->k) {
        case Stmt::Launch: {
          size_t idx = 0;
          for (; idx < p.kernels.size(); ++idx)
            if (p.kernels[idx].name == s->fname) break;
          os << "(launch " << idx << " " << s->grid.x << " " << s->grid.y << " " << s->grid.z << " " << s->block.x << " "
             << s->block.y << " " << s->block.z << " (args";
          for (auto& a : s->args) os << " " << hexpr(a);
          os << "))";
          break;
        }
        case Stmt::PersistentLaunch: {
          size_t idx = 0;
          for (; idx < p.kernels.size(); ++idx)
            if (p.kernels[idx].name == s->fname) break;
          os << "(persist " << idx << " " << s->grid.x << " " << s->grid.y << " " << s->grid.z << " " << s->block.x << " "
             << s->block.y << " " << s->block.z << " (args";
          for (auto& a : s->args) os << " " << hexpr(a);
          os << ") (body ";
          stmts(s->body);
          os << ") " << std::max<int64_t>(s->iv, 1) << ")";
          break;
        }
        case Stmt::For:
          os << "(for " << sx_quote(s->id.str()) << " " << hexpr(s->lo) << " " << hexpr(s->hi) << " " << s->step << " (body ";
          stmts(s->body);
          os << "))";
          break;
        case Stmt::While:
          os << "(while " << hexpr(s->expr) << " (body ";
          stmts(s->body);
          os << "))";
          break;
        case Stmt::If:
          os << "(if " << hexpr(s->expr) << " (then ";
          stmts(s->body);
          os << ") (else ";
          stmts(s->els);
          os << "))";
          break;
        case Stmt::Def: os << "(def " << sx_quote(s->id.str()) << " " << kind_of(s->ty) << " " << hexpr(s->expr) << ")"; break;
        case Stmt::Assign: os << "(set " << sx_quote(s->dst->name.str()) << " " << hexpr(s->expr) << ")"; break;
        case Stmt::Alloc: os << "(alloc " << sx_quote(s->id.str()) << " " << s->iv * elem_bytes(s->ty.sz) << ")"; break;
        case Stmt::Free: os << "(free " << sx_quote(s->id.str()) << ")"; break;
        default: fail_rt(s->i, "Statement not supported in host code (internal error)");
      }
      os << " ";
    }
  }

  std::string run() {
    os << "(plan " << sx_quote(p.name) << " (params";
    for (auto& q : p.entry_params) os << " (" << sx_quote(q.id.str()) << " ptr)";
    os << ") (kernels";
    for (auto& k : p.kernels) {
      os << " (" << sx_quote(k.name) << " (params";
      for (auto& q : k.params) os << " " << kind_of(q.ty);
      os << "))";
    }
    os << ") (body ";
    stmts(p.host);
    os << "))";
    return os.str();
  }
};

// pseudo host code for the human-readable listing
void list_host(std::ostringstream& os, const Stmts& ss, int n) {
  std::string pad(n, ' ');
  for (auto& s : ss) {
    switch (s->k) {
      case Stmt::Launch: {
        os << pad << s->fname << "<<<dim3(" << s->grid.x << ", " << s->grid.y << ", " << s->grid.z << "), dim3(" << s->block.x
           << ", " << s->block.y << ", " << s->block.z << "), 0, 0>>>(";
        for (size_t i = 0; i < s->args.size(); ++i) os << (i ? ", " : "") << print_expr(s->args[i]);
        os << ");\n";
        break;
      }
      case Stmt::PersistentLaunch:
        os << pad << "if (parpy_grid_fits_device(" << s->fname << ")) {   // all workgroups resident: the loop runs inside one kernel\n";
        os << pad << "  " << s->fname << "<<<dim3(" << s->grid.x << ", " << s->grid.y << ", " << s->grid.z << "), dim3(" << s->block.x
           << ", " << s->block.y << ", " << s->block.z << "), 0, 0>>>(";
        for (size_t i = 0; i < s->args.size(); ++i) os << (i ? ", " : "") << print_expr(s->args[i]);
        os << ", parpy_barrier_counter, parpy_barrier_status, parpy_barrier_limit);\n";
        os << pad << "} else {\n";
        list_host(os, s->body, n + 2);
        os << pad << "}\n";
        break;
      case Stmt::For:
        os << pad << "for (int64_t " << s->id.str() << " = " << print_expr(s->lo) << "; " << s->id.str() << (s->step > 0 ? " < " : " > ")
           << print_expr(s->hi) << "; " << s->id.str() << " += " << s->step << ") {\n";
        list_host(os, s->body, n + 2);
        os << pad << "}\n";
        break;
      case Stmt::While:
        os << pad << "while (" << print_expr(s->expr) << ") {\n";
        list_host(os, s->body, n + 2);
        os << pad << "}\n";
        break;
      case Stmt::If:
        os << pad << "if (" << print_expr(s->expr) << ") {\n";
        list_host(os, s->body, n + 2);
        if (!s->els.empty()) {
          os << pad << "} else {\n";
          list_host(os, s->els, n + 2);
        }
        os << pad << "}\n";
        break;
      case Stmt::Def: os << pad << "auto " << s->id.str() << " = " << print_expr(s->expr) << ";\n"; break;
      case Stmt::Assign: os << pad << print_expr(s->dst) << " = " << print_expr(s->expr) << ";\n"; break;
      case Stmt::Alloc:
        os << pad << elem_ctype(s->ty.sz) << "* " << s->id.str() << " = (" << elem_ctype(s->ty.sz) << "*)parpy_alloc_buffer("
           << s->iv * elem_bytes(s->ty.sz) << ");\n";
        break;
      case Stmt::Free: os << pad << "parpy_free_buffer(" << s->id.str() << ");\n"; break;
      default: break;
    }
  }
}

}  // namespace

std::string hip_print_device(const Program& p, const Options& opts) {
  std::ostringstream out;
  out << PREAMBLE;
  for (auto& inc : p.includes) out << "#include \"" << inc << "\"\n";
  // headers of the external device functions the kernels call (written as given: <x.h> or "x.h")
  std::set<std::string> headers;
  for (auto& k : p.kernels)
    visit_stmts(k.body, [&](const S& st) {
      auto scan = [&](const E& e) {
        visit_exprs(e, [&](const E& x) { if (x->k == Expr::Call && x->ext && !x->ext->header.empty()) headers.insert(x->ext->header); });
      };
      scan(st->dst); scan(st->expr); scan(st->lo); scan(st->hi);
      for (auto& a : st->args) scan(a);
    });
  for (auto& h : headers) out << "#include " << ((h[0] == '<' || h[0] == '"') ? h : "\"" + h + "\"") << "\n";
  for (auto& d : p.preamble) out << d << "\n";
  DevicePrinter dp(opts);
  for (auto& f : p.device_funs) out << "\n" << dp.device_function_text(f);
  for (auto& k : p.kernels) out << "\n" << dp.kernel_text(k);
  return out.str();
}

std::string hip_print_plan(const Program& p) { return PlanPrinter(p).run(); }

std::string hip_print_listing(const Program& p, const Options& opts) {
  std::ostringstream out;
  out << hip_print_device(p, opts);
  out << "\n// host side: executed by the runtime's launch-plan interpreter (hipModuleLaunchKernel on stream 0)\n";
  out << "extern \"C\" int32_t " << p.name << "(";
  for (size_t i = 0; i < p.entry_params.size(); ++i)
    out << (i ? ", " : "") << elem_ctype(p.entry_params[i].ty.sz) << "* " << p.entry_params[i].id.str();
  out << ") {\n";
  list_host(out, p.host, 2);
  out << "  return 0;\n}\n";
  return out.str();
}

}  // namespace parpy
