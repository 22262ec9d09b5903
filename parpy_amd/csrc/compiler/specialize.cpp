// Call-time specialisation: bind parameters to the argument descriptors,
// inline every scalar as a literal, resolve indices, turn slice statements
// into loops and type-check the result.
//
// Counterpart of the reference's src/py/mod.rs:45-109 pipeline:
// type_check.rs:129-160 (parameter types), inline_const.rs:97-147 (scalars and
// 0-d arrays become literals, including dict fields), indices.rs:15-58
// (negative / omitted bounds), slices.rs:269-486 (slices -> loops, reductions
// -> labelled reduction loops) and type_check.rs:162-1010 (typing with
// coercions inside one numeric family).
#include <algorithm>
#include <sstream>

#include "passes.hpp"

namespace parpy {

// ---------------------------------------------------------------- descriptors
namespace {

ArgDesc parse_arg(const SXP& x) {
  ArgDesc a;
  const std::string& h = x->head();
  if (h == "int") { a.k = ArgDesc::Int; a.iv = x->at(1)->as_int(); }
  else if (h == "float") { a.k = ArgDesc::Float; a.fv = x->at(1)->as_double(); }
  else if (h == "scalar") {
    a.k = ArgDesc::Scalar;
    if (!parse_elem_tag(x->at(1)->atom, &a.sz)) throw std::runtime_error("bad scalar dtype " + x->at(1)->atom);
    if (is_float(a.sz)) a.fv = x->at(2)->as_double();
    else if (a.sz == ElemSize::Bool) a.iv = x->at(2)->atom == "true" || x->at(2)->atom == "1";
    else a.iv = x->at(2)->as_int();
  } else if (h == "tensor") {
    a.k = ArgDesc::Tensor;
    if (!parse_elem_tag(x->at(1)->atom, &a.sz)) throw std::runtime_error("bad tensor dtype " + x->at(1)->atom);
    for (auto& d : x->at(2)->items) a.shape.push_back(d->as_int());
  } else if (h == "dict") {
    a.k = ArgDesc::Dict;
    for (size_t k = 1; k < x->size(); ++k) a.fields.emplace_back(x->at(k)->at(0)->atom, parse_arg(x->at(k)->at(1)));
    std::sort(a.fields.begin(), a.fields.end(), [](auto& l, auto& r) { return l.first < r.first; });
  } else {
    throw std::runtime_error("unknown argument descriptor '" + h + "'");
  }
  return a;
}

}  // namespace

std::vector<ArgDesc> parse_args(const std::string& sexpr) {
  SXP x = parse_sexpr(sexpr);
  std::vector<ArgDesc> r;
  for (size_t k = 1; k < x->size(); ++k) r.push_back(parse_arg(x->at(k)));
  return r;
}

Options parse_options(const std::string& sexpr) {
  SXP x = parse_sexpr(sexpr);
  Options o;
  for (size_t k = 1; k < x->size(); ++k) {
    const SXP& f = x->at(k);
    const std::string& h = f->head();
    auto flag = [&]() { return f->at(1)->as_int() != 0; };
    if (h == "par") {
      for (size_t j = 1; j < f->size(); ++j) {
        const SXP& p = f->at(j);
        LoopPar lp;
        lp.nthreads = p->at(1)->as_int();
        lp.reduction = p->at(2)->as_int() != 0;
        lp.tpb = p->at(3)->as_int();
        if (lp.tpb <= 0 || lp.tpb % WAVE_SIZE != 0)
          fail_rt(Info(), "The number of threads per block must be a positive integer divisible by 64.");
        o.parallelize[p->at(0)->atom] = lp;
      }
    } else if (h == "debug_print") o.debug_print = flag();
    else if (h == "use_graphs") o.use_graphs = flag();
    else if (h == "persistent_loops") o.persistent_loops = flag();
    else if (h == "device_functions") o.device_functions = flag();
    else if (h == "force_int_size") { o.has_force_int = parse_elem_tag(f->at(1)->atom, &o.force_int); }
    else if (h == "force_float_size") { o.has_force_float = parse_elem_tag(f->at(1)->atom, &o.force_float); }
    else if (h == "includes") { for (size_t j = 1; j < f->size(); ++j) o.includes.push_back(f->at(j)->atom); }
    else if (h == "opt_vectorize") o.opt_vectorize = flag();
    else if (h == "opt_lds_rows") o.opt_lds_rows = flag();
    else if (h == "opt_reg_cache") o.opt_reg_cache = flag();
    else if (h == "opt_hoist_invariant") o.opt_hoist_invariant = flag();
    else if (h == "opt_narrow_index") o.opt_narrow_index = flag();
    else if (h == "opt_mfma_sddmm") o.opt_mfma_sddmm = flag();
    else if (h == "opt_unswitch") o.opt_unswitch = flag();
    else if (h == "opt_nontemporal") o.opt_nontemporal = flag();
    else if (h == "opt_lane_split") o.opt_lane_split = flag();
    else if (h == "opt_drop_barriers") o.opt_drop_barriers = flag();
    else if (h == "opt_unswitch_uniform") o.opt_unswitch_uniform = flag();
    else if (h == "opt_offset32") o.opt_offset32 = flag();
    else if (h == "opt_if_convert") o.opt_if_convert = flag();
    else if (h == "opt_noalias_scopes") o.opt_noalias_scopes = flag();
    else if (h == "opt_gather_transpose") o.opt_gather_transpose = flag();
    else if (h == "opt_expand_short_loops") o.opt_expand_short_loops = flag();
    else if (h == "opt_guard_bounds") o.opt_guard_bounds = flag();
    else if (h == "opt_pack_accesses") o.opt_pack_accesses = flag();
    else if (h == "opt_share_iterations") o.opt_share_iterations = flag();
    else if (h == "opt_fence_iterations") o.opt_fence_iterations = flag();
    else if (h == "opt_keep_stored") o.opt_keep_stored = flag();
    else if (h == "opt_keep_own") o.opt_keep_own = flag();
    else if (h == "opt_prefetch_steps") o.opt_prefetch_steps = flag();
    else if (h == "reg_budget") o.reg_budget = f->at(1)->as_int();
    else if (h == "reg_budget_scale") o.reg_budget_scale = f->at(1)->as_int();
    else if (h == "assume_aligned") o.assume_aligned = flag();
    else if (h == "backend") {
      const std::string& b = f->at(1)->atom;
      o.backend = b == "hip" ? Backend::Hip : b == "cuda" ? Backend::Cuda : b == "metal" ? Backend::Metal : Backend::Auto;
    }
  }
  return o;
}

namespace {

// ---------------------------------------------------------------- parameter binding
struct Binding {
  enum Kind { Literal, Array, Dict } k = Literal;
  E lit;                                   // Literal
  Name id;                                 // Array: flattened parameter
  Type ty;                                 // Array type
  std::map<std::string, Binding> fields;   // Dict
};

struct Specializer {
  const Options& opts;
  NameGen& gen;
  std::map<Name, Binding> binds;
  std::vector<Param> flat_params;

  Specializer(const Options& o, NameGen& g) : opts(o), gen(g) {}

  Binding bind(const std::string& name, const ArgDesc& a, const Info& i, bool in_dict) {
    Binding b;
    switch (a.k) {
      case ArgDesc::Int: b.lit = mk_int(a.iv, opts.int_size(), i); break;
      case ArgDesc::Float: b.lit = mk_float(a.fv, opts.float_size(), i); break;
      case ArgDesc::Scalar:
        if (is_float(a.sz)) b.lit = mk_float(a.fv, a.sz, i);
        else if (a.sz == ElemSize::Bool) b.lit = mk_bool(a.iv != 0, i);
        else b.lit = mk_int(a.iv, a.sz, i);
        break;
      case ArgDesc::Tensor: {
        b.k = Binding::Array;
        b.id = gen.fresh(name);
        b.ty = Type::tensor(a.sz, a.shape);
        flat_params.push_back(Param{b.id, b.ty, i});
        break;
      }
      case ArgDesc::Dict: {
        if (in_dict) fail_rt(i, "Nested dictionary arguments are not supported");
        b.k = Binding::Dict;
        for (auto& f : a.fields) b.fields[f.first] = bind(name + "_" + f.first, f.second, i, true);
        break;
      }
    }
    return b;
  }

  // ---- substitution of parameters (and dict lookups) in expressions
  E subst(const E& e) {
    if (!e) return e;
    if (e->k == Expr::Var) {
      auto it = binds.find(e->name);
      if (it == binds.end()) return e;
      const Binding& b = it->second;
      if (b.k == Binding::Literal) { auto r = std::make_shared<Expr>(*b.lit); r->i = e->i; return r; }
      if (b.k == Binding::Array) return mk_var(b.id, b.ty, e->i);
      fail_ty(e->i, "Dictionary argument " + e->name.s + " must be accessed with a string key");
    }
    if (e->k == Expr::Subscript && e->args[0]->k == Expr::Var && e->args[1]->k == Expr::Str) {
      auto it = binds.find(e->args[0]->name);
      if (it != binds.end() && it->second.k == Binding::Dict) {
        auto f = it->second.fields.find(e->args[1]->sval);
        if (f == it->second.fields.end())
          fail_ty(e->i, "Field " + e->args[1]->sval + " not present in dictionary " + e->args[0]->name.s);
        const Binding& b = f->second;
        if (b.k == Binding::Literal) { auto r = std::make_shared<Expr>(*b.lit); r->i = e->i; return r; }
        return mk_var(b.id, b.ty, e->i);
      }
    }
    return map_children(e, [&](const E& c) { return subst(c); });
  }

  Stmts subst_stmts(const Stmts& ss) {
    Stmts out;
    for (auto& s : ss) {
      if (s->k == Stmt::Assign && s->dst->k == Expr::Var) {
        auto it = binds.find(s->dst->name);
        if (it != binds.end() && it->second.k == Binding::Literal)
          fail_ty(s->i, "Cannot assign to scalar parameter " + s->dst->name.s + ", which is a compile-time constant");
      }
      auto r = std::const_pointer_cast<Stmt>(std::static_pointer_cast<const Stmt>(map_exprs(s, [&](const E& e) { return subst(e); })));
      r->body = subst_stmts(s->body);
      r->els = subst_stmts(s->els);
      out.push_back(r);
    }
    return out;
  }
};

// ---------------------------------------------------------------- slices -> loops
struct SliceExpander {
  NameGen& gen;
  std::map<Name, Type> arrays;  // array-typed variables visible (parameters and aliases)

  std::vector<E> index_list(const E& idx) {
    if (idx->k == Expr::Tuple) return idx->args;
    return {idx};
  }

  static int count_slices_idx(const E& idx) {
    int n = 0;
    if (idx->k == Expr::Slice) return 1;
    if (idx->k == Expr::Tuple)
      for (auto& a : idx->args) n += a->k == Expr::Slice ? 1 : 0;
    return n;
  }

  int count_slices(const E& e) {
    if (!e) return 0;
    if (e->k == Expr::Subscript) {
      int t = count_slices(e->args[0]);
      return std::max(t, count_slices_idx(e->args[1]));
    }
    int n = 0;
    for (auto& a : e->args) n = std::max(n, count_slices(a));
    return n;
  }

  const Type& target_type(const E& target, const Info& i) {
    if (target->k != Expr::Var) fail_rt(i, "Target of slice must be a variable.");
    auto it = arrays.find(target->name);
    if (it == arrays.end() || !it->second.is_array())
      fail_rt(i, "Target of slice subscript operation has invalid type.");
    return it->second;
  }

  // extents of the sliced dimensions of one subscript
  std::vector<int64_t> slice_shape(const E& sub) {
    const Type& ty = target_type(sub->args[0], sub->i);
    auto idxs = index_list(sub->args[1]);
    if (idxs.size() != ty.shape.size())
      fail_rt(sub->i, "Subscript operations containing slices must refer to all dimensions of the target. Target has " +
                          std::to_string(ty.shape.size()) + " dimensions, but only " + std::to_string(idxs.size()) +
                          " dimensions are addressed by the index.");
    std::vector<int64_t> r;
    for (size_t d = 0; d < idxs.size(); ++d) {
      if (idxs[d]->k != Expr::Slice) continue;
      int64_t lo = 0, hi = ty.shape[d];
      if (idxs[d]->args[0]) {
        E l = fold_expr(idxs[d]->args[0]);
        if (l->k != Expr::Int) fail_ty(idxs[d]->i, "Lower-bound of slice must be fixed.");
        lo = l->iv;
      }
      if (idxs[d]->args[1]) {
        E h = fold_expr(idxs[d]->args[1]);
        if (h->k != Expr::Int) fail_ty(idxs[d]->i, "Upper-bound of slice must be fixed.");
        hi = h->iv;
      }
      if (lo < 0) lo += ty.shape[d];
      if (hi < 0) hi += ty.shape[d];
      if (lo >= hi)
        fail_ty(idxs[d]->i, "Lower-bound " + std::to_string(lo) + " of slice must be less than its upper-bound " + std::to_string(hi) + ".");
      if (lo < 0 || hi > ty.shape[d])
        fail_ty(idxs[d]->i, "Slice dimensions " + std::to_string(lo) + " and " + std::to_string(hi) + " out of range for shape " +
                                std::to_string(ty.shape[d]));
      r.push_back(hi - lo);
    }
    return r;
  }

  // shape of an expression containing slices: every sliced subscript must agree
  void collect_shape(const E& e, std::vector<int64_t>& shape, bool& found) {
    if (!e) return;
    if (e->k == Expr::Subscript && count_slices_idx(e->args[1]) > 0) {
      auto s = slice_shape(e);
      if (!found) { shape = s; found = true; }
      else if (s.size() == shape.size() && s != shape) {
        std::ostringstream a, b;
        for (auto v : shape) a << v << " ";
        for (auto v : s) b << v << " ";
        fail_ty(e->i, "Found incompatible shapes " + a.str() + "and " + b.str());
      } else if (s.size() > shape.size()) {
        shape = s;
      }
      return;
    }
    for (auto& a : e->args) collect_shape(a, shape, found);
  }

  // replace the k-th slice of every subscript by lo + ids[k]
  E insert_ids(const E& e, const std::vector<Name>& ids) {
    if (!e) return e;
    if (e->k == Expr::Subscript && count_slices_idx(e->args[1]) > 0) {
      const Type& ty = target_type(e->args[0], e->i);
      auto idxs = index_list(e->args[1]);
      size_t k = 0;
      std::vector<E> nidx;
      for (size_t d = 0; d < idxs.size(); ++d) {
        if (idxs[d]->k != Expr::Slice) { nidx.push_back(insert_ids(idxs[d], ids)); continue; }
        int64_t lo = 0;
        if (idxs[d]->args[0]) lo = fold_expr(idxs[d]->args[0])->iv;
        if (lo < 0) lo += ty.shape[d];
        auto v = std::make_shared<Expr>();
        v->k = Expr::Var;
        v->name = ids.at(k++);
        v->i = idxs[d]->i;
        E var = v;
        if (lo != 0) {
          auto l = std::make_shared<Expr>();
          l->k = Expr::Int;
          l->iv = lo;
          l->i = idxs[d]->i;
          auto add = std::make_shared<Expr>();
          add->k = Expr::BinOpE;
          add->bop = BinOp::Add;
          add->args = {E(l), var};
          add->i = idxs[d]->i;
          var = add;
        }
        nidx.push_back(var);
      }
      auto r = std::make_shared<Expr>(*e);
      if (nidx.size() == 1) r->args[1] = nidx[0];
      else {
        auto t = std::make_shared<Expr>();
        t->k = Expr::Tuple;
        t->args = nidx;
        t->i = e->args[1]->i;
        r->args[1] = t;
      }
      return r;
    }
    return map_children(e, [&](const E& c) { return insert_ids(c, ids); });
  }

  E subst_vars(const E& e, const std::map<Name, E>& m) {
    if (!e) return e;
    if (e->k == Expr::Var) {
      auto it = m.find(e->name);
      return it == m.end() ? e : it->second;
    }
    return map_children(e, [&](const E& c) { return subst_vars(c, m); });
  }

  static bool reduction_builtin(const E& e, BinOp* op) {
    if (e->k != Expr::BuiltinE || e->args.size() != 1) return false;
    switch (e->fn) {
      case Builtin::Sum: *op = BinOp::Add; return true;
      case Builtin::Prod: *op = BinOp::Mul; return true;
      case Builtin::Max: *op = BinOp::Max; return true;
      case Builtin::Min: *op = BinOp::Min; return true;
      default: return false;
    }
  }

  E untyped_int(int64_t v, const Info& i) {
    auto l = std::make_shared<Expr>();
    l->k = Expr::Int;
    l->iv = v;
    l->i = i;
    return l;
  }

  S make_for(const Name& id, int64_t n, Stmts body, std::vector<std::string> labels, const Info& i) {
    auto f = std::make_shared<Stmt>();
    f->k = Stmt::For;
    f->i = i;
    f->id = id;
    f->lo = untyped_int(0, i);
    f->hi = untyped_int(n, i);
    f->step = 1;
    f->body = std::move(body);
    f->labels = std::move(labels);
    return f;
  }

  // Shapes of slice statements are checked before they are expanded, the way the reference
  // type-checks shapes first (src/py/type_check.rs:235-270 unification with broadcasting from
  // the right, :720-738 rank of a subscript).
  static std::string shape_str(const std::vector<int64_t>& s, const char* sep) {
    std::string r;
    for (size_t k = 0; k < s.size(); ++k) r += (k ? sep : "") + std::to_string(s[k]);
    return r;
  }

  std::vector<int64_t> unify(const std::vector<int64_t>& l, const std::vector<int64_t>& r, const Info& i) {
    std::vector<int64_t> acc;
    size_t n = std::max(l.size(), r.size());
    for (size_t k = 0; k < n; ++k) {
      bool hl = k < l.size(), hr = k < r.size();
      int64_t a = hl ? l[l.size() - 1 - k] : 0, b = hr ? r[r.size() - 1 - k] : 0;
      if (hl && hr && !(a == b || a == 1 || b == 1))
        fail_ty(i, "Found incompatible shapes " + shape_str(l, ", ") + " and " + shape_str(r, ", "));
      acc.push_back(hl ? a : b);
    }
    std::reverse(acc.begin(), acc.end());
    return acc;
  }

  std::vector<int64_t> shape_of(const E& e) {
    if (!e) return {};
    switch (e->k) {
      case Expr::Var: {
        auto it = arrays.find(e->name);
        return it != arrays.end() && it->second.is_array() ? it->second.shape : std::vector<int64_t>{};
      }
      case Expr::Subscript: {
        if (e->args[0]->k != Expr::Var) fail_rt(e->i, "Target of slice must be a variable.");
        auto it = arrays.find(e->args[0]->name);
        if (it == arrays.end() || !it->second.is_array()) return {};
        const auto& full = it->second.shape;
        auto idxs = index_list(e->args[1]);
        if (idxs.size() > full.size())
          fail_ty(e->i, "Indexing with " + std::to_string(idxs.size()) + " dimensions on tensor of shape [" + shape_str(full, ",") + "]");
        std::vector<int64_t> r;
        if (count_slices_idx(e->args[1]) > 0 && idxs.size() == full.size()) r = slice_shape(e);
        for (size_t d = idxs.size(); d < full.size(); ++d) r.push_back(full[d]);
        return r;
      }
      case Expr::BinOpE: return unify(shape_of(e->args[0]), shape_of(e->args[1]), e->i);
      case Expr::IfExpr: return unify(shape_of(e->args[1]), shape_of(e->args[2]), e->i);
      case Expr::BuiltinE: {
        BinOp op;
        if (reduction_builtin(e, &op)) {
          auto s = shape_of(e->args[0]);
          if (!e->has_axis) return {};
          int64_t n = (int64_t)s.size(), ax = e->iv;
          if (n == 0 || ax >= n || ax < -n) return s;   // reported with the slice counts below
          s.erase(s.begin() + (size_t)(((ax % n) + n) % n));
          return s;
        }
        std::vector<int64_t> r;
        for (auto& a : e->args) r = unify(r, shape_of(a), e->i);
        return r;
      }
      case Expr::UnOpE: case Expr::Convert: return shape_of(e->args[0]);
      case Expr::Call: {
        std::vector<int64_t> r;
        for (size_t k = 0; k < e->args.size(); ++k)
          if (!(e->ext && k < e->ext->params.size() && e->ext->params[k].is_pointer())) r = unify(r, shape_of(e->args[k]), e->i);
        return r;
      }
      default: return {};
    }
  }

  // src/py/slices.rs:362-486
  S expand_assignment(const S& s) {
    bool is_def = s->k == Stmt::Def;
    E lhs = is_def ? E() : s->dst;
    E rhs = s->expr;
    int lslices = is_def ? 0 : count_slices(lhs);
    int rslices = count_slices(rhs);
    int nslices = std::max(lslices, rslices);
    if (nslices == 0) return s;
    const Info& i = s->i;
    {
      auto rs = shape_of(rhs);
      if (!is_def) unify(shape_of(lhs), rs, i);
    }
    std::vector<std::string> labels = s->labels;

    BinOp op = BinOp::Add;
    bool is_reduce = reduction_builtin(rhs, &op);
    bool reduce_all = is_reduce && !rhs->has_axis;

    std::vector<Name> ids;
    for (int k = 0; k < nslices; ++k) ids.push_back(gen.fresh("slice_dim"));
    std::vector<int64_t> shape;
    bool found = false;
    if (!is_reduce) {
      if (lslices < rslices)
        fail_rt(i, "Slice statements cannot have more slice dimensions in the right-hand side expression than in "
                   "the left-hand side expression.");
      if (is_def) fail_rt(i, "Slice expression cannot be assigned to fresh variable " + s->id.s + ".");
      collect_shape(lhs, shape, found);
    } else {
      collect_shape(rhs->args[0], shape, found);
    }
    if (!found || (int)shape.size() != nslices) fail_rt(i, "Invalid type of slice operation");
    // every sliced subscript on the other side must agree with the iteration shape
    {
      std::vector<int64_t> other;
      bool f2 = false;
      collect_shape(is_reduce ? lhs : rhs, other, f2);
      if (f2 && !is_reduce && other.size() == shape.size() && other != shape) fail_ty(i, "Found incompatible shapes in slice statement");
    }
    E lhs_i = lhs ? insert_ids(lhs, ids) : E();
    E rhs_i = insert_ids(rhs, ids);

    auto mk_target = [&]() -> E {
      if (!is_def) return lhs_i;
      auto v = std::make_shared<Expr>();
      v->k = Expr::Var;
      v->name = s->id;
      v->i = i;
      return v;
    };

    auto reduce_nest = [&](E target, E arg, Name rid, int64_t niters, std::vector<std::string> rlabel,
                           std::vector<std::pair<Name, int64_t>> outer, std::vector<std::string> outer_labels) -> S {
      if (niters <= 0) fail_rt(i, "Cannot apply reduction on empty dimension");
      auto upd = std::make_shared<Expr>();
      upd->k = Expr::BinOpE;
      upd->bop = op;
      upd->args = {target, arg};
      upd->i = i;
      S inner = mk_assign(target, upd, i);
      rlabel.push_back(REDUCE_PAR_LABEL);
      S loop = make_for(rid, niters, {inner}, rlabel, i);
      // the neutral element takes the type of the reduced expression (first iteration)
      auto ne = std::make_shared<Expr>();
      ne->k = Expr::NeutralElement;
      ne->bop = op;
      std::map<Name, E> zero{{rid, untyped_int(0, i)}};
      ne->args = {subst_vars(arg, zero)};
      ne->i = i;
      S pre;
      if (is_def) pre = mk_def(s->id, Type(), ne, i);
      else pre = mk_assign(target, ne, i);
      auto g = std::make_shared<Stmt>();
      g->k = Stmt::WithGpu;
      g->i = i;
      g->body = {pre, loop};
      S stmt = g;
      for (size_t k = outer.size(); k-- > 0;) {
        std::vector<std::string> l;
        if (!outer_labels.empty()) { l.push_back(outer_labels.back()); outer_labels.pop_back(); }
        stmt = make_for(outer[k].first, outer[k].second, {stmt}, l, i);
      }
      return stmt;
    };

    if (is_reduce && !reduce_all) {
      if (lslices != rslices - 1)
        fail_rt(i, "When reducing along one dimension, the number of slice dimensions of the left-hand side "
                   "expression must be one less than in the right-hand side.");
      if (!labels.empty() && (int)labels.size() != nslices)
        fail_rt(i, "Expected zero or " + std::to_string(nslices) + " labels, found " + std::to_string(labels.size()));
      int64_t ax = rhs->iv;
      if (ax >= nslices || ax < -nslices)
        fail_ty(i, "Invalid axis value " + std::to_string(ax) + " for tensor of " + std::to_string(nslices) + " dimensions.");
      size_t idx = (size_t)(((ax % nslices) + nslices) % nslices);
      // the lhs slices are numbered without the reduced dimension: re-number them
      std::vector<Name> lhs_ids;
      for (size_t k = 0; k < ids.size(); ++k)
        if (k != idx) lhs_ids.push_back(ids[k]);
      if (lhs) lhs_i = insert_ids(lhs, lhs_ids);
      std::vector<std::pair<Name, int64_t>> outer;
      for (size_t k = 0; k < ids.size(); ++k)
        if (k != idx) outer.emplace_back(ids[k], shape[k]);
      std::vector<std::string> rlabel;
      if (idx < labels.size()) { rlabel.push_back(labels[idx]); labels.erase(labels.begin() + idx); }
      return reduce_nest(mk_target(), rhs_i->args[0], ids[idx], shape[idx], rlabel, outer, labels);
    }
    if (reduce_all) {
      if (lslices != 0)
        fail_rt(i, "When reducing along all dimensions, the left-hand side expression must be a scalar.");
      if (labels.size() > 1)
        fail_rt(i, "Expected zero or one labels for full reduction operation, found " + std::to_string(labels.size()));
      Name rid = gen.fresh("reduce_dim");
      // row-major recovery of the per-dimension indices from the flat reduction index
      std::map<Name, E> m;
      auto v = std::make_shared<Expr>();
      v->k = Expr::Var;
      v->name = rid;
      v->i = i;
      E cur = v;
      for (size_t k = ids.size(); k-- > 1;) {
        auto rem = std::make_shared<Expr>();
        rem->k = Expr::BinOpE;
        rem->bop = BinOp::Rem;
        rem->args = {cur, untyped_int(shape[k], i)};
        rem->i = i;
        m[ids[k]] = rem;
        auto div = std::make_shared<Expr>();
        div->k = Expr::BinOpE;
        div->bop = BinOp::FloorDiv;
        div->args = {cur, untyped_int(shape[k], i)};
        div->i = i;
        cur = div;
      }
      m[ids[0]] = cur;
      int64_t total = 1;
      for (auto d : shape) total *= d;
      return reduce_nest(mk_target(), subst_vars(rhs_i->args[0], m), rid, total, labels, {}, {});
    }
    // plain mapping statement
    if (lslices < rslices)
      fail_rt(i, "Slice statements cannot have more slice dimensions in the right-hand side expression than in "
                 "the left-hand side expression.");
    if (!labels.empty() && (int)labels.size() != nslices)
      fail_rt(i, "Expected zero or " + std::to_string(nslices) + " labels, found " + std::to_string(labels.size()));
    S stmt = mk_assign(lhs_i, rhs_i, i);
    for (size_t k = ids.size(); k-- > 0;) {
      std::vector<std::string> l;
      if (!labels.empty()) { l.push_back(labels.back()); labels.pop_back(); }
      stmt = make_for(ids[k], shape[k], {stmt}, l, i);
    }
    return stmt;
  }

  void check_no_slices(const E& e) {
    if (count_slices(e) > 0) fail_rt(e->i, "Slice expressions are only allowed in assignment statements.");
  }

  Stmts run(const Stmts& ss) {
    Stmts out;
    for (auto& s : ss) {
      if (s->k == Stmt::Def || s->k == Stmt::Assign) {
        S r = expand_assignment(s);
        out.push_back(r);
        // array aliases (`alpha_src = alpha2`) stay usable as slice targets
        if (r->k == Stmt::Def && r->expr->k == Expr::Var) {
          auto it = arrays.find(r->expr->name);
          if (it != arrays.end()) arrays[r->id] = it->second;
        }
        continue;
      }
      if (s->expr) check_no_slices(s->expr);
      if (s->lo) check_no_slices(s->lo);
      if (s->hi) check_no_slices(s->hi);
      auto r = std::make_shared<Stmt>(*s);
      r->body = run(s->body);
      r->els = run(s->els);
      out.push_back(r);
    }
    return out;
  }
};

// ---------------------------------------------------------------- type checking
bool lub_elem(ElemSize l, ElemSize r, ElemSize* out) {  // src/py/type_check.rs:162-187
  if (l == ElemSize::Bool && r == ElemSize::Bool) { *out = r; return true; }
  if ((is_signed(l) && is_signed(r)) || (is_unsigned(l) && is_unsigned(r)) || (is_float(l) && is_float(r))) {
    *out = elem_bytes(l) >= elem_bytes(r) ? l : r;
    return true;
  }
  return false;
}

struct TypeChecker {
  const Options& opts;
  std::map<Name, Type> vars;
  Type res_ty = Type::vvoid();
  // Functions called inside expressions that stay functions (device_functions option): one typed instance per callee
  // and argument types, shared by the checker of the main function and those of the callees, callees first.
  struct Instances {
    std::map<std::string, std::shared_ptr<const FunDef>> by_key;
    std::vector<std::shared_ptr<const FunDef>> in_order;
    std::set<std::string> open;   // being checked: a function that reaches itself cannot be compiled
    int next = 0;
  };
  std::shared_ptr<Instances> instances = std::make_shared<Instances>();
  std::set<Name> pending;             // result variables of inlined calls that have not been assigned yet
  std::map<Name, Type> resolved;      // ... and the type their first assignment gave them

  explicit TypeChecker(const Options& o) : opts(o) {}

  // definitions left without a value get the zero of the type they were resolved to
  Stmts finish(const Stmts& ss) {
    Stmts out;
    for (auto& s : ss) {
      auto r = std::make_shared<Stmt>(*s);
      if (s->k == Stmt::Def && s->expr->k == Expr::NeutralElement && s->expr->args.empty()) {
        auto it = resolved.find(s->id);
        if (it == resolved.end()) fail_ty(s->i, "Unknown return type of a called function (no value is ever returned)");
        r->ty = it->second;
        r->expr = is_float(r->ty.sz) ? mk_float(0.0, r->ty.sz, s->i) : r->ty.sz == ElemSize::Bool ? mk_bool(false, s->i) : mk_int(0, r->ty.sz, s->i);
      }
      r->body = finish(s->body);
      r->els = finish(s->els);
      out.push_back(r);
    }
    return out;
  }

  static bool is_scalar_of(const Type& t, bool (*pred)(ElemSize)) { return t.is_scalar() && pred(t.sz); }

  E ensure_scalar(const E& e, ElemSize expected) {
    const Type& ty = e->ty;
    if (!ty.is_scalar())
      fail_ty(e->i, std::string("Expected element of scalar type ") + elem_pyname(expected) + ", but found type " + ty.str() + ".");
    ElemSize l;
    if (!lub_elem(ty.sz, expected, &l))
      fail_ty(e->i, std::string("Expected element of type ") + elem_pyname(expected) + ", found incompatible element type " +
                        elem_pyname(ty.sz) + ".");
    return mk_convert(e, expected);
  }

  E coerce(const E& e, const Type& expected) {
    if (e->ty == expected) return e;
    if (e->ty.k == Type::Tensor && expected.k == Type::Tensor) {
      if (e->ty.shape.empty() && expected.shape.empty()) return ensure_scalar(e, expected.sz);
      fail_ty(e->i, "Cannot coerce incompatible tensor types (" + e->ty.str() + " != " + expected.str() + ")");
    }
    fail_ty(e->i, "Cannot coerce expression " + print_expr(e) + " of type " + e->ty.str() + " to type " + expected.str());
  }

  Type lub(const Type& l, const Type& r, const Info& i) {
    if (l.k == Type::Unknown) return r;
    if (r.k == Type::Unknown) return l;
    if (l.k == Type::Tensor && r.k == Type::Tensor && l.shape == r.shape) {
      ElemSize sz;
      if (lub_elem(l.sz, r.sz, &sz)) return Type::tensor(sz, l.shape);
      fail_ty(i, "Incompatible element types");
    }
    if (l == r) return l;
    fail_ty(i, "Types " + l.str() + " and " + r.str() + " are incompatible");
  }

  E unop_node(UnOp op, E a, const Info& i) { return mk_unop(op, a, a->ty, i); }

  E builtin(const E& e) {
    const Info& i = e->i;
    std::vector<E> args;
    for (auto& a : e->args) args.push_back(expr(a));
    auto nargs = args.size();
    switch (e->fn) {
      case Builtin::Inf:
        if (nargs == 0) return mk_float(HUGE_VAL, opts.float_size(), i);
        break;
      case Builtin::Exp: case Builtin::Log: case Builtin::Cos: case Builtin::Sin: case Builtin::Sqrt: case Builtin::Tanh:
        if (nargs == 1) {
          if (!is_scalar_of(args[0]->ty, is_float))
            fail_ty(i, "Unexpected type " + args[0]->ty.str() + " of unary builtin (expected float)");
          UnOp op = e->fn == Builtin::Exp ? UnOp::Exp : e->fn == Builtin::Log ? UnOp::Log : e->fn == Builtin::Cos ? UnOp::Cos
                  : e->fn == Builtin::Sin ? UnOp::Sin : e->fn == Builtin::Sqrt ? UnOp::Sqrt : UnOp::Tanh;
          return unop_node(op, args[0], i);
        }
        break;
      case Builtin::Abs:
        if (nargs == 1) {
          if (is_scalar_of(args[0]->ty, is_unsigned)) return args[0];
          if (is_scalar_of(args[0]->ty, is_signed) || is_scalar_of(args[0]->ty, is_float)) return unop_node(UnOp::Abs, args[0], i);
          fail_ty(i, "Unexpected type " + args[0]->ty.str() + " of abs builtin");
        }
        break;
      case Builtin::Convert:
        if (nargs == 1) {
          if (!args[0]->ty.is_scalar()) fail_ty(i, "Expected scalar type in type conversion, found " + args[0]->ty.str());
          auto r = std::make_shared<Expr>();
          r->k = Expr::Convert;
          r->ty = Type::scalar(e->ty.sz);
          r->i = i;
          r->args = {args[0]};
          return r;
        }
        break;
      case Builtin::Max: case Builtin::Min: case Builtin::Atan2:
        if (nargs == 2) {
          Type ty = lub(args[0]->ty, args[1]->ty, i);
          if (!ty.is_scalar()) fail_ty(i, "Unexpected type " + ty.str() + " of builtin");
          if (e->fn == Builtin::Atan2 && !is_float(ty.sz)) fail_ty(i, "Operation atan2 is only supported for floats.");
          BinOp op = e->fn == Builtin::Max ? BinOp::Max : e->fn == Builtin::Min ? BinOp::Min : BinOp::Atan2;
          return mk_binop(op, coerce(args[0], ty), coerce(args[1], ty), ty, i);
        }
        if (nargs == 1) fail_ty(i, "Reduction builtins must be applied to a slice expression in an assignment");
        break;
      case Builtin::Sum: case Builtin::Prod:
        if (nargs == 1) fail_ty(i, "Reduction builtins must be applied to a slice expression in an assignment");
        break;
      default:
        break;
    }
    fail_ty(i, "Unsupported use of builtin with " + std::to_string(nargs) + " args.");
  }

  E subscript(const E& e) {
    E target = expr(e->args[0]);
    if (target->ty.k != Type::Tensor || target->ty.shape.empty())
      fail_ty(e->i, "Cannot index into a value of type " + target->ty.str());
    std::vector<E> idxs = e->args[1]->k == Expr::Tuple ? e->args[1]->args : std::vector<E>{e->args[1]};
    const auto& shape = target->ty.shape;
    if (idxs.size() > shape.size())
      fail_ty(e->i, "Indexing with " + std::to_string(idxs.size()) + " dimensions on tensor of shape " + target->ty.str());
    std::vector<E> typed;
    for (size_t d = 0; d < idxs.size(); ++d) {
      E x = fold_expr(expr(idxs[d]));
      if (!(x->ty.is_scalar() && is_int(x->ty.sz)))
        fail_ty(idxs[d]->i, "Index must be an integer scalar, found " + x->ty.str());
      if (x->k == Expr::Int) {  // src/py/indices.rs:15-58
        int64_t v = x->iv < 0 ? x->iv + shape[d] : x->iv;
        if (v < 0 || v >= shape[d])
          fail_ty(idxs[d]->i, "Index " + std::to_string(x->iv) + " out of range for shape " + std::to_string(shape[d]));
        x = mk_int(v, opts.int_size(), x->i);
      } else if (is_signed(x->ty.sz)) {
        x = mk_convert(x, opts.int_size());
      } else {
        // unsigned indices are reinterpreted in the default (signed) index type
        auto c = std::make_shared<Expr>();
        c->k = Expr::Convert;
        c->ty = Type::scalar(opts.int_size());
        c->i = x->i;
        c->args = {x};
        x = c;
      }
      typed.push_back(x);
    }
    auto r = std::make_shared<Expr>();
    r->k = Expr::Subscript;
    r->i = e->i;
    auto t = std::make_shared<Expr>();
    t->k = Expr::Tuple;
    t->args = typed;
    t->i = e->args[1]->i;
    r->args = {target, E(t)};
    r->ty = Type::tensor(target->ty.sz, std::vector<int64_t>(shape.begin() + idxs.size(), shape.end()));
    return r;
  }

  // Call of an external device function (src/py/type_check.rs:854-877): scalar arguments are
  // coerced to the declared types, pointer arguments must be arrays of the declared element type,
  // and every call of one external must pass arrays of the same shapes.
  std::map<std::string, std::vector<Type>> ext_arg_types;

  // A call of a jitted function that stays a call (src/py/insert_called_functions.rs:12-88 collects such callees,
  // src/gpu/codegen.rs:573-585 makes them device functions): the callee is type-checked with the types of this call's
  // arguments and becomes a function of its own, once per combination of argument types.
  E fun_call(const E& e) {
    const FunDef& f = *e->callee;
    auto r = std::make_shared<Expr>(*e);
    // (the text of the callee is part of the key: two functions of one name -- a callee redefined after another of
    // its callers was declared -- are different functions)
    std::string key = f.id.s + "#" + std::to_string(std::hash<std::string>{}(print_fun(f))) + "(";
    std::vector<Type> tys;
    for (size_t k = 0; k < e->args.size(); ++k) {
      E a = expr(e->args[k]);
      if (!a->ty.is_scalar())
        fail_ty(a->i, "Found incompatible types in function call:\nargument " + std::to_string(k + 1) + " of " + f.id.s + " has type " +
                          a->ty.str() + ", and a function called inside an expression takes scalars when it is compiled as a device function");
      if (f.params[k].ty.k == Type::Tensor && f.params[k].ty.shape.empty()) a = ensure_scalar(a, f.params[k].ty.sz);   // annotated
      tys.push_back(a->ty);
      key += std::string(k ? "," : "") + elem_pyname(a->ty.sz);
      r->args[k] = a;
    }
    key += ")";
    auto it = instances->by_key.find(key);
    if (it == instances->by_key.end()) {
      if (instances->open.count(key)) fail_rt(e->i, "Call to unknown function " + f.id.s + " (a function cannot call itself)");
      instances->open.insert(key);
      TypeChecker tc(opts);
      tc.instances = instances;
      auto d = std::make_shared<FunDef>();
      d->id = Name{f.id.s + "_fn" + std::to_string(++instances->next), 0};
      d->i = f.i;
      for (size_t k = 0; k < f.params.size(); ++k) {
        tc.vars[f.params[k].id] = tys[k];
        d->params.push_back(Param{f.params[k].id, tys[k], f.params[k].i});
      }
      Stmts body = tc.finish(tc.stmts(f.body));
      if (!tc.res_ty.is_scalar()) fail_ty(e->i, "Unknown return type of function " + f.id.s);
      d->res_ty = tc.res_ty;
      // every return statement yields the common type of all of them
      std::function<Stmts(const Stmts&)> fix = [&](const Stmts& ss) {
        Stmts out;
        for (auto& st : ss) {
          auto c = std::make_shared<Stmt>(*st);
          if (st->k == Stmt::Return) c->expr = tc.coerce(st->expr, d->res_ty);
          c->body = fix(st->body);
          c->els = fix(st->els);
          out.push_back(c);
        }
        return out;
      };
      d->body = fold_stmts(fix(body));
      instances->open.erase(key);
      instances->by_key[key] = d;
      instances->in_order.push_back(d);
      it = instances->by_key.find(key);
    }
    r->callee = it->second;
    r->sval = it->second->id.str();
    r->ty = it->second->res_ty;
    return r;
  }

  E ext_call(const E& e) {
    if (e->callee) return fun_call(e);
    if (!e->ext || e->ext->backend != (int)opts.backend) fail_rt(e->i, "Call to unknown function " + e->sval);
    const ExtSig& sig = *e->ext;
    if (sig.params.size() != e->args.size())
      fail_rt(e->i, "Function " + sig.py_name + " expected " + std::to_string(sig.params.size()) + " arguments, but received " +
                        std::to_string(e->args.size()) + ".");
    auto r = std::make_shared<Expr>(*e);
    std::vector<Type> tys;
    for (size_t k = 0; k < e->args.size(); ++k) {
      E a = expr(e->args[k]);
      if (sig.params[k].is_pointer()) {
        if (!a->ty.is_array() || a->ty.sz != sig.params[k].sz)
          fail_ty(a->i, "Found incompatible types in function call:\nargument " + std::to_string(k + 1) + " of " + sig.py_name +
                            " has type " + a->ty.str() + ", expected an array of " + Type::scalar(sig.params[k].sz).str());
      } else {
        if (!a->ty.is_scalar())
          fail_ty(a->i, "Found incompatible types in function call:\nargument " + std::to_string(k + 1) + " of " + sig.py_name +
                            " has type " + a->ty.str() + ", expected " + sig.params[k].str());
        a = ensure_scalar(a, sig.params[k].sz);
      }
      tys.push_back(a->ty);
      r->args[k] = a;
    }
    auto seen = ext_arg_types.find(sig.py_name);
    if (seen == ext_arg_types.end()) ext_arg_types[sig.py_name] = tys;
    else
      for (size_t k = 0; k < tys.size(); ++k)
        if (tys[k] != seen->second[k])
          fail_ty(e->i, "Found incompatible types in function call:\n" + tys[k].str() + " and " + seen->second[k].str() +
                            " for argument " + std::to_string(k + 1) + " of " + sig.py_name);
    r->ty = sig.ret;
    return r;
  }

  E binop(const E& e) {
    E a = expr(e->args[0]), b = expr(e->args[1]);
    const Info& i = e->i;
    Type ty = lub(a->ty, b->ty, i);
    if (!ty.is_scalar()) fail_ty(i, "Invalid type " + ty.str() + " of binary operation");
    a = coerce(a, ty);
    b = coerce(b, ty);
    Type rty = ty;
    bool isint = is_int(ty.sz), isflt = is_float(ty.sz), isbool = ty.sz == ElemSize::Bool;
    switch (e->bop) {
      case BinOp::Add: case BinOp::Sub: case BinOp::Mul: case BinOp::Div:
        if (!isint && !isflt) fail_ty(i, "Invalid type " + ty.str() + " of arithmetic operation");
        break;
      case BinOp::FloorDiv: case BinOp::Rem:
        if (!isint) fail_ty(i, "Invalid type " + ty.str() + " of integer arithmetic operation");
        break;
      case BinOp::Pow:
        if (!(ty.sz == ElemSize::F32 || ty.sz == ElemSize::F64))
          fail_ty(i, "Invalid type " + ty.str() + " of floating-point arithmetic operation");
        break;
      case BinOp::And: case BinOp::Or:
        if (!isbool) fail_ty(i, "Invalid type " + ty.str() + " of boolean operation");
        break;
      case BinOp::BitAnd: case BinOp::BitOr: case BinOp::BitXor: case BinOp::BitShl: case BinOp::BitShr:
        if (!isint) fail_ty(i, "Invalid type " + ty.str() + " of bitwise operation");
        break;
      case BinOp::Eq: case BinOp::Neq: case BinOp::Leq: case BinOp::Geq: case BinOp::Lt: case BinOp::Gt:
        rty = Type::scalar(ElemSize::Bool);
        break;
      case BinOp::Max: case BinOp::Min:
        if (!isint && !isflt) fail_ty(i, "Invalid type " + ty.str() + " of comparison operation");
        break;
      default:
        fail_ty(i, "Type-checking not implemented for this operator");
    }
    return mk_binop(e->bop, a, b, rty, i);
  }

  E expr(const E& e) {
    switch (e->k) {
      case Expr::Var: {
        if (e->ty.k != Type::Unknown) return e;  // substituted parameter
        auto it = vars.find(e->name);
        if (it == vars.end()) fail_name(e->i, "Found reference to unknown variable " + e->name.s);
        return with_type(e, it->second);
      }
      case Expr::Int: return e->ty.k == Type::Unknown ? with_type(e, Type::scalar(opts.int_size())) : e;
      case Expr::Float: return e->ty.k == Type::Unknown ? with_type(e, Type::scalar(opts.float_size())) : e;
      case Expr::Bool: return with_type(e, Type::scalar(ElemSize::Bool));
      case Expr::Str: fail_ty(e->i, "String literals may only be used as dictionary keys");
      case Expr::UnOpE: {
        E a = expr(e->args[0]);
        const Type& ty = a->ty;
        switch (e->uop) {
          case UnOp::Sub:
            if (!(is_scalar_of(ty, is_int) || is_scalar_of(ty, is_float))) fail_ty(e->i, "Invalid type " + ty.str() + " of unary minus");
            break;
          case UnOp::Not:
            if (!(ty.is_scalar() && ty.sz == ElemSize::Bool)) fail_ty(e->i, "Invalid type " + ty.str() + " of boolean negation");
            break;
          case UnOp::BitNeg:
            if (!is_scalar_of(ty, is_int)) fail_ty(e->i, "Invalid type " + ty.str() + " of bitwise negation");
            break;
          default: break;
        }
        return mk_unop(e->uop, a, ty, e->i);
      }
      case Expr::BinOpE: return binop(e);
      case Expr::IfExpr: {
        E c = expr(e->args[0]), a = expr(e->args[1]), b = expr(e->args[2]);
        if (!c->ty.is_scalar()) fail_ty(e->i, "Unsupported type " + c->ty.str() + " of conditional expression");
        Type ty = lub(a->ty, b->ty, e->i);
        return mk_ifexpr(c, coerce(a, ty), coerce(b, ty), ty, e->i);
      }
      case Expr::Subscript: return subscript(e);
      case Expr::Slice: fail_rt(e->i, "Slice expressions are only allowed in assignment statements.");
      case Expr::Tuple: fail_ty(e->i, "Tuple expressions are only supported as indices");
      case Expr::BuiltinE: return builtin(e);
      case Expr::Call: return ext_call(e);
      case Expr::Convert: {
        E a = expr(e->args[0]);
        auto r = std::make_shared<Expr>(*e);
        r->args = {a};
        return r;
      }
      case Expr::NeutralElement: {
        E t = expr(e->args[0]);
        if (!t->ty.is_scalar()) fail_ty(e->i, "Reduction over non-scalar elements of type " + t->ty.str());
        return neutral_element(e->bop, t->ty.sz, e->i);
      }
      default: return e;
    }
  }

  E condition(const E& c) {
    E r = expr(c);
    if (!r->ty.is_scalar()) fail_ty(c->i, "Unsupported type " + r->ty.str() + " of conditional expression");
    return r;
  }

  Stmts stmts(const Stmts& ss) {
    Stmts out;
    for (auto& s : ss) out.push_back(stmt(s));
    return out;
  }

  S stmt(const S& s) {
    auto r = std::make_shared<Stmt>(*s);
    switch (s->k) {
      case Stmt::Def: {
        if (s->expr->k == Expr::NeutralElement && s->expr->args.empty()) {
          // the result variable of an inlined call with several returns: typed by its first assignment
          pending.insert(s->id);
          break;
        }
        r->expr = expr(s->expr);
        r->ty = r->expr->ty;
        if (r->ty.k != Type::Tensor) fail_ty(s->i, "Unsupported type " + r->ty.str() + " of variable " + s->id.s);
        vars[s->id] = r->ty;
        break;
      }
      case Stmt::Assign: {
        if (s->dst->k == Expr::Var && pending.count(s->dst->name)) {
          r->expr = expr(s->expr);
          if (!r->expr->ty.is_scalar()) fail_ty(s->i, "Unsupported type " + r->expr->ty.str() + " of the value returned by a called function");
          vars[s->dst->name] = r->expr->ty;
          resolved[s->dst->name] = r->expr->ty;
          pending.erase(s->dst->name);
          r->dst = with_type(s->dst, r->expr->ty);
          break;
        }
        r->dst = expr(s->dst);
        r->expr = coerce(expr(s->expr), r->dst->ty);
        break;
      }
      case Stmt::For: {
        r->lo = ensure_scalar(expr(s->lo), opts.int_size());
        r->hi = ensure_scalar(expr(s->hi), opts.int_size());
        vars[s->id] = Type::scalar(opts.int_size());
        r->body = stmts(s->body);
        break;
      }
      case Stmt::While:
        r->expr = condition(s->expr);
        r->body = stmts(s->body);
        break;
      case Stmt::If:
        r->expr = condition(s->expr);
        r->body = stmts(s->body);
        r->els = stmts(s->els);
        break;
      case Stmt::WithGpu:
        r->body = stmts(s->body);
        break;
      case Stmt::Return:
        r->expr = expr(s->expr);
        res_ty = res_ty.k == Type::Void ? r->expr->ty : lub(res_ty, r->expr->ty, s->i);
        break;
      case Stmt::CallStmt:
        fail_ty(s->i, "Call to function " + s->fname + " should have been inlined (internal error)");
      default:
        break;
    }
    return r;
  }
};

bool has_parallelism(const Stmts& ss, const std::map<std::string, LoopPar>& par) {  // src/py/par.rs:14-55
  for (auto& s : ss) {
    for (auto& l : s->labels)
      if (par.count(l)) return true;
    if (s->k == Stmt::WithGpu) return true;
    if (has_parallelism(s->body, par) || has_parallelism(s->els, par)) return true;
  }
  return false;
}

bool has_return(const Stmts& ss) {
  for (auto& s : ss)
    if (s->k == Stmt::Return || has_return(s->body) || has_return(s->els)) return true;
  return false;
}

}  // namespace

FunDef specialize(const ParsedFun& pf, const std::vector<ArgDesc>& args, const Options& opts, NameGen& gen) {
  if (!opts.device_functions && pf.inline_error) throw *pf.inline_error;
  const FunDef& f = opts.device_functions ? pf.fun_calls : pf.fun;
  if (!has_parallelism(f.body, opts.parallelize))
    fail_rt(f.i, "The function " + f.id.s +
                     " does not contain any parallelism, which is not allowed. Try adding a label ('parpy.label') in "
                     "front of a parallelizable statement, and specify its parallelism using the 'parallelize' keyword "
                     "argument. Alternatively, if you want to run sequential code on the GPU, wrap the code in a GPU "
                     "context as 'with parpy.gpu: ...'.");
  if (args.size() != f.params.size())
    fail_ty(f.i, "Function " + f.id.s + " expected " + std::to_string(f.params.size()) + " arguments, but received " +
                     std::to_string(args.size()) + ".");
  if (has_return(f.body)) fail_rt(f.i, "The called function " + f.id.s + " cannot return a value");  // src/py/no_return.rs:10-16

  Specializer sp(opts, gen);
  for (size_t k = 0; k < args.size(); ++k)
    sp.binds[f.params[k].id] = sp.bind(f.params[k].id.s, args[k], f.params[k].i, false);

  FunDef out;
  out.id = f.id;
  out.i = f.i;
  out.params = sp.flat_params;
  out.res_ty = Type::vvoid();
  Stmts body = fold_stmts(sp.subst_stmts(f.body));

  SliceExpander se{gen, {}};
  for (auto& p : out.params) se.arrays[p.id] = p.ty;
  body = se.run(body);

  TypeChecker tc(opts);
  for (auto& p : out.params) tc.vars[p.id] = p.ty;
  body = tc.finish(tc.stmts(body));
  out.body = fold_stmts(body);
  out.device_funs = tc.instances->in_order;
  return out;
}

}  // namespace parpy
