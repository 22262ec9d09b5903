// Decoration-time front end: S-expression -> untyped AST, symbol binding,
// label association and inlining of statement calls.
//
// Counterpart of the reference's src/py/mod.rs:34-43 (parse_untyped_ast),
// src/py/symbolize.rs, src/py/labels.rs:16-98 and src/py/inline_calls.rs:13-111.
#include "passes.hpp"

namespace parpy {

namespace {

Info parse_info(const SXP& a) {
  Info i;
  if (a->is_list || a->atom.empty() || a->atom[0] != '@') return i;
  sscanf(a->atom.c_str(), "@%d:%d:%d:%d", &i.l0, &i.c0, &i.l1, &i.c1);
  return i;
}

struct Reader {
  std::shared_ptr<Expr> node(Expr::Kind k, const Info& i) {
    auto e = std::make_shared<Expr>();
    e->k = k;
    e->ty = Type();
    e->i = i;
    return e;
  }

  UnOp unop(const std::string& s, const Info& i) {
    if (s == "sub") return UnOp::Sub;
    if (s == "not") return UnOp::Not;
    if (s == "bitneg") return UnOp::BitNeg;
    fail_rt(i, "Unsupported unary expression " + s);
  }

  BinOp binop(const std::string& s, const Info& i) {
    static const std::map<std::string, BinOp> m = {
        {"add", BinOp::Add}, {"sub", BinOp::Sub}, {"mul", BinOp::Mul}, {"div", BinOp::Div},
        {"floordiv", BinOp::FloorDiv}, {"rem", BinOp::Rem}, {"pow", BinOp::Pow}, {"and", BinOp::And},
        {"or", BinOp::Or}, {"bitand", BinOp::BitAnd}, {"bitor", BinOp::BitOr}, {"bitxor", BinOp::BitXor},
        {"shl", BinOp::BitShl}, {"shr", BinOp::BitShr}, {"eq", BinOp::Eq}, {"neq", BinOp::Neq},
        {"leq", BinOp::Leq}, {"geq", BinOp::Geq}, {"lt", BinOp::Lt}, {"gt", BinOp::Gt}};
    auto it = m.find(s);
    if (it == m.end()) fail_rt(i, "Unsupported binary operation: " + s);
    return it->second;
  }

  E expr(const SXP& x) {
    if (!x->is_list || x->size() < 2) throw std::runtime_error("malformed expression node");
    const std::string& h = x->head();
    Info i = parse_info(x->at(1));
    if (h == "var") {
      auto e = node(Expr::Var, i);
      e->name = Name{x->at(2)->atom, 0};
      return e;
    }
    if (h == "int") { auto e = node(Expr::Int, i); e->iv = x->at(2)->as_int(); return e; }
    if (h == "float") { auto e = node(Expr::Float, i); e->fv = x->at(2)->as_double(); return e; }
    if (h == "bool") { auto e = node(Expr::Bool, i); e->bv = x->at(2)->atom == "true"; return e; }
    if (h == "str") { auto e = node(Expr::Str, i); e->sval = x->at(2)->atom; return e; }
    if (h == "unop") {
      auto e = node(Expr::UnOpE, i);
      e->uop = unop(x->at(2)->atom, i);
      e->args = {expr(x->at(3))};
      return e;
    }
    if (h == "binop") {
      auto e = node(Expr::BinOpE, i);
      e->bop = binop(x->at(2)->atom, i);
      e->args = {expr(x->at(3)), expr(x->at(4))};
      return e;
    }
    if (h == "ifexp") {
      auto e = node(Expr::IfExpr, i);
      e->args = {expr(x->at(2)), expr(x->at(3)), expr(x->at(4))};
      return e;
    }
    if (h == "sub") {
      auto e = node(Expr::Subscript, i);
      e->args = {expr(x->at(2)), expr(x->at(3))};
      return e;
    }
    if (h == "slice") {
      auto e = node(Expr::Slice, i);
      e->args = {x->at(2)->is_sym("none") ? E() : expr(x->at(2)), x->at(3)->is_sym("none") ? E() : expr(x->at(3))};
      return e;
    }
    if (h == "tuple") {
      auto e = node(Expr::Tuple, i);
      for (size_t k = 2; k < x->size(); ++k) e->args.push_back(expr(x->at(k)));
      return e;
    }
    if (h == "call") {
      auto e = node(Expr::Call, i);
      e->sval = x->at(2)->atom;
      for (size_t k = 3; k < x->size(); ++k) e->args.push_back(expr(x->at(k)));
      return e;
    }
    if (h == "builtin") {
      auto e = node(Expr::BuiltinE, i);
      const std::string& n = x->at(2)->atom;
      static const std::map<std::string, Builtin> m = {
          {"exp", Builtin::Exp}, {"inf", Builtin::Inf}, {"log", Builtin::Log}, {"min", Builtin::Min},
          {"max", Builtin::Max}, {"abs", Builtin::Abs}, {"cos", Builtin::Cos}, {"sin", Builtin::Sin},
          {"sqrt", Builtin::Sqrt}, {"tanh", Builtin::Tanh}, {"atan2", Builtin::Atan2}, {"sum", Builtin::Sum},
          {"prod", Builtin::Prod}, {"label", Builtin::Label}, {"gpu", Builtin::Gpu}};
      if (n.rfind("convert_", 0) == 0) {
        e->fn = Builtin::Convert;
        ElemSize sz;
        if (!parse_elem_tag(n.substr(8), &sz)) fail_rt(i, "Unknown conversion " + n);
        e->ty = Type::scalar(sz);  // target type is carried in ty until type checking
      } else {
        auto it = m.find(n);
        if (it == m.end()) fail_rt(i, "Unknown built-in operator " + n);
        e->fn = it->second;
      }
      if (!x->at(3)->is_sym("none")) { e->has_axis = true; e->iv = x->at(3)->as_int(); }
      for (size_t k = 4; k < x->size(); ++k) e->args.push_back(expr(x->at(k)));
      return e;
    }
    throw std::runtime_error("unknown expression node '" + h + "'");
  }

  Stmts stmts(const SXP& lst, size_t from = 1) {
    Stmts r;
    for (size_t k = from; k < lst->size(); ++k) r.push_back(stmt(lst->at(k)));
    return r;
  }

  S stmt(const SXP& x) {
    const std::string& h = x->head();
    Info i = parse_info(x->at(1));
    auto s = std::make_shared<Stmt>();
    s->i = i;
    if (h == "for") {
      s->k = Stmt::For;
      s->id = Name{x->at(2)->atom, 0};
      s->lo = expr(x->at(3));
      s->hi = expr(x->at(4));
      s->step = x->at(5)->as_int();
      s->body = stmts(x->at(6));
      s->par = LoopPar();
    } else if (h == "while") {
      s->k = Stmt::While;
      s->expr = expr(x->at(2));
      s->body = stmts(x->at(3));
    } else if (h == "if") {
      s->k = Stmt::If;
      s->expr = expr(x->at(2));
      s->body = stmts(x->at(3));
      s->els = stmts(x->at(4));
    } else if (h == "assign") {
      s->k = Stmt::Assign;
      s->dst = expr(x->at(2));
      s->expr = expr(x->at(3));
    } else if (h == "withgpu") {
      s->k = Stmt::WithGpu;
      s->body = stmts(x->at(2));
    } else if (h == "callstmt") {
      s->k = Stmt::CallStmt;
      s->fname = x->at(2)->atom;
      for (size_t k = 3; k < x->size(); ++k) s->args.push_back(expr(x->at(k)));
    } else if (h == "label") {
      s->k = Stmt::Label;
      s->fname = x->at(2)->atom;
    } else if (h == "return") {
      s->k = Stmt::Return;
      s->expr = expr(x->at(2));
    } else {
      throw std::runtime_error("unknown statement node '" + h + "'");
    }
    return s;
  }

  Type annotation(const SXP& x, const Info& i) {
    if (x->is_sym("none")) return Type();
    ElemSize sz;
    if (!x->is_list || x->size() != 2 || !parse_elem_tag(x->at(1)->atom, &sz))
      fail_rt(i, "Unsupported parameter type annotation");
    if (x->head() == "scalar") return Type::scalar(sz);
    if (x->head() == "pointer") return Type::pointer(sz);
    fail_rt(i, "Unsupported parameter type annotation");
  }

  FunDef fun(const SXP& x) {
    if (x->head() != "fun") throw std::runtime_error("expected (fun ...)");
    FunDef f;
    f.id = Name{x->at(1)->atom, 0};
    f.i = parse_info(x->at(2));
    f.res_ty = annotation(x->at(3), f.i);
    const SXP& ps = x->at(4);
    for (size_t k = 1; k < ps->size(); ++k) {
      const SXP& p = ps->at(k);
      Param q;
      q.id = Name{p->at(1)->atom, 0};
      q.i = parse_info(p->at(3));
      q.ty = annotation(p->at(2), q.i);
      f.params.push_back(q);
    }
    f.body = stmts(x->at(5));
    return f;
  }
};

// ---------------------------------------------------------------- symbolize
// The first assignment to a name that is not bound in an enclosing scope
// becomes a definition (src/py/symbolize.rs:104-122).  Scopes follow the block
// structure because the emitted code is C++.
struct Symbolizer {
  NameGen& gen;
  std::vector<std::map<std::string, Name>> scopes;

  explicit Symbolizer(NameGen& g) : gen(g) {}

  const Name* lookup(const std::string& s) const {
    for (auto it = scopes.rbegin(); it != scopes.rend(); ++it) {
      auto f = it->find(s);
      if (f != it->end()) return &f->second;
    }
    return nullptr;
  }

  E expr(const E& e) {
    if (!e) return e;
    if (e->k == Expr::Var) {
      if (e->name.id != 0) return e;
      const Name* n = lookup(e->name.s);
      if (!n) fail_name(e->i, "Found reference to unknown variable " + e->name.s);
      auto r = std::make_shared<Expr>(*e);
      r->name = *n;
      return r;
    }
    return map_children(e, [&](const E& c) { return expr(c); });
  }

  Stmts block(const Stmts& ss) {
    scopes.emplace_back();
    Stmts r;
    for (auto& s : ss) r.push_back(stmt(s));
    scopes.pop_back();
    return r;
  }

  S stmt(const S& s) {
    auto r = std::make_shared<Stmt>(*s);
    switch (s->k) {
      case Stmt::Assign: {
        r->expr = expr(s->expr);
        if (s->dst->k == Expr::Var && !lookup(s->dst->name.s)) {
          r->k = Stmt::Def;
          r->id = gen.fresh(s->dst->name.s);
          r->ty = Type();
          r->dst = nullptr;
          scopes.back()[r->id.s] = r->id;
        } else {
          r->dst = expr(s->dst);
        }
        break;
      }
      case Stmt::For: {
        r->lo = expr(s->lo);
        r->hi = expr(s->hi);
        scopes.emplace_back();
        r->id = gen.fresh(s->id.s);
        scopes.back()[r->id.s] = r->id;
        r->body = block(s->body);
        scopes.pop_back();
        break;
      }
      case Stmt::While:
        r->expr = expr(s->expr);
        r->body = block(s->body);
        break;
      case Stmt::If:
        r->expr = expr(s->expr);
        r->body = block(s->body);
        r->els = block(s->els);
        break;
      case Stmt::WithGpu: {
        // a GPU context is transparent for scoping: what it defines stays visible after it
        Stmts b;
        for (auto& c : s->body) b.push_back(stmt(c));
        r->body = b;
        break;
      }
      case Stmt::CallStmt:
        for (auto& a : r->args) a = expr(a);
        break;
      case Stmt::Return:
        r->expr = expr(s->expr);
        break;
      default:
        break;
    }
    return r;
  }
};

// ---------------------------------------------------------------- labels
S add_labels(const S& s, std::vector<std::string>& l) {
  if (s->k != Stmt::Def && s->k != Stmt::Assign && s->k != Stmt::For)
    fail_rt(s->i, "Cannot associate label with non-parallelizable statement");
  auto r = std::make_shared<Stmt>(*s);
  for (auto& x : l) r->labels.push_back(x);
  l.clear();
  return r;
}

Stmts associate_labels(const Stmts& ss) {
  Stmts out;
  std::vector<std::string> labels;
  for (auto& s0 : ss) {
    if (s0->k == Stmt::Label) {
      labels.push_back(s0->fname);
      continue;
    }
    S s = labels.empty() ? s0 : add_labels(s0, labels);
    if (!s->body.empty() || !s->els.empty()) {
      auto r = std::make_shared<Stmt>(*s);
      r->body = associate_labels(s->body);
      r->els = associate_labels(s->els);
      s = r;
    }
    out.push_back(s);
  }
  if (!labels.empty())
    fail_rt(out.empty() ? Info() : out.back()->i, "Found labels not associated with any statement");
  return out;
}

// ---------------------------------------------------------------- inlining of statement calls
struct Inliner {
  NameGen& gen;
  const std::map<std::string, const ParsedFun*>& tops;
  // Calls of jitted functions inside expressions stay calls (for the device_functions option) when the callee only
  // uses its parameters as scalars; statement calls are inlined either way.
  bool keep_expr_calls = false;

  const FunDef& body_of(const ParsedFun* pf) const {
    if (!keep_expr_calls && pf->inline_error) throw *pf->inline_error;
    return keep_expr_calls ? pf->fun_calls : pf->fun;
  }

  // no parameter is subscripted or sliced: the callee can take its arguments by value
  static bool scalar_parameters_only(const FunDef& f) {
    std::set<Name> params;
    for (auto& q : f.params) params.insert(q.id);
    bool ok = true;
    std::function<void(const Stmts&)> walk = [&](const Stmts& ss) {
      for (auto& st : ss) {
        auto scan = [&](const E& root) {
          visit_exprs(root, [&](const E& x) {
            if (x->k == Expr::Slice) ok = false;
            if (x->k == Expr::Subscript && x->args[0]->k == Expr::Var && params.count(x->args[0]->name)) ok = false;
          });
        };
        scan(st->dst); scan(st->expr); scan(st->lo); scan(st->hi);
        for (auto& a : st->args) scan(a);
        if (!st->labels.empty() || st->k == Stmt::WithGpu || st->k == Stmt::CallStmt) ok = false;
        walk(st->body);
        walk(st->els);
      }
    };
    walk(f.body);
    return ok;
  }

  // substitute parameters by argument expressions and give every callee-local
  // name a fresh identity in the caller
  struct Sub {
    std::map<Name, E> params;
    std::map<Name, Name> locals;
  };

  E sub_expr(const E& e, Sub& sub) {
    if (!e) return e;
    if (e->k == Expr::Var) {
      auto p = sub.params.find(e->name);
      if (p != sub.params.end()) {
        auto r = std::make_shared<Expr>(*p->second);
        r->i = e->i;
        return r;
      }
      auto l = sub.locals.find(e->name);
      if (l != sub.locals.end()) {
        auto r = std::make_shared<Expr>(*e);
        r->name = l->second;
        return r;
      }
      return e;
    }
    E r = map_children(e, [&](const E& c) { return sub_expr(c, sub); });
    return merge_subscripts(r);
  }

  // A parameter bound to a partially indexed array (`f(x[i])`) turns the callee's `x[j]` into
  // `x[i][j]`: one subscript with the indices in sequence.
  static E merge_subscripts(const E& e) {
    if (e->k != Expr::Subscript || e->args[0]->k != Expr::Subscript) return e;
    const E& inner = e->args[0];
    auto list = [](const E& idx) { return idx->k == Expr::Tuple ? idx->args : std::vector<E>{idx}; };
    std::vector<E> idxs = list(inner->args[1]);
    for (auto& x : idxs)
      if (x->k == Expr::Slice || x->k == Expr::Str) return e;  // slices of slices are rejected later; d["key"][i] stays a field access
    for (auto& x : list(e->args[1])) idxs.push_back(x);
    auto t = std::make_shared<Expr>();
    t->k = Expr::Tuple;
    t->args = idxs;
    t->i = e->args[1]->i;
    auto r = std::make_shared<Expr>(*e);
    r->args = {inner->args[0], E(t)};
    return merge_subscripts(r);
  }

  // Calls inside expressions.  A call of an external stays a call (its signature is attached); a
  // call of a jitted function is replaced by the value it returns, with the statements in front
  // of its final `return` placed before the statement that contains the call.
  E inline_expr(const E& e, Stmts& pre) {
    if (!e) return e;
    E r = map_children(e, [&](const E& c) { return inline_expr(c, pre); });
    if (r->k != Expr::Call) return r;
    auto it = tops.find(r->sval);
    if (it == tops.end()) fail_rt(r->i, "Call to unknown function " + r->sval);
    const ParsedFun* pf = it->second;
    if (pf->ext) {
      auto c = std::make_shared<Expr>(*r);
      c->ext = pf->ext;
      return c;
    }
    const FunDef& f = body_of(pf);
    if (f.params.size() != r->args.size())
      fail_rt(r->i, "Function " + f.id.s + " expected " + std::to_string(f.params.size()) + " arguments, but received " +
                        std::to_string(r->args.size()) + ".");
    if (f.body.empty() || !always_returns(f.body))
      fail_ty(r->i, "Unknown return type of function " + f.id.s);
    if (keep_expr_calls && scalar_parameters_only(f)) {
      auto c = std::make_shared<Expr>(*r);
      c->callee = std::make_shared<FunDef>(f);
      return c;
    }
    Sub sub;
    for (size_t k = 0; k < f.params.size(); ++k) {
      E a = r->args[k];
      if (f.params[k].ty.k == Type::Tensor && f.params[k].ty.shape.empty()) {
        // an annotated scalar parameter: the argument is converted to the declared type
        auto c = std::make_shared<Expr>();
        c->k = Expr::BuiltinE;
        c->fn = Builtin::Convert;
        c->ty = Type::scalar(f.params[k].ty.sz);
        c->args = {a};
        c->i = a->i;
        a = c;
      }
      sub.params[f.params[k].id] = a;
    }
    if (count_returns(f.body) == 1 && f.body.back()->k == Stmt::Return) {
      Stmts head(f.body.begin(), f.body.end() - 1);
      for (auto& st : sub_stmts(head, sub)) pre.push_back(st);
      return sub_expr(f.body.back()->expr, sub);
    }
    // Several return statements (`if c: return a` ... `return b`).  The reference keeps such a callee as a device
    // function (src/py/insert_called_functions.rs:12-88); here the body is inlined like any other with the
    // returned value in a variable: what follows a conditional that returns moves into the branch that goes on,
    // every `return e` becomes `result = e`.  The variable takes the type of the first value assigned to it.
    if (return_in_loop(f.body, false))
      fail_rt(r->i, "A return statement inside a loop of function " + f.id.s + " is not supported when the call is part of an expression");
    Name res = gen.fresh(f.id.s + "_result");
    E resv = mk_var(res, Type(), r->i);
    auto marker = std::make_shared<Expr>();
    marker->k = Expr::NeutralElement;   // without operand: a definition whose type comes from the first assignment
    marker->bop = BinOp::Add;
    marker->i = r->i;
    pre.push_back(mk_def(res, Type(), marker, r->i));
    for (auto& st : sub_stmts(lower_returns(f.body, resv), sub)) pre.push_back(st);
    return resv;
  }

  static int count_returns(const Stmts& ss) {
    int n = 0;
    for (auto& s : ss) n += (s->k == Stmt::Return) + count_returns(s->body) + count_returns(s->els);
    return n;
  }

  static bool return_in_loop(const Stmts& ss, bool in_loop) {
    for (auto& s : ss) {
      if (s->k == Stmt::Return && in_loop) return true;
      bool loop = in_loop || s->k == Stmt::For || s->k == Stmt::While;
      if (return_in_loop(s->body, loop) || return_in_loop(s->els, loop)) return true;
    }
    return false;
  }

  static bool always_returns(const Stmts& ss) {
    if (ss.empty()) return false;
    const S& last = ss.back();
    if (last->k == Stmt::Return) return true;
    return last->k == Stmt::If && always_returns(last->body) && always_returns(last->els);
  }

  static Stmts lower_returns(const Stmts& ss, const E& res) {
    Stmts out;
    for (size_t i = 0; i < ss.size(); ++i) {
      const S& s = ss[i];
      if (s->k == Stmt::Return) {
        out.push_back(mk_assign(res, s->expr, s->i));
        return out;   // nothing after a return runs
      }
      if (s->k == Stmt::If && (count_returns(s->body) || count_returns(s->els))) {
        Stmts rest(ss.begin() + i + 1, ss.end());
        Stmts b = s->body, e = s->els;
        if (!always_returns(b)) b.insert(b.end(), rest.begin(), rest.end());
        if (!always_returns(e)) e.insert(e.end(), rest.begin(), rest.end());
        auto r = std::make_shared<Stmt>(*s);
        r->body = lower_returns(b, res);
        r->els = lower_returns(e, res);
        out.push_back(r);
        return out;
      }
      out.push_back(s);
    }
    return out;
  }

  Stmts sub_stmts(const Stmts& ss, Sub& sub) {
    Stmts out;
    for (auto& s : ss) {
      auto r = std::make_shared<Stmt>(*s);
      if (s->k == Stmt::Def || s->k == Stmt::For) {
        Name n = gen.fresh(s->id.s);
        sub.locals[s->id] = n;
        r->id = n;
      }
      if (s->k == Stmt::Return) fail_rt(s->i, "Cannot inline a call to a function containing a return statement");
      if (r->dst) {
        if (r->dst->k == Expr::Var && sub.params.count(r->dst->name) && sub.params[r->dst->name]->k != Expr::Var)
          fail_rt(s->i, "Cannot assign to a parameter bound to a non-variable argument in an inlined call");
        r->dst = sub_expr(r->dst, sub);
      }
      if (r->expr) r->expr = sub_expr(r->expr, sub);
      if (r->lo) r->lo = sub_expr(r->lo, sub);
      if (r->hi) r->hi = sub_expr(r->hi, sub);
      for (auto& a : r->args) a = sub_expr(a, sub);
      r->body = sub_stmts(s->body, sub);
      r->els = sub_stmts(s->els, sub);
      out.push_back(r);
    }
    return out;
  }

  Stmts run(const Stmts& ss) {
    Stmts out;
    for (auto& s : ss) {
      if (s->k == Stmt::CallStmt) {
        auto it = tops.find(s->fname);
        if (it == tops.end()) fail_rt(s->i, "Reference to unknown function " + s->fname + ".");
        const FunDef& f = body_of(it->second);
        if (f.params.size() != s->args.size())
          fail_rt(f.i, "Function " + f.id.s + " expected " + std::to_string(f.params.size()) +
                           " arguments, but received " + std::to_string(s->args.size()) + ".");
        if (it->second->ext) fail_rt(s->i, "Cannot inline call to external function " + s->fname);
        Sub sub;
        for (size_t k = 0; k < f.params.size(); ++k) sub.params[f.params[k].id] = inline_expr(s->args[k], out);
        Stmts body = sub_stmts(f.body, sub);
        for (auto& b : body) out.push_back(b);
        continue;
      }
      auto r = std::make_shared<Stmt>(*s);
      Stmts pre;
      if (r->dst) r->dst = inline_expr(r->dst, pre);
      if (r->expr) r->expr = inline_expr(r->expr, pre);
      if (r->lo) r->lo = inline_expr(r->lo, pre);
      if (r->hi) r->hi = inline_expr(r->hi, pre);
      if (!pre.empty() && s->k == Stmt::While)
        fail_rt(s->i, "A function called in the condition of a while loop must consist of a single return statement");
      for (auto& q : pre) out.push_back(q);
      r->body = run(s->body);
      r->els = run(s->els);
      out.push_back(r);
    }
    return out;
  }
};

}  // namespace

std::unique_ptr<ParsedFun> parse_function(const std::string& sexpr,
                                          const std::map<std::string, const ParsedFun*>& tops) {
  SXP x = parse_sexpr(sexpr);
  auto pf = std::make_unique<ParsedFun>();
  Reader rd;
  if (x->head() == "ext") {
    // (ext "python name" "target name" <return annotation> (params (p name annotation info)...) "header" backend nthreads info)
    auto sig = std::make_shared<ExtSig>();
    sig->py_name = x->at(1)->atom;
    sig->name = x->at(2)->atom;
    Info i = parse_info(x->at(8));
    if (x->at(3)->is_sym("none")) fail_rt(i, "Unsupported return type annotation on external function");
    sig->ret = rd.annotation(x->at(3), i);
    if (!sig->ret.is_scalar()) fail_rt(i, "Unsupported return type annotation on external function");
    const SXP& ps = x->at(4);
    for (size_t k = 1; k < ps->size(); ++k) {
      Info pi = parse_info(ps->at(k)->at(3));
      if (ps->at(k)->at(2)->is_sym("none")) fail_rt(pi, "Unsupported parameter type annotation");
      sig->params.push_back(rd.annotation(ps->at(k)->at(2), pi));
    }
    sig->header = x->at(5)->atom;
    sig->backend = (int)x->at(6)->as_int();
    sig->par_threads = x->at(7)->as_int();
    pf->fun.id = Name{sig->py_name, 0};
    pf->fun.i = i;
    pf->ext = sig;
    pf->source_text = "external " + sig->py_name + " = " + sig->name;
    return pf;
  }
  pf->fun = rd.fun(x);

  // symbolize: parameters first, then the body
  Symbolizer sym(pf->gen);
  sym.scopes.emplace_back();
  for (auto& p : pf->fun.params) {
    p.id = pf->gen.fresh(p.id.s);
    sym.scopes.back()[p.id.s] = p.id;
  }
  Stmts body;
  for (auto& s : pf->fun.body) body.push_back(sym.stmt(s));
  pf->fun.body = associate_labels(body);

  pf->fun_calls = pf->fun;
  pf->gen_calls = pf->gen;
  Inliner keep{pf->gen_calls, tops};
  keep.keep_expr_calls = true;
  pf->fun_calls.body = keep.run(pf->fun_calls.body);
  // what only the inlined form cannot express (a callee that returns from inside a loop) is reported when that form
  // is asked for; everything else has already been reported by the run above
  try {
    Inliner inl{pf->gen, tops};
    pf->fun.body = inl.run(pf->fun.body);
  } catch (const CompileError& e) {
    pf->inline_error = std::make_shared<CompileError>(e);
  }
  pf->source_text = print_fun(pf->inline_error ? pf->fun_calls : pf->fun);
  return pf;
}

}  // namespace parpy
