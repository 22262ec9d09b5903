// C ABI of the compiler core (declared in include/parpy_hipc.h).
#include <cstring>
#include <chrono>
#include <sstream>

#include "../../../include/parpy_hipc.h"
#include "passes.hpp"

using namespace parpy;

struct parpy_hipc_fun {
  std::unique_ptr<ParsedFun> pf;
  std::string name;
};

namespace {
thread_local std::string g_error;
thread_local int32_t g_error_kind = 0;
thread_local int32_t g_error_span[4] = {0, 0, 0, 0};

void set_error(const std::string& msg, int32_t kind, const Info& i) {
  g_error = msg;
  g_error_kind = kind;
  g_error_span[0] = i.l0;
  g_error_span[1] = i.c0;
  g_error_span[2] = i.l1;
  g_error_span[3] = i.c1;
}

char* dup_string(const std::string& s) {
  char* r = (char*)malloc(s.size() + 1);
  memcpy(r, s.c_str(), s.size() + 1);
  return r;
}

template <class F> int32_t guarded(F f) {
  try {
    f();
    return 0;
  } catch (const CompileError& e) {
    set_error(e.what(), (int32_t)e.kind, e.info);
  } catch (const std::exception& e) {
    set_error(e.what(), 0, Info());
  }
  return 1;
}
}  // namespace

extern "C" {

int32_t parpy_hipc_parse(const char* sexpr, const char* const* top_names, const parpy_hipc_fun* const* tops,
                         int32_t ntops, parpy_hipc_fun** out) {
  return guarded([&] {
    std::map<std::string, const ParsedFun*> m;
    for (int32_t k = 0; k < ntops; ++k) m[top_names[k]] = tops[k]->pf.get();
    auto f = new parpy_hipc_fun();
    try {
      f->pf = parse_function(sexpr, m);
    } catch (...) {
      delete f;
      throw;
    }
    f->name = f->pf->fun.id.s;
    *out = f;
  });
}

void parpy_hipc_fun_free(parpy_hipc_fun* f) { delete f; }

const char* parpy_hipc_fun_name(const parpy_hipc_fun* f) { return f->name.c_str(); }

const char* parpy_hipc_fun_print(const parpy_hipc_fun* f) { return f->pf->source_text.c_str(); }

int32_t parpy_hipc_compile(const parpy_hipc_fun* f, const char* args, const char* opts_text, char** device_src,
                           char** plan, char** listing, char** debug_log) {
  return guarded([&] {
    std::vector<ArgDesc> a = parse_args(args);
    Options opts = parse_options(opts_text);
    // the parsed function is shared: every compilation numbers its names from the same start
    NameGen gen = opts.device_functions ? f->pf->gen_calls : f->pf->gen;
    std::ostringstream dbg;
    // every dump carries the time since the start of the compilation (src/utils/debug.rs:10-37)
    auto t0 = std::chrono::steady_clock::now();
    auto stage = [&](const char* name, const std::string& text) {
      if (!opts.debug_print) return;
      auto us = std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now() - t0).count();
      dbg << "=== " << name << " (time: " << us << " us) ===\n" << text << "\n";
    };
    FunDef spec = specialize(*f->pf, a, opts, gen);
    stage("specialised and type-checked", print_fun(spec));
    FunDef low = lower(spec, opts, gen);
    stage("lowered", print_fun(low));
    Program prog = gpu_codegen(low, opts, gen);
    if (opts.debug_print) {
      std::ostringstream ks;
      for (auto& k : prog.kernels) ks << "kernel " << k.name << ":\n" << print_stmts(k.body, 2);
      ks << "host:\n" << print_stmts(prog.host, 2);
      stage("kernels", ks.str());
    }
    hip_optimize(prog, opts, gen);
    if (opts.debug_print) {
      std::ostringstream ks;
      for (auto& k : prog.kernels) ks << "kernel " << k.name << ":\n" << print_stmts(k.body, 2);
      stage("after memory code generation", ks.str());
    }
    std::string dev = hip_print_device(prog, opts);
    std::string pl = hip_print_plan(prog);
    std::string ls = hip_print_listing(prog, opts);
    *device_src = dup_string(dev);
    *plan = dup_string(pl);
    *listing = dup_string(ls);
    if (debug_log) *debug_log = dup_string(dbg.str());
  });
}

void parpy_hipc_free_string(char* s) { free(s); }

const char* parpy_hipc_last_error(void) { return g_error.c_str(); }
int32_t parpy_hipc_last_error_kind(void) { return g_error_kind; }
void parpy_hipc_last_error_span(int32_t* span) { memcpy(span, g_error_span, sizeof g_error_span); }

}  // extern "C"
