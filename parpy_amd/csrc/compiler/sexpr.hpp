// Minimal S-expression reader/writer shared by the compiler core and the
// runtime's launch-plan loader.  Atoms are symbols, numbers or double-quoted
// strings; lists are parenthesised.
#pragma once
#include <cstdint>
#include <cmath>
#include <cstdlib>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace parpy {

struct SX;
using SXP = std::shared_ptr<SX>;

struct SX {
  bool is_list = false;
  bool is_str = false;      // quoted string atom
  std::string atom;         // atom text (unquoted / unescaped)
  std::vector<SXP> items;   // list items

  bool is_atom() const { return !is_list; }
  bool is_sym(const char* s) const { return !is_list && !is_str && atom == s; }
  size_t size() const { return items.size(); }
  const SXP& at(size_t i) const {
    if (!is_list || i >= items.size()) throw std::runtime_error("S-expression index out of range");
    return items[i];
  }
  // head symbol of a list, "" otherwise
  const std::string& head() const {
    static const std::string empty;
    if (is_list && !items.empty() && !items[0]->is_list) return items[0]->atom;
    return empty;
  }
  int64_t as_int() const { return std::strtoll(atom.c_str(), nullptr, 10); }
  double as_double() const {
    if (atom == "inf") return HUGE_VAL;
    if (atom == "-inf") return -HUGE_VAL;
    if (atom == "nan") return std::strtod("nan", nullptr);
    return std::strtod(atom.c_str(), nullptr);
  }
};

class SXParser {
 public:
  explicit SXParser(const std::string& text) : s_(text) {}
  SXP parse() {
    skip();
    SXP r = read();
    skip();
    if (p_ != s_.size()) throw std::runtime_error("trailing characters after S-expression");
    return r;
  }

 private:
  const std::string& s_;
  size_t p_ = 0;
  void skip() {
    while (p_ < s_.size() && (s_[p_] == ' ' || s_[p_] == '\n' || s_[p_] == '\t' || s_[p_] == '\r')) ++p_;
  }
  SXP read() {
    if (p_ >= s_.size()) throw std::runtime_error("unexpected end of S-expression");
    auto n = std::make_shared<SX>();
    char c = s_[p_];
    if (c == '(') {
      ++p_;
      n->is_list = true;
      for (;;) {
        skip();
        if (p_ >= s_.size()) throw std::runtime_error("unterminated list in S-expression");
        if (s_[p_] == ')') { ++p_; break; }
        n->items.push_back(read());
      }
      return n;
    }
    if (c == ')') throw std::runtime_error("unexpected ')' in S-expression");
    if (c == '"') {
      ++p_;
      n->is_str = true;
      while (p_ < s_.size() && s_[p_] != '"') {
        if (s_[p_] == '\\' && p_ + 1 < s_.size()) {
          char e = s_[p_ + 1];
          n->atom.push_back(e == 'n' ? '\n' : e);
          p_ += 2;
        } else {
          n->atom.push_back(s_[p_++]);
        }
      }
      if (p_ >= s_.size()) throw std::runtime_error("unterminated string in S-expression");
      ++p_;
      return n;
    }
    size_t b = p_;
    while (p_ < s_.size() && s_[p_] != ' ' && s_[p_] != '\n' && s_[p_] != '\t' && s_[p_] != '\r' &&
           s_[p_] != '(' && s_[p_] != ')')
      ++p_;
    n->atom = s_.substr(b, p_ - b);
    return n;
  }
};

inline SXP parse_sexpr(const std::string& text) { return SXParser(text).parse(); }

inline std::string sx_quote(const std::string& s) {
  std::string r = "\"";
  for (char c : s) {
    if (c == '\\' || c == '"') { r.push_back('\\'); r.push_back(c); }
    else if (c == '\n') r += "\\n";
    else r.push_back(c);
  }
  r.push_back('"');
  return r;
}

}  // namespace parpy
