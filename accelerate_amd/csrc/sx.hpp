// S-expression reader for the textual array program (one list per AST constructor of the
// reference's DelayedOpenAcc / OpenExp terms; de Bruijn indices preserved).
#pragma once
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace acchip {

struct Error : std::runtime_error {
  using std::runtime_error::runtime_error;
};

struct Sx {
  bool atom = false;
  std::string s;            // atom text
  std::vector<Sx> kids;     // list elements

  bool is(const char* head) const { return !atom && !kids.empty() && kids[0].atom && kids[0].s == head; }
  bool isAtom(const char* a) const { return atom && s == a; }
  const std::string& head() const {
    static const std::string none;
    if (atom) return s;
    return (!kids.empty() && kids[0].atom) ? kids[0].s : none;
  }
  const Sx& at(size_t i) const {
    if (atom || i >= kids.size()) throw Error("malformed term near '" + str().substr(0, 80) + "'");
    return kids[i];
  }
  size_t size() const { return kids.size(); }
  long long asInt() const {
    if (!atom) throw Error("expected integer, got list");
    return std::stoll(s, nullptr, 0);
  }
  std::string str() const {
    if (atom) return s;
    std::string r = "(";
    for (size_t i = 0; i < kids.size(); ++i) {
      if (i) r += ' ';
      r += kids[i].str();
    }
    return r + ")";
  }
};

inline Sx parseSx(const char* text, size_t len) {
  size_t pos = 0;
  auto skip = [&]() {
    while (pos < len && (text[pos] == ' ' || text[pos] == '\n' || text[pos] == '\t' || text[pos] == '\r')) ++pos;
  };
  struct Rec {
    static Sx go(const char* t, size_t n, size_t& p, int depth) {
      if (depth > 4096) throw Error("program text nested too deeply");
      while (p < n && (t[p] == ' ' || t[p] == '\n' || t[p] == '\t' || t[p] == '\r')) ++p;
      if (p >= n) throw Error("unexpected end of program text");
      Sx out;
      if (t[p] == '(') {
        ++p;
        for (;;) {
          while (p < n && (t[p] == ' ' || t[p] == '\n' || t[p] == '\t' || t[p] == '\r')) ++p;
          if (p >= n) throw Error("unbalanced '(' in program text");
          if (t[p] == ')') { ++p; break; }
          out.kids.push_back(go(t, n, p, depth + 1));
        }
        return out;
      }
      if (t[p] == ')') throw Error("unbalanced ')' in program text");
      size_t b = p;
      while (p < n && t[p] != '(' && t[p] != ')' && t[p] != ' ' && t[p] != '\n' && t[p] != '\t' && t[p] != '\r') ++p;
      out.atom = true;
      out.s.assign(t + b, p - b);
      return out;
    }
  };
  Sx r = Rec::go(text, len, pos, 0);
  skip();
  if (pos != len) throw Error("trailing input after program text");
  return r;
}

}  // namespace acchip
