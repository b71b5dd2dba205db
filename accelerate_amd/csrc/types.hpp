// Representation types of the array language: scalar leaves, tuple trees, array types
// (reference: Type.hs:112-152, Representation/Type.hs, Representation/Array.hs:43-60).
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "sx.hpp"

namespace acchip {

enum class ST : int { I8, I16, I32, I64, U8, U16, U32, U64, F16, F32, F64 };

// SIMD vector types `Vec n t` (Type.hs VectorType; n in 2, 3, 4, 8, 16), written v<n><t>:
// one leaf whose n components are stored next to each other, n*size(t) bytes per element
// with the alignment of t (Array/Data.hs:119, 190: a buffer of w * size scalars).  Encoded
// in ST as base | n << 8.
inline int stWidth(ST t) { return ((int)t >> 8) ? ((int)t >> 8) : 1; }
inline ST stBase(ST t) { return (ST)((int)t & 0xff); }
inline bool stIsVec(ST t) { return ((int)t >> 8) != 0; }
inline ST stVec(ST base, int n) { return (ST)((int)base | (n << 8)); }
inline bool stVecWidthOk(int n) { return n == 2 || n == 3 || n == 4 || n == 8 || n == 16; }

inline const char* stName(ST t) {
  static const char* n[] = {"i8", "i16", "i32", "i64", "u8", "u16", "u32", "u64", "f16", "f32", "f64"};
  if (!stIsVec(t)) return n[(int)t];
  static const std::vector<std::string> names = [] {
    std::vector<std::string> v(17 * 16);
    for (int w = 2; w <= 16; ++w)
      for (int b = 0; b < 11; ++b) v[w * 16 + b] = "v" + std::to_string(w) + n[b];
    return v;
  }();
  return names[stWidth(t) * 16 + (int)stBase(t)].c_str();
}
inline int stAlign(ST t) {
  static const int n[] = {1, 2, 4, 8, 1, 2, 4, 8, 2, 4, 8};
  return n[(int)stBase(t)];
}
inline int stSize(ST t) { return stAlign(t) * stWidth(t); }
inline int stBits(ST t) { return stSize(t) * 8; }
inline bool stIsFloat(ST t) { return t == ST::F16 || t == ST::F32 || t == ST::F64; }
inline bool stIsSigned(ST t) { return (int)t <= (int)ST::I64; }
inline bool stIsInt(ST t) { return !stIsVec(t) && !stIsFloat(t); }
inline ST stUnsigned(ST t) { return stIsSigned(t) ? (ST)((int)t + 4) : t; }
// type the wrap-around arithmetic of an integer type is carried out in
inline const char* stWide(ST t) { return stSize(t) == 8 ? "u64" : "u32"; }

inline bool parseSTName(const std::string& s, ST& out) {
  for (int i = 0; i <= (int)ST::F64; ++i)
    if (s == stName((ST)i)) {
      out = (ST)i;
      return true;
    }
  if (s.size() >= 4 && s[0] == 'v' && s[1] >= '1' && s[1] <= '9') {
    size_t p = 1;
    int w = 0;
    while (p < s.size() && s[p] >= '0' && s[p] <= '9' && w < 100) w = w * 10 + (s[p++] - '0');
    ST base;
    if (stVecWidthOk(w) && parseSTName(s.substr(p), base) && !stIsVec(base)) {
      out = stVec(base, w);
      return true;
    }
  }
  return false;
}
inline ST parseST(const Sx& s) {
  ST t;
  if (s.atom && parseSTName(s.s, t)) return t;
  throw Error("unknown scalar type '" + s.str() + "'");
}
inline bool isST(const Sx& s) {
  ST t;
  return s.atom && parseSTName(s.s, t);
}

struct Type;
using TypeP = std::shared_ptr<const Type>;
struct Type {
  enum K { Unit, Scalar, Pair } k = Unit;
  ST st = ST::I64;
  TypeP a, b;
};

inline TypeP tUnit() {
  static TypeP u = std::make_shared<Type>();
  return u;
}
inline TypeP tScalar(ST s) {
  auto t = std::make_shared<Type>();
  t->k = Type::Scalar;
  t->st = s;
  return t;
}
inline TypeP tPair(TypeP a, TypeP b) {
  auto t = std::make_shared<Type>();
  t->k = Type::Pair;
  t->a = a;
  t->b = b;
  return t;
}
inline TypeP tShape(int rank) {
  TypeP t = tUnit();
  for (int i = 0; i < rank; ++i) t = tPair(t, tScalar(ST::I64));
  return t;
}
inline TypeP parseType(const Sx& s) {
  if (s.isAtom("unit")) return tUnit();
  if (s.atom) return tScalar(parseST(s));
  if (s.is("pair") && s.size() == 3) return tPair(parseType(s.at(1)), parseType(s.at(2)));
  throw Error("malformed type '" + s.str() + "'");
}
inline void typeLeaves(const TypeP& t, std::vector<ST>& out) {
  if (t->k == Type::Scalar) out.push_back(t->st);
  else if (t->k == Type::Pair) {
    typeLeaves(t->a, out);
    typeLeaves(t->b, out);
  }
}
inline std::vector<ST> typeLeaves(const TypeP& t) {
  std::vector<ST> v;
  typeLeaves(t, v);
  return v;
}
inline bool typeEq(const TypeP& x, const TypeP& y) {
  if (x->k != y->k) return false;
  if (x->k == Type::Scalar) return x->st == y->st;
  if (x->k == Type::Pair) return typeEq(x->a, y->a) && typeEq(x->b, y->b);
  return true;
}
inline std::string typeStr(const TypeP& t) {
  if (t->k == Type::Unit) return "unit";
  if (t->k == Type::Scalar) return stName(t->st);
  return "(pair " + typeStr(t->a) + " " + typeStr(t->b) + ")";
}

struct ArrayR {
  int rank = 0;
  TypeP elt;
};
inline ArrayR parseArrayR(const Sx& s) {
  if (!s.is("array") || s.size() != 3) throw Error("malformed array type '" + s.str() + "'");
  ArrayR r;
  r.rank = (int)s.at(1).asInt();
  if (r.rank < 0 || r.rank > 8) throw Error("array rank out of range (0..8)");
  r.elt = parseType(s.at(2));
  return r;
}

}  // namespace acchip
