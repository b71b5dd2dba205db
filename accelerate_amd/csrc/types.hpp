// Representation types of the array language: scalar leaves, tuple trees, array types
// (reference: Type.hs:112-152, Representation/Type.hs, Representation/Array.hs:43-60).
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "sx.hpp"

namespace acchip {

enum class ST : int { I8, I16, I32, I64, U8, U16, U32, U64, F16, F32, F64 };

inline const char* stName(ST t) {
  static const char* n[] = {"i8", "i16", "i32", "i64", "u8", "u16", "u32", "u64", "f16", "f32", "f64"};
  return n[(int)t];
}
inline int stSize(ST t) {
  static const int n[] = {1, 2, 4, 8, 1, 2, 4, 8, 2, 4, 8};
  return n[(int)t];
}
inline int stBits(ST t) { return stSize(t) * 8; }
inline bool stIsFloat(ST t) { return t == ST::F16 || t == ST::F32 || t == ST::F64; }
inline bool stIsSigned(ST t) { return (int)t <= (int)ST::I64; }
inline bool stIsInt(ST t) { return !stIsFloat(t); }
inline ST stUnsigned(ST t) { return stIsSigned(t) ? (ST)((int)t + 4) : t; }
// type the wrap-around arithmetic of an integer type is carried out in
inline const char* stWide(ST t) { return stSize(t) == 8 ? "u64" : "u32"; }

inline ST parseST(const Sx& s) {
  if (s.atom) {
    for (int i = 0; i <= (int)ST::F64; ++i)
      if (s.s == stName((ST)i)) return (ST)i;
  }
  throw Error("unknown scalar type '" + s.str() + "'");
}
inline bool isST(const Sx& s) {
  if (!s.atom) return false;
  for (int i = 0; i <= (int)ST::F64; ++i)
    if (s.s == stName((ST)i)) return true;
  return false;
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
