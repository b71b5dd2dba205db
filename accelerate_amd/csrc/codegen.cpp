#include "codegen.hpp"

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <regex>
#include <set>

namespace acchip {

// ------------------------------------------------------------------------------------
// values

ValP vUnit() {
  static ValP u = std::make_shared<Val>();
  return u;
}
ValP vLeaf(ST st, const std::string& ex) {
  auto v = std::make_shared<Val>();
  v->k = Val::Leaf;
  v->st = st;
  v->ex = ex;
  return v;
}
ValP vPair(ValP a, ValP b) {
  auto v = std::make_shared<Val>();
  v->k = Val::Pair;
  v->a = std::move(a);
  v->b = std::move(b);
  return v;
}
TypeP valType(const ValP& v) {
  if (v->k == Val::Unit) return tUnit();
  if (v->k == Val::Leaf) return tScalar(v->st);
  return tPair(valType(v->a), valType(v->b));
}
void valLeaves(const ValP& v, std::vector<ValP>& out) {
  if (v->k == Val::Leaf) out.push_back(v);
  else if (v->k == Val::Pair) {
    valLeaves(v->a, out);
    valLeaves(v->b, out);
  }
}
static std::vector<ValP> leavesOf(const ValP& v) {
  std::vector<ValP> o;
  valLeaves(v, o);
  return o;
}

static const ValP& leaf1(const ValP& v, const char* what) {
  if (v->k != Val::Leaf) throw Error(std::string("expected a scalar operand for ") + what);
  return v;
}

// ------------------------------------------------------------------------------------
// literals

std::string literalText(ST st, const std::string& tok) {
  char buf[96];
  if (stIsFloat(st)) {
    double d;
    if (tok == "nan") d = NAN;
    else if (tok == "inf") d = INFINITY;
    else if (tok == "-inf") d = -INFINITY;
    else {
      char* end = nullptr;
      d = std::strtod(tok.c_str(), &end);
      if (!end || *end) throw Error("malformed floating literal '" + tok + "'");
    }
    const char* T = stName(st);
    if (std::isnan(d)) { snprintf(buf, sizeof buf, "((%s)__builtin_nanf(\"\"))", T); return buf; }
    if (std::isinf(d)) { snprintf(buf, sizeof buf, "((%s)%s__builtin_inff())", T, d < 0 ? "-" : ""); return buf; }
    if (st == ST::F64) snprintf(buf, sizeof buf, "(%a)", d);
    else if (st == ST::F32) snprintf(buf, sizeof buf, "(%af)", (double)(float)d);
    else snprintf(buf, sizeof buf, "((f16)%af)", (double)(float)d);
    return buf;
  }
  // integers: accept anything that fits the signed or unsigned range, wrap to the type
  errno = 0;
  char* end = nullptr;
  unsigned long long u;
  if (!tok.empty() && tok[0] == '-') u = (unsigned long long)std::strtoll(tok.c_str(), &end, 0);
  else u = std::strtoull(tok.c_str(), &end, 0);
  if (!end || *end || tok.empty()) throw Error("malformed integer literal '" + tok + "'");
  int bits = stBits(st);
  if (bits < 64) u &= ((1ULL << bits) - 1);
  snprintf(buf, sizeof buf, "((%s)0x%llxULL)", stName(st), u);
  return buf;
}

// ------------------------------------------------------------------------------------
// array slots

const ArraySlot& Codegen::slotForVar(int idx) {
  if (idx < 0 || idx >= (int)aenv_.size()) throw Error("array variable index out of range");
  std::string name = "a" + std::to_string(idx);
  auto it = used_.find(name);
  if (it == used_.end()) {
    ArraySlot s;
    s.name = name;
    s.r = aenv_[idx];
    s.index = idx;
    it = used_.emplace(name, s).first;
  }
  return it->second;
}

std::string Codegen::addTemp(const ArrayR& r) {
  ArraySlot s;
  s.name = "t" + std::to_string(temps_.size());
  s.r = r;
  s.temp = true;
  s.index = (int)temps_.size();
  temps_.push_back(s);
  return s.name;
}

const ArraySlot& Codegen::slotByName(const std::string& name) {
  auto it = used_.find(name);
  if (it != used_.end()) return it->second;
  if (name[0] == 't') {
    int k = std::atoi(name.c_str() + 1);
    if (k < 0 || k >= (int)temps_.size()) throw Error("unknown temporary slot " + name);
    return used_.emplace(name, temps_[k]).first->second;
  }
  if (name == "out") throw Error("output extent slot not declared");
  return slotForVar(std::atoi(name.c_str() + 1));
}

// ------------------------------------------------------------------------------------
// small emit helpers

ValP Codegen::bindLeaf(ST st, const std::string& ex, Emit& em) {
  std::string n = fresh();
  em.line(std::string("const ") + stName(st) + " " + n + " = " + ex + ";");
  return vLeaf(st, n);
}

ValP Codegen::declareVars(const TypeP& t, Emit& em) {
  if (t->k == Type::Unit) return vUnit();
  if (t->k == Type::Scalar) {
    std::string n = fresh();
    em.line(std::string(stName(t->st)) + " " + n + ";");
    return vLeaf(t->st, n);
  }
  ValP a = declareVars(t->a, em);
  return vPair(a, declareVars(t->b, em));
}

void Codegen::assign(const ValP& dst, const ValP& src, Emit& em) {
  auto d = leavesOf(dst), s = leavesOf(src);
  if (d.size() != s.size()) throw Error("internal: assignment between values of different shape");
  for (size_t i = 0; i < d.size(); ++i) {
    if (d[i]->st != s[i]->st) throw Error("type mismatch between branches of a conditional or loop");
    em.line(d[i]->ex + " = " + s[i]->ex + ";");
  }
}

ValP Codegen::copyToVars(const ValP& v, Emit& em) {
  if (v->k == Val::Unit) return v;
  if (v->k == Val::Leaf) {
    std::string n = fresh();
    em.line(std::string(stName(v->st)) + " " + n + " = " + v->ex + ";");
    return vLeaf(v->st, n);
  }
  ValP a = copyToVars(v->a, em);
  return vPair(a, copyToVars(v->b, em));
}

static void pushLhs(const Sx& lhs, const ValP& v, Codegen::Env& env) {
  if (lhs.is("single")) {
    if (v->k != Val::Leaf) throw Error("left-hand side binds a scalar but the value is a tuple: " + lhs.str());
    env.push_back(v);
  } else if (lhs.is("wild")) {
  } else if (lhs.is("pair")) {
    if (v->k != Val::Pair) throw Error("left-hand side is a pair but the value is not: " + lhs.str());
    pushLhs(lhs.at(1), v->a, env);
    pushLhs(lhs.at(2), v->b, env);
  } else {
    throw Error("malformed left-hand side " + lhs.str());
  }
}

ValP Codegen::shapeOf(const ArraySlot& s) {
  ValP v = vUnit();
  for (int d = 0; d < s.r.rank; ++d) v = vPair(v, vLeaf(ST::I64, "env." + s.name + "_d" + std::to_string(d)));
  return v;
}

static void shapeDims(const ValP& sh, std::vector<std::string>& out) {
  if (sh->k == Val::Unit) return;
  if (sh->k != Val::Pair || sh->b->k != Val::Leaf) throw Error("expected a shape value");
  shapeDims(sh->a, out);
  out.push_back(sh->b->ex);
}

std::string Codegen::toIndex(const ValP& sh, const ValP& ix, Emit& em) {
  std::vector<std::string> d, i;
  shapeDims(sh, d);
  shapeDims(ix, i);
  if (d.size() != i.size()) throw Error("toIndex: rank mismatch between shape and index");
  if (d.empty()) return "((i64)0)";
  if (d.size() == 1) return i[0];
  std::string e = i[0];
  for (size_t k = 1; k < d.size(); ++k) e = "(" + e + " * " + d[k] + " + " + i[k] + ")";
  return bindLeaf(ST::I64, e, em)->ex;
}

ValP Codegen::fromIndex(int rank, const ValP& sh, const std::string& lin, Emit& em) {
  std::vector<std::string> d;
  shapeDims(sh, d);
  if ((int)d.size() != rank) throw Error("fromIndex: rank mismatch");
  if (rank == 0) return vUnit();
  std::vector<std::string> ix(rank);
  std::string cur = lin;
  for (int k = rank - 1; k >= 1; --k) {
    // one division per dimension: the remainder follows from the quotient
    const std::string q = bindLeaf(ST::I64, "acc_quot(" + cur + ", " + d[k] + ")", em)->ex;
    ix[k] = bindLeaf(ST::I64, cur + " - " + q + " * " + d[k], em)->ex;
    cur = q;
  }
  ix[0] = cur;  // the outermost component needs no remainder (Shape.hs:110-120)
  ValP v = vUnit();
  for (int k = 0; k < rank; ++k) v = vPair(v, vLeaf(ST::I64, ix[k]));
  return v;
}

ValP Codegen::readArray(const ArraySlot& s, const std::string& lin, Emit& em) {
  int leaf = 0;
  struct R {
    static ValP go(Codegen& cg, const TypeP& t, const ArraySlot& s, const std::string& lin, int& leaf, Emit& em) {
      if (t->k == Type::Unit) return vUnit();
      if (t->k == Type::Scalar)
      {
        const std::string at = "env." + s.name + "_" + std::to_string(leaf++) + "[" + lin + "]";
        // read at the skeleton's own linear index: each element once, in order
        return cg.bindLeaf(t->st, lin == "i" ? "acc_ld<kStream>(&" + at + ")" : at, em);
      }
      ValP a = go(cg, t->a, s, lin, leaf, em);
      return vPair(a, go(cg, t->b, s, lin, leaf, em));
    }
  };
  return R::go(*this, s.r.elt, s, lin, leaf, em);
}

ValP Codegen::operandLinear(const Operand& o, const std::string& lin, Emit& em) {
  if (o.delayed) return applyFun(o.linearD, {vLeaf(ST::I64, lin)}, {}, em);
  return readArray(slotByName(o.slot), lin, em);
}

ValP Codegen::operandIndex(const Operand& o, const ValP& ix, Emit& em) {
  if (o.delayed) return applyFun(o.indexD, {ix}, {}, em);
  const ArraySlot& s = slotByName(o.slot);
  return readArray(s, toIndex(shapeOf(s), ix, em), em);
}

ValP Codegen::operandShape(const Operand& o, Emit& em) {
  if (o.delayed) return exp(o.extent, {}, em);
  return shapeOf(slotByName(o.slot));
}

// ------------------------------------------------------------------------------------
// primitives (semantics: Interpreter.hs:1154-1416)

static int primTypeParams(const std::string& n) {
  if (n == "land" || n == "lor" || n == "lnot") return 0;
  if (n == "truncate" || n == "round" || n == "floor" || n == "ceiling" || n == "fromintegral" || n == "tofloating")
    return 2;
  return 1;
}

ValP Codegen::prim(const std::string& name, const std::vector<ST>& tys, const ValP& arg, Emit& em) {
  auto T = [](ST t) { return std::string(stName(t)); };
  auto bin = [&](std::string& a, std::string& b) {
    if (arg->k != Val::Pair) throw Error("primitive '" + name + "' expects a pair argument");
    a = leaf1(arg->a, name.c_str())->ex;
    b = leaf1(arg->b, name.c_str())->ex;
  };
  auto un = [&]() { return leaf1(arg, name.c_str())->ex; };
  auto fcall1 = [&](ST t, const char* fn, const std::string& a) {
    if (t == ST::F64) return std::string(fn) + "(" + a + ")";
    if (t == ST::F32) return std::string(fn) + "f(" + a + ")";
    return "(f16)" + std::string(fn) + "f((f32)" + a + ")";
  };
  auto fcall2 = [&](ST t, const char* fn, const std::string& a, const std::string& b) {
    if (t == ST::F64) return std::string(fn) + "(" + a + ", " + b + ")";
    if (t == ST::F32) return std::string(fn) + "f(" + a + ", " + b + ")";
    return "(f16)" + std::string(fn) + "f((f32)" + a + ", (f32)" + b + ")";
  };
  auto arith = [&](ST t, const char* op, const std::string& a, const std::string& b) {
    if (stIsInt(t)) return "(" + T(t) + ")((" + stWide(t) + ")" + a + " " + op + " (" + stWide(t) + ")" + b + ")";
    if (t == ST::F16) return "(f16)((f32)" + a + " " + op + " (f32)" + b + ")";
    return a + " " + op + " " + b;
  };
  auto needInt = [&](ST t) {
    if (!stIsInt(t)) throw Error("primitive '" + name + "' needs an integral type");
  };
  auto needFloat = [&](ST t) {
    if (!stIsFloat(t)) throw Error("primitive '" + name + "' needs a floating type");
  };
  for (ST ty : tys)
    if (stIsVec(ty)) throw Error("primitive '" + name + "' applied at a SIMD vector type");
  const ST t = tys.empty() ? ST::U8 : tys[0];
  const std::string bits = std::to_string(stBits(t));
  const std::string U = T(stUnsigned(t));
  std::string a, b;

  if (name == "add" || name == "sub" || name == "mul") {
    bin(a, b);
    return bindLeaf(t, arith(t, name == "add" ? "+" : name == "sub" ? "-" : "*", a, b), em);
  }
  if (name == "neg") {
    a = un();
    if (stIsInt(t)) return bindLeaf(t, "(" + T(t) + ")((" + stWide(t) + ")0 - (" + stWide(t) + ")" + a + ")", em);
    return bindLeaf(t, "-" + a, em);
  }
  if (name == "abs") {
    a = un();
    if (stIsInt(t)) {
      if (!stIsSigned(t)) return arg;
      return bindLeaf(t, "(" + a + " < 0) ? (" + T(t) + ")((" + stWide(t) + ")0 - (" + stWide(t) + ")" + a + ") : " + a, em);
    }
    return bindLeaf(t, fcall1(t, "fabs", a), em);
  }
  if (name == "sig") {
    a = un();
    if (stIsInt(t)) return bindLeaf(t, "(" + T(t) + ")((" + a + " > 0) - (" + a + " < 0))", em);
    // GHC.Float: signum x | x > 0 = 1 | x < 0 = -1 | otherwise = x
    return bindLeaf(t, "(" + a + " > 0) ? (" + T(t) + ")1 : ((" + a + " < 0) ? (" + T(t) + ")-1 : " + a + ")", em);
  }
  if (name == "quot" || name == "rem" || name == "idiv" || name == "mod" || name == "quotrem" || name == "divmod") {
    needInt(t);
    bin(a, b);
    ValP q = bindLeaf(t, "(" + T(t) + ")(" + a + " / " + b + ")", em);
    ValP r = bindLeaf(t, "(" + T(t) + ")(" + a + " % " + b + ")", em);
    if (name == "quot") return q;
    if (name == "rem") return r;
    if (name == "quotrem") return vPair(q, r);
    if (!stIsSigned(t)) return name == "idiv" ? q : name == "mod" ? r : vPair(q, r);
    // floor division (Haskell div / mod): adjust when the remainder's sign differs from the divisor's
    ValP adj = bindLeaf(ST::U8, "(u8)((" + r->ex + " != 0) & ((" + r->ex + " < 0) != (" + b + " < 0)))", em);
    ValP d = bindLeaf(t, adj->ex + " ? (" + T(t) + ")(" + q->ex + " - 1) : " + q->ex, em);
    ValP m = bindLeaf(t, adj->ex + " ? (" + T(t) + ")(" + r->ex + " + " + b + ") : " + r->ex, em);
    if (name == "idiv") return d;
    if (name == "mod") return m;
    return vPair(d, m);
  }
  if (name == "band" || name == "bor" || name == "bxor") {
    needInt(t);
    bin(a, b);
    const char* op = name == "band" ? "&" : name == "bor" ? "|" : "^";
    return bindLeaf(t, "(" + T(t) + ")(" + a + " " + op + " " + b + ")", em);
  }
  if (name == "bnot") {
    needInt(t);
    return bindLeaf(t, "(" + T(t) + ")(~" + un() + ")", em);
  }
  if (name == "shl") {
    needInt(t);
    bin(a, b);
    return bindLeaf(t, "((u64)" + b + " >= " + bits + ") ? (" + T(t) + ")0 : (" + T(t) + ")((" + stWide(t) + ")" + a + " << " + b + ")", em);
  }
  if (name == "shr") {
    needInt(t);
    bin(a, b);
    std::string over = stIsSigned(t) ? "(" + T(t) + ")(" + a + " < 0 ? -1 : 0)" : "(" + T(t) + ")0";
    return bindLeaf(t, "((u64)" + b + " >= " + bits + ") ? " + over + " : (" + T(t) + ")(" + a + " >> " + b + ")", em);
  }
  if (name == "rotl" || name == "rotr") {
    needInt(t);
    bin(a, b);
    // rotate by (n mod bits), Data.Bits semantics; rotr n = rotl (-n)
    std::string n = name == "rotl" ? b : "(-" + b + ")";
    ValP k = bindLeaf(ST::I32, "(i32)(((" + n + " % " + bits + ") + " + bits + ") % " + bits + ")", em);
    ValP u = bindLeaf(stUnsigned(t), "(" + U + ")" + a, em);
    std::string W = stWide(t);
    return bindLeaf(t, "(" + k->ex + " == 0) ? " + a + " : (" + T(t) + ")(((" + W + ")" + u->ex + " << " + k->ex + ") | ((" + W + ")" + u->ex + " >> (" + bits + " - " + k->ex + ")))", em);
  }
  if (name == "popcount") {
    needInt(t);
    return bindLeaf(ST::I64, "(i64)__builtin_popcountll((u64)(" + U + ")" + un() + ")", em);
  }
  if (name == "clz") {
    needInt(t);
    a = un();
    return bindLeaf(ST::I64, "((" + U + ")" + a + " == 0) ? (i64)" + bits + " : (i64)(__builtin_clzll((u64)(" + U + ")" + a + ") - (64 - " + bits + "))", em);
  }
  if (name == "ctz") {
    needInt(t);
    a = un();
    return bindLeaf(ST::I64, "((" + U + ")" + a + " == 0) ? (i64)" + bits + " : (i64)__builtin_ctzll((u64)(" + U + ")" + a + ")", em);
  }
  if (name == "fdiv") {
    needFloat(t);
    bin(a, b);
    return bindLeaf(t, arith(t, "/", a, b), em);
  }
  if (name == "recip") {
    needFloat(t);
    return bindLeaf(t, arith(t, "/", "(" + T(t) + ")1", un()), em);
  }
  static const char* unaryMath[] = {"sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh", "tanh",
                                    "asinh", "acosh", "atanh", "exp", "sqrt", "log"};
  for (const char* m : unaryMath)
    if (name == m) {
      needFloat(t);
      return bindLeaf(t, fcall1(t, m, un()), em);
    }
  if (name == "fpow") {
    needFloat(t);
    bin(a, b);
    return bindLeaf(t, fcall2(t, "pow", a, b), em);
  }
  if (name == "atan2") {
    needFloat(t);
    bin(a, b);
    return bindLeaf(t, fcall2(t, "atan2", a, b), em);
  }
  if (name == "logbase") {  // logBase x y = log y / log x
    needFloat(t);
    bin(a, b);
    ValP ly = bindLeaf(t, fcall1(t, "log", b), em), lx = bindLeaf(t, fcall1(t, "log", a), em);
    return bindLeaf(t, arith(t, "/", ly->ex, lx->ex), em);
  }
  if (name == "truncate" || name == "round" || name == "floor" || name == "ceiling") {
    if (tys.size() != 2) throw Error("primitive '" + name + "' needs two type parameters");
    needFloat(tys[0]);
    if (!stIsInt(tys[1])) throw Error("primitive '" + name + "' converts to an integral type");
    const char* fn = name == "truncate" ? "trunc" : name == "round" ? "rint" : name == "floor" ? "floor" : "ceil";
    std::string x = tys[0] == ST::F64 ? std::string(fn) + "(" + un() + ")" : std::string(fn) + "f((f32)" + un() + ")";
    // go through i64 so that narrow targets wrap like fromIntegral would
    return bindLeaf(tys[1], "(" + T(tys[1]) + ")(i64)" + x, em);
  }
  if (name == "isnan" || name == "isinf") {
    needFloat(t);
    std::string x = t == ST::F16 ? "(f32)" + un() : un();
    return bindLeaf(ST::U8, std::string("(u8)(") + (name == "isnan" ? "__builtin_isnan(" : "__builtin_isinf(") + x + ") != 0)", em);
  }
  static const struct { const char* n; const char* op; } cmps[] = {{"lt", "<"}, {"gt", ">"}, {"lte", "<="},
                                                                   {"gte", ">="}, {"eq", "=="}, {"neq", "!="}};
  for (auto& c : cmps)
    if (name == c.n) {
      bin(a, b);
      return bindLeaf(ST::U8, "(u8)(" + a + " " + c.op + " " + b + ")", em);
    }
  if (name == "max") {  // Ord default: max x y = if x <= y then y else x
    bin(a, b);
    return bindLeaf(t, "(" + a + " <= " + b + ") ? " + b + " : " + a, em);
  }
  if (name == "min") {  // min x y = if x <= y then x else y
    bin(a, b);
    return bindLeaf(t, "(" + a + " <= " + b + ") ? " + a + " : " + b, em);
  }
  if (name == "land" || name == "lor") {
    bin(a, b);
    return bindLeaf(ST::U8, "(u8)((" + a + " != 0) " + (name == "land" ? "&" : "|") + " (" + b + " != 0))", em);
  }
  if (name == "lnot") return bindLeaf(ST::U8, "(u8)(" + un() + " == 0)", em);
  if (name == "fromintegral" || name == "tofloating") {
    if (tys.size() != 2) throw Error("primitive '" + name + "' needs two type parameters");
    a = un();
    ST to = tys[1];
    if (to == ST::F16 && stIsInt(tys[0])) return bindLeaf(to, "(f16)(f32)" + a, em);  // Half goes through Float
    ValP r = bindLeaf(to, "(" + T(to) + ")" + a, em);
    if (stIsInt(tys[0]) && !stIsVec(tys[0]) && stSize(tys[0]) <= 4 && stIsInt(to) && !stIsVec(to) && stSize(to) == 8) {
      r->narrowEx = a;
      r->narrowSt = tys[0];
    }
    return r;
  }
  throw Error("unknown primitive '" + name + "'");
}

// ------------------------------------------------------------------------------------
// expressions

static void sliceRestrict(const Sx& spec, size_t k, const ValP& slix, const ValP& sh, ValP& out) {
  // IndexSlice (Interpreter.hs:944-953); spec lists all/fixed from the innermost dimension outwards
  if (k == spec.size()) { out = vUnit(); return; }
  if (slix->k != Val::Pair || sh->k != Val::Pair) throw Error("indexslice: slice index does not match the specification");
  ValP rest;
  sliceRestrict(spec, k + 1, slix->a, sh->a, rest);
  out = spec.at(k).isAtom("all") ? vPair(rest, sh->b) : rest;
}

static void sliceExtend(const Sx& spec, size_t k, const ValP& slix, const ValP& sl, ValP& out) {
  // IndexFull (Interpreter.hs:955-965)
  if (k == spec.size()) { out = vUnit(); return; }
  if (slix->k != Val::Pair) throw Error("indexfull: slice index does not match the specification");
  ValP rest;
  if (spec.at(k).isAtom("all")) {
    if (sl->k != Val::Pair) throw Error("indexfull: slice shape does not match the specification");
    sliceExtend(spec, k + 1, slix->a, sl->a, rest);
    out = vPair(rest, sl->b);
  } else {
    sliceExtend(spec, k + 1, slix->a, sl, rest);
    out = vPair(rest, slix->b);
  }
}

ValP Codegen::applyFun(const Sx& f, const std::vector<ValP>& args, const Env& env, Emit& em) {
  Env e2 = env;
  const Sx* cur = &f;
  for (const ValP& a : args) {
    if (!cur->is("lam")) throw Error("function applied to too many arguments: " + f.str().substr(0, 120));
    pushLhs(cur->at(1), a, e2);
    cur = &cur->at(2);
  }
  if (cur->is("lam")) throw Error("function applied to too few arguments");
  return exp(*cur, e2, em);
}

ValP Codegen::exp(const Sx& e, const Env& env, Emit& em) {
  if (e.isAtom("nil")) return vUnit();
  if (e.atom) throw Error("unexpected atom '" + e.s + "' in scalar expression");
  const std::string& h = e.head();
  if (h == "var") {
    long long ix = e.at(1).asInt();
    if (ix < 0 || ix >= (long long)env.size()) throw Error("scalar variable index out of range");
    return env[env.size() - 1 - ix];
  }
  if (h == "let") {
    ValP v = exp(e.at(2), env, em);
    Env e2 = env;
    pushLhs(e.at(1), v, e2);
    return exp(e.at(3), e2, em);
  }
  if (h == "pair") {
    ValP a = exp(e.at(1), env, em);
    return vPair(a, exp(e.at(2), env, em));
  }
  if (h == "const") {
    ST t = parseST(e.at(1));
    if (stIsVec(t)) {  // (const v<n><t> (lit ..))
      const Sx& ls = e.at(2);
      if (ls.atom || (int)ls.size() != stWidth(t)) throw Error("vector constant needs one literal per component");
      std::string x = std::string(stName(t)) + "{{";
      for (int k = 0; k < stWidth(t); ++k) x += (k ? ", " : "") + literalText(stBase(t), ls.at(k).s);
      return vLeaf(t, x + "}}");
    }
    return vLeaf(t, literalText(t, e.at(2).s));
  }
  if (h == "undef") {
    ST t = parseST(e.at(1));
    if (stIsVec(t)) return vLeaf(t, std::string(stName(t)) + "{}");
    return vLeaf(t, literalText(t, "0"));
  }
  if (h == "vecpack" || h == "vecunpack") {  // (vecpack N T e) / (vecunpack N T e): Interpreter.hs:942-943
    const int w = (int)e.at(1).asInt();
    const ST base = parseST(e.at(2));
    if (!stVecWidthOk(w) || stIsVec(base)) throw Error("malformed vector type in " + h);
    const ST vt = stVec(base, w);
    ValP v = exp(e.at(3), env, em);
    if (h == "vecpack") {
      std::vector<ValP> parts;
      valLeaves(v, parts);
      if ((int)parts.size() != w) throw Error("vecpack: expected a tuple of " + std::to_string(w) + " components");
      std::string x = std::string(stName(vt)) + "{{";
      for (int k = 0; k < w; ++k) {
        if (parts[k]->st != base) throw Error("vecpack: component type does not match the vector type");
        x += (k ? ", " : "") + parts[k]->ex;
      }
      return bindLeaf(vt, x + "}}", em);
    }
    ValP l = leaf1(v, "vecunpack");
    if (l->st != vt) throw Error("vecunpack: operand is not of the stated vector type");
    ValP l2 = bindLeaf(vt, l->ex, em);  // a name, so that components can be selected
    ValP out = vUnit();
    for (int k = 0; k < w; ++k) out = vPair(out, bindLeaf(base, l2->ex + ".e[" + std::to_string(k) + "]", em));
    return out;
  }
  if (h == "minbound" || h == "maxbound") {
    ST t = parseST(e.at(1));
    if (!stIsInt(t)) throw Error(h + " needs an integral type");
    int bits = stBits(t);
    unsigned long long v;
    if (h == "minbound") v = stIsSigned(t) ? (1ULL << (bits - 1)) : 0ULL;
    else v = stIsSigned(t) ? ((1ULL << (bits - 1)) - 1) : (bits == 64 ? ~0ULL : ((1ULL << bits) - 1));
    char buf[64];
    snprintf(buf, sizeof buf, "((%s)0x%llxULL)", stName(t), v);
    return vLeaf(t, buf);
  }
  if (h == "pi") {
    ST t = parseST(e.at(1));
    return vLeaf(t, literalText(t, "0x1.921fb54442d18p+1"));
  }
  if (h == "prim") {
    std::string name = e.at(1).s;
    int nt = primTypeParams(name);
    std::vector<ST> tys;
    for (int k = 0; k < nt; ++k) tys.push_back(parseST(e.at(2 + k)));
    ValP arg = exp(e.at(2 + nt), env, em);
    return prim(name, tys, arg, em);
  }
  if (h == "toindex") {
    ValP sh = exp(e.at(2), env, em), ix = exp(e.at(3), env, em);
    return vLeaf(ST::I64, toIndex(sh, ix, em));
  }
  if (h == "fromindex") {
    ValP sh = exp(e.at(2), env, em), i = exp(e.at(3), env, em);
    return fromIndex((int)e.at(1).asInt(), sh, leaf1(i, "fromindex")->ex, em);
  }
  if (h == "indexslice" || h == "indexfull") {
    ValP slix = exp(e.at(2), env, em), sh = exp(e.at(3), env, em), out;
    if (h == "indexslice") sliceRestrict(e.at(1), 0, slix, sh, out);
    else sliceExtend(e.at(1), 0, slix, sh, out);
    return out;
  }
  if (h == "cond") {
    ValP c = exp(e.at(1), env, em);
    Emit et, ee;
    et.ind = ee.ind = em.ind + 2;
    ValP tv = exp(e.at(2), env, et), ev = exp(e.at(3), env, ee);
    if (!typeEq(valType(tv), valType(ev))) throw Error("branches of a conditional have different types");
    const std::string cx = "(" + leaf1(c, "cond")->ex + " != 0)";
    if (et.code.empty() && ee.code.empty()) {
      auto tl = leavesOf(tv), el = leavesOf(ev);
      std::vector<ValP> rl;
      for (size_t i = 0; i < tl.size(); ++i)
        rl.push_back(tl[i]->ex == el[i]->ex ? tl[i] : bindLeaf(tl[i]->st, cx + " ? " + tl[i]->ex + " : " + el[i]->ex, em));
      size_t pos = 0;
      struct B {
        static ValP go(const ValP& shape, const std::vector<ValP>& rl, size_t& pos) {
          if (shape->k == Val::Unit) return shape;
          if (shape->k == Val::Leaf) return rl[pos++];
          ValP a = go(shape->a, rl, pos);
          return vPair(a, go(shape->b, rl, pos));
        }
      };
      return B::go(tv, rl, pos);
    }
    // only the chosen branch may run (a branch can guard an out-of-bounds index)
    ValP res = declareVars(valType(tv), em);
    em.line("if " + cx + " {");
    em.code += et.code;
    em.ind += 2;
    assign(res, tv, em);
    em.ind -= 2;
    em.line("} else {");
    em.code += ee.code;
    em.ind += 2;
    assign(res, ev, em);
    em.ind -= 2;
    em.line("}");
    return res;
  }
  if (h == "case") {
    ValP tag = exp(e.at(1), env, em);
    const Sx& alts = e.at(2);
    std::vector<Emit> ems(alts.size() + 1);
    std::vector<ValP> vals;
    for (size_t k = 0; k < alts.size(); ++k) {
      ems[k].ind = em.ind + 4;
      vals.push_back(exp(alts.at(k).at(1), env, ems[k]));
    }
    bool hasDef = !e.at(3).isAtom("none");
    if (hasDef) {
      ems.back().ind = em.ind + 4;
      vals.push_back(exp(e.at(3), env, ems.back()));
    }
    if (vals.empty()) throw Error("case without alternatives");
    ValP res = declareVars(valType(vals[0]), em);
    em.line("switch ((int)" + leaf1(tag, "case")->ex + ") {");
    for (size_t k = 0; k < vals.size(); ++k) {
      bool def = k == alts.size();
      em.line(def ? "  default: {" : "  case " + std::to_string(alts.at(k).at(0).asInt()) + ": {");
      em.code += ems[k].code;
      em.ind += 4;
      assign(res, vals[k], em);
      em.ind -= 4;
      em.line("  } break;");
    }
    em.line("}");
    return res;
  }
  if (h == "while") {
    ValP seed = exp(e.at(3), env, em);
    ValP st = copyToVars(seed, em);
    em.line("for (;;) {");
    em.ind += 2;
    ValP c = applyFun(e.at(1), {st}, env, em);
    em.line("if (" + leaf1(c, "while")->ex + " == 0) break;");
    ValP nv = applyFun(e.at(2), {st}, env, em);
    ValP tmp = copyToVars(nv, em);  // the new state may mention the old one
    assign(st, tmp, em);
    em.ind -= 2;
    em.line("}");
    return st;
  }
  if (h == "index") {
    const ArraySlot& s = slotForVar((int)e.at(1).asInt());
    ValP ix = exp(e.at(2), env, em);
    return readArray(s, toIndex(shapeOf(s), ix, em), em);
  }
  if (h == "linearindex") {
    const ArraySlot& s = slotForVar((int)e.at(1).asInt());
    ValP i = exp(e.at(2), env, em);
    return readArray(s, leaf1(i, "linearindex")->ex, em);
  }
  if (h == "shape") return shapeOf(slotForVar((int)e.at(1).asInt()));
  if (h == "shapesize") {
    ValP sh = exp(e.at(2), env, em);
    std::vector<std::string> d;
    shapeDims(sh, d);
    if (d.empty()) return vLeaf(ST::I64, "((i64)1)");
    std::string neg, prod;
    for (size_t k = 0; k < d.size(); ++k) {
      neg += (k ? " || " : "") + ("(" + d[k] + " <= 0)");
      prod += (k ? " * " : "") + d[k];
    }
    return bindLeaf(ST::I64, "(" + neg + ") ? (i64)0 : (i64)(" + prod + ")", em);
  }
  if (h == "coerce") {
    ST t1 = parseST(e.at(1)), t2 = parseST(e.at(2));
    if (stSize(t1) != stSize(t2)) throw Error("coerce between types of different width");
    ValP v = exp(e.at(3), env, em);
    return bindLeaf(t2, std::string("__builtin_bit_cast(") + stName(t2) + ", (" + stName(t1) + ")" + leaf1(v, "coerce")->ex + ")", em);
  }
  if (h == "foreign") {
    ValP v = exp(e.at(2), env, em);
    return applyFun(e.at(1), {v}, {}, em);  // the pure fallback, in an empty environment
  }
  throw Error("unknown scalar expression '" + h + "'");
}

TypeP Codegen::typeOfExp(const Sx& e) {
  Emit scratch;
  int save = next_;
  auto usedSave = used_;
  TypeP t = valType(exp(e, {}, scratch));
  next_ = save;
  used_ = usedSave;
  return t;
}

// ------------------------------------------------------------------------------------
// translation-unit assembly

static std::string leafDecls(const std::vector<ST>& leaves, const char* prefix, bool pointer, bool constPtr) {
  std::string s;
  for (size_t k = 0; k < leaves.size(); ++k) {
    s += "  ";
    if (pointer && constPtr) s += "const ";
    s += stName(leaves[k]);
    if (pointer) s += "*";
    s += " " + std::string(prefix) + std::to_string(k) + ";\n";
  }
  return s;
}

std::string Codegen::eltStruct(const TypeP& t, const std::string& name) {
  return "struct " + name + " {\n" + leafDecls(typeLeaves(t), "c", false, false) + "};\n";
}

std::string Codegen::outStruct(const std::vector<ST>& leaves) {
  return "struct Out {\n  i64 _pad;\n" + leafDecls(leaves, "o", true, false) + "};\n";
}

std::string Codegen::envStruct(std::vector<ArraySlot>& order) {
  std::string s = "struct Env {\n  i64 _pad;\n";
  order.clear();
  for (auto& kv : used_) order.push_back(kv.second);
  for (auto& a : order) {
    auto lv = typeLeaves(a.r.elt);
    for (size_t k = 0; k < lv.size(); ++k)
      s += std::string("  const ") + stName(lv[k]) + "* __restrict__ " + a.name + "_" + std::to_string(k) + ";\n";
    for (int d = 0; d < a.r.rank; ++d) s += "  i64 " + a.name + "_d" + std::to_string(d) + ";\n";
  }
  return s + "};\n";
}

ValP Codegen::eltVal(const TypeP& t, const std::string& var) {
  int leaf = 0;
  struct R {
    static ValP go(const TypeP& t, const std::string& var, int& leaf) {
      if (t->k == Type::Unit) return vUnit();
      if (t->k == Type::Scalar) return vLeaf(t->st, var + ".c" + std::to_string(leaf++));
      ValP a = go(t->a, var, leaf);
      return vPair(a, go(t->b, var, leaf));
    }
  };
  return R::go(t, var, leaf);
}

std::string Codegen::returnElt(const ValP& v, Emit& em) {
  auto lv = leavesOf(v);
  em.line("Elt r_;");
  for (size_t k = 0; k < lv.size(); ++k) em.line("r_.c" + std::to_string(k) + " = " + lv[k]->ex + ";");
  em.line("return r_;");
  return em.code;
}

bool Codegen::isCommutative(const Sx& f, std::string* op, ST* st) {
  // \x y -> prim OP T (x, y)   or   (y, x), for OP in a fixed set of commutative primitives
  if (!f.is("lam") || !f.at(1).is("single")) return false;
  const Sx& g = f.at(2);
  if (!g.is("lam") || !g.at(1).is("single")) return false;
  const Sx& b = g.at(2);
  if (!b.is("prim") || b.size() != 4) return false;
  static const char* ops[] = {"add", "mul", "min", "max", "band", "bor", "bxor"};
  bool ok = false;
  for (const char* o : ops) ok = ok || b.at(1).s == o;
  if (!ok || !isST(b.at(2))) return false;
  const Sx& arg = b.at(3);
  if (!arg.is("pair") || !arg.at(1).is("var") || !arg.at(2).is("var")) return false;
  long long i = arg.at(1).at(1).asInt(), j = arg.at(2).at(1).asInt();
  if (!((i == 0 && j == 1) || (i == 1 && j == 0))) return false;
  if (op) *op = b.at(1).s;
  if (st) *st = parseST(b.at(2));
  return true;
}

// Is f a component-wise combination of tuples, \(x0, .., xn) (y0, .., yn) -> (x0 (+)0 y0, ..),
// with every (+)k one of the commutative primitives that exist as hardware atomics?  Then the
// components can be combined independently of each other, one atomic each.  Accepts the form
// the front end produces: both arguments bound by fully destructuring left-hand sides, the body
// a tuple of primitive applications to the matching pair of variables (in either order).
static bool componentwiseAtomic(const Sx& f, const std::vector<ST>& leaves, std::vector<std::string>& ops,
                                bool anyCommutative = false) {
  struct Lhs {
    static bool singles(const Sx& l, int& n) {  // counts variables; false on wildcards
      if (l.is("single")) { ++n; return true; }
      if (l.is("pair") && l.size() == 3) return singles(l.at(1), n) && singles(l.at(2), n);
      if (l.is("wild")) return l.at(1).isAtom("unit");
      return false;
    }
    static bool flat(const Sx& e, std::vector<const Sx*>& out) {  // leaves of a tuple expression
      if (e.isAtom("nil")) return true;
      if (e.is("pair") && e.size() == 3) return flat(e.at(1), out) && flat(e.at(2), out);
      out.push_back(&e);
      return true;
    }
  };
  const int n = (int)leaves.size();
  if (n < 2 || !f.is("lam")) return false;
  const Sx& g = f.at(2);
  if (!g.is("lam")) return false;
  int nx = 0, ny = 0;
  if (!Lhs::singles(f.at(1), nx) || !Lhs::singles(g.at(1), ny) || nx != n || ny != n) return false;
  std::vector<const Sx*> parts;
  if (!Lhs::flat(g.at(2), parts) || (int)parts.size() != n) return false;
  ops.clear();
  for (int k = 0; k < n; ++k) {
    const Sx& b = *parts[k];
    if (!b.is("prim") || b.size() != 4 || !isST(b.at(2)) || parseST(b.at(2)) != leaves[k]) return false;
    const ST t = leaves[k];
    const std::string& o = b.at(1).s;
    if (anyCommutative) {  // for reductions: any commutative primitive at any scalar type
      if (stIsVec(t) || !(o == "add" || o == "mul" || o == "min" || o == "max" || o == "band" || o == "bor" || o == "bxor"))
        return false;
    } else {
      if (stIsVec(t) || (stSize(t) != 4 && stSize(t) != 8)) return false;
      const bool okOp = o == "add" || (stIsInt(t) && (o == "min" || o == "max" || o == "band" || o == "bor" || o == "bxor"));
      if (!okOp) return false;
    }
    const Sx& arg = b.at(3);
    if (!arg.is("pair") || !arg.at(1).is("var") || !arg.at(2).is("var")) return false;
    // variable levels: x_k = k, y_k = n + k; de Bruijn index = 2n - 1 - level
    const long long ix = 2 * n - 1 - k, iy = n - 1 - k;
    const long long a = arg.at(1).at(1).asInt(), c = arg.at(2).at(1).asInt();
    if (!((a == ix && c == iy) || (a == iy && c == ix))) return false;
    ops.push_back(o);
  }
  return true;
}

static int vecFor(const std::vector<ST>& leaves, const std::vector<ArraySlot>& arrays) {
  int maxLeaf = 1, eltBytes = 0;
  for (ST s : leaves) {
    maxLeaf = std::max(maxLeaf, stSize(s));
    eltBytes += stSize(s);
  }
  for (auto& a : arrays)
    for (ST s : typeLeaves(a.r.elt)) maxLeaf = std::max(maxLeaf, stSize(s));
  int v = 16 / maxLeaf;
  while (v > 1 && v * eltBytes > 64) v >>= 1;
  return std::max(1, std::min(v, 8));
}

KernelSource Codegen::finish(const std::string& specBody, const TypeP& elt, const std::vector<ST>& outLeaves,
                             const std::string& skeleton, int vec, bool ownStore) {
  KernelSource ks;
  std::string envS = envStruct(ks.arrays);
  ks.outLeaves = outLeaves;
  ks.vec = vec > 0 ? vec : vecFor(outLeaves, ks.arrays);
  // ACCHIP_KERNEL_DEFINES="NAME=VALUE ...": macros put in front of every generated translation unit
  // (the skeletons' tuning constants are #ifndef-guarded); part of the source, hence of the cache key
  std::string s;
  if (const char* defs = std::getenv("ACCHIP_KERNEL_DEFINES")) {
    std::string tok;
    for (const char* c = defs;; ++c) {
      if (*c && *c != ' ' && *c != ',') {
        tok += *c;
        continue;
      }
      if (!tok.empty()) {
        const size_t eq = tok.find('=');
        s += "#define " + (eq == std::string::npos ? tok + " 1" : tok.substr(0, eq) + " " + tok.substr(eq + 1)) + "\n";
        tok.clear();
      }
      if (!*c) break;
    }
  }
  s += deviceHeader("prelude.hpp");
  s += "\n" + envS + eltStruct(elt, "Elt") + outStruct(outLeaves);
  s += "struct Spec {\n  typedef ::Env Env;\n  typedef ::Elt Elt;\n  typedef ::Out Out;\n";
  s += "  static constexpr int V = " + std::to_string(ks.vec) + ";\n";
  s += specBody;
  // Out <-> Elt when both have the same leaves
  auto el = typeLeaves(elt);
  if (el == outLeaves && !ownStore) {
    s += "  ACC_DEV Elt load(const Out& o, i64 i) {\n    Elt r_;\n";
    for (size_t k = 0; k < el.size(); ++k) s += "    r_.c" + std::to_string(k) + " = o.o" + std::to_string(k) + "[i];\n";
    s += "    return r_;\n  }\n";
    s += "  template <bool kStream = false>\n  ACC_DEV void store(const Out& o, i64 i, const Elt& v) {\n";
    for (size_t k = 0; k < el.size(); ++k)
      s += "    acc_st<kStream>(&o.o" + std::to_string(k) + "[i], v.c" + std::to_string(k) + ");\n";
    s += "  }\n";
    // V consecutive results at once: one wide request per leaf whatever the compiler can
    // prove about the alignment of position i
    s += "  ACC_DEV void store_run(const Out& o, i64 i, const Elt* v) {\n";
    for (size_t k = 0; k < el.size(); ++k) {
      const std::string K = std::to_string(k), T = stName(el[k]);
      s += "    {\n      acc_run<" + T + ", V> r_;\n#pragma unroll\n      for (int k_ = 0; k_ < V; ++k_) r_.e[k_] = v[k_].c" + K +
           ";\n      *(acc_run<" + T + ", V>*)&o.o" + K + "[i] = r_;\n    }\n";
    }
    s += "  }\n";
  }
  s += "};\n\n";
  for (size_t b = 0; b <= skeleton.size();) {  // one or more headers joined by '+'
    size_t e = skeleton.find('+', b);
    if (e == std::string::npos) e = skeleton.size();
    s += deviceHeader(skeleton.substr(b, e - b)) + "\n";
    b = e + 1;
  }
  ks.source = std::move(s);
  return ks;
}

// ------------------------------------------------------------------------------------
// skeleton instantiations

static std::string fnHead(const char* ret, const char* name, const char* params) {
  return std::string("  ACC_DEV ") + ret + " " + name + "(" + params + ") {\n";
}

// a function with a streaming variant: kStream selects non-temporal reads at index i
static std::string streamHead(const char* ret, const char* name, const char* params) {
  return "  template <bool kStream = false>\n" + fnHead(ret, name, params);
}

static void structLayout(const std::vector<ST>& leaves, int& size, int& align);

static int structWords(const std::vector<ST>& leaves);

KernelSource Codegen::fold(const Sx& f, const Sx* seed, const Operand& src) {
  const TypeP elt = src.r.elt;
  std::string body;
  bool comm = isCommutative(f);
  {
    // component-wise combinations of tuples of commutative primitives commute as a whole
    std::vector<std::string> ops;
    if (!comm && componentwiseAtomic(f, typeLeaves(elt), ops, true)) comm = true;
  }
  body += std::string("  static constexpr bool kCommutative = ") + (comm ? "true" : "false") + ";\n";
  body += std::string("  static constexpr bool kSeeded = ") + (seed ? "true" : "false") + ";\n";
  {
    Emit em;
    em.ind = 4;
    ValP r = applyFun(f, {eltVal(elt, "x"), eltVal(elt, "y")}, {}, em);
    if (!typeEq(valType(r), elt)) throw Error("fold: combination function does not return the element type");
    body += fnHead("Elt", "combine", "const Env& env, const Elt& x, const Elt& y") + returnElt(r, em) + "  }\n";
  }
  {
    Emit em;
    em.ind = 4;
    if (seed) {
      ValP z = exp(*seed, {}, em);
      if (!typeEq(valType(z), elt)) throw Error("fold: seed does not have the element type");
      returnElt(z, em);
    } else {
      em.line("Elt r_{};");
      em.line("return r_;");
    }
    body += fnHead("Elt", "seed", "const Env& env") + em.code + "  }\n";
  }
  {
    Emit em;
    em.ind = 4;
    ValP v = operandLinear(src, "i", em);
    if (!typeEq(valType(v), elt)) throw Error("fold: fused producer does not return the element type");
    body += streamHead("Elt", "in_linear", "const Env& env, i64 i") + returnElt(v, em) + "  }\n";
  }
  // geometry of the kernel for many short rows (acc_fold_rows): 256 threads, about 64 bytes
  // of (value, flag) pairs per lane
  auto leaves = typeLeaves(elt);
  int eltBytes = 4;
  for (ST st : leaves) eltBytes += stSize(st);
  std::vector<ArraySlot> tmpOrder;
  for (auto& kv : used_) tmpOrder.push_back(kv.second);
  const int vec = vecFor(leaves, tmpOrder);
  const int g = std::max(1, std::min(8, 64 / std::max(1, vec * eltBytes)));
  body += "  static constexpr int G = " + std::to_string(g) + ";\n";
  body += "#define ACC_SCAN_BLOCK 256\n";
  {
    int sz = 0, al = 1;
    std::vector<ST> flagged = leaves;
    flagged.push_back(ST::U32);
    structLayout(flagged, sz, al);
    if (g > 1 && 4L * (64 * (g + 1) + 1) * sz <= 64 * 1024) body += "#define ACC_ROWS_RAKE 1\n";
  }
  KernelSource ks = finish(body, elt, leaves, "scan.hpp+fold.hpp", vec);
  ks.commutative = comm;
  ks.words = structWords(leaves);
  ks.group = g;
  ks.block = 256;
  ks.streaming = true;
  return ks;
}

// size and alignment of `struct { leaf0; leaf1; .. }` under the C++ layout rules
static void structLayout(const std::vector<ST>& leaves, int& size, int& align) {
  int off = 0;
  align = 1;
  for (ST s : leaves) {
    int a = stAlign(s);
    off = (off + a - 1) / a * a + stSize(s);
    align = std::max(align, a);
  }
  if (off == 0) off = 1;
  size = (off + align - 1) / align * align;
}
static int structWords(const std::vector<ST>& leaves) {
  int size, align;
  structLayout(leaves, size, align);
  return (size + 3) / 4;
}
// words of `struct { Elt v; u32 f; }`
static int flaggedWords(const std::vector<ST>& leaves) {
  int size, align;
  structLayout(leaves, size, align);
  int off = (size + 3) / 4 * 4 + 4;
  align = std::max(align, 4);
  return ((off + align - 1) / align * align + 3) / 4;
}

// Bytes of elements a lane holds in a scan tile (tuning knob: ACCHIP_SCAN_BYTES).  Measured
// on MI355X for 2^28-element scans with 1024-thread workgroups: 128 B 822 us, 192 B 795 us,
// 256 B 1124 us (register spills) for Int64; 440 / 416 / 410 us for Float32.
static int scanBytesPerLane() {
  const char* e = std::getenv("ACCHIP_SCAN_BYTES");
  int v = e ? std::atoi(e) : 192;
  return v >= 16 && v <= 512 ? v : 192;
}

// threads per workgroup of the scan-family kernels (tuning knob: ACCHIP_SCAN_BLOCK)
static int scanBlock() {
  const char* e = std::getenv("ACCHIP_SCAN_BLOCK");
  int v = e ? std::atoi(e) : 1024;
  return (v == 256 || v == 512 || v == 1024) ? v : 1024;
}

KernelSource Codegen::foldSeg(const Sx& f, const Sx* seed, const Operand& src, const Operand& seg, ST segType) {
  const TypeP elt = src.r.elt;
  std::string body;
  body += std::string("  static constexpr bool kSeeded = ") + (seed ? "true" : "false") + ";\n";
  auto leaves = typeLeaves(elt);
  int eltBytes = 4;
  for (ST s : leaves) eltBytes += stSize(s);
  {
    Emit em;
    em.ind = 4;
    ValP r = applyFun(f, {eltVal(elt, "x"), eltVal(elt, "y")}, {}, em);
    if (!typeEq(valType(r), elt)) throw Error("foldSeg: combination function does not return the element type");
    body += fnHead("Elt", "combine", "const Env& env, const Elt& x, const Elt& y") + returnElt(r, em) + "  }\n";
  }
  {
    Emit em;
    em.ind = 4;
    if (seed) {
      ValP z = exp(*seed, {}, em);
      if (!typeEq(valType(z), elt)) throw Error("foldSeg: seed does not have the element type");
      returnElt(z, em);
    } else {
      em.line("Elt r_{};");
      em.line("return r_;");
    }
    body += fnHead("Elt", "seed", "const Env& env") + em.code + "  }\n";
  }
  {
    Emit em;
    em.ind = 4;
    ValP v = operandLinear(src, "i", em);
    if (!typeEq(valType(v), elt)) throw Error("foldSeg: fused producer does not return the element type");
    body += fnHead("Elt", "in_linear", "const Env& env, i64 i") + returnElt(v, em) + "  }\n";
  }
  {
    Emit em;
    em.ind = 4;
    ValP v = operandLinear(seg, "s", em);
    if (v->k != Val::Leaf || v->st != segType) throw Error("foldSeg: segment descriptor does not have the declared integral type");
    em.line("return (i64)" + v->ex + ";");
    body += fnHead("i64", "seg_at", "const Env& env, i64 s") + em.code + "  }\n";
  }
  std::vector<ArraySlot> tmpOrder;
  for (auto& kv : used_)
    if (kv.second.name != seg.slot) tmpOrder.push_back(kv.second);
  int vec = vecFor(leaves, tmpOrder);
  // Geometry of the segmented fold, with its own knobs: a lane's run is two 128-bit loads
  // long (ACCHIP_FOLDSEG_VECMUL), which halves the number of wave scans per element; a lane
  // holds ACCHIP_FOLDSEG_BYTES of (value, flag) pairs; workgroups of ACCHIP_FOLDSEG_BLOCK
  // threads (smaller ones lose less at the barriers).  The tile also pays for 2 bytes of LDS
  // per element.  Measured on 2^27 Int32 values in 2^20 segments, whole pipeline: 256
  // threads x 256 B 136 us, 256 x 128 B 154, 512 x 256 B 157, 512 x 128 B 150, 1024 x 256 B 173.
  const char* vm = std::getenv("ACCHIP_FOLDSEG_VECMUL");
  vec *= vm ? std::max(1, std::min(4, std::atoi(vm))) : 2;
  const char* fe = std::getenv("ACCHIP_FOLDSEG_BYTES");
  int fbytes = fe ? std::atoi(fe) : 256;
  if (fbytes < 16 || fbytes > 512) fbytes = 256;
  int g = std::max(1, std::min(8, fbytes / std::max(1, vec * eltBytes)));
  body += "  static constexpr int G = " + std::to_string(g) + ";\n";
  const char* fb = std::getenv("ACCHIP_FOLDSEG_BLOCK");
  int fblock = fb ? std::atoi(fb) : 256;
  if (fblock != 256 && fblock != 512 && fblock != 1024) fblock = 256;
  body += "#define ACC_SCAN_BLOCK " + std::to_string(fblock) + "\n";
  KernelSource ks = finish(body, elt, leaves, "scan.hpp+foldseg.hpp", vec);
  ks.block = fblock;
  ks.group = g;
  ks.words = flaggedWords(leaves);
  return ks;
}

// The pipelined scan moves its input with direct global -> LDS loads: the operand must be an
// array in memory (nothing fused into it) whose elements are one scalar of 4 or 8 bytes, read
// left to right.
bool Codegen::scanPipeable(const Operand& src, bool right) {
  (void)right;  // both directions: a right scan walks over the row's mirror image
  // (a fused producer may still turn out not to be a function of one array's element at the
  // same place: Codegen::scan then throws ScanNotPipeable)
  auto leaves = typeLeaves(src.r.elt);
  return leaves.size() == 1 && !stIsVec(leaves[0]) && (stSize(leaves[0]) == 4 || stSize(leaves[0]) == 8);
}

KernelSource Codegen::scan(const Sx& f, const Sx* seed, const Operand& src, bool right, int kind, int variant,
                           const Sx* post, const TypeP& postElt) {
  const TypeP elt = src.r.elt;
  const bool small = variant == 1, pipe = variant == 2;
  if (pipe && !scanPipeable(src, right)) throw Error("scan: this operand cannot take the pipelined kernel");
  if (post && (pipe || kind == 2)) throw Error("scan: this variant applies no function to its results");
  std::string pipeSlot;  // the array the pipelined kernel moves
  if (kind != 0 && !seed) throw Error("scan: this variant needs a seed");
  std::string body;
  body += std::string("  static constexpr bool kSeeded = ") + (seed ? "true" : "false") + ";\n";
  body += std::string("  static constexpr bool kRight = ") + (right ? "true" : "false") + ";\n";
  body += "  static constexpr int kKind = " + std::to_string(kind) + ";\n";
  body += "  ACC_DEV bool stops(const Elt&) { return false; }\n";
  auto leaves = typeLeaves(elt);
  int eltBytes = 0;
  for (ST s : leaves) eltBytes += stSize(s);
  {
    // combine(earlier, later) in traversal order; right scans apply f with the input on the
    // left (Interpreter.hs:524-526, 547-549)
    Emit em;
    em.ind = 4;
    ValP a = eltVal(elt, "x"), b = eltVal(elt, "y");
    ValP r = right ? applyFun(f, {b, a}, {}, em) : applyFun(f, {a, b}, {}, em);
    if (!typeEq(valType(r), elt)) throw Error("scan: combination function does not return the element type");
    body += fnHead("Elt", "combine", "const Env& env, const Elt& x, const Elt& y") + returnElt(r, em) + "  }\n";
  }
  {
    Emit em;
    em.ind = 4;
    if (seed) {
      ValP z = exp(*seed, {}, em);
      if (!typeEq(valType(z), elt)) throw Error("scan: seed does not have the element type");
      returnElt(z, em);
    } else {
      em.line("Elt r_{};");
      em.line("return r_;");
    }
    body += fnHead("Elt", "seed", "const Env& env") + em.code + "  }\n";
  }
  {
    Emit em;
    em.ind = 4;
    ValP v = operandLinear(src, "i", em);
    if (!typeEq(valType(v), elt)) throw Error("scan: fused producer does not return the element type");
    body += fnHead("Elt", "in_linear", "const Env& env, i64 i") + returnElt(v, em) + "  }\n";
  }
  // V from the widest leaf; G so that a lane holds scanBytesPerLane() bytes of elements (192)
  std::vector<ArraySlot> tmpOrder;
  for (auto& kv : used_) tmpOrder.push_back(kv.second);
  int vec = vecFor(leaves, tmpOrder);
  if (pipe) vec = 16 / stSize(leaves[0]);  // a lane's share of a row is one 128-bit load
  // Large tiles keep the number of look-back steps on the critical path small, but a row of
  // a few tiles cannot fill 256 CUs and a row shorter than a tile leaves most of a large
  // workgroup idle: short rows get 256-thread workgroups with 256 bytes per lane (one row
  // of 2^20 Int32: 8 us against 15 us with the large tiles; the large tiles win from 2^24 on).
  int g = std::max(1, std::min(16, scanBytesPerLane() / std::max(1, vec * std::max(1, eltBytes))));
  const int block = small ? 256 : scanBlock();
  if (small) {
    const char* sb = std::getenv("ACCHIP_SCAN_SMALL_BYTES");
    const char* sl = std::getenv("ACCHIP_SCAN_SMALL_LB");
    // 256 B per lane (64 KiB tiles): 2^21 / 2^22 / 2^23 Float32 in 9.8 / 13.5 / 21.9 us against 10.9 /
    // 17.7 / 30.8 with 128 B (and 10.7 / 17.3 / 26.7 with the large tiles)
    const int bytes = sb ? std::atoi(sb) : 256;
    g = std::max(1, std::min(16, bytes / std::max(1, vec * std::max(1, eltBytes))));
    body += "#define ACC_SCAN_LBWAVES " + std::to_string(sl ? std::max(1, std::min(4, std::atoi(sl))) : 1) + "\n";
  }
  if (pipe) {
    // bytes of elements a lane holds per tile of the pipelined kernel (ACCHIP_SCAN_PIPE_BYTES)
    const char* pb = std::getenv("ACCHIP_SCAN_PIPE_BYTES");
    // 4-byte elements: 112 B, so that the rake area (57 KiB) fits beside the load buffer (112 KiB)
    // and the next tile's loads can leave in the middle of the rake; 8-byte elements would have to
    // come down to 96 B for that, which gains nothing over 128 B with the rake area over the buffer
    const int bytes = pb ? std::atoi(pb) : (eltBytes == 4 ? 112 : 128);
    g = std::max(2, std::min(9, bytes / 16));
    const std::string T = stName(leaves[0]);
    std::string rawT = T, fromRaw = "    Elt r_;\n    r_.c0 = raw_;\n    return r_;\n";
    if (!src.delayed) {
      pipeSlot = slotByName(src.slot).name;
    } else {
      // A producer fused into the scan (scanl f z (map g xs)) can ride along when it is a
      // function of the element of one array at the scan's own position: the kernel moves that
      // array and applies the function to what arrives in LDS.  The function's code is the
      // producer's with its one load replaced; anything else that depends on the position
      // (another array read there, the index itself) disqualifies it.
      Emit em;
      em.ind = 4;
      ValP v = operandLinear(src, "i", em);
      if (!typeEq(valType(v), elt)) throw Error("scan: fused producer does not return the element type");
      std::string code = returnElt(v, em);
      static const std::regex load("acc_ld<kStream>\\(&env\\.(\\w+)_0\\[i\\]\\)");
      for (std::sregex_iterator it(code.begin(), code.end(), load), end; it != end; ++it) {
        const std::string name = (*it)[1].str();
        if (!pipeSlot.empty() && pipeSlot != name) throw ScanNotPipeable();
        pipeSlot = name;
      }
      if (pipeSlot.empty()) throw ScanNotPipeable();
      code = std::regex_replace(code, load, "raw_");
      if (std::regex_search(code, std::regex("\\bi\\b"))) throw ScanNotPipeable();
      const ArraySlot& as = slotByName(pipeSlot);
      auto rl = typeLeaves(as.r.elt);
      if (rl.size() != 1 || stIsVec(rl[0]) || stSize(rl[0]) != stSize(leaves[0]) || as.r.rank != src.r.rank) throw ScanNotPipeable();
      rawT = stName(rl[0]);
      fromRaw = code;
    }
    const std::string at = "env." + pipeSlot + "_0";
    body += "  typedef " + rawT + " Raw;\n  typedef " + T + " RawOut;\n";
    body += "  ACC_DEV const Raw* in_base(const Env& env) { return " + at + "; }\n";
    body += "  ACC_DEV RawOut* out_base(const Out& o) { return o.o0; }\n";
    body += "  ACC_DEV Elt from_raw(const Env& env, Raw raw_) {\n" + fromRaw + "  }\n";
    body += "  ACC_DEV RawOut to_raw(const Elt& e) { return e.c0; }\n";
  }
  body += "  static constexpr int G = " + std::to_string(g) + ";\n";
  body += "#define ACC_SCAN_BLOCK " + std::to_string(pipe ? 1024 : block) + "\n";
  int rowsG = g;
  if (!pipe) {
    // prefixes of the lane totals by raking through LDS, when the totals of a workgroup fit
    int sz = 0, al = 1;
    structLayout(leaves, sz, al);
    const long rake = (long)(block / 64) * (64 * (g + 1) + 1) * sz;
    const char* re = std::getenv("ACCHIP_SCAN_RAKE");
    if (g > 1 && rake <= 112 * 1024 && !(re && re[0] == '0')) body += "#define ACC_SCAN_RAKE 1\n";
    // the same for the rows kernel, whose values carry a head flag (only the 256-thread variant runs it)
    std::vector<ST> flagged = leaves;
    flagged.push_back(ST::U32);
    structLayout(flagged, sz, al);
    // (the rows kernel keeps 128 B per lane: its values travel with their flags, and 256 B of them
    // do not fit the registers -- 2^20 rows of 256 Int32: 406 us against 730)
    rowsG = std::max(1, std::min(g, 128 / std::max(1, vec * std::max(1, eltBytes))));
    if (small) body += "#define ACC_ROWS_G " + std::to_string(rowsG) + "\n";
    if (small && rowsG > 1 && (long)(block / 64) * (64 * (rowsG + 1) + 1) * sz <= 64 * 1024 && !(re && re[0] == '0'))
      body += "#define ACC_ROWS_RAKE 1\n";
  }
  std::vector<ST> outLeaves = leaves;
  if (post) {
    // the results leave through store / store_run, which here apply the function first.  They are
    // not handed the environment: a function that reads arrays stays a launch of its own.
    Emit em;
    em.ind = 6;
    ValP r = applyFun(*post, {eltVal(elt, "v")}, {}, em);
    if (!typeEq(valType(r), postElt)) throw Error("map: function result does not match the declared element type");
    if (em.code.find("env.") != std::string::npos) throw ScanPostNotFusable();
    auto lv = leavesOf(r);
    for (auto& l : lv)
      if (l->ex.find("env.") != std::string::npos) throw ScanPostNotFusable();
    outLeaves = typeLeaves(postElt);
    body += "  template <bool kStream = false>\n  ACC_DEV void store(const Out& o, i64 i, const Elt& v) {\n" + em.code;
    for (size_t k = 0; k < lv.size(); ++k)
      body += "      acc_st<kStream>(&o.o" + std::to_string(k) + "[i], (" + stName(outLeaves[k]) + ")(" + lv[k]->ex + "));\n";
    body += "  }\n";
    body += "  ACC_DEV void store_run(const Out& o, i64 i, const Elt* vs_) {\n";
    for (size_t k = 0; k < lv.size(); ++k)
      body += std::string("    acc_run<") + stName(outLeaves[k]) + ", V> r" + std::to_string(k) + "_;\n";
    body += "#pragma unroll\n    for (int k_ = 0; k_ < V; ++k_) {\n      const Elt& v = vs_[k_];\n" + em.code;
    for (size_t k = 0; k < lv.size(); ++k) body += "      r" + std::to_string(k) + "_.e[k_] = " + lv[k]->ex + ";\n";
    body += "    }\n";
    for (size_t k = 0; k < lv.size(); ++k)
      body += std::string("    *(acc_run<") + stName(outLeaves[k]) + ", V>*)&o.o" + std::to_string(k) + "[i] = r" + std::to_string(k) + "_;\n";
    body += "  }\n";
  }
  KernelSource ks = finish(body, elt, outLeaves, pipe ? "scan.hpp+scan_pipe.hpp" : "scan.hpp+scan_kernel.hpp", vec, post != nullptr);
  ks.block = pipe ? 1024 : block;
  ks.group = g;
  ks.words = structWords(leaves);
  ks.scanRight = right;
  ks.pipeSlot = pipeSlot;
  ks.rowsGroup = rowsG;
  return ks;
}

// Producers of rank >= 2 that need the multi-dimensional index of a result: the skeleton splits
// the linear index of a thread's first result once (the divisions) and steps from result to
// result, instead of dividing for every result.
std::string Codegen::indexedFns(int rank, const ArraySlot& o) {
  std::string fns;
  Emit ef;
  ef.ind = 4;
  ValP ix0 = fromIndex(rank, shapeOf(o), "i", ef);
  std::vector<std::string> c;
  shapeDims(ix0, c);
  for (int d = 0; d < rank; ++d) ef.line("ix[" + std::to_string(d) + "] = " + c[d] + ";");
  fns += fnHead("void", "from_index", "const Env& env, i64 i, i64* ix") + ef.code + "  }\n";
  std::vector<std::string> od;
  shapeDims(shapeOf(o), od);
  Emit en;
  en.ind = 4;
  for (int d = rank - 1; d >= 1; --d) {
    en.line("if (++ix[" + std::to_string(d) + "] < " + od[d] + ") return;");
    en.line("ix[" + std::to_string(d) + "] = 0;");
  }
  en.line("++ix[0];");
  fns += fnHead("void", "next_index", "const Env& env, i64* ix") + en.code + "  }\n";
  return fns;
}

ValP Codegen::indexedIx(int rank) {
  ValP v = vUnit();
  for (int d = 0; d < rank; ++d) v = vPair(v, vLeaf(ST::I64, "ix[" + std::to_string(d) + "]"));
  return v;
}

std::string Codegen::indexedTail(int rank) {
  return "  static constexpr int kRank = " + std::to_string(rank) + ";\n#define ACC_MAP_INDEXED 1\n";
}

KernelSource Codegen::map(const TypeP& outElt, const Sx* f, const Operand& src) {
  Emit em;
  em.ind = 4;
  ValP v = operandLinear(src, "i", em);
  ValP r = f ? applyFun(*f, {v}, {}, em) : v;
  if (!typeEq(valType(r), outElt)) throw Error("map: function result does not match the declared element type");
  std::string body = streamHead("Elt", "produce", "const Env& env, i64 i") + returnElt(r, em) + "  }\n";
  KernelSource ks = finish(body, outElt, typeLeaves(outElt), "map.hpp", 0);
  ks.streaming = true;
  return ks;
}

static void declareOut(std::map<std::string, ArraySlot>& used, int rank) {
  ArraySlot s;
  s.name = "out";
  s.r.rank = rank;
  s.r.elt = tUnit();
  s.index = -1;
  used.emplace("out", s);
}

KernelSource Codegen::zipWith(const TypeP& outElt, const Sx& f, const Operand& a, const Operand& b, int rank) {
  Emit em;
  em.ind = 4;
  ValP x, y;
  if (rank <= 1) {
    // rank <= 1: the linear index of the intersection is the linear index of both operands
    x = operandLinear(a, "i", em);
    y = operandLinear(b, "i", em);
  } else {
    declareOut(used_, rank);
    ArraySlot o = used_.at("out");
    ValP ix = indexedIx(rank);
    x = operandIndex(a, ix, em);
    y = operandIndex(b, ix, em);
    ValP r = applyFun(f, {x, y}, {}, em);
    if (!typeEq(valType(r), outElt)) throw Error("zipWith: function result does not match the declared element type");
    std::string body = indexedFns(rank, o) + fnHead("Elt", "produce_at", "const Env& env, i64 i, const i64* ix") +
                       returnElt(r, em) + "  }\n" + indexedTail(rank);
    return finish(body, outElt, typeLeaves(outElt), "map.hpp", 0);
  }
  ValP r = applyFun(f, {x, y}, {}, em);
  if (!typeEq(valType(r), outElt)) throw Error("zipWith: function result does not match the declared element type");
  std::string body = streamHead("Elt", "produce", "const Env& env, i64 i") + returnElt(r, em) + "  }\n";
  KernelSource ks = finish(body, outElt, typeLeaves(outElt), "map.hpp", 0);
  ks.streaming = true;
  return ks;
}

KernelSource Codegen::generate(const ArrayR& out, const Sx& f) {
  Emit em;
  em.ind = 4;
  declareOut(used_, out.rank);
  ArraySlot o = used_.at("out");
  if (out.rank >= 2) {
    ValP r = applyFun(f, {indexedIx(out.rank)}, {}, em);
    if (!typeEq(valType(r), out.elt)) throw Error("generate: function result does not match the declared element type");
    std::string body = indexedFns(out.rank, o) + fnHead("Elt", "produce_at", "const Env& env, i64 i, const i64* ix") +
                       returnElt(r, em) + "  }\n" + indexedTail(out.rank);
    return finish(body, out.elt, typeLeaves(out.elt), "map.hpp", 0);
  }
  ValP ix = fromIndex(out.rank, shapeOf(o), "i", em);
  ValP r = applyFun(f, {ix}, {}, em);
  if (!typeEq(valType(r), out.elt)) throw Error("generate: function result does not match the declared element type");
  std::string body = streamHead("Elt", "produce", "const Env& env, i64 i") + returnElt(r, em) + "  }\n";
  KernelSource ks = finish(body, out.elt, typeLeaves(out.elt), "map.hpp", 0);
  ks.streaming = true;
  return ks;
}

KernelSource Codegen::backpermute(int outRank, const Sx& p, const Sx* f, const TypeP& outElt, const Operand& src) {
  Emit em;
  em.ind = 4;
  declareOut(used_, outRank);
  ArraySlot o = used_.at("out");
  ValP ix = outRank >= 2 ? indexedIx(outRank) : fromIndex(outRank, shapeOf(o), "i", em);
  ValP sx = applyFun(p, {ix}, {}, em);
  ValP v = operandIndex(src, sx, em);
  ValP r = f ? applyFun(*f, {v}, {}, em) : v;
  if (!typeEq(valType(r), outElt)) throw Error("backpermute: result does not match the declared element type");
  if (outRank >= 2) {
    std::string body = indexedFns(outRank, o) + fnHead("Elt", "produce_at", "const Env& env, i64 i, const i64* ix") +
                       returnElt(r, em) + "  }\n" + indexedTail(outRank);
    // Transpositions -- index functions that walk the source along another dimension than the
    // result's innermost one (Language.hs:821-842) -- can go through tiles in LDS, 64 x 65
    // elements of up to 16 bytes (acc_map_xpose).
    int esz = 0, eal = 1;
    structLayout(typeLeaves(outElt), esz, eal);
    const bool fits = esz <= 16;
    if (fits) body += "#define ACC_MAP_XPOSE 1\n";
    KernelSource ks = finish(body, outElt, typeLeaves(outElt), "map.hpp", 0);
    ks.xpose = fits;
    ks.words = structWords(typeLeaves(outElt));
    return ks;
  }
  std::string body = streamHead("Elt", "produce", "const Env& env, i64 i") + returnElt(r, em) + "  }\n";
  KernelSource ks = finish(body, outElt, typeLeaves(outElt), "map.hpp", 0);
  ks.streaming = true;
  return ks;
}

// does the function's second argument (the old value) go unused?  `\x _ -> ..`
static bool ignoresSecond(const Sx& f) {
  if (!f.is("lam")) return false;
  const Sx& g = f.at(2);
  if (!g.is("lam")) return false;
  struct W {
    static bool allWild(const Sx& lhs) {
      if (lhs.is("wild")) return true;
      if (lhs.is("pair")) return allWild(lhs.at(1)) && allWild(lhs.at(2));
      return false;
    }
  };
  return W::allWild(g.at(1));
}

KernelSource Codegen::permute(const Sx& f, const ArrayR& dst, const Sx& p, const Operand& src, const Sx* freshInit) {
  const TypeP elt = dst.elt;
  if (!typeEq(elt, src.r.elt)) throw Error("permute: source and defaults have different element types");
  auto leaves = typeLeaves(elt);
  std::string body;
  {
    Emit em;
    em.ind = 4;
    ValP r = applyFun(f, {eltVal(elt, "x"), eltVal(elt, "y")}, {}, em);
    if (!typeEq(valType(r), elt)) throw Error("permute: combination function does not return the element type");
    body += fnHead("Elt", "combine", "const Env& env, const Elt& x, const Elt& y") + returnElt(r, em) + "  }\n";
  }
  {
    Emit em;
    em.ind = 4;
    ValP v = operandLinear(src, "i", em);
    if (!typeEq(valType(v), elt)) throw Error("permute: fused producer does not return the element type");
    body += fnHead("Elt", "in_linear", "const Env& env, i64 i") + returnElt(v, em) + "  }\n";
  }
  std::string target32, preamble;
  {
    // source index -> PrimMaybe destination index = (tag, ((), dst))  (AST.hs:202)
    Emit em;
    em.ind = 4;
    declareOut(used_, dst.rank);
    ArraySlot o = used_.at("out");
    ValP ssh = operandShape(src, em);
    ValP ix = fromIndex(src.r.rank, ssh, "i", em);
    ValP m = applyFun(p, {ix}, {}, em);
    if (m->k != Val::Pair || m->a->k != Val::Leaf || m->b->k != Val::Pair)
      throw Error("permute: index function must return a Maybe index (tag, ((), ix))");
    std::string tag = m->a->ex;
    {
      // a target outside the destination is an error in the reference (toIndex's bounds check,
      // Shape.hs:98-106); here it is dropped instead of written, and the skeleton reports it.  The
      // function stays free of stores and branches, so that the loads of many sources can be in
      // flight.  0: Nothing, 1: j is the target, 2: the target lies outside the destination.
      std::vector<std::string> dd, ii;
      shapeDims(shapeOf(o), dd);
      shapeDims(m->b->b, ii);
      if (dd.size() != ii.size()) throw Error("permute: index function returns an index of the wrong rank");
      std::string bad;
      for (size_t d = 0; d < dd.size(); ++d)
        bad += (bad.empty() ? "" : " | ") + std::string("((u64)") + ii[d] + " >= (u64)" + dd[d] + ")";
      if (bad.empty()) bad = "false";
      preamble = em.code;
      em.line("j = " + toIndex(shapeOf(o), m->b->b, em) + ";");
      em.line("return " + tag + " == 0 ? 0 : ((" + bad + ") ? 2 : 1);");
    }
    body += fnHead("int", "target", "const Env& env, i64 i, i64& j") + em.code + "  }\n";
    // For a destination of rank 1 and fewer than 2^31 elements (the caller's to check) whose index
    // was widened from an integer of at most 32 bits: the index in 32 bits, untested (the skeleton
    // compares it with the extent when it uses it, not when it is loaded); returns the Maybe's
    // tag.  An index below zero wraps to a number no such destination has.
    std::vector<ValP> il;
    valLeaves(m->b->b, il);
    if (il.size() == 1 && !il[0]->narrowEx.empty()) {
      std::vector<std::string> dd;
      shapeDims(shapeOf(o), dd);
      const ST ns = il[0]->narrowSt;
      const std::string widened = stIsSigned(ns) ? "(u32)(i32)(" + il[0]->narrowEx + ")" : "(u32)(" + il[0]->narrowEx + ")";
      target32 = "#define ACC_PERMUTE_TARGET32 1\n" + fnHead("int", "target32", "const Env& env, i64 i, u32& j") + preamble +
                 "    j = " + widened + ";\n    return " + tag + " != 0 ? 1 : 0;\n  }\n";
      body += target32;
    }
  }
  // how to combine into the destination
  std::string mode = "lock", op;
  ST st = ST::I32;
  const bool single = leaves.size() == 1;
  const bool wide = single && !stIsVec(leaves[0]) && (stSize(leaves[0]) == 4 || stSize(leaves[0]) == 8);
  if (ignoresSecond(f) && (fastPermuteConst || wide)) mode = "store";
  else if (wide && isCommutative(f, &op, &st) && st == leaves[0] &&
           (op == "add" ? (st != ST::F16) : (op != "mul" && stIsInt(st))))
    mode = "atomic";
  else if (wide) mode = "cas";
  std::vector<std::string> leafOps;
  if (mode == "lock" && componentwiseAtomic(f, leaves, leafOps)) mode = "atomics";
  std::string lds;
  std::string u = "  ACC_DEV void update(const Env& env, const Out& out, i64 j, const Elt& x, u32* locks, u32* err) {\n";
  if (mode == "store") {
    u += "    Elt y_{};\n    store(out, j, combine(env, x, y_));\n";
  } else if (mode == "atomic") {
    std::string fn = op == "add" ? "__hip_atomic_fetch_add" : op == "min" ? "__hip_atomic_fetch_min"
                   : op == "max" ? "__hip_atomic_fetch_max" : op == "band" ? "__hip_atomic_fetch_and"
                   : op == "bor" ? "__hip_atomic_fetch_or" : "__hip_atomic_fetch_xor";
    u += "    (void)" + fn + "(&out.o0[j], x.c0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n";
    leafOps = {op};
  } else if (mode == "atomics") {
    // component-wise combination: the components do not see each other, one atomic each
    for (size_t k = 0; k < leaves.size(); ++k) {
      const std::string& o = leafOps[k];
      std::string fn = o == "add" ? "__hip_atomic_fetch_add" : o == "min" ? "__hip_atomic_fetch_min"
                     : o == "max" ? "__hip_atomic_fetch_max" : o == "band" ? "__hip_atomic_fetch_and"
                     : o == "bor" ? "__hip_atomic_fetch_or" : "__hip_atomic_fetch_xor";
      const std::string K = std::to_string(k);
      u += "    (void)" + fn + "(&out.o" + K + "[j], x.c" + K + ", __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n";
    }
  } else if (mode == "cas") {
    std::string B = stSize(leaves[0]) == 4 ? "u32" : "u64", T = stName(leaves[0]);
    u += "    " + B + "* a_ = (" + B + "*)&out.o0[j];\n";
    u += "    " + B + " old_ = __hip_atomic_load(a_, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n";
    u += "    for (;;) {\n      Elt y_;\n      y_.c0 = __builtin_bit_cast(" + T + ", old_);\n";
    u += "      Elt r_ = combine(env, x, y_);\n      " + B + " new_ = __builtin_bit_cast(" + B + ", r_.c0);\n";
    u += "      if (__hip_atomic_compare_exchange_strong(a_, &old_, new_, __ATOMIC_RELAXED, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) break;\n    }\n";
  } else {
    // The loop runs until every lane of the wave is done (wave-uniform exit through the
    // ballot).  With a per-lane exit the compiler may move the critical section behind the
    // loop, where a lane that won the lock waits for the lanes still spinning on it: two
    // lanes of one wave with the same destination then never finish.
    // The wait for a lock is bounded: a wave that sees none of its lanes win a lock for
    // ACC_LOCK_SPIN_LIMIT rounds in a row (many seconds) reports through err and drops the updates
    // still waiting, so that the kernel always ends.  The count starts again whenever a lane of
    // the wave wins, so heavy but legitimate contention -- millions of sources for one cell -- is
    // slow, not an error, as long as the wave's own updates keep landing.
    u += "    u32* lk_ = locks + j;\n    bool done_ = false;\n    u32 rounds_ = 0;\n    while (__ballot(!done_) != 0ull) {\n";
    u += "      if (++rounds_ > ACC_LOCK_SPIN_LIMIT) {\n        if (!done_) __hip_atomic_store(err, 4u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);\n        break;\n      }\n";
    // Lock word and element are only ever touched by relaxed device-scope atomics, which go past
    // the caches that are not coherent across the device; what orders them is that a wave's
    // accesses have completed before its next ones leave: the exchange's result is waited for by
    // the branch on it, and the element's stores are waited for (s_waitcnt) before the store that
    // frees the lock.  Acquire / release orderings on the lock would add a cache invalidation and a
    // write-back of the whole L2 per update, which nothing here needs: 2^24 pairs into 2^24
    // elements 17.0 -> 2.3 ms, into 2^20 elements 29.0 -> 2.2 ms.  ACCHIP_LOCK_ORDER=fences
    // generates the orderings instead.
    const char* lo = std::getenv("ACCHIP_LOCK_ORDER");
    const bool relaxedLock = !(lo && std::string(lo) == "fences");
    if (relaxedLock)
      u += "      const bool won_ = !done_ && __hip_atomic_exchange(lk_, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u;\n";
    else
      u += "      const bool won_ = !done_ && __hip_atomic_exchange(lk_, 1u, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) == 0u;\n";
    u += "      if (__ballot(won_) != 0ull) rounds_ = 0;\n";
    u += "      if (won_) {\n        Elt y_;\n";
    if (relaxedLock) u += "        asm volatile(\"\" ::: \"memory\");  // (the compiler keeps the element's loads behind the exchange)\n";
    // leaf by leaf (component by component for SIMD vector leaves) through relaxed atomics
    auto each = [&](size_t k, const std::function<void(const std::string& cell, const std::string& field)>& fn) {
      const std::string cell = "out.o" + std::to_string(k) + "[j]", field = ".c" + std::to_string(k);
      if (!stIsVec(leaves[k])) return fn(cell, field);
      for (int m = 0; m < stWidth(leaves[k]); ++m) fn(cell + ".e[" + std::to_string(m) + "]", field + ".e[" + std::to_string(m) + "]");
    };
    for (size_t k = 0; k < leaves.size(); ++k)
      each(k, [&](const std::string& cell, const std::string& field) {
        u += "        y_" + field + " = __hip_atomic_load(&" + cell + ", __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n";
      });
    u += "        Elt r_ = combine(env, x, y_);\n";
    for (size_t k = 0; k < leaves.size(); ++k)
      each(k, [&](const std::string& cell, const std::string& field) {
        u += "        __hip_atomic_store(&" + cell + ", r_" + field + ", __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n";
      });
    if (relaxedLock)
      u += "        asm volatile(\"s_waitcnt vmcnt(0)\" ::: \"memory\");\n        __hip_atomic_store(lk_, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n        done_ = true;\n      }\n    }\n";
    else
      u += "        __hip_atomic_store(lk_, 0u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);\n        done_ = true;\n      }\n    }\n";
  }
  if (mode == "atomic" || mode == "atomics") {
    // pieces of the LDS-privatised variant (permute.hpp): one private array per component, its
    // identity, the LDS update and the addition of a private value to the destination
    int bytes = 0;
    for (ST t : leaves) bytes += stSize(t);
    lds = "#define ACC_PERMUTE_LDS 1\n  static constexpr int kPart = 131072 / " + std::to_string(bytes) + ";\n  struct Priv {\n";
    std::string init, upd, flush;
    for (size_t k = 0; k < leaves.size(); ++k) {
      const ST t = leaves[k];
      const std::string& o = leafOps[k];
      const std::string T = stName(t), K = std::to_string(k);
      std::string fn = o == "add" ? "__hip_atomic_fetch_add" : o == "min" ? "__hip_atomic_fetch_min"
                     : o == "max" ? "__hip_atomic_fetch_max" : o == "band" ? "__hip_atomic_fetch_and"
                     : o == "bor" ? "__hip_atomic_fetch_or" : "__hip_atomic_fetch_xor";
      std::string idv;
      if (o == "add" || o == "bor" || o == "bxor") idv = "(" + T + ")0";
      else if (o == "band") idv = "(" + T + ")~(" + T + ")0";
      else {
        int bits = stBits(t);
        unsigned long long mx = stIsSigned(t) ? ((1ULL << (bits - 1)) - 1) : (bits == 64 ? ~0ULL : ((1ULL << bits) - 1));
        unsigned long long mn = stIsSigned(t) ? (1ULL << (bits - 1)) : 0ULL;
        char buf[64];
        snprintf(buf, sizeof buf, "(%s)0x%llxULL", T.c_str(), o == "min" ? mx : mn);
        idv = buf;
      }
      lds += "    " + T + " c" + K + "[kPart];\n";
      init += "    p.c" + K + "[i] = " + idv + ";\n";
      upd += "    (void)" + fn + "(&p.c" + K + "[i], x.c" + K + ", __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);\n";
      flush += "    {\n      const " + T + " v_ = p.c" + K + "[i];\n      if (v_ != " + idv + ") (void)" + fn + "(&out.o" + K +
               "[j], v_, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n    }\n";
    }
    lds += "  };\n";
    lds += "  ACC_DEV void lds_init(Priv& p, int i) {\n" + init + "  }\n";
    lds += "  ACC_DEV void lds_update(Priv& p, int i, const Elt& x) {\n" + upd + "  }\n";
    lds += "  ACC_DEV void lds_flush(const Priv& p, int i, const Out& out, i64 j) {\n" + flush + "  }\n";
  }
  if (mode == "lock" || mode == "cas") {
    // The same privatisation for combinations that need the lock, or the compare-and-swap loop
    // (2^24 Int64 products into 384 / 4096 elements: 498 / 25 ms of retries): a private copy of a destination
    // range in LDS, one state word per element (bit 0: locked, bit 1: holds a value -- no identity
    // of the function is known, so the first source of an element is stored as it is), updated
    // under LDS locks; the workgroups leave their copies in memory, and a second launch combines
    // them element by element.
    int bytes = 4;
    for (ST t : leaves) bytes += stSize(t);
    lds = "#define ACC_PERMUTE_LDS 1\n#define ACC_PERMUTE_LDS_LOCKED 1\n  static constexpr int kPart = 131072 / " + std::to_string(bytes) +
          ";\n  struct Priv {\n    u32 st[kPart];\n";
    std::string rd, wr;
    for (size_t k = 0; k < leaves.size(); ++k) {
      const std::string T = stName(leaves[k]), K = std::to_string(k);
      lds += "    " + T + " c" + K + "[kPart];\n";
      rd += "          y_.c" + K + " = p.c" + K + "[i];\n";
      wr += "        p.c" + K + "[i] = r_.c" + K + ";\n";
    }
    lds += "  };\n";
    lds += "  ACC_DEV void lds_init(Priv& p, int i) { p.st[i] = 0u; }\n";
    // (the loop ends for the whole wave at once, like the one of update(), and for the same reason)
    lds += "  ACC_DEV void lds_update(const Env& env, Priv& p, int i, const Elt& x, u32* err) {\n"
           "    bool done_ = false;\n    u32 rounds_ = 0;\n    while (__ballot(!done_) != 0ull) {\n"
           "      if (++rounds_ > ACC_LOCK_SPIN_LIMIT) {\n        if (!done_) __hip_atomic_store(err, 4u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);\n        break;\n      }\n"
           "      u32 old_ = 1u;\n"
           "      if (!done_) old_ = __hip_atomic_fetch_or(&p.st[i], 1u, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP);\n"
           "      const bool won_ = (old_ & 1u) == 0u;\n"
           "      if (__ballot(won_) != 0ull) rounds_ = 0;\n"
           "      if (won_) {\n        Elt r_ = x;\n        if (old_ & 2u) {\n          Elt y_;\n" + rd +
           "          r_ = combine(env, x, y_);\n        }\n" + wr +
           "        __hip_atomic_store(&p.st[i], 2u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);\n        done_ = true;\n      }\n    }\n  }\n";
    std::string spill, take;
    for (size_t k = 0; k < leaves.size(); ++k) {
      const std::string K = std::to_string(k);
      spill += "      g->c" + K + "[i] = p.c" + K + "[i];\n";
      take += "      x_.c" + K + " = g[c_].c" + K + "[i];\n";
    }
    lds += "  ACC_DEV void lds_spill(const Priv& p, int i, Priv* g) {\n    const u32 s_ = p.st[i];\n    g->st[i] = s_;\n"
           "    if (s_ & 2u) {\n" + spill + "    }\n  }\n";
    // (the copies' values are loaded whether they hold one or not, so that the loads of several
    // copies can be in flight together)
    lds += "  ACC_DEV void lds_merge(const Env& env, const Out& out, i64 j, const Priv* g, i64 groups, int i) {\n"
           "    bool have_ = false;\n    Elt acc_{};\n#pragma unroll 4\n    for (i64 c_ = 0; c_ < groups; ++c_) {\n"
           "      const u32 s_ = g[c_].st[i];\n      Elt x_;\n" + take +
           "      if (s_ & 2u) {\n        acc_ = have_ ? combine(env, x_, acc_) : x_;\n        have_ = true;\n      }\n    }\n"
           "    if (have_) store(out, j, combine(env, acc_, load(out, j)));\n  }\n";
  }
  // A sum of one and the same constant per source (a histogram: `permute (+) zeros p ones`, the ones
  // fused into a constant producer): the skeleton only counts, in 16-bit LDS counters, and adds
  // count * constant (acc_permute_count).
  bool countable = false, countSet = false;
  if (mode == "atomic" && op == "add" && stIsInt(st) && src.delayed && src.linearD.is("lam") &&
      src.linearD.at(2).is("const") && isST(src.linearD.at(2).at(1)) && parseST(src.linearD.at(2).at(1)) == st) {
    countable = true;
    const std::string T = stName(st), U = stName(stUnsigned(st));
    lds += "#define ACC_PERMUTE_COUNT 1\n";
    lds += "  ACC_DEV void count_flush(const Out& out, i64 j, u32 n) {\n    (void)__hip_atomic_fetch_add(&out.o0[j], (" + T +
           ")((" + U + ")n * (" + U + ")(" + literalText(st, src.linearD.at(2).at(2).s) +
           ")), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n  }\n";
    if (freshInit && freshInit->is("const") && isST(freshInit->at(1)) && parseST(freshInit->at(1)) == st) {
      countSet = true;
      lds += "#define ACC_PERMUTE_COUNT_SET 1\n";
      lds += "  ACC_DEV void count_set(const Out& out, i64 j, u32 n) {\n    out.o0[j] = (" + T + ")((" + U + ")(" +
             literalText(st, freshInit->at(2).s) + ") + (" + U + ")n * (" + U + ")(" + literalText(st, src.linearD.at(2).at(2).s) +
             "));\n  }\n";
    }
  }
  u += "  }\n" + lds;
  // update() uses store()/combine(): it must come after them, and finish() appends load/store
  // last, so emit our own forward-safe copies by placing update in a trailing block
  KernelSource ks = finish(body + "//@UPDATE@\n", elt, leaves, "permute.hpp", 1);
  size_t at = ks.source.find("//@UPDATE@\n");
  size_t endSpec = ks.source.find("};\n\n", at);
  ks.source.erase(at, std::strlen("//@UPDATE@\n"));
  endSpec -= std::strlen("//@UPDATE@\n");
  ks.source.insert(endSpec, u);
  ks.permuteMode = mode;
  ks.permuteCount = countable;
  ks.permuteCountSet = countSet;
  ks.permuteTarget32 = !target32.empty();
  return ks;
}

static int stencilWidth(const Sx& sr) {
  const std::string& h = sr.head();
  if (h.compare(0, 4, "unit") == 0) return std::atoi(h.c_str() + 4);
  if (h.compare(0, 3, "tup") == 0) return std::atoi(h.c_str() + 3);
  throw Error("malformed stencil pattern " + sr.str());
}

// halo of a stencil pattern per dimension (outermost first)
static void stencilHalo(const Sx& sr, int dim, std::vector<int>& halo) {
  const int w = stencilWidth(sr);
  if ((int)halo.size() <= dim) halo.resize(dim + 1, 0);
  halo[dim] = std::max(halo[dim], w / 2);
  if (sr.head().compare(0, 4, "unit") != 0)
    for (size_t r = 1; r < sr.size(); ++r) stencilHalo(sr.at(r), dim + 1, halo);
}

std::vector<int> stencilHaloOf(const Sx& pattern) {
  std::vector<int> halo;
  stencilHalo(pattern, 0, halo);
  return halo;
}

KernelSource Codegen::stencil(const std::vector<Sx>& patterns, const TypeP& outElt, const Sx& f,
                              const std::vector<Sx>& boundaries, const std::vector<Operand>& srcs) {
  Emit em;
  em.ind = 4;
  const int rank = srcs.at(0).r.rank;
  if (rank < 1) throw Error("stencil: rank must be at least 1");
  declareOut(used_, rank);
  ArraySlot o = used_.at("out");
  // the focus arrives as a multi-dimensional index: the skeleton splits the linear index
  // of a thread's first result once and steps to the following results by increments
  std::vector<std::string> fx(rank);
  for (int d = 0; d < rank; ++d) fx[d] = "ix[" + std::to_string(d) + "]";
  std::string indexFns = indexedFns(rank, o);

  // stencilAccess (Interpreter.hs:670-794): the outermost tuple walks the left-most
  // dimension, offsets -k..+k left to right
  struct Rec {
    static ValP go(const Sx& sr, int dim, int rank, std::vector<int>& off,
                   const std::function<ValP(const std::vector<int>&)>& access) {
      int w = stencilWidth(sr), k = w / 2;
      bool unit = sr.head().compare(0, 4, "unit") == 0;
      if (unit != (dim == rank - 1)) throw Error("stencil pattern does not match the array rank");
      if (!unit && (int)sr.size() != w + 1) throw Error("malformed stencil pattern " + sr.str());
      ValP v = vUnit();
      for (int d = -k; d <= k; ++d) {
        off[dim] = d;
        v = vPair(v, unit ? access(off) : go(sr.at(1 + d + k), dim + 1, rank, off, access));
      }
      off[dim] = 0;
      return v;
    }
  };
  auto mk = [&](const std::vector<std::string>& c) {
    ValP v = vUnit();
    for (int d = 0; d < rank; ++d) v = vPair(v, vLeaf(ST::I64, c[d]));
    return v;
  };

  // extents of the sources, and the condition under which no tap of this focus leaves them
  std::vector<std::vector<std::string>> dimsOf(srcs.size());
  std::string interior;
  for (size_t a = 0; a < srcs.size(); ++a) {
    const std::string kind = boundaries[a].atom ? boundaries[a].s : boundaries[a].head();
    if (kind != "clamp" && kind != "mirror" && kind != "wrap" && kind != "constant" && kind != "function")
      throw Error("unknown stencil boundary '" + kind + "'");
    ValP sh = operandShape(srcs[a], em);
    shapeDims(sh, dimsOf[a]);
    std::vector<int> halo;
    stencilHalo(patterns[a], 0, halo);
    if ((int)halo.size() != rank) throw Error("stencil pattern does not match the array rank");
    for (int d = 0; d < rank; ++d) {
      if (halo[d] == 0) continue;
      interior += (interior.empty() ? "" : " && ") + std::string("(") + fx[d] + " >= (i64)" + std::to_string(halo[d]) +
                  ") && (" + fx[d] + " + (i64)" + std::to_string(halo[d]) + " < " + dimsOf[a][d] + ")";
    }
  }

  // Away from the borders (almost every focus of a large array) no tap needs the boundary
  // condition: a stencil over one array reads at constant distances from the focus' linear
  // index, which costs one addition per tap instead of an index computation per tap.
  Emit ei;
  ei.ind = em.ind + 2;
  ValP ri;
  std::vector<std::string> focusLin, focusDefs;
  {
    // every source is read at its own linear index of the focus (for one source that is the
    // result's linear index; for two, whose extents may differ, it is computed from ix)
    std::vector<std::vector<std::string>> stride(srcs.size(), std::vector<std::string>(rank));
    for (size_t a = 0; a < srcs.size(); ++a) {
      std::string acc = "(i64)1";
      for (int d = rank - 1; d >= 0; --d) {
        stride[a][d] = acc;
        if (d > 0) acc = bindLeaf(ST::I64, acc + " * " + dimsOf[a][d], em)->ex;
      }
      if (srcs.size() == 1) {
        focusLin.push_back("i");
      } else {
        std::string e = fx[0];
        for (int d = 1; d < rank; ++d) e = "(" + e + " * " + dimsOf[a][d] + " + " + fx[d] + ")";
        focusLin.push_back("b" + std::to_string(a));
        focusDefs.push_back("const i64 b" + std::to_string(a) + " = " + e);
      }
    }
    std::vector<ValP> args;
    for (size_t a = 0; a < srcs.size(); ++a) {
      auto access = [&](const std::vector<int>& off) -> ValP {
        std::string lin = focusLin[a];
        for (int d = 0; d < rank; ++d)
          if (off[d] != 0) lin += " + (i64)" + std::to_string(off[d]) + " * " + stride[a][d];
        return operandLinear(srcs[a], bindLeaf(ST::I64, lin, ei)->ex, ei);
      };
      std::vector<int> off(rank, 0);
      args.push_back(Rec::go(patterns[a], 0, rank, off, access));
    }
    ri = applyFun(f, args, {}, ei);
  }

  // At the borders: bounded (Interpreter.hs:797-839) decides every tap
  Emit eb;
  eb.ind = em.ind + 2;
  std::vector<ValP> stencilArgs;
  for (size_t a = 0; a < srcs.size(); ++a) {
    const Operand& src = srcs[a];
    const Sx& bnd = boundaries[a];
    const std::string kind = bnd.atom ? bnd.s : bnd.head();
    const std::vector<std::string>& dims = dimsOf[a];
    auto access = [&](const std::vector<int>& off) -> ValP {
      Emit& em = eb;
      std::vector<std::string> raw(rank), idx(rank);
      std::string inside;
      for (int d = 0; d < rank; ++d) {
        if (off[d] == 0) {
          raw[d] = idx[d] = fx[d];
          continue;
        }
        raw[d] = bindLeaf(ST::I64, fx[d] + " + (i64)" + std::to_string(off[d]), em)->ex;
        const std::string& j = raw[d];
        const std::string& sz = dims[d];
        if (kind == "clamp")
          idx[d] = bindLeaf(ST::I64, off[d] < 0 ? "(" + j + " < 0) ? (i64)0 : " + j
                                                : "(" + j + " >= " + sz + ") ? " + sz + " - 1 : " + j, em)->ex;
        else if (kind == "mirror")
          idx[d] = bindLeaf(ST::I64, off[d] < 0 ? "(" + j + " < 0) ? -" + j + " : " + j
                                                : "(" + j + " >= " + sz + ") ? " + sz + " - (" + j + " - " + sz + " + 2) : " + j, em)->ex;
        else if (kind == "wrap")
          idx[d] = bindLeaf(ST::I64, off[d] < 0 ? "(" + j + " < 0) ? " + sz + " + " + j + " : " + j
                                                : "(" + j + " >= " + sz + ") ? " + j + " - " + sz + " : " + j, em)->ex;
        else {
          idx[d] = j;
          inside += (inside.empty() ? "" : " && ") + (off[d] < 0 ? "(" + j + " >= 0)" : "(" + j + " < " + sz + ")");
        }
      }
      if ((kind != "constant" && kind != "function") || inside.empty()) return operandIndex(src, mk(idx), em);
      // Constant / Function: the whole index decides (no per-dimension remapping)
      Emit ein, eo;
      ein.ind = eo.ind = em.ind + 2;
      ValP vin = operandIndex(src, mk(idx), ein);
      ValP vout = kind == "constant" ? exp(bnd.at(1), {}, eo) : applyFun(bnd.at(1), {mk(raw)}, {}, eo);
      if (!typeEq(valType(vin), valType(vout))) throw Error("stencil: boundary value does not have the element type");
      ValP res = declareVars(valType(vin), em);
      em.line("if (" + inside + ") {");
      em.code += ein.code;
      em.ind += 2;
      assign(res, vin, em);
      em.ind -= 2;
      em.line("} else {");
      em.code += eo.code;
      em.ind += 2;
      assign(res, vout, em);
      em.ind -= 2;
      em.line("}");
      return res;
    };
    std::vector<int> off(rank, 0);
    stencilArgs.push_back(Rec::go(patterns[a], 0, rank, off, access));
  }
  ValP rb = applyFun(f, stencilArgs, {}, eb);
  if (!typeEq(valType(rb), outElt) || !typeEq(valType(ri), outElt))
    throw Error("stencil: function result does not match the declared element type");

  // A thread whose V results and all their taps lie inside one row of the array evaluates
  // them without any test (interior_run / produce_in): the taps of neighbouring results are
  // then the same loads, and what is left becomes a few wide requests.
  std::string runFns;
  if (!interior.empty()) {
    std::string cond;
    for (size_t a = 0; a < srcs.size(); ++a) {
      std::vector<int> halo;
      stencilHalo(patterns[a], 0, halo);
      for (int d = 0; d < rank; ++d) {
        const bool inner = d == rank - 1;
        if (halo[d] == 0 && !inner) continue;
        cond += (cond.empty() ? "" : " && ") + std::string("(") + fx[d] + " >= (i64)" + std::to_string(halo[d]) + ") && (" +
                fx[d] + " + (i64)" + std::to_string(halo[d]) + (inner ? " + (i64)(V - 1)" : "") + " < " + dimsOf[a][d] + ")";
      }
    }
    Emit er;
    er.ind = 4;
    er.code = em.code;  // extents and strides bound so far
    er.line("return " + cond + ";");
    runFns += fnHead("bool", "interior_run", "const Env& env, const i64* ix") + er.code + "  }\n";
    // result k of the run that starts at ix (i: its linear index in the result)
    Emit ep;
    ep.ind = 4;
    ep.code = em.code;
    for (const std::string& d : focusDefs) ep.line(d + " + (i64)k;");
    ep.code += ei.code;
    runFns += fnHead("Elt", "produce_in", "const Env& env, i64 i, const i64* ix, int k") + returnElt(ri, ep) + "  }\n";
    runFns += "#define ACC_MAP_INTERIOR_RUN 1\n";
  }

  ValP r = rb;
  if (interior.empty()) {
    em.code += eb.code;  // no halo at all: nothing can leave the array (eb was emitted one level deeper)
  } else {
    r = declareVars(outElt, em);
    em.line("if (" + interior + ") {");
    em.ind += 2;
    for (const std::string& d : focusDefs) em.line(d + ";");
    em.ind -= 2;
    em.code += ei.code;
    em.ind += 2;
    assign(r, ri, em);
    em.ind -= 2;
    em.line("} else {");
    em.code += eb.code;
    em.ind += 2;
    assign(r, rb, em);
    em.ind -= 2;
    em.line("}");
  }
  std::string body = indexFns + runFns + fnHead("Elt", "produce_at", "const Env& env, i64 i, const i64* ix") + returnElt(r, em) + "  }\n";
  body += "  static constexpr int kRank = " + std::to_string(rank) + ";\n#define ACC_MAP_INDEXED 1\n";
  if (rank >= 2) body += "#define ACC_MAP_XCD 1\n";
  return finish(body, outElt, typeLeaves(outElt), "map.hpp", 0);
}

// Results per stencil tile: 256 columns x 8 rows (16 rows when the halo is wider than one
// row, to keep the share of halo rows down).  Measured on the 8192 x 8192 Jacobi sweep (us
// per sweep, one tile per workgroup): 256x8 92, 128x16 94, 256x16 94, 64x16 97, 128x32 99,
// 128x8 100.  Tuning knobs: ACCHIP_STENCIL_H, ACCHIP_STENCIL_W.
int stencilTileH(int hy) {
  const char* e = std::getenv("ACCHIP_STENCIL_H");
  const int dflt = hy <= 1 ? 8 : 16;
  int v = e ? std::atoi(e) : dflt;
  return (v == 8 || v == 16 || v == 32 || v == 64) ? v : dflt;
}

int stencilTileW() {
  const char* e = std::getenv("ACCHIP_STENCIL_W");
  int v = e ? std::atoi(e) : 256;
  return (v == 64 || v == 128 || v == 256) ? v : 256;
}

KernelSource Codegen::stencil2d(const Sx& pattern, const TypeP& outElt, const Sx& f, const Sx& bnd,
                                const Operand& src) {
  const TypeP srcElt = src.r.elt;
  auto sleaves = typeLeaves(srcElt);
  const std::string kind = bnd.atom ? bnd.s : bnd.head();
  if (kind != "clamp" && kind != "mirror" && kind != "wrap" && kind != "constant" && kind != "function")
    throw Error("unknown stencil boundary '" + kind + "'");
  if (pattern.head().compare(0, 3, "tup") != 0) throw Error("stencil2d: pattern is not of rank 2");
  const int hy = stencilWidth(pattern) / 2;
  int hx = 0;
  for (size_t r = 1; r < pattern.size(); ++r) hx = std::max(hx, stencilWidth(pattern.at(r)) / 2);
  const int tileH = stencilTileH(hy);
  const int tileW = stencilTileW();
  const int hxp = (hx + 3) / 4 * 4;  // halo columns padded so that result columns stay 16-byte aligned in LDS
  const int pw = tileW + 2 * hxp, ph = tileH + 2 * hy;
  std::string body;
  body += "#define ACC_ST_H " + std::to_string(tileH) + "\n";
  body += "#define ACC_ST_W " + std::to_string(tileW) + "\n";
  body += "  static constexpr int HY = " + std::to_string(hy) + ";\n  static constexpr int HX = " + std::to_string(hx) + ";\n  static constexpr int HXP = " + std::to_string(hxp) + ";\n";
  body += "  struct SrcElt {\n" + leafDecls(sleaves, "c", false, false) + "  };\n  struct Tile {\n";
  for (size_t k = 0; k < sleaves.size(); ++k)
    body += std::string("    __attribute__((aligned(16))) ") + stName(sleaves[k]) + " c" + std::to_string(k) + "[" + std::to_string(pw * ph) + "];\n";
  body += "  };\n  ACC_DEV void stage(Tile& t, int idx, const SrcElt& v) {\n";
  for (size_t k = 0; k < sleaves.size(); ++k)
    body += "    t.c" + std::to_string(k) + "[idx] = v.c" + std::to_string(k) + ";\n";
  body += "  }\n";
  auto retSrc = [&](const ValP& v, Emit& em) {
    auto lv = leavesOf(v);
    em.line("SrcElt r_;");
    for (size_t k = 0; k < lv.size(); ++k) em.line("r_.c" + std::to_string(k) + " = " + lv[k]->ex + ";");
    em.line("return r_;");
  };
  auto idx2 = [](const std::string& y, const std::string& x) {
    return vPair(vPair(vUnit(), vLeaf(ST::I64, y)), vLeaf(ST::I64, x));
  };
  {
    Emit em;
    em.ind = 4;
    ValP v = operandIndex(src, idx2("y", "x"), em);
    if (!typeEq(valType(v), srcElt)) throw Error("stencil: fused producer does not return the element type");
    retSrc(v, em);
    body += fnHead("SrcElt", "src_in", "const Env& env, i64 y, i64 x") + em.code + "  }\n";
  }
  {
    // bounded (Interpreter.hs:797-839) at an index that may lie outside on either side
    Emit em;
    em.ind = 4;
    std::vector<std::string> dims;
    shapeDims(operandShape(src, em), dims);
    const char* raw[2] = {"y", "x"};
    std::string idx[2], inside;
    for (int d = 0; d < 2; ++d) {
      const std::string j = raw[d], sz = dims[d];
      if (kind == "clamp") idx[d] = bindLeaf(ST::I64, "(" + j + " < 0) ? (i64)0 : ((" + j + " >= " + sz + ") ? " + sz + " - 1 : " + j + ")", em)->ex;
      else if (kind == "mirror") idx[d] = bindLeaf(ST::I64, "(" + j + " < 0) ? -" + j + " : ((" + j + " >= " + sz + ") ? " + sz + " - (" + j + " - " + sz + " + 2) : " + j + ")", em)->ex;
      else if (kind == "wrap") idx[d] = bindLeaf(ST::I64, "(" + j + " < 0) ? " + sz + " + " + j + " : ((" + j + " >= " + sz + ") ? " + j + " - " + sz + " : " + j + ")", em)->ex;
      else {
        idx[d] = j;
        inside += std::string(inside.empty() ? "" : " && ") + "(" + j + " >= 0) && (" + j + " < " + sz + ")";
      }
    }
    if (kind == "constant" || kind == "function") {
      Emit ei, eo;
      ei.ind = eo.ind = em.ind + 2;
      ValP vin = operandIndex(src, idx2(idx[0], idx[1]), ei);
      ValP vout = kind == "constant" ? exp(bnd.at(1), {}, eo) : applyFun(bnd.at(1), {idx2("y", "x")}, {}, eo);
      if (!typeEq(valType(vin), valType(vout))) throw Error("stencil: boundary value does not have the element type");
      ValP res = declareVars(valType(vin), em);
      em.line("if (" + inside + ") {");
      em.code += ei.code;
      em.ind += 2;
      assign(res, vin, em);
      em.ind -= 2;
      em.line("} else {");
      em.code += eo.code;
      em.ind += 2;
      assign(res, vout, em);
      em.ind -= 2;
      em.line("}");
      retSrc(res, em);
    } else {
      retSrc(operandIndex(src, idx2(idx[0], idx[1]), em), em);
    }
    body += fnHead("SrcElt", "src_at", "const Env& env, i64 y, i64 x") + em.code + "  }\n";
  }
  {
    // the stencil function over taps read from the staged tile; c is the focus inside the tile
    Emit em;
    em.ind = 4;
    const int k0 = stencilWidth(pattern) / 2;
    ValP arg = vUnit();
    for (int dy = -k0; dy <= k0; ++dy) {
      const Sx& row = pattern.at(1 + dy + k0);
      if (row.head().compare(0, 4, "unit") != 0) throw Error("stencil2d: pattern is not of rank 2");
      const int k1 = stencilWidth(row) / 2;
      ValP rv = vUnit();
      for (int dx = -k1; dx <= k1; ++dx) {
        int leaf = 0;
        struct R {
          static ValP go(Codegen& cg, const TypeP& t, int& leaf, const std::string& at, Emit& em) {
            if (t->k == Type::Unit) return vUnit();
            if (t->k == Type::Scalar) return cg.bindLeaf(t->st, "t.c" + std::to_string(leaf++) + "[" + at + "]", em);
            ValP a = go(cg, t->a, leaf, at, em);
            return vPair(a, go(cg, t->b, leaf, at, em));
          }
        };
        std::string at = "c + (" + std::to_string(dy * pw + dx) + ")";
        rv = vPair(rv, R::go(*this, srcElt, leaf, at, em));
      }
      arg = vPair(arg, rv);
    }
    ValP r = applyFun(f, {arg}, {}, em);
    if (!typeEq(valType(r), outElt)) throw Error("stencil: function result does not match the declared element type");
    body += fnHead("Elt", "apply", "const Env& env, const Tile& t, int c, i64 gy, i64 gx") + returnElt(r, em) + "  }\n";
  }
  KernelSource ks = finish(body, outElt, typeLeaves(outElt), "stencil2d.hpp", 1);
  ks.group = tileH;
  ks.words = tileW;
  return ks;
}

// Rank-3 stencils: tiles of ACC_ST_H x ACC_ST_W results in (y, x) that march along z with a
// ring of 2*HZ+1 staged planes in LDS (stencil3d.hpp).  Same generated members as for rank 2,
// with a z coordinate; apply() receives the LDS offsets of the planes z-HZ .. z+HZ.
KernelSource Codegen::stencil3d(const Sx& pattern, const TypeP& outElt, const Sx& f, const Sx& bnd,
                                const Operand& src) {
  const TypeP srcElt = src.r.elt;
  auto sleaves = typeLeaves(srcElt);
  const std::string kind = bnd.atom ? bnd.s : bnd.head();
  if (kind != "clamp" && kind != "mirror" && kind != "wrap" && kind != "constant" && kind != "function")
    throw Error("unknown stencil boundary '" + kind + "'");
  std::vector<int> halo;
  stencilHalo(pattern, 0, halo);
  if (halo.size() != 3) throw Error("stencil3d: pattern is not of rank 3");
  const int hz = halo[0], hy = halo[1], hx = halo[2];
  const int tileH = stencilTileH(hy), tileW = stencilTileW();
  const int pw = tileW + 2 * hx, ph = tileH + 2 * hy, np = 2 * hz + 1;
  std::string body;
  body += "#define ACC_ST_H " + std::to_string(tileH) + "\n";
  body += "#define ACC_ST_W " + std::to_string(tileW) + "\n";
  body += "  static constexpr int HZ = " + std::to_string(hz) + ";\n  static constexpr int HY = " + std::to_string(hy) +
          ";\n  static constexpr int HX = " + std::to_string(hx) + ";\n";
  body += "  struct SrcElt {\n" + leafDecls(sleaves, "c", false, false) + "  };\n  struct Tile {\n";
  for (size_t k = 0; k < sleaves.size(); ++k)
    body += std::string("    ") + stName(sleaves[k]) + " c" + std::to_string(k) + "[" + std::to_string(np * pw * ph) + "];\n";
  body += "  };\n  ACC_DEV void stage(Tile& t, int idx, const SrcElt& v) {\n";
  for (size_t k = 0; k < sleaves.size(); ++k)
    body += "    t.c" + std::to_string(k) + "[idx] = v.c" + std::to_string(k) + ";\n";
  body += "  }\n";
  auto retSrc = [&](const ValP& v, Emit& em) {
    auto lv = leavesOf(v);
    em.line("SrcElt r_;");
    for (size_t k = 0; k < lv.size(); ++k) em.line("r_.c" + std::to_string(k) + " = " + lv[k]->ex + ";");
    em.line("return r_;");
  };
  auto idx3 = [](const std::string& z, const std::string& y, const std::string& x) {
    return vPair(vPair(vPair(vUnit(), vLeaf(ST::I64, z)), vLeaf(ST::I64, y)), vLeaf(ST::I64, x));
  };
  {
    Emit em;
    em.ind = 4;
    ValP v = operandIndex(src, idx3("z", "y", "x"), em);
    if (!typeEq(valType(v), srcElt)) throw Error("stencil: fused producer does not return the element type");
    retSrc(v, em);
    body += fnHead("SrcElt", "src_in", "const Env& env, i64 z, i64 y, i64 x") + em.code + "  }\n";
  }
  {
    // bounded (Interpreter.hs:797-839) at an index that may lie outside on either side
    Emit em;
    em.ind = 4;
    std::vector<std::string> dims;
    shapeDims(operandShape(src, em), dims);
    const char* raw[3] = {"z", "y", "x"};
    std::string idx[3], inside;
    for (int d = 0; d < 3; ++d) {
      const std::string j = raw[d], sz = dims[d];
      if (kind == "clamp") idx[d] = bindLeaf(ST::I64, "(" + j + " < 0) ? (i64)0 : ((" + j + " >= " + sz + ") ? " + sz + " - 1 : " + j + ")", em)->ex;
      else if (kind == "mirror") idx[d] = bindLeaf(ST::I64, "(" + j + " < 0) ? -" + j + " : ((" + j + " >= " + sz + ") ? " + sz + " - (" + j + " - " + sz + " + 2) : " + j + ")", em)->ex;
      else if (kind == "wrap") idx[d] = bindLeaf(ST::I64, "(" + j + " < 0) ? " + sz + " + " + j + " : ((" + j + " >= " + sz + ") ? " + j + " - " + sz + " : " + j + ")", em)->ex;
      else {
        idx[d] = j;
        inside += std::string(inside.empty() ? "" : " && ") + "(" + j + " >= 0) && (" + j + " < " + sz + ")";
      }
    }
    if (kind == "constant" || kind == "function") {
      Emit ei, eo;
      ei.ind = eo.ind = em.ind + 2;
      ValP vin = operandIndex(src, idx3(idx[0], idx[1], idx[2]), ei);
      ValP vout = kind == "constant" ? exp(bnd.at(1), {}, eo) : applyFun(bnd.at(1), {idx3("z", "y", "x")}, {}, eo);
      if (!typeEq(valType(vin), valType(vout))) throw Error("stencil: boundary value does not have the element type");
      ValP res = declareVars(valType(vin), em);
      em.line("if (" + inside + ") {");
      em.code += ei.code;
      em.ind += 2;
      assign(res, vin, em);
      em.ind -= 2;
      em.line("} else {");
      em.code += eo.code;
      em.ind += 2;
      assign(res, vout, em);
      em.ind -= 2;
      em.line("}");
      retSrc(res, em);
    } else {
      retSrc(operandIndex(src, idx3(idx[0], idx[1], idx[2]), em), em);
    }
    body += fnHead("SrcElt", "src_at", "const Env& env, i64 z, i64 y, i64 x") + em.code + "  }\n";
  }
  {
    // the stencil function over taps read from the staged planes; c is the focus inside a
    // plane, pl[dz + HZ] the LDS offset of plane z + dz
    Emit em;
    em.ind = 4;
    ValP arg = vUnit();
    for (int dz = -hz; dz <= hz; ++dz) {
      const Sx& plane = pattern.at(1 + dz + hz);
      const int k1 = stencilWidth(plane) / 2;
      ValP pv = vUnit();
      for (int dy = -k1; dy <= k1; ++dy) {
        const Sx& row = plane.at(1 + dy + k1);
        if (row.head().compare(0, 4, "unit") != 0) throw Error("stencil3d: pattern is not of rank 3");
        const int k2 = stencilWidth(row) / 2;
        ValP rv = vUnit();
        for (int dx = -k2; dx <= k2; ++dx) {
          int leaf = 0;
          struct R {
            static ValP go(Codegen& cg, const TypeP& t, int& leaf, const std::string& at, Emit& em) {
              if (t->k == Type::Unit) return vUnit();
              if (t->k == Type::Scalar) return cg.bindLeaf(t->st, "t.c" + std::to_string(leaf++) + "[" + at + "]", em);
              ValP a = go(cg, t->a, leaf, at, em);
              return vPair(a, go(cg, t->b, leaf, at, em));
            }
          };
          std::string at = "pl[" + std::to_string(dz + hz) + "] + c + (" + std::to_string(dy * pw + dx) + ")";
          rv = vPair(rv, R::go(*this, srcElt, leaf, at, em));
        }
        pv = vPair(pv, rv);
      }
      arg = vPair(arg, pv);
    }
    ValP r = applyFun(f, {arg}, {}, em);
    if (!typeEq(valType(r), outElt)) throw Error("stencil: function result does not match the declared element type");
    body += fnHead("Elt", "apply", "const Env& env, const Tile& t, const int* pl, int c") + returnElt(r, em) + "  }\n";
  }
  KernelSource ks = finish(body, outElt, typeLeaves(outElt), "stencil3d.hpp", 1);
  ks.group = tileH;
  ks.words = tileW;
  ks.block = np;  // planes in the ring
  return ks;
}

KernelSource Codegen::scalarKernel(const Sx& e) {
  Emit em;
  em.ind = 4;
  ValP r = exp(e, {}, em);
  TypeP t = valType(r);
  std::string body = streamHead("Elt", "produce", "const Env& env, i64 i") + returnElt(r, em) + "  }\n";
  return finish(body, t, typeLeaves(t), "map.hpp", 1);
}

}  // namespace acchip
