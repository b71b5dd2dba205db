#include "exec.hpp"

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>

namespace acchip {

// ------------------------------------------------------------------------------------
// array types

static ATyP atUnit() {
  static ATyP u = std::make_shared<ATy>();
  return u;
}
static ATyP atArr(const ArrayR& r) {
  auto t = std::make_shared<ATy>();
  t->k = ATy::Arr;
  t->r = r;
  return t;
}
static ATyP atPair(ATyP a, ATyP b) {
  auto t = std::make_shared<ATy>();
  t->k = ATy::Pair;
  t->a = std::move(a);
  t->b = std::move(b);
  return t;
}
static const ArrayR& oneArray(const ATyP& t, const char* what) {
  if (t->k != ATy::Arr) throw Error(std::string(what) + ": expected a single array");
  return t->r;
}

static AValP avUnit() {
  static AValP u = std::make_shared<AVal>();
  return u;
}
static AValP avArr(DArrayP a) {
  auto v = std::make_shared<AVal>();
  v->k = AVal::Arr;
  v->arr = std::move(a);
  return v;
}
static AValP avPair(AValP a, AValP b) {
  auto v = std::make_shared<AVal>();
  v->k = AVal::Pair;
  v->a = std::move(a);
  v->b = std::move(b);
  return v;
}

static ATyP lhsType(const Sx& lhs) {
  if (lhs.is("single")) return atArr(parseArrayR(lhs.at(1)));
  if (lhs.is("wild")) {
    const Sx& t = lhs.at(1);
    if (t.isAtom("unit")) return atUnit();
    if (t.is("array")) return atArr(parseArrayR(t));
    if (t.is("pair")) {
      Sx l, r;
      l.kids = {Sx{true, "wild", {}}, t.at(1)};
      r.kids = {Sx{true, "wild", {}}, t.at(2)};
      return atPair(lhsType(l), lhsType(r));
    }
    throw Error("malformed array left-hand side " + lhs.str());
  }
  if (lhs.is("pair")) return atPair(lhsType(lhs.at(1)), lhsType(lhs.at(2)));
  throw Error("malformed array left-hand side " + lhs.str());
}

static void pushTypes(const Sx& lhs, std::vector<ArrayR>& tenv) {
  if (lhs.is("single")) tenv.push_back(parseArrayR(lhs.at(1)));
  else if (lhs.is("pair")) {
    pushTypes(lhs.at(1), tenv);
    pushTypes(lhs.at(2), tenv);
  }
}
static int lhsCount(const Sx& lhs) {
  if (lhs.is("single")) return 1;
  if (lhs.is("pair")) return lhsCount(lhs.at(1)) + lhsCount(lhs.at(2));
  return 0;
}
static void pushVals(const Sx& lhs, const AValP& v, std::vector<DArrayP>& aenv) {
  if (lhs.is("single")) {
    if (v->k != AVal::Arr) throw Error("array left-hand side binds one array but the value is a tuple");
    aenv.push_back(v->arr);
  } else if (lhs.is("pair")) {
    if (v->k != AVal::Pair) throw Error("array left-hand side is a pair but the value is not");
    pushVals(lhs.at(1), v->a, aenv);
    pushVals(lhs.at(2), v->b, aenv);
  }
}

// ------------------------------------------------------------------------------------
// host evaluation of simple scalar expressions (extents, predicates)

static HValP hvUnit() {
  static HValP u = std::make_shared<HVal>();
  return u;
}
static HValP hvInt(ST st, int64_t i) {
  auto v = std::make_shared<HVal>();
  v->k = HVal::Leaf;
  v->st = st;
  v->i = i;
  return v;
}
static HValP hvPair(HValP a, HValP b) {
  auto v = std::make_shared<HVal>();
  v->k = HVal::Pair;
  v->a = std::move(a);
  v->b = std::move(b);
  return v;
}

static bool hostPrimOk(const std::string& n) {
  static const char* ok[] = {"add", "sub", "mul", "min", "max", "quot", "rem", "idiv", "mod", "lt", "gt", "lte",
                             "gte", "eq", "neq", "land", "lor", "lnot", "fromintegral", "neg", "abs"};
  for (const char* o : ok)
    if (n == o) return true;
  return false;
}

// thrown by hostEval when it needs the contents of an array the host does not know
struct HostUnknown {};

// structural test: can hostEval handle this term without touching array contents?  With
// `scalars`, reading a rank-0 array is allowed too (it succeeds at run time when the host
// knows that array's value).
static bool hostSupported(const Sx& e, bool scalars = false) {
  if (e.isAtom("nil")) return true;
  if (e.atom) return false;
  const std::string& h = e.head();
  if (h == "var" || h == "shape") return true;
  if (scalars && (h == "index" || h == "linearindex")) return hostSupported(e.at(2), true);
  if (h == "const") return isST(e.at(1)) && !stIsFloat(parseST(e.at(1)));
  if (h == "let") return hostSupported(e.at(2), scalars) && hostSupported(e.at(3), scalars);
  if (h == "pair") return hostSupported(e.at(1), scalars) && hostSupported(e.at(2), scalars);
  if (h == "cond") return hostSupported(e.at(1), scalars) && hostSupported(e.at(2), scalars) && hostSupported(e.at(3), scalars);
  if (h == "toindex" || h == "fromindex") return hostSupported(e.at(2), scalars) && hostSupported(e.at(3), scalars);
  if (h == "indexslice" || h == "indexfull") return hostSupported(e.at(2), scalars) && hostSupported(e.at(3), scalars);
  if (h == "shapesize") return hostSupported(e.at(2), scalars);
  if (h == "prim") {
    if (!hostPrimOk(e.at(1).s)) return false;
    for (size_t k = 2; k + 1 < e.size(); ++k)
      if (!isST(e.at(k)) || stIsFloat(parseST(e.at(k)))) return false;
    return hostSupported(e.at(e.size() - 1), scalars);
  }
  return false;
}

static int64_t wrapTo(ST st, int64_t v) {
  switch (st) {
    case ST::I8: return (int8_t)v;
    case ST::I16: return (int16_t)v;
    case ST::I32: return (int32_t)v;
    case ST::U8: return (uint8_t)v;
    case ST::U16: return (uint16_t)v;
    case ST::U32: return (uint32_t)v;
    default: return v;
  }
}

static void hPush(const Sx& lhs, const HValP& v, std::vector<HValP>& env) {
  if (lhs.is("single")) env.push_back(v);
  else if (lhs.is("pair")) {
    if (v->k != HVal::Pair) throw Error("host evaluation: left-hand side does not match the value");
    hPush(lhs.at(1), v->a, env);
    hPush(lhs.at(2), v->b, env);
  }
}

static void hDims(const HValP& sh, std::vector<int64_t>& out) {
  if (sh->k == HVal::Unit) return;
  if (sh->k != HVal::Pair || sh->b->k != HVal::Leaf) throw Error("host evaluation: expected a shape");
  hDims(sh->a, out);
  out.push_back(sh->b->i);
}
static void hLeaves(const HValP& v, std::vector<int64_t>& out) {
  if (v->k == HVal::Leaf) out.push_back(v->i);
  else if (v->k == HVal::Pair) {
    hLeaves(v->a, out);
    hLeaves(v->b, out);
  }
}
static HValP hShape(const std::vector<int64_t>& d) {
  HValP v = hvUnit();
  for (int64_t x : d) v = hvPair(v, hvInt(ST::I64, x));
  return v;
}

static HValP hostEval(const Sx& e, std::vector<HValP> env, const std::vector<DArrayP>& aenv) {
  if (e.isAtom("nil")) return hvUnit();
  const std::string& h = e.head();
  if (h == "var") {
    size_t ix = (size_t)e.at(1).asInt();
    if (ix >= env.size()) throw Error("host evaluation: scalar variable out of range");
    return env[env.size() - 1 - ix];
  }
  if (h == "shape") {
    size_t ix = (size_t)e.at(1).asInt();
    if (ix >= aenv.size()) throw Error("host evaluation: array variable out of range");
    return hShape(aenv[aenv.size() - 1 - ix]->shape);
  }
  if (h == "index" || h == "linearindex") {
    size_t ix = (size_t)e.at(1).asInt();
    if (ix >= aenv.size()) throw Error("host evaluation: array variable out of range");
    const DArrayP& a = aenv[aenv.size() - 1 - ix];
    if (!a->hostKnown) throw HostUnknown();
    auto leaves = typeLeaves(a->r.elt);
    return hvInt(leaves.at(0), a->hostValue);
  }
  if (h == "const") {
    ST st = parseST(e.at(1));
    const std::string& tok = e.at(2).s;
    int64_t v = (!tok.empty() && tok[0] == '-') ? std::strtoll(tok.c_str(), nullptr, 0)
                                                 : (int64_t)std::strtoull(tok.c_str(), nullptr, 0);
    return hvInt(st, wrapTo(st, v));
  }
  if (h == "let") {
    HValP v = hostEval(e.at(2), env, aenv);
    hPush(e.at(1), v, env);
    return hostEval(e.at(3), env, aenv);
  }
  if (h == "pair") {
    HValP a = hostEval(e.at(1), env, aenv);
    return hvPair(a, hostEval(e.at(2), env, aenv));
  }
  if (h == "cond") {
    HValP c = hostEval(e.at(1), env, aenv);
    return hostEval(c->i != 0 ? e.at(2) : e.at(3), env, aenv);
  }
  if (h == "toindex") {
    std::vector<int64_t> d, i;
    hDims(hostEval(e.at(2), env, aenv), d);
    hDims(hostEval(e.at(3), env, aenv), i);
    if (d.size() != i.size()) throw Error("host evaluation: toIndex rank mismatch");
    int64_t lin = 0;
    for (size_t k = 0; k < d.size(); ++k) lin = lin * d[k] + i[k];
    return hvInt(ST::I64, lin);
  }
  if (h == "fromindex") {
    std::vector<int64_t> d;
    hDims(hostEval(e.at(2), env, aenv), d);
    int64_t cur = hostEval(e.at(3), env, aenv)->i;
    std::vector<int64_t> ix(d.size());
    for (size_t k = d.size(); k-- > 1;) {
      if (d[k] == 0) throw Error("host evaluation: fromIndex into an empty shape");
      ix[k] = cur % d[k];
      cur /= d[k];
    }
    if (!d.empty()) ix[0] = cur;
    return hShape(ix);
  }
  if (h == "shapesize") {
    std::vector<int64_t> d;
    hDims(hostEval(e.at(2), env, aenv), d);
    int64_t n = 1;
    for (int64_t x : d) {
      if (x <= 0) return hvInt(ST::I64, 0);
      n *= x;
    }
    return hvInt(ST::I64, n);
  }
  if (h == "indexslice" || h == "indexfull") {
    const Sx& spec = e.at(1);
    HValP slix = hostEval(e.at(2), env, aenv), sh = hostEval(e.at(3), env, aenv);
    struct R {
      static HValP restrict_(const Sx& spec, size_t k, const HValP& slix, const HValP& sh) {
        if (k == spec.size()) return hvUnit();
        if (slix->k != HVal::Pair || sh->k != HVal::Pair) throw Error("host evaluation: malformed slice");
        HValP rest = restrict_(spec, k + 1, slix->a, sh->a);
        return spec.at(k).isAtom("all") ? hvPair(rest, sh->b) : rest;
      }
      static HValP extend(const Sx& spec, size_t k, const HValP& slix, const HValP& sl) {
        if (k == spec.size()) return hvUnit();
        if (slix->k != HVal::Pair) throw Error("host evaluation: malformed slice");
        if (spec.at(k).isAtom("all")) {
          if (sl->k != HVal::Pair) throw Error("host evaluation: malformed slice");
          return hvPair(extend(spec, k + 1, slix->a, sl->a), sl->b);
        }
        return hvPair(extend(spec, k + 1, slix->a, sl), slix->b);
      }
    };
    return h == "indexslice" ? R::restrict_(spec, 0, slix, sh) : R::extend(spec, 0, slix, sh);
  }
  if (h == "prim") {
    const std::string& n = e.at(1).s;
    HValP arg = hostEval(e.at(e.size() - 1), env, aenv);
    ST st = e.size() > 3 ? parseST(e.at(2)) : ST::U8;
    auto B = [](bool b) { return hvInt(ST::U8, b ? 1 : 0); };
    if (n == "lnot") return B(arg->i == 0);
    if (n == "neg") return hvInt(st, wrapTo(st, (int64_t)(0 - (uint64_t)arg->i)));
    if (n == "abs") return hvInt(st, wrapTo(st, arg->i < 0 ? (int64_t)(0 - (uint64_t)arg->i) : arg->i));
    if (n == "fromintegral") {
      ST to = parseST(e.at(3));
      return hvInt(to, wrapTo(to, arg->i));
    }
    if (arg->k != HVal::Pair) throw Error("host evaluation: primitive expects a pair");
    int64_t a = arg->a->i, b = arg->b->i;
    bool uns = !stIsSigned(st) && stSize(st) == 8;
    uint64_t ua = (uint64_t)a, ub = (uint64_t)b;
    if (n == "add") return hvInt(st, wrapTo(st, (int64_t)(ua + ub)));
    if (n == "sub") return hvInt(st, wrapTo(st, (int64_t)(ua - ub)));
    if (n == "mul") return hvInt(st, wrapTo(st, (int64_t)(ua * ub)));
    auto le = [&](int64_t x, int64_t y) { return uns ? (uint64_t)x <= (uint64_t)y : x <= y; };
    auto ltf = [&](int64_t x, int64_t y) { return uns ? (uint64_t)x < (uint64_t)y : x < y; };
    if (n == "min") return hvInt(st, le(a, b) ? a : b);
    if (n == "max") return hvInt(st, le(a, b) ? b : a);
    if (n == "lt") return B(ltf(a, b));
    if (n == "gt") return B(ltf(b, a));
    if (n == "lte") return B(le(a, b));
    if (n == "gte") return B(le(b, a));
    if (n == "eq") return B(a == b);
    if (n == "neq") return B(a != b);
    if (n == "land") return B(a != 0 && b != 0);
    if (n == "lor") return B(a != 0 || b != 0);
    if (b == 0) throw Error("divide by zero");
    if (uns) {
      if (n == "quot" || n == "idiv") return hvInt(st, (int64_t)(ua / ub));
      return hvInt(st, (int64_t)(ua % ub));
    }
    // minBound `quot` (-1) overflows: the reference raises (GHC.Real overflowError), C would trap
    if (b == -1) {
      if (n == "rem" || n == "mod") return hvInt(st, 0);
      const int64_t lowest = stSize(st) == 8 ? INT64_MIN : -((int64_t)1 << (8 * stSize(st) - 1));
      if (a == lowest) throw Error("arithmetic overflow");
      return hvInt(st, wrapTo(st, (int64_t)(0 - (uint64_t)a)));
    }
    int64_t q = a / b, r = a % b;
    if (n == "quot") return hvInt(st, wrapTo(st, q));
    if (n == "rem") return hvInt(st, wrapTo(st, r));
    bool adj = r != 0 && ((r < 0) != (b < 0));
    if (n == "idiv") return hvInt(st, wrapTo(st, adj ? q - 1 : q));
    if (n == "mod") return hvInt(st, wrapTo(st, adj ? r + b : r));
  }
  throw Error("host evaluation: unsupported expression '" + h + "'");
}

// ------------------------------------------------------------------------------------
// preparation (type inference + code generation for every node)

Program::Program(Context& ctx, const char* text, size_t len) : ctx_(ctx) {
  root_ = parseSx(text, len);
  const Sx* f = &root_;
  // (acchip-ir VERSION afun): the version of the term grammar; a bare term is read as version 1
  if (f->is("acchip-ir")) {
    if (f->size() != 3 || !f->at(1).atom) throw Error("malformed program header");
    if (f->at(1).s != "1") throw Error("unsupported wire format version " + f->at(1).s + " (this library reads version 1)");
    f = &f->at(2);
  }
  TEnv tenv;
  while (f->is("alam")) {
    argTypes.push_back(lhsType(f->at(1)));
    pushTypes(f->at(1), tenv);
    lams_.push_back(f);
    f = &f->at(2);
  }
  body_ = f;
  resultType = prepare(*body_, tenv);
  // the kernels were handed to the compiler as they were generated; collect them (and what the
  // compiler had to say) before the program is handed out
  for (auto& kv : plans_) {
    ctx_.wait(kv.second.k);
    ctx_.wait(kv.second.k2);
    ctx_.wait(kv.second.k3);
    for (auto& sk : kv.second.scalarKernels) ctx_.wait(sk.second);
  }
  // a program that is one scan can be run without allocating (runInto): its code objects are
  // loaded now, so that no launch of it has set-up work left
  if (ctx_.hasDevice() && (body_->is("scan") || body_->is("scan'"))) {
    const Plan& plan = plans_.at(body_);
    ctx_.preload(plan.k, {"acc_scan", "acc_scan_rows"});
    ctx_.preload(plan.k2, {"acc_scan", "acc_scan_rows"});
    if (plan.k3) ctx_.preload(plan.k3, {"acc_scan_pipe", "acc_scan_pipe_tail"});
  }
}

std::vector<std::string> Program::kernelKeys() const {
  std::vector<std::string> keys;
  for (auto& kv : plans_) {
    for (const KernelP& k : {kv.second.k, kv.second.k2, kv.second.k3})
      if (k) keys.push_back(k->hash);
    for (auto& sk : kv.second.scalarKernels)
      if (sk.second) keys.push_back(sk.second->hash);
  }
  std::sort(keys.begin(), keys.end());
  keys.erase(std::unique(keys.begin(), keys.end()), keys.end());
  return keys;
}

std::vector<ArrayR> Program::aenvOf(const TEnv& tenv) {
  std::vector<ArrayR> a(tenv.rbegin(), tenv.rend());  // index 0 = most recently bound
  return a;
}

Operand Program::operandOf(const Sx& o, Codegen& cg, TEnv& tenv, Plan& plan) {
  Operand op;
  if (o.is("delayed")) {
    op.delayed = true;
    op.r = parseArrayR(o.at(1));
    op.extent = o.at(2);
    op.indexD = o.at(3);
    op.linearD = o.at(4);
    prepareHostExp(o.at(2), tenv, plan);
    return op;
  }
  if (o.is("avar")) {
    size_t ix = (size_t)o.at(1).asInt();
    if (ix >= tenv.size()) throw Error("array variable index out of range");
    op.r = tenv[tenv.size() - 1 - ix];
    op.slot = "a" + std::to_string(ix);
    return op;
  }
  // a nested manifest term: evaluated to a temporary before this node's kernel runs
  ATyP t = prepare(o, tenv);
  op.r = oneArray(t, "array operand");
  op.slot = cg.addTemp(op.r);
  plan.temps.push_back(&o);
  return op;
}

void Program::prepareHostExp(const Sx& e, TEnv& tenv, Plan& plan) {
  if (hostSupported(e)) return;
  Codegen cg(aenvOf(tenv));
  plan.scalarKernels[&e] = ctx_.kernel(cg.scalarKernel(e));
}

ATyP Program::prepareFun(const Sx& f, TEnv& tenv, std::vector<ATyP>* params) {
  if (f.is("alam")) {
    if (params) params->push_back(lhsType(f.at(1)));
    size_t mark = tenv.size();
    pushTypes(f.at(1), tenv);
    ATyP r = prepareFun(f.at(2), tenv, params);
    tenv.resize(mark);
    return r;
  }
  return prepare(f, tenv);
}

ATyP Program::prepare(const Sx& n, TEnv& tenv) {
  if (n.isAtom("anil")) return atUnit();
  if (n.atom) throw Error("unexpected atom '" + n.s + "' in array term");
  const std::string& h = n.head();
  auto seedOf = [&](const Sx& s) -> const Sx* {
    if (s.isAtom("nothing")) return nullptr;
    if (s.is("just")) return &s.at(1);
    throw Error("expected (just e) or nothing, got " + s.str());
  };

  if (h == "avar") {
    size_t ix = (size_t)n.at(1).asInt();
    if (ix >= tenv.size()) throw Error("array variable index out of range");
    return atArr(tenv[tenv.size() - 1 - ix]);
  }
  if (h == "alet") {
    prepare(n.at(2), tenv);
    size_t mark = tenv.size();
    pushTypes(n.at(1), tenv);
    ATyP r = prepare(n.at(3), tenv);
    tenv.resize(mark);
    return r;
  }
  if (h == "apair") {
    ATyP a = prepare(n.at(1), tenv);
    return atPair(a, prepare(n.at(2), tenv));
  }
  if (h == "apply") {
    prepare(n.at(2), tenv);
    return prepareFun(n.at(1), tenv, nullptr);
  }
  if (h == "atrace") {  // (atrace hex-of-message as bs): Interpreter.hs:215
    prepare(n.at(2), tenv);
    return prepare(n.at(3), tenv);
  }
  if (h == "aforeign") {  // (aforeign hex-of-name afun acc): the pure fallback, closed (Interpreter.hs:217)
    prepare(n.at(3), tenv);
    TEnv empty;
    return prepareFun(n.at(2), empty, nullptr);
  }
  if (h == "acond") {
    Plan& plan = plans_[&n];
    prepareHostExp(n.at(1), tenv, plan);
    ATyP a = prepare(n.at(2), tenv);
    prepare(n.at(3), tenv);
    return a;
  }
  if (h == "awhile") {
    ATyP t = prepare(n.at(3), tenv);
    prepareFun(n.at(1), tenv, nullptr);
    prepareFun(n.at(2), tenv, nullptr);
    return t;
  }
  if (h == "use") return atArr(parseArrayR(n.at(1)));
  if (h == "delayed") throw Error("expected manifest array");  // Interpreter.hs:180

  {
    // a node is planned once, however many variants of its consumer ask for it as an operand
    // (its own nested operands would otherwise be listed, and evaluated, once per request)
    auto known = plans_.find(&n);
    if (known != plans_.end() && known->second.ty) return known->second.ty;
  }
  Plan& plan = plans_[&n];
  Codegen cg(aenvOf(tenv));
  cg.fastPermuteConst = ctx_.flag(Context::kFastPermuteConst);
  auto done = [&](const ArrayR& r) {
    plan.ty = atArr(r);
    return plan.ty;
  };

  if (h == "unit") {
    ArrayR r;
    r.rank = 0;
    r.elt = parseType(n.at(1));
    plan.k = ctx_.kernel(cg.scalarKernel(n.at(2)));
    return done(r);
  }
  if (h == "reshape") {
    prepareHostExp(n.at(2), tenv, plan);
    ATyP t = prepare(n.at(3), tenv);
    ArrayR r = oneArray(t, "reshape");
    r.rank = (int)n.at(1).asInt();
    return done(r);
  }
  if (h == "generate") {
    ArrayR r = parseArrayR(n.at(1));
    prepareHostExp(n.at(2), tenv, plan);
    plan.k = ctx_.kernel(cg.generate(r, n.at(3)));
    return done(r);
  }
  if (h == "transform") {
    ArrayR r = parseArrayR(n.at(1));
    prepareHostExp(n.at(2), tenv, plan);
    Operand src = operandOf(n.at(5), cg, tenv, plan);
    plan.k = ctx_.kernel(cg.backpermute(r.rank, n.at(3), &n.at(4), r.elt, src));
    return done(r);
  }
  if (h == "backpermute") {
    int rank = (int)n.at(1).asInt();
    prepareHostExp(n.at(2), tenv, plan);
    Operand src = operandOf(n.at(4), cg, tenv, plan);
    ArrayR r;
    r.rank = rank;
    r.elt = src.r.elt;
    plan.k = ctx_.kernel(cg.backpermute(rank, n.at(3), nullptr, r.elt, src));
    return done(r);
  }
  if (h == "map") {
    if (n.at(3).is("scan") && ctx_.knobs.scan_post != 0) {
      // map g (scan f z xs) with the scan written out as an operand (not let-bound: nobody else
      // reads it): the scan applies g as it stores, where g reads no arrays
      Plan trial;
      try {
        prepareScan(n.at(3), tenv, trial, &n.at(2), parseType(n.at(1)));
        trial.mode = "scan";
        plan = std::move(trial);
        return plan.ty;
      } catch (const ScanPostNotFusable&) {
      }
    }
    Operand src = operandOf(n.at(3), cg, tenv, plan);
    ArrayR r;
    r.rank = src.r.rank;
    r.elt = parseType(n.at(1));
    plan.k = ctx_.kernel(cg.map(r.elt, &n.at(2), src));
    return done(r);
  }
  if (h == "zipwith") {
    Operand a = operandOf(n.at(3), cg, tenv, plan);
    Operand b = operandOf(n.at(4), cg, tenv, plan);
    if (a.r.rank != b.r.rank) throw Error("zipWith: operands of different rank");
    ArrayR r;
    r.rank = a.r.rank;
    r.elt = parseType(n.at(1));
    plan.k = ctx_.kernel(cg.zipWith(r.elt, n.at(2), a, b, r.rank));
    return done(r);
  }
  if (h == "fold") {
    Operand src = operandOf(n.at(3), cg, tenv, plan);
    if (src.r.rank < 1) throw Error("fold: operand must have rank >= 1");
    plan.k = ctx_.kernel(cg.fold(n.at(1), seedOf(n.at(2)), src));
    ArrayR r;
    r.rank = src.r.rank - 1;
    r.elt = src.r.elt;
    return done(r);
  }
  if (h == "permute") {
    // (permute f defaults p source); the defaults operand is always manifest (Fusion.hs:213)
    ATyP dt = prepare(n.at(2), tenv);
    ArrayR dr = oneArray(dt, "permute defaults");
    Operand src = operandOf(n.at(4), cg, tenv, plan);
    // defaults that are one constant everywhere (`generate sh (\_ -> c)`, what `fill` becomes)
    const Sx* freshInit = nullptr;
    if (n.at(2).is("generate") && n.at(2).at(3).is("lam") && n.at(2).at(3).at(2).is("const")) freshInit = &n.at(2).at(3).at(2);
    KernelSource ks = cg.permute(n.at(1), dr, n.at(3), src, freshInit);
    plan.mode = ks.permuteMode;
    plan.k = ctx_.kernel(ks);
    return done(dr);
  }
  if (h == "stencil" || h == "stencil2") {
    const bool two = h == "stencil2";
    std::vector<Sx> pats, bnds;
    std::vector<Operand> srcs;
    TypeP outElt;
    const Sx* f;
    if (!two) {
      pats = {n.at(1)};
      outElt = parseType(n.at(2));
      f = &n.at(3);
      bnds = {n.at(4)};
      srcs.push_back(operandOf(n.at(5), cg, tenv, plan));
    } else {
      // (looked up before the lists are built: an operand that is missing throws here, not in the middle of a list)
      const Sx &p0 = n.at(1), &p1 = n.at(2), &b0 = n.at(5), &b1 = n.at(7);
      pats = {p0, p1};
      outElt = parseType(n.at(3));
      f = &n.at(4);
      bnds = {b0, b1};
      srcs.push_back(operandOf(n.at(6), cg, tenv, plan));
      srcs.push_back(operandOf(n.at(8), cg, tenv, plan));
      if (srcs[0].r.rank != srcs[1].r.rank) throw Error("stencil2: operands of different rank");
    }
    // the LDS-tiled skeletons move 32-bit and 128-bit words; SIMD vector leaves go the generic way
    bool simd = false;
    for (ST st : typeLeaves(outElt)) simd = simd || stIsVec(st);
    for (ST st : typeLeaves(srcs[0].r.elt)) simd = simd || stIsVec(st);
    if (simd) {
      plan.k = ctx_.kernel(cg.stencil(pats, outElt, *f, bnds, srcs));
    } else if (!two && srcs[0].r.rank == 2 && !ctx_.knobs.stencil_no2d) {
      plan.k = ctx_.kernel(cg.stencil2d(pats[0], outElt, *f, bnds[0], srcs[0]));
      plan.mode = "lds2d";
    } else if (!two && srcs[0].r.rank == 3 && !ctx_.knobs.stencil_no3d) {
      plan.k = ctx_.kernel(cg.stencil3d(pats[0], outElt, *f, bnds[0], srcs[0]));
      plan.mode = "lds3d";
    } else {
      plan.k = ctx_.kernel(cg.stencil(pats, outElt, *f, bnds, srcs));
    }
    ArrayR r;
    r.rank = srcs[0].r.rank;
    r.elt = outElt;
    return done(r);
  }
  if (h == "foldseg") {
    ST ity = parseST(n.at(1));
    if (!stIsInt(ity)) throw Error("foldSeg: segment descriptor must be integral");
    Operand src = operandOf(n.at(4), cg, tenv, plan);
    Operand seg = operandOf(n.at(5), cg, tenv, plan);
    if (src.r.rank < 1 || seg.r.rank != 1) throw Error("foldSeg: operands have the wrong rank");
    plan.k = ctx_.kernel(cg.foldSeg(n.at(2), seedOf(n.at(3)), src, seg, ity));
    return done(src.r);
  }
  if (h == "scan" || h == "scan'") return prepareScan(n, tenv, plan, nullptr, nullptr);
  throw Error("unsupported array term '" + h + "'");
}

// (scan dir f seed operand) and (scan' ...), optionally with the function of a `map` around it
// applied to the results as they are stored (post; not for scan', whose results are a pair)
ATyP Program::prepareScan(const Sx& n, TEnv& tenv, Plan& plan, const Sx* post, const TypeP& postElt) {
  const bool prime = n.is("scan'");
  auto seedOf = [&](const Sx& s) -> const Sx* {
    if (s.isAtom("nothing")) return nullptr;
    if (s.is("just")) return &s.at(1);
    throw Error("expected (just e) or nothing, got " + s.str());
  };
  const std::string& dir = n.at(1).s;
  if (dir != "l" && dir != "r") throw Error("scan direction must be l or r");
  Codegen cg(aenvOf(tenv));
  Operand src = operandOf(n.at(4), cg, tenv, plan);
  if (src.r.rank < 1) throw Error("scan: operand must have rank >= 1");
  const Sx* z = prime ? &n.at(3) : seedOf(n.at(3));
  int kind = prime ? 2 : (z ? 1 : 0);
  plan.k = ctx_.kernel(cg.scan(n.at(2), z, src, dir == "r", kind, 0, post, postElt));
  {
    // the same scan with small tiles, chosen at launch for short rows
    Codegen cgs(aenvOf(tenv));
    Plan scratch;
    Operand srcS = operandOf(n.at(4), cgs, tenv, scratch);
    plan.k2 = ctx_.kernel(cgs.scan(n.at(2), z, srcS, dir == "r", kind, 1, post, postElt));
  }
  if (!post && Codegen::scanPipeable(src, dir == "r")) {
    // and as a pipeline in persistent workgroups, chosen at launch for long rows
    Codegen cgp(aenvOf(tenv));
    Plan scratch;
    Operand srcP = operandOf(n.at(4), cgp, tenv, scratch);
    try {
      plan.k3 = ctx_.kernel(cgp.scan(n.at(2), z, srcP, dir == "r", kind, 2));
    } catch (const ScanNotPipeable&) {
    }
  }
  if (prime) {
    ArrayR tr = src.r;
    tr.rank -= 1;
    plan.ty = atPair(atArr(src.r), atArr(tr));
    return plan.ty;
  }
  ArrayR r = src.r;
  if (post) r.elt = postElt;
  plan.ty = atArr(r);
  return plan.ty;
}

// ------------------------------------------------------------------------------------
// execution

DArrayP Program::alloc(const ArrayR& r, const std::vector<int64_t>& shape) {
  if (noAlloc_) {
    if (destNext_ >= dest_.size())
      throw Error("this program needs device memory beyond its results, which acchip_execute_into does not provide");
    const DArrayP& d = dest_[destNext_++];
    if (d->r.rank != r.rank || !typeEq(d->r.elt, r.elt))
      throw Error("result array has the wrong type: the program yields rank " + std::to_string(r.rank) + ", " +
                  typeStr(r.elt));
    if (d->shape != shape) {
      std::string want;
      for (int64_t x : shape) want += (want.empty() ? "" : " x ") + std::to_string(x);
      throw Error("result array has the wrong extents: the program yields " + (want.empty() ? std::string("a scalar") : want));
    }
    return d;
  }
  auto a = std::make_shared<DArray>();
  a->r = r;
  a->shape = shape;
  int64_t n = a->size();
  for (ST st : typeLeaves(r.elt)) {
    auto b = std::make_shared<Buffer>();
    b->ctx = ctx_.shared_from_this();
    b->bytes = (size_t)n * stSize(st);
    b->p = ctx_.malloc(b->bytes);
    if (!b->p) throw Error("Remote memory exhausted");  // Array/Remote/LRU.hs:250-341
    b->owned = true;
    a->bufs.push_back(b);
  }
  return a;
}

void Program::packOut(std::vector<uint64_t>& args, const DArray& a) {
  args.push_back(0);
  for (auto& b : a.bufs) args.push_back((uint64_t)(uintptr_t)b->p);
}

// A scalar the host computed (`unit` of index arithmetic) reaches the device only when
// something there reads it: a kernel that takes the array, a copy, or the caller.
void Program::materialize(DArray& a) {
  if (!a.hostKnown || a.onDevice) return;
  if (noAlloc_) throw Error("an argument of acchip_execute_into has not been written to the device yet");
  auto leaves = typeLeaves(a.r.elt);
  void* p = a.bufs.at(0)->p;
  const uint64_t v = (uint64_t)a.hostValue;
  hipStream_t st = ctx_.stream();
  switch (stSize(leaves.at(0))) {
    case 1: hipCheck(hipMemsetD8Async(p, (unsigned char)v, 1, st), "hipMemsetD8Async"); break;
    case 2: hipCheck(hipMemsetD16Async(p, (unsigned short)v, 1, st), "hipMemsetD16Async"); break;
    case 4: hipCheck(hipMemsetD32Async(p, (int)(uint32_t)v, 1, st), "hipMemsetD32Async"); break;
    default:
      hipCheck(hipMemsetD32Async(p, (int)(uint32_t)v, 1, st), "hipMemsetD32Async");
      hipCheck(hipMemsetD32Async(static_cast<char*>(p) + 4, (int)(uint32_t)(v >> 32), 1, st), "hipMemsetD32Async");
  }
  a.onDevice = true;
}

void Program::materializeAll(const AValP& v) {
  if (!v) return;
  if (v->k == AVal::Arr) materialize(*v->arr);
  else if (v->k == AVal::Pair) {
    materializeAll(v->a);
    materializeAll(v->b);
  }
}

std::vector<uint64_t> Program::packArgs(const KernelSource& ks, const AEnv& aenv, const std::vector<DArrayP>& temps,
                                        const std::vector<int64_t>& outShape) {
  std::vector<uint64_t> args;
  args.push_back(0);
  for (const ArraySlot& s : ks.arrays) {
    if (s.name == "out") {
      if ((int)outShape.size() != s.r.rank) throw Error("internal: result rank does not match the generated kernel");
      for (int64_t d : outShape) args.push_back((uint64_t)d);
      continue;
    }
    DArrayP a;
    if (s.temp) {
      if (s.index >= (int)temps.size()) throw Error("internal: missing temporary operand");
      a = temps[s.index];
    } else {
      if (s.index >= (int)aenv.size()) throw Error("internal: array variable out of range at launch");
      a = aenv[aenv.size() - 1 - s.index];
    }
    if (a->r.rank != s.r.rank || !typeEq(a->r.elt, s.r.elt))
      throw Error("array bound to " + s.name + " does not have the type the program declares (rank " +
                  std::to_string(s.r.rank) + ", " + typeStr(s.r.elt) + ")");
    materialize(*a);
    for (auto& b : a->bufs) args.push_back((uint64_t)(uintptr_t)b->p);
    for (int64_t d : a->shape) args.push_back((uint64_t)d);
  }
  return args;
}

// text carried as the hexadecimal digits of its bytes ("-" for the empty string)
static std::string unhex(const std::string& h) {
  std::string out;
  if (h == "-") return out;
  if (h.size() % 2) throw Error("malformed hexadecimal text '" + h + "'");
  auto nib = [&](char c) -> int {
    if (c >= '0' && c <= '9') return c - '0';
    if (c >= 'a' && c <= 'f') return c - 'a' + 10;
    if (c >= 'A' && c <= 'F') return c - 'A' + 10;
    throw Error("malformed hexadecimal text '" + h + "'");
  };
  for (size_t i = 0; i < h.size(); i += 2) out.push_back((char)(nib(h[i]) * 16 + nib(h[i + 1])));
  return out;
}

static int64_t arrayBytes(const DArray& a) {
  int64_t per = 0;
  for (ST st : typeLeaves(a.r.elt)) per += stSize(st);
  return a.size() * per;
}

bool Program::streams(const KernelSource& ks, const AEnv& aenv, const std::vector<DArrayP>& temps, int64_t more) {
  if (!ks.streaming) return false;
  // Measured on MI355X (256 MiB last-level cache): the non-temporal variants win once a launch
  // moves more than about twice that, and lose below.
  const int64_t threshold = ctx_.knobs.stream_bytes;
  int64_t bytes = more;
  for (const ArraySlot& s : ks.arrays) {
    if (s.name == "out") continue;
    const DArrayP& a = s.temp ? temps.at(s.index) : aenv.at(aenv.size() - 1 - s.index);
    bytes += arrayBytes(*a);
  }
  return bytes >= threshold;
}

HValP Program::hostExp(const Sx& e, const AEnv& aenv, const Plan& plan) {
  auto it = plan.scalarKernels.find(&e);
  if (it == plan.scalarKernels.end()) return hostEval(e, {}, aenv);
  if (hostSupported(e, true)) {
    try {
      return hostEval(e, {}, aenv);  // only reads scalars the host knows
    } catch (const HostUnknown&) {
    }
  }
  // one-thread kernel, then read the leaves back
  const KernelP& k = it->second;
  ArrayR r;
  r.rank = 0;
  TypeP t = tUnit();
  // rebuild the element type from the leaves (flat tuple is enough to hold them)
  for (ST st : k->meta.outLeaves) t = tPair(t, tScalar(st));
  r.elt = t;
  DArrayP out = alloc(r, {});
  std::vector<uint64_t> args = packArgs(k->meta, aenv, {}, {});
  packOut(args, *out);
  args.push_back(1);
  args.push_back(0);
  ctx_.launch(k, "acc_map", 1, 256, args);
  std::vector<HValP> leaves;
  for (size_t i = 0; i < out->bufs.size(); ++i) {
    ST st = k->meta.outLeaves[i];
    unsigned char raw[8] = {0};
    if (stIsVec(st)) throw Error("a SIMD vector value cannot be read back as a host scalar");
    ctx_.peek(raw, out->bufs[i]->p, stSize(st));
    auto v = std::make_shared<HVal>();
    v->k = HVal::Leaf;
    v->st = st;
    switch (st) {
      case ST::I8: v->i = *(int8_t*)raw; break;
      case ST::I16: v->i = *(int16_t*)raw; break;
      case ST::I32: v->i = *(int32_t*)raw; break;
      case ST::I64: v->i = *(int64_t*)raw; break;
      case ST::U8: v->i = *(uint8_t*)raw; break;
      case ST::U16: v->i = *(uint16_t*)raw; break;
      case ST::U32: v->i = *(uint32_t*)raw; break;
      case ST::U64: v->i = (int64_t) * (uint64_t*)raw; break;
      case ST::F32: v->f = *(float*)raw; break;
      case ST::F64: v->f = *(double*)raw; break;
      case ST::F16: {  // binary16 -> double
        const unsigned h16 = *(uint16_t*)raw, ex = (h16 >> 10) & 31, fr = h16 & 1023;
        double mag = ex == 0 ? std::ldexp((double)fr, -24)
                   : ex == 31 ? (fr ? std::nan("") : HUGE_VAL)
                              : std::ldexp((double)(fr | 1024), (int)ex - 25);
        v->f = (h16 & 0x8000) ? -mag : mag;
        break;
      }
    }
    leaves.push_back(v);
  }
  // the caller only needs shapes / predicates: hand back a left-nested tuple of the leaves
  HValP v = hvUnit();
  if (leaves.size() == 1) return leaves[0];
  for (auto& l : leaves) v = hvPair(v, l);
  return v;
}

std::vector<int64_t> Program::hostShape(const Sx& e, const AEnv& aenv, const Plan& plan, int rank) {
  HValP v = hostExp(e, aenv, plan);
  std::vector<int64_t> d;
  hLeaves(v, d);
  if ((int)d.size() != rank) throw Error("shape expression has rank " + std::to_string(d.size()) + ", expected " + std::to_string(rank));
  return d;
}

std::vector<DArrayP> Program::evalTemps(const std::vector<const Sx*>& temps, AEnv& aenv) {
  std::vector<DArrayP> out;
  for (const Sx* t : temps) {
    AValP v = eval(*t, aenv);
    if (v->k != AVal::Arr) throw Error("array operand evaluated to a tuple");
    out.push_back(v->arr);
  }
  return out;
}

std::vector<int64_t> Program::operandExtent(const Sx& o, const AEnv& aenv, const Plan& plan,
                                            const std::vector<DArrayP>& temps, size_t& cursor) {
  if (o.is("delayed")) return hostShape(o.at(2), aenv, plan, parseArrayR(o.at(1)).rank);
  if (o.is("avar")) {
    size_t ix = (size_t)o.at(1).asInt();
    return aenv[aenv.size() - 1 - ix]->shape;
  }
  return temps.at(cursor++)->shape;
}

void Program::launchMap(const KernelP& k, const AEnv& aenv, const std::vector<DArrayP>& temps, DArray& out) {
  int64_t n = out.size();
  if (n == 0) return;
  std::vector<uint64_t> args = packArgs(k->meta, aenv, temps, out.shape);
  packOut(args, out);
  args.push_back((uint64_t)n);
  args.push_back(0);
  int64_t per = (int64_t)256 * k->meta.vec;
  const bool st = streams(k->meta, aenv, temps, arrayBytes(out));
  // a launch holds fewer than 2^32 threads: larger index spaces take several
  // (the knob lets tests cover an index space with several launches at a small size)
  const int64_t blocks = (n + per - 1) / per, most = std::max<int64_t>(1, ctx_.knobs.map_max_blocks);
  for (int64_t base = 0; base < blocks; base += most) {
    args.back() = (uint64_t)base;
    ctx_.launch(k, st ? "acc_map_stream" : "acc_map", (uint64_t)std::min(most, blocks - base), 256, args);
  }
}

AValP Program::evalFun(const Sx& f, AEnv& aenv, const std::vector<AValP>& args) {
  size_t mark = aenv.size();
  const Sx* cur = &f;
  for (const AValP& a : args) {
    if (!cur->is("alam")) throw Error("array function applied to too many arguments");
    pushVals(cur->at(1), a, aenv);
    cur = &cur->at(2);
  }
  if (cur->is("alam")) throw Error("array function applied to too few arguments");
  AValP r = eval(*cur, aenv);
  aenv.resize(mark);
  return r;
}

AValP Program::run(const std::vector<AValP>& args, const std::vector<DArrayP>& uses) {
  if (args.size() != lams_.size())
    throw Error("program expects " + std::to_string(lams_.size()) + " arguments, got " + std::to_string(args.size()));
  uses_ = &uses;
  AEnv aenv;
  for (size_t i = 0; i < args.size(); ++i) pushVals(lams_[i]->at(1), args[i], aenv);
  AValP r = eval(*body_, aenv);
  materializeAll(r);  // what the caller gets is on the device
  return r;
}

void Program::runInto(const std::vector<AValP>& args, const std::vector<DArrayP>& uses, const AValP& dest) {
  if (args.size() != lams_.size())
    throw Error("program expects " + std::to_string(lams_.size()) + " arguments, got " + std::to_string(args.size()));
  const bool prime = body_->is("scan'");
  if (!prime && !body_->is("scan"))
    throw Error("acchip_execute_into runs programs whose body is a single scan; this one is not");
  const Plan& plan = plans_.at(body_);
  if (!plan.temps.empty() || !plan.scalarKernels.empty())
    throw Error("acchip_execute_into: the scan's operand must be an array variable or a fused producer whose extent "
                "the host can compute");
  std::vector<DArrayP> d;
  if (prime) {
    if (dest->k != AVal::Pair || dest->a->k != AVal::Arr || dest->b->k != AVal::Arr)
      throw Error("acchip_execute_into: the result of scanl' / scanr' is a pair (array, totals)");
    d = {dest->a->arr, dest->b->arr};
  } else {
    if (dest->k != AVal::Arr) throw Error("acchip_execute_into: the result is a single array");
    d = {dest->arr};
  }
  struct Mode {  // left again however the call ends
    Program& p;
    ~Mode() {
      p.noAlloc_ = false;
      p.dest_.clear();
      p.destNext_ = 0;
    }
  } mode{*this};
  noAlloc_ = true;
  dest_ = std::move(d);
  destNext_ = 0;
  uses_ = &uses;
  AEnv aenv;
  for (size_t i = 0; i < args.size(); ++i) pushVals(lams_[i]->at(1), args[i], aenv);
  eval(*body_, aenv);
  if (destNext_ != dest_.size()) throw Error("internal: acchip_execute_into left a result unwritten");
}

AValP Program::eval(const Sx& n, AEnv& aenv) {
  if (n.isAtom("anil")) return avUnit();
  const std::string& h = n.head();
  if (h == "avar") {
    size_t ix = (size_t)n.at(1).asInt();
    return avArr(aenv[aenv.size() - 1 - ix]);
  }
  if (h == "alet") {
    AValP v = eval(n.at(2), aenv);
    size_t mark = aenv.size();
    pushVals(n.at(1), v, aenv);
    AValP r = eval(n.at(3), aenv);
    aenv.resize(mark);
    return r;
  }
  if (h == "apair") {
    AValP a = eval(n.at(1), aenv);
    return avPair(a, eval(n.at(2), aenv));
  }
  if (h == "apply") {
    AValP a = eval(n.at(2), aenv);
    return evalFun(n.at(1), aenv, {a});
  }
  if (h == "atrace") {
    // evaluate the traced arrays, hand them over complete, then go on with the body
    AValP traced = eval(n.at(2), aenv);
    materializeAll(traced);
    ctx_.sync();
    const std::string msg = unhex(n.at(1).str());
    if (ctx_.traceSink) {
      ctx_.traceSink(msg, traced);
    } else {
      std::string line = msg;
      std::function<void(const AValP&)> show = [&](const AValP& v) {
        if (v->k == AVal::Pair) {
          show(v->a);
          show(v->b);
        } else if (v->k == AVal::Arr) {
          line += line.size() > msg.size() ? ", " : ": ";
          line += "Array (Z";
          for (int64_t d : v->arr->shape) line += " :. " + std::to_string(d);
          line += ") " + typeStr(v->arr->r.elt);
        }
      };
      show(traced);
      std::fprintf(stderr, "%s\n", line.c_str());
      std::fflush(stderr);
    }
    return eval(n.at(3), aenv);
  }
  if (h == "aforeign") {
    AValP a = eval(n.at(3), aenv);
    AEnv closed;
    return evalFun(n.at(2), closed, {a});
  }
  if (h == "acond") {
    const Plan& plan = plans_.at(&n);
    HValP c = hostExp(n.at(1), aenv, plan);
    return eval(c->i != 0 ? n.at(2) : n.at(3), aenv);
  }
  if (h == "awhile") {
    // host loop reading one byte back per iteration (Interpreter.hs:222-229)
    AValP x = eval(n.at(3), aenv);
    for (;;) {
      AValP p = evalFun(n.at(1), aenv, {x});
      if (p->k != AVal::Arr || p->arr->bufs.size() != 1) throw Error("awhile: predicate must be a scalar boolean array");
      unsigned char flag = 0;
      if (p->arr->hostKnown) flag = p->arr->hostValue != 0;  // no round trip to the device
      else ctx_.peek(&flag, p->arr->bufs[0]->p, 1);
      if (!flag) break;
      x = evalFun(n.at(2), aenv, {x});
    }
    return x;
  }
  if (h == "use") {
    size_t slot = (size_t)n.at(2).asInt();
    if (!uses_ || slot >= uses_->size()) throw Error("use: no array supplied for slot " + std::to_string(slot));
    return avArr((*uses_)[slot]);
  }

  const Plan& plan = plans_.at(&n);
  auto seeded = [&](const Sx& s) { return !s.isAtom("nothing"); };

  if (h == "unit") {
    DArrayP out = alloc(plan.ty->r, {});
    // the host follows integral scalars made of index arithmetic and other such scalars; the
    // device copy is written only if something reads it there (materialize)
    if (plan.ty->r.elt->k == Type::Scalar && !stIsFloat(plan.ty->r.elt->st) && hostSupported(n.at(2), true)) {
      try {
        HValP v = hostEval(n.at(2), {}, aenv);
        if (v->k == HVal::Leaf) {
          out->hostKnown = true;
          out->hostValue = wrapTo(plan.ty->r.elt->st, v->i);
          out->onDevice = false;
          return avArr(out);
        }
      } catch (const HostUnknown&) {
      }
    }
    launchMap(plan.k, aenv, {}, *out);
    return avArr(out);
  }
  if (h == "reshape") {
    AValP v = eval(n.at(3), aenv);
    int rank = (int)n.at(1).asInt();
    std::vector<int64_t> sh = hostShape(n.at(2), aenv, plan, rank);
    auto a = std::make_shared<DArray>(*v->arr);
    a->shape = sh;
    a->r.rank = rank;
    if (a->size() != v->arr->size()) throw Error("shape mismatch");  // Interpreter.hs:295
    return avArr(a);
  }
  if (h == "generate" || h == "transform" || h == "backpermute") {
    std::vector<DArrayP> temps = evalTemps(plan.temps, aenv);
    const ArrayR& r = plan.ty->r;
    DArrayP out = alloc(r, hostShape(n.at(2), aenv, plan, r.rank));
    // index-permuting producers of rank >= 2 go over two-dimensional tiles of the result
    // (acc_map_tiled): a transposition then uses whole cache lines of its source
    const int64_t w = r.rank >= 2 ? out->shape.back() : 0;
    const int64_t cols = 8 * (int64_t)plan.k->meta.vec;
    const long long te = ctx_.knobs.map_tiled;  // 0 / 1: override, for tests
    bool tiled = h != "generate" && r.rank >= 2 && w >= cols && out->size() / w >= 32;
    int xposeAxis = -1;  // a transposition: the dimension of the result that the source's memory follows
    if (tiled && te < 0) {
      // Tiles pay off only when neighbouring results read far-apart sources.  Where the index
      // function is pure index arithmetic it is evaluated here at two neighbouring result
      // indices; one that reads index arrays (a gather) keeps the linear order.
      tiled = false;
      const Sx& perm = n.at(3);
      if (perm.is("lam") && hostSupported(perm.at(2))) {
        size_t cur = 0;
        const std::vector<int64_t> sext = operandExtent(n.at(h == "transform" ? 5 : 4), aenv, plan, temps, cur);
        auto sourceAt = [&](const std::vector<int64_t>& ix) {
          HValP v = hvUnit();
          for (int64_t c : ix) v = hvPair(v, hvInt(ST::I64, c));
          std::vector<HValP> env;
          hPush(perm.at(1), v, env);
          std::vector<int64_t> sx;
          hDims(hostEval(perm.at(2), env, aenv), sx);
          if (sx.size() != sext.size()) throw Error("backpermute: index function does not return a source index");
          int64_t lin = 0;
          for (size_t k = 0; k < sx.size(); ++k) lin = lin * sext[k] + sx[k];
          return lin;
        };
        std::vector<int64_t> a;
        for (int64_t dim : out->shape) a.push_back(dim / 2);
        std::vector<int64_t> b = a;
        b.back() += b.back() + 1 < out->shape.back() ? 1 : -1;
        try {
          const int64_t at = sourceAt(a);
          const int64_t step = sourceAt(b) - at;
          tiled = step > 1 || step < -1;
          // which other dimension of the result walks the source one element at a time?
          for (int d = r.rank - 2; tiled && d >= 0 && xposeAxis < 0; --d) {
            if (out->shape[d] < 2) continue;
            std::vector<int64_t> e = a;
            e[d] += e[d] + 1 < out->shape[d] ? 1 : -1;
            const int64_t sd = sourceAt(e) - at;
            if (sd == 1 || sd == -1) xposeAxis = d;
          }
        } catch (const Error&) {
          tiled = false;  // the probe is only a hint
          xposeAxis = -1;
        }
      }
    }
    if (tiled && te < 0 && xposeAxis >= 0 && plan.k->meta.xpose) {
      // tiles of the (that dimension, innermost dimension) plane through LDS
      int64_t no = 1, nm = 1;
      for (int d = 0; d < xposeAxis; ++d) no *= out->shape[d];
      for (int d = xposeAxis + 1; d + 1 < r.rank; ++d) nm *= out->shape[d];
      const int64_t na = out->shape[xposeAxis], nw = out->shape.back();
      const int64_t tilesA = (na + 63) / 64, tilesW = (nw + 63) / 64;
      if (no * nm * tilesA * tilesW > 0x7fffffffLL) throw Error("too many tiles for one launch");
      std::vector<uint64_t> args = packArgs(plan.k->meta, aenv, temps, out->shape);
      packOut(args, *out);
      args.push_back((uint64_t)na);
      args.push_back((uint64_t)nm);
      args.push_back((uint64_t)nw);
      args.push_back((uint64_t)tilesA);
      args.push_back((uint64_t)tilesW);
      args.push_back((uint64_t)xposeAxis);
      // (a quarter of what the streaming kernels wait for: 4000 x 9000 Float32, 288 MB moved, 74 -> 54 us;
      // 4096 x 4096 the same either way)
      args.push_back(2 * arrayBytes(*out) >= ctx_.knobs.stream_bytes / 4 ? 1 : 0);
      ctx_.launch(plan.k, "acc_map_xpose", (uint64_t)(no * nm * tilesA * tilesW), 256, args);
      return avArr(out);
    }
    if (te == 0) tiled = false;
    if (te == 1) tiled = h != "generate" && r.rank >= 2 && out->size() > 0;
    if (tiled) {
      const int64_t rows = out->size() / w;
      const int64_t tilesX = (w + cols - 1) / cols, tilesY = (rows + 31) / 32;
      if (tilesX * tilesY > 0x7fffffffLL) throw Error("too many tiles for one launch");
      std::vector<uint64_t> args = packArgs(plan.k->meta, aenv, temps, out->shape);
      packOut(args, *out);
      args.push_back((uint64_t)rows);
      args.push_back((uint64_t)w);
      args.push_back((uint64_t)tilesX);
      ctx_.launch(plan.k, "acc_map_tiled", (uint64_t)(tilesX * tilesY), 256, args);
      return avArr(out);
    }
    launchMap(plan.k, aenv, temps, *out);
    return avArr(out);
  }
  if (h == "map" && plan.mode != "scan") {
    std::vector<DArrayP> temps = evalTemps(plan.temps, aenv);
    size_t cur = 0;
    std::vector<int64_t> ext = operandExtent(n.at(3), aenv, plan, temps, cur);
    DArrayP out = alloc(plan.ty->r, ext);
    launchMap(plan.k, aenv, temps, *out);
    return avArr(out);
  }
  if (h == "zipwith") {
    std::vector<DArrayP> temps = evalTemps(plan.temps, aenv);
    size_t cur = 0;
    std::vector<int64_t> e1 = operandExtent(n.at(3), aenv, plan, temps, cur);
    std::vector<int64_t> e2 = operandExtent(n.at(4), aenv, plan, temps, cur);
    for (size_t k = 0; k < e1.size(); ++k) e1[k] = std::min(e1[k], e2[k]);  // intersect, Shape.hs:81-82
    DArrayP out = alloc(plan.ty->r, e1);
    launchMap(plan.k, aenv, temps, *out);
    return avArr(out);
  }
  if (h == "fold") {
    std::vector<DArrayP> temps = evalTemps(plan.temps, aenv);
    size_t cur = 0;
    std::vector<int64_t> ext = operandExtent(n.at(3), aenv, plan, temps, cur);
    int64_t len = std::max<int64_t>(ext.back(), 0);
    ext.pop_back();
    if (!seeded(n.at(2)) && len <= 0) throw Error("empty array");  // fold1, Interpreter.hs:386
    DArrayP out = alloc(plan.ty->r, ext);
    int64_t rows = out->size();
    if (rows == 0) return avArr(out);
    {
      // many rows of up to a few thousand elements: a few lanes of a wave per row (acc_fold_wrows;
      // under an operator that is not commutative a lane takes a stretch of the row instead of
      // every so-many-th run).  fold_rows: 2 forces it, 0 and 1 keep it off.
      const KernelSource& m = plan.k->meta;
      const long long fr = ctx_.knobs.fold_rows;
      // (in order, a lane's stretch of more than two runs no longer lets the wave's loads cover
      // consecutive memory: rows of 1024 Int64 1.9 TB/s against 3.9 - 4.5 several rows per workgroup;
      // rows of 16 / 256: 4.2 / 4.2 against 3.6 / 3.8, Float32 5.2 / 5.3 against 3.9 / 3.9)
      const bool wave = len >= 1 && (fr == 2 || (fr < 0 && rows >= 256 && (m.commutative ? len < 4096 : len <= 128 * m.vec)));
      if (wave) {
        const int64_t runs = (len + m.vec - 1) / m.vec;
        int64_t lanes = 1;
        while (lanes < 64 && lanes < runs) lanes *= 2;
        const int64_t perStep = 4 * (64 / lanes);  // rows the four waves of a workgroup work on at a time
        // about 32 KiB of 4-byte elements per workgroup
        const int64_t rpg = std::max<int64_t>(perStep, ((8192 + len - 1) / len + perStep - 1) / perStep * perStep);
        const int64_t groups = (rows + rpg - 1) / rpg;
        if (groups > 0x7fffffffLL) throw Error("fold: too many rows for one launch");
        std::vector<uint64_t> args = packArgs(m, aenv, temps, {});
        packOut(args, *out);
        packOut(args, *out);
        args.push_back((uint64_t)rows);
        args.push_back((uint64_t)len);
        args.push_back((uint64_t)lanes);
        args.push_back((uint64_t)rpg);
        const bool st = streams(m, aenv, temps, 0);
        ctx_.launch(plan.k, st ? "acc_fold_wrows_stream" : "acc_fold_wrows", (uint64_t)groups, 256, args);
        return avArr(out);
      }
    }
    {
      // many short rows: several whole rows per workgroup (acc_fold_rows)
      const KernelSource& m = plan.k->meta;
      const int64_t rowsTile = (int64_t)m.block * m.group * m.vec;
      const long long fr = ctx_.knobs.fold_rows;  // 0 / 1: override, for tests
      bool useRows = len >= 1 && rows >= 64 && 4 * len <= rowsTile;
      if (fr == 0) useRows = false;
      if (fr == 1) useRows = len >= 1 && len <= rowsTile;
      if (useRows) {
        const int64_t rpt = rowsTile / len;
        const int64_t groups = (rows + rpt - 1) / rpt;
        if (groups > 0x7fffffffLL) throw Error("fold: too many rows for one launch");
        std::vector<uint64_t> args = packArgs(m, aenv, temps, {});
        packOut(args, *out);
        packOut(args, *out);
        args.push_back((uint64_t)rows);
        args.push_back((uint64_t)len);
        args.push_back((uint64_t)rpt);
        ctx_.launch(plan.k, "acc_fold_rows", (uint64_t)groups, (unsigned)m.block, args);
        return avArr(out);
      }
    }
    // geometry: enough workgroups to fill the chip, each with at least a few tiles of work
    const int64_t tile = (int64_t)4 * 64 * plan.k->meta.vec;
    // workgroups aimed at; long rows take a quarter of them (two per CU: dotp over 2^24 / 2^26 / 2^28
    // elements 21.2 / 80.2 / 306 us against 21.8 / 82.2 / 311; rows of 2^22 would lose with fewer)
    int64_t target = std::max<int64_t>(1, ctx_.knobs.fold_target);
    if (rows == 1 && len >= ((int64_t)1 << 23)) target = std::max<int64_t>(1, target / 4);
    int64_t bpr = 1;
    if (rows < target && len > 8 * tile)
      bpr = std::min((target + rows - 1) / rows, (len + 8 * tile - 1) / (8 * tile));
    int64_t chunk = ((len + bpr - 1) / bpr + tile - 1) / tile * tile;
    if (chunk == 0) chunk = tile;
    bpr = std::max<int64_t>(1, (len + chunk - 1) / chunk);
    const int64_t most = std::max<int64_t>(1, std::min<int64_t>(ctx_.knobs.fold_max_blocks, 0xffffffffLL / 256));
    // A single row cut into chunks is finished by the workgroup that publishes last (no second
    // launch): the chunk results travel as tagged words in the scans' descriptor memory.
    const bool oneLaunch = rows == 1 && bpr > 1 && bpr <= most && ctx_.knobs.fold_one_launch != 0;
    DArrayP tmp = out;
    if (bpr > 1 && !oneLaunch) {
      ArrayR tr = plan.ty->r;
      tr.rank = 1;
      tmp = alloc(tr, {rows * bpr});
    }
    std::vector<uint64_t> args = packArgs(plan.k->meta, aenv, temps, {});
    packOut(args, *out);
    packOut(args, *tmp);
    args.push_back((uint64_t)rows);
    args.push_back((uint64_t)len);
    args.push_back((uint64_t)bpr);
    args.push_back((uint64_t)chunk);
    args.push_back(0);  // FoldParams::first
    const size_t firstAt = args.size() - 1;
    if (oneLaunch) {
      const size_t descBytes = (size_t)bpr * plan.k->meta.words * sizeof(uint64_t);
      ScanState& ss = noAlloc_ ? staticScanState(ctx_.device(), ctx_.stream(), descBytes) : ctx_.scanState(descBytes);
      args.push_back((uint64_t)(uintptr_t)ss.desc);
      args.push_back((uint64_t)ss.epoch);
      args.push_back((uint64_t)std::max<long long>(1, ctx_.knobs.scan_spin_limit));
      args.push_back((uint64_t)(uintptr_t)ctx_.errorWord());
    } else {
      for (int k = 0; k < 4; ++k) args.push_back(0);
    }
    const bool st = streams(plan.k->meta, aenv, temps, 0);
    // An operator that is not commutative over chunks of 64 KiB and more: the kernel that turns
    // blocks of tiles over in LDS (a wave then joins its lanes once per 8 KiB instead of once per
    // KiB: a single row of 2^27 Int64 3.1 -> 6.6 TB/s; its staging area would cost shorter rows
    // their occupancy).  Elements of up to 64 bytes a run (AccFoldStage).
    int64_t eltBytes = 0;
    for (ST t : plan.k->meta.outLeaves) eltBytes += stSize(t);
    const bool staged = !plan.k->meta.commutative && chunk * eltBytes >= 65536 && plan.k->meta.vec * eltBytes <= 64 &&
                        ctx_.knobs.fold_staged != 0;
    const char* entry = staged ? (st ? "acc_fold_main_staged_stream" : "acc_fold_main_staged") : (st ? "acc_fold_main_stream" : "acc_fold_main");
    // a launch holds fewer than 2^32 threads: more rows than that many workgroups take several launches
    for (int64_t first = 0; first < rows * bpr; first += most) {
      args[firstAt] = (uint64_t)first;
      ctx_.launch(plan.k, entry, (uint64_t)std::min(most, rows * bpr - first), 256, args);
    }
    args[firstAt] = 0;
    if (bpr > 1 && !oneLaunch) ctx_.launch(plan.k, "acc_fold_final", (uint64_t)rows, 256, args);
    return avArr(out);
  }
  if (h == "permute") {
    // the destination starts as the defaults; a defaults operand that is not a variable is
    // a fresh array nobody else can see and is updated in place (Trafo/Fusion.hs:559-566)
    std::vector<DArrayP> temps = evalTemps(plan.temps, aenv);
    size_t cur = 0;
    std::vector<int64_t> ext = operandExtent(n.at(4), aenv, plan, temps, cur);
    int64_t cnt = 1;
    for (int64_t d : ext) cnt *= std::max<int64_t>(d, 0);
    // the counting kernels' launch geometry for a destination of `size` elements (false: they do not apply)
    struct CountGeometry {
      int64_t nparts, part, groups, chunk;
      bool viaPartials;
    };
    auto countGeometry = [&](int64_t size, CountGeometry& g) {
      // every range of the destination reads all the sources again (from the XCD's L2), so the
      // counting kernels lose to plain global atomics beyond about 90 ranges (2^26 keys: 26 us per
      // range against 2.5 ms)
      const int64_t maxParts = std::min<int64_t>(ctx_.knobs.permute_parts, 88);
      const bool many = cnt >= (1 << 20) || (cnt >= (1 << 12) && cnt >= 4 * size);
      if (!(plan.k->meta.permuteCount && many && size > 0 && size <= maxParts * 65536 && ctx_.knobs.permute_count != 0)) return false;
      g.nparts = (size + 65535) / 65536;
      g.part = g.nparts == 1 ? size : 65536;
      const long long ge = ctx_.knobs.permute_groups;
      g.groups = ge > 0 ? ge : std::min<int64_t>(256 / g.nparts, cnt / 16384);
      g.groups = std::max<int64_t>(8, g.groups / 8 * 8);
      g.chunk = ((cnt + g.groups - 1) / g.groups + 3) / 4 * 4;
      // The workgroups leave their counters in memory and a second launch sums them, unless there
      // are so few workgroups that adding them to the destination directly is as cheap.
      g.viaPartials = g.groups >= 32;
      if (ctx_.knobs.permute_partials >= 0) g.viaPartials = ctx_.knobs.permute_partials != 0;
      return true;
    };
    // Defaults of one constant under the counting kernels with a second launch: that launch
    // writes constant + count to every element, and the defaults are never materialised (a
    // workgroup must then note its reliefs in a list of 15 entries: chunk < 15 * 32768).
    DArrayP out;
    bool freshDefaults = false;
    if (plan.k->meta.permuteCountSet && ctx_.flag(Context::kInplace) && ctx_.knobs.permute_fresh != 0) {
      const Sx& gen = n.at(2);
      const Plan& gp = plans_.at(&gen);
      const ArrayR& gr = gp.ty->r;
      std::vector<int64_t> shp = hostShape(gen.at(2), aenv, gp, gr.rank);
      int64_t size = 1;
      for (int64_t d : shp) size *= std::max<int64_t>(d, 0);
      CountGeometry g;
      if (cnt > 0 && countGeometry(size, g) && g.viaPartials && g.chunk < 15 * 32768) {
        out = alloc(gr, shp);
        freshDefaults = true;
      }
    }
    if (!out) {
      AValP dv = eval(n.at(2), aenv);
      if (dv->k != AVal::Arr) throw Error("permute: defaults must be a single array");
      materialize(*dv->arr);
      out = dv->arr;
      static const char* fresh[] = {"generate", "map", "zipwith", "transform", "backpermute", "fold", "foldseg",
                                    "scan", "permute", "stencil", "stencil2", "unit"};
      bool inPlace = false;
      for (const char* k : fresh) inPlace = inPlace || n.at(2).is(k);
      inPlace = inPlace && ctx_.flag(Context::kInplace);  // -fno-inplace: always a copy (cbits/flags.h:25)
      if (!inPlace) {
        out = alloc(dv->arr->r, dv->arr->shape);
        for (size_t k = 0; k < out->bufs.size(); ++k) ctx_.copy(out->bufs[k]->p, dv->arr->bufs[k]->p, out->bufs[k]->bytes);
      }
    }
    if (cnt == 0 || out->size() == 0) return avArr(out);
    std::vector<uint64_t> args = packArgs(plan.k->meta, aenv, temps, out->shape);
    packOut(args, *out);
    // Many sources into a destination of a few LDS-fuls with a hardware-atomic combination:
    // combine in workgroup-private LDS copies first (see permute.hpp).
    int64_t eltBytes = 0;
    for (ST st : plan.k->meta.outLeaves) eltBytes += stSize(st);
    const bool statefulCopies = plan.mode == "lock" || plan.mode == "cas";
    if (statefulCopies) eltBytes += 4;  // the private copy's state word
    const int64_t partMax = 131072 / std::max<int64_t>(1, eltBytes);  // Spec::kPart
    // Up to 128 LDS-fuls: every share re-reads the sources (from its XCD's L2), so the cost grows
    // with the destination -- 2^26 keys into 2^20 / 2^22 Int32 bins take 0.5 / 2.0 ms, which is
    // where plain global atomics are for uniform keys (2.5 ms); for Zipf keys those take 110 ms.
    // (the privatised permute: 80 us per range for 2^26 sources, against 2.5 - 3.2 ms of global atomics)
    // (a compare-and-swap loop without contention does 2^24 updates in 0.8 ms, ten ranges' worth)
    const int64_t maxParts = std::min<int64_t>(ctx_.knobs.permute_parts, plan.mode == "cas" ? 10 : 32);
    // From 2^20 sources on, and from 2^12 on when every destination element receives several of
    // them (few destinations under many sources contend in the memory-side atomic units: 2^16
    // keys into 256 bins take 33 us through global atomics, 2^14 keys into 16 bins 47 us,
    // against 9 us this way).
    const bool many = cnt >= (1 << 20) || (cnt >= (1 << 12) && cnt >= 4 * out->size());
    CountGeometry cg;
    if (countGeometry(out->size(), cg)) {
      // a sum of one constant per source: 16-bit counters, 65536 destination elements per LDS-ful
      const int64_t nparts = cg.nparts, groups = cg.groups;
      args.push_back((uint64_t)cnt);
      args.push_back((uint64_t)cg.chunk);
      args.push_back((uint64_t)nparts);
      args.push_back((uint64_t)cg.part);
      args.push_back((uint64_t)out->size());
      args.push_back((uint64_t)(uintptr_t)ctx_.errorWord());
      DArrayP partials;
      if (cg.viaPartials) {
        ArrayR pr;
        pr.rank = 1;
        pr.elt = tScalar(ST::U32);
        partials = alloc(pr, {nparts * groups * (32768 + 16)});  // ACC_COUNT_STRIDE words per workgroup
      }
      args.push_back(partials ? (uint64_t)(uintptr_t)partials->bufs[0]->p : 0);
      args.push_back((uint64_t)groups);
      args.push_back(freshDefaults ? 1 : 0);
      ctx_.launch(plan.k, "acc_permute_count", (uint64_t)(groups * nparts), 1024, args);
      if (partials) ctx_.launch(plan.k, "acc_permute_count_reduce", (uint64_t)(nparts * (32768 / 128)), 256, args);
      return avArr(out);
    }
    // (under the lock, contended elements cost milliseconds each way: 2^24 pairs into 384 elements
    // took 6.4 s through global locks alone)
    if ((plan.mode == "atomic" || plan.mode == "atomics" || statefulCopies) && many && out->size() <= maxParts * partMax) {
      const int64_t nparts = (out->size() + partMax - 1) / partMax;
      const int64_t part = (out->size() + nparts - 1) / nparts;
      // one workgroup per CU in total (each holds 128 KiB of LDS): fewer, longer workgroups
      // mean fewer private copies to add into the destination at the end; at least 16 Ki
      // sources per workgroup
      const long long ge = ctx_.knobs.permute_groups;
      int64_t groups = ge > 0 ? ge : std::min<int64_t>(256 / nparts, cnt / 16384);
      groups = std::max<int64_t>(8, groups / 8 * 8);
      int64_t chunk = ((cnt + groups - 1) / groups + 3) / 4 * 4;
      args.push_back((uint64_t)cnt);
      args.push_back((uint64_t)chunk);
      args.push_back((uint64_t)nparts);
      args.push_back((uint64_t)part);
      args.push_back((uint64_t)out->size());
      args.push_back((uint64_t)(uintptr_t)ctx_.errorWord());
      DArrayP copies;
      if (statefulCopies) {
        // the workgroups' private copies, one Spec::Priv each (128 KiB and the padding between its arrays at most)
        ArrayR pr;
        pr.rank = 1;
        pr.elt = tScalar(ST::U32);
        const int64_t privBytes = 131072 + 16 * ((int64_t)plan.k->meta.outLeaves.size() + 2);
        copies = alloc(pr, {nparts * groups * privBytes / 4});
      }
      args.push_back(copies ? (uint64_t)(uintptr_t)copies->bufs[0]->p : 0);  // (otherwise a field of the counting variant)
      args.push_back((uint64_t)groups);
      args.push_back(0);
      ctx_.launch(plan.k, "acc_permute_lds", (uint64_t)(groups * nparts), 1024, args);
      if (copies) ctx_.launch(plan.k, "acc_permute_lds_merge", (uint64_t)(nparts * ((part + 255) / 256)), 256, args);
      return avArr(out);
    }
    DArrayP locks;
    if (plan.mode == "lock") {
      ArrayR lr;
      lr.rank = 1;
      lr.elt = tScalar(ST::U32);
      locks = alloc(lr, {out->size()});
      ctx_.fill0(locks->bufs[0]->p, locks->bufs[0]->bytes);
    }
    args.push_back((uint64_t)cnt);
    args.push_back(locks ? (uint64_t)(uintptr_t)locks->bufs[0]->p : 0);
    args.push_back((uint64_t)(uintptr_t)ctx_.errorWord());
    int64_t grid = std::min<int64_t>((cnt + 255) / 256, 256 * 32);
    ctx_.launch(plan.k, "acc_permute", (uint64_t)grid, 256, args);
    return avArr(out);
  }
  if (h == "stencil" || h == "stencil2") {
    const bool two = h == "stencil2";
    std::vector<DArrayP> temps = evalTemps(plan.temps, aenv);
    size_t cur = 0;
    std::vector<int64_t> ext = operandExtent(n.at(two ? 6 : 5), aenv, plan, temps, cur);
    if (two) {
      std::vector<int64_t> e2 = operandExtent(n.at(8), aenv, plan, temps, cur);
      for (size_t k = 0; k < ext.size(); ++k) ext[k] = std::min(ext[k], e2[k]);
    }
    // Mirror and Wrap remap an outside index once (Interpreter.hs:824-839); on an extent shorter
    // than the taps reach (Mirror: extent <= halo, Wrap: extent < halo) the remapped index is
    // still outside, which the reference reports when it indexes the source (indexCheck in
    // toIndex, Shape.hs:98-106).  The kernels do not test their reads, so this is decided here.
    {
      bool nonEmpty = true;
      for (int64_t d : ext) nonEmpty = nonEmpty && d > 0;
      size_t cur2 = 0;
      for (int a = 0; nonEmpty && a < (two ? 2 : 1); ++a) {
        const Sx& bnd = n.at(two ? (a == 0 ? 5 : 7) : 4);
        const std::vector<int64_t> sext = operandExtent(n.at(two ? (a == 0 ? 6 : 8) : 5), aenv, plan, temps, cur2);
        const bool mirror = bnd.isAtom("mirror"), wrap = bnd.isAtom("wrap");
        if (!mirror && !wrap) continue;
        const std::vector<int> halo = stencilHaloOf(n.at(two ? 1 + a : 1));
        for (size_t d = 0; d < halo.size() && d < sext.size(); ++d)
          if (halo[d] > 0 && sext[d] < halo[d] + (mirror ? 1 : 0))
            throw Error("index out of bounds: a " + std::string(mirror ? "mirror" : "wrap") + " boundary on an extent of " +
                        std::to_string(sext[d]) + " under a stencil that reaches " + std::to_string(halo[d]) +
                        " beyond the focus");
      }
    }
    DArrayP out = alloc(plan.ty->r, ext);
    if (plan.mode == "lds2d") {
      if (out->size() == 0) return avArr(out);
      const int64_t th = plan.k->meta.group;  // rows per tile chosen by the code generator
      const int64_t tw = plan.k->meta.words;  // and columns per tile
      const int64_t tilesY = (ext[0] + th - 1) / th, tilesX = (ext[1] + tw - 1) / tw;
      if (tilesX * tilesY > 0x7fffffffLL) throw Error("stencil: too many tiles for one launch");
      std::vector<uint64_t> args = packArgs(plan.k->meta, aenv, temps, ext);
      packOut(args, *out);
      args.push_back((uint64_t)ext[0]);
      args.push_back((uint64_t)ext[1]);
      args.push_back((uint64_t)tilesX);
      args.push_back((uint64_t)tilesY);
      // a workgroup can chain several tiles down a column, prefetching the next one; with
      // 128-bit staging one tile per workgroup measured best (92 us against 103 / 107 us for
      // chains of 2 / 4 on the 8192 x 8192 Jacobi sweep), so chains are only a knob
      const long long ce = ctx_.knobs.stencil_chain;
      int64_t chain = ce > 0 ? ce : 1;
      chain = std::max<int64_t>(1, std::min(chain, tilesY));
      args.push_back((uint64_t)chain);
      const int64_t chunksY = (tilesY + chain - 1) / chain;
      ctx_.launch(plan.k, "acc_stencil2d", (uint64_t)(tilesX * chunksY), 256, args);
      return avArr(out);
    }
    if (plan.mode == "lds3d") {
      if (out->size() == 0) return avArr(out);
      const int64_t th = plan.k->meta.group, tw = plan.k->meta.words;
      const int64_t tilesY = (ext[1] + th - 1) / th, tilesX = (ext[2] + tw - 1) / tw;
      // planes per workgroup: long enough to amortise the 2*HZ planes staged before the first
      // result, short enough that the grid fills the device
      const long long ce = ctx_.knobs.stencil_chain;
      int64_t chain = ce > 0 ? ce : 16;  // measured on 512^3: 8..32 planes within 5 %
      while (ce <= 0 && chain > 4 && tilesX * tilesY * ((ext[0] + chain - 1) / chain) < 2048) chain /= 2;
      chain = std::max<int64_t>(1, std::min(chain, ext[0]));
      const int64_t chunksZ = (ext[0] + chain - 1) / chain;
      if (tilesX * tilesY * chunksZ > 0x7fffffffLL) throw Error("stencil: too many tiles for one launch");
      std::vector<uint64_t> args = packArgs(plan.k->meta, aenv, temps, ext);
      packOut(args, *out);
      for (int k = 0; k < 3; ++k) args.push_back((uint64_t)ext[k]);
      args.push_back((uint64_t)tilesX);
      args.push_back((uint64_t)tilesY);
      args.push_back((uint64_t)chain);
      ctx_.launch(plan.k, "acc_stencil3d", (uint64_t)(tilesX * tilesY * chunksZ), 256, args);
      return avArr(out);
    }
    launchMap(plan.k, aenv, temps, *out);
    return avArr(out);
  }
  if (h == "foldseg") {
    std::vector<DArrayP> temps = evalTemps(plan.temps, aenv);
    size_t cur = 0;
    std::vector<int64_t> ext = operandExtent(n.at(4), aenv, plan, temps, cur);
    std::vector<int64_t> sext = operandExtent(n.at(5), aenv, plan, temps, cur);
    if (sext[0] <= 0) throw Error("empty segment descriptor");  // Interpreter.hs:400
    const int64_t len = std::max<int64_t>(ext.back(), 0), nseg = sext[0] - 1;
    std::vector<int64_t> oshape(ext.begin(), ext.end() - 1);
    int64_t rows = 1;
    for (int64_t d : oshape) rows *= std::max<int64_t>(d, 0);
    oshape.push_back(nseg);
    DArrayP out = alloc(plan.ty->r, oshape);
    if (rows == 0 || nseg == 0) return avArr(out);
    const KernelSource& m = plan.k->meta;
    const int64_t tile = (int64_t)m.block * m.group * m.vec;
    const int64_t total = rows * len;
    const int64_t tiles = std::max<int64_t>(1, (total + tile - 1) / tile);
    if (tiles > 0x7f000000LL) throw Error("foldSeg: too many tiles for one launch");
    ArrayR pr;
    pr.rank = 1;
    pr.elt = tScalar(ST::I64);
    DArrayP part = alloc(pr, {tiles + 1});
    // per tile a descriptor of its carry and one of its pending end (value + boundary number), in
    // the scans' descriptor memory
    ScanState& st = ctx_.scanState((size_t)tiles * (2 * (size_t)m.words + 4) * sizeof(uint64_t));
    std::vector<uint64_t> args = packArgs(m, aenv, temps, {});
    packOut(args, *out);
    args.push_back((uint64_t)rows);
    args.push_back((uint64_t)len);
    args.push_back((uint64_t)nseg);
    args.push_back((uint64_t)total);
    args.push_back((uint64_t)tiles);
    args.push_back((uint64_t)(uintptr_t)part->bufs[0]->p);
    args.push_back((uint64_t)(uintptr_t)st.desc);
    args.push_back((uint64_t)st.epoch);
    args.push_back((uint64_t)std::max<long long>(1, ctx_.knobs.scan_spin_limit));
    args.push_back((uint64_t)(uintptr_t)ctx_.errorWord());
    const int64_t boundaries = rows * (nseg + 1);
    if ((boundaries + 255) / 256 > 0x7fffffffLL) throw Error("foldSeg: too many segments for one launch");
    ctx_.launch(plan.k, "acc_foldseg_partition", (uint64_t)((boundaries + 255) / 256), 256, args);
    // behind the tiles, the workgroups that complete the segment ends reaching across tile borders
    const uint64_t fixGroups = (uint64_t)((tiles + m.block - 1) / m.block);
    if (ctx_.knobs.foldseg_one_launch != 0) {
      ctx_.launch(plan.k, "acc_foldseg", (uint64_t)tiles + fixGroups, (unsigned)m.block, args);
    } else {
      ctx_.launch(plan.k, "acc_foldseg", (uint64_t)tiles, (unsigned)m.block, args);
      ctx_.launch(plan.k, "acc_foldseg_fixup", fixGroups, (unsigned)m.block, args);
    }
    return avArr(out);
  }
  if (h == "scan" || h == "scan'" || (h == "map" && plan.mode == "scan")) {
    const Sx& sn = h == "map" ? n.at(3) : n;  // the scan inside a map whose function it applies itself
    const bool prime = h == "scan'";
    const int kind = prime ? 2 : (seeded(sn.at(3)) ? 1 : 0);
    std::vector<DArrayP> temps = evalTemps(plan.temps, aenv);
    size_t cur = 0;
    std::vector<int64_t> ext = operandExtent(sn.at(4), aenv, plan, temps, cur);
    const int64_t len = std::max<int64_t>(ext.back(), 0);
    std::vector<int64_t> outer(ext.begin(), ext.end() - 1);
    std::vector<int64_t> oshape = outer;
    oshape.push_back(kind == 1 ? len + 1 : len);
    const ArrayR& ar = prime ? plan.ty->a->r : plan.ty->r;
    DArrayP out = alloc(ar, oshape);
    DArrayP tot = out;
    if (prime) tot = alloc(plan.ty->b->r, outer);
    int64_t rows = 1;
    for (int64_t d : outer) rows *= std::max<int64_t>(d, 0);
    AValP result = prime ? avPair(avArr(out), avArr(tot)) : avArr(out);
    if (rows == 0 || (kind == 0 && len == 0)) return result;
    // large tiles when they fill the device, small ones otherwise
    const KernelSource& big = plan.k->meta;
    const int64_t bigTile = (int64_t)big.block * big.group * big.vec;
    bool small = false;
    if (plan.k2) {
      const KernelSource& sm = plan.k2->meta;
      const int64_t smallTile = (int64_t)sm.block * sm.group * sm.vec;
      // (measured, large against small tiles: Float32 171 large tiles 26.7 / 21.9 us, 341 tiles 36.0 /
      // 39.4; Int64 85 tiles 13.3 / 13.2, 171 tiles 18.0 / 21.7 -- elements of 4 bytes and fewer keep
      // the small tiles for longer because a large tile's lanes hold twice as many of them)
      const int64_t fewer = big.words <= 1 ? 256 : 100;
      small = rows * ((len + bigTile - 1) / bigTile) < fewer || len <= 2 * smallTile;
      // and as long as all small tiles are on the device at once, for then they need no tickets
      // (Float32 2^24, 1024 tiles: 27.9 us against 36.1 with the large tiles and 37.2 pipelined;
      // Int64 2^23: 25.4 against 32.1 and 27.0)
      if (!small && ctx_.knobs.scan_ticketless != 0 && ctx_.knobs.scan_test_skew == 0)
        small = rows * ((len + smallTile - 1) / smallTile) <= ctx_.residentGroups(plan.k2, "acc_scan", (unsigned)sm.block);
    }
    const long long forcedTiles = ctx_.knobs.scan_tiles;  // 1 large / 2 small / 3 rows: override, for tests
    if (forcedTiles == 1 || forcedTiles == 4) small = false;
    if (forcedTiles == 2 && plan.k2) small = true;
    if (plan.k2 && len >= 1) {
      // many short rows: several whole rows per workgroup (acc_scan_rows)
      const KernelSource& sm = plan.k2->meta;
      const int64_t rowsTile = (int64_t)sm.block * sm.rowsGroup * sm.vec;
      const bool forced = forcedTiles == 3;
      // (up to a whole tile of it: a row alone in its workgroup still moves group by group, while
      // a tile of acc_scan that its row does not fill goes through the code for ragged ends)
      if ((forced && len <= rowsTile) || (forcedTiles == 0 && rows >= 2 && len <= rowsTile)) {
        const int64_t rpt = rowsTile / len;
        const int64_t groups = (rows + rpt - 1) / rpt;
        if (groups > 0x7fffffffLL) throw Error("scan: too many rows for one launch");
        std::vector<uint64_t> args = packArgs(sm, aenv, temps, {});
        packOut(args, *out);
        packOut(args, *tot);
        args.push_back((uint64_t)rows);
        args.push_back((uint64_t)len);
        args.push_back((uint64_t)rpt);
        ctx_.launch(plan.k2, "acc_scan_rows", (uint64_t)groups, (unsigned)sm.block, args);
        return result;
      }
    }
    // Long rows of a plain array: the pipelined kernel (persistent workgroups, one per CU).  Its
    // direct global -> LDS loads move 16 bytes per lane from 16-byte aligned addresses.
    bool pipe = false;
    if (plan.k3 && !small) {
      const KernelSource& pm = plan.k3->meta;
      const int64_t pipeTile = (int64_t)pm.block * pm.group * pm.vec;
      const int64_t eltBytes = 16 / pm.vec;
      // the array the kernel moves: the operand itself, or the one array a fused producer reads
      DArrayP srcArr;
      for (const ArraySlot& sl : pm.arrays)
        if (sl.name == pm.pipeSlot) srcArr = sl.temp ? temps.at(sl.index) : aenv.at(aenv.size() - 1 - sl.index);
      // (a right scan's tiles are counted from the end of each row; a producer must cover its array exactly)
      const bool aligned = srcArr && !srcArr->bufs.empty() && ((uintptr_t)srcArr->bufs[0]->p & 15) == 0 &&
                           srcArr->shape == ext && ((rows == 1 && !pm.scanRight) || (len * eltBytes) % 16 == 0);
      const int64_t tprP = (len + pipeTile - 1) / pipeTile;
      // measured on 2^28 elements: Float32 350 us against 395 us for a workgroup per tile, Int64 706
      // against 742; from two tiles per CU on it is level or ahead (Int64 2^23, 512 tiles: 27 against
      // 32 us; Float32 2^24, 585 tiles: 37 against 36; with 256 tiles 18.7 against 18.0)
      pipe = aligned && (forcedTiles == 4 ? len >= pipeTile
                                          : (forcedTiles == 0 && tprP >= 16 && rows * tprP >= 2 * ctx_.computeUnits()));
    }
    const KernelP& kern = pipe ? plan.k3 : (small ? plan.k2 : plan.k);
    const KernelSource& m = kern->meta;
    const int64_t tile = (int64_t)m.block * m.group * m.vec;
    const int64_t tpr = std::max<int64_t>(1, (len + tile - 1) / tile);
    const int64_t tiles = rows * tpr;
    if (tiles > 0x7fffffffLL) throw Error("scan: too many tiles for one launch");
    const size_t descBytes = (size_t)tiles * m.words * sizeof(uint64_t);
    ScanState& st = noAlloc_ ? staticScanState(ctx_.device(), ctx_.stream(), descBytes) : ctx_.scanState(descBytes);
    std::vector<uint64_t> args = packArgs(m, aenv, temps, {});
    packOut(args, *out);
    packOut(args, *tot);
    args.push_back((uint64_t)rows);
    args.push_back((uint64_t)len);
    args.push_back((uint64_t)tpr);
    args.push_back((uint64_t)(uintptr_t)st.desc);
    args.push_back((uint64_t)(uintptr_t)st.ticket);
    const size_t ticketAt = args.size() - 1;
    // fault injection for the test of the bounded look-back wait: a ticket base that lags the
    // counter by `skew` gives every tile a number `skew` too high, so the first tiles wait for
    // predecessors that never run, give up after `spin` polls and report
    const uint64_t skew = (uint64_t)std::max<long long>(0, ctx_.knobs.scan_test_skew);
    // a legitimate wait lasts microseconds; 2^22 polls are several seconds
    const uint64_t spin = (uint64_t)std::max<long long>(1, ctx_.knobs.scan_spin_limit);
    args.push_back((uint64_t)(st.ticketBase - skew));
    args.push_back((uint64_t)st.epoch);
    args.push_back(spin);
    args.push_back((uint64_t)(uintptr_t)ctx_.errorWord());
    const int64_t tprFull = len / tile;
    args.push_back((uint64_t)tprFull);
    if (pipe) {
      // the full tiles of every row; every workgroup takes tickets until it meets the first one
      // beyond them.  Then, with the same epoch, the rows' last tiles where they are partial.
      const int64_t fullTiles = rows * tprFull;
      const uint64_t groups = (uint64_t)std::min<int64_t>(fullTiles, ctx_.computeUnits());
      ctx_.launch(kern, "acc_scan_pipe", groups, (unsigned)m.block, args);
      // (a workgroup stops at the first ticket beyond the tiles: with the test's skew that is `skew` tickets earlier)
      st.ticketBase += (uint64_t)std::max<int64_t>(0, fullTiles - (int64_t)skew) + groups;
      if (tprFull < tpr) ctx_.launch(kern, "acc_scan_pipe_tail", (uint64_t)rows, (unsigned)m.block, args);
      return result;
    }
    // A launch whose tiles are all on the device at once needs no tickets: a tile's number is its
    // workgroup's, nobody waits for a tile that cannot start, and every workgroup is spared the
    // counter's round trip in front of its loads (one row of 2^20 Int32: 7.5 -> 6.5 us).
    const bool ticketless = skew == 0 && ctx_.knobs.scan_ticketless != 0 && tiles <= ctx_.residentGroups(kern, "acc_scan", (unsigned)m.block);
    if (ticketless) args[ticketAt] = 0;
    ctx_.launch(kern, "acc_scan", (uint64_t)tiles, (unsigned)m.block, args);
    if (!ticketless) st.ticketBase += (uint64_t)tiles;
    return result;
  }
  throw Error("unsupported array term '" + h + "'");
}

}  // namespace acchip
