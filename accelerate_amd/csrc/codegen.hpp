// Lowering of the scalar language (OpenExp / OpenFun / PrimFun, AST.hs:494-753) to HIP C++
// text, and assembly of one translation unit per array node: prelude + generated `Spec`
// (element type, scalar functions, fused producers) + one hand-written skeleton.
#pragma once
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "types.hpp"

namespace acchip {

// A value during code generation: a tree whose leaves are C++ expressions that are cheap
// and pure to repeat (a variable name or a literal).
struct Val;
using ValP = std::shared_ptr<Val>;
struct Val {
  enum K { Unit, Leaf, Pair } k = Unit;
  ST st = ST::I64;
  std::string ex;
  ValP a, b;
  // set on a 64-bit integer leaf that is the widening of an integer of at most 32 bits: the
  // expression and type it was widened from (a permute's index test can then stay in 32 bits)
  std::string narrowEx;
  ST narrowSt = ST::I64;
};
ValP vUnit();
ValP vLeaf(ST st, const std::string& ex);
ValP vPair(ValP a, ValP b);
TypeP valType(const ValP& v);
void valLeaves(const ValP& v, std::vector<ValP>& out);

// An array a kernel reads: a variable of the node's array environment, or a temporary the
// executor materialised for a nested manifest operand.
struct ArraySlot {
  std::string name;   // "a<deBruijn>" or "t<k>"
  ArrayR r;
  bool temp = false;
  int index = 0;      // de Bruijn index or temporary number
};

// Operand of a consumer: fused (Delayed) or a real array.
struct Operand {
  bool delayed = false;
  ArrayR r;
  Sx extent, indexD, linearD;  // when delayed
  std::string slot;            // when manifest: name of the array slot
};

// thrown by Codegen::scan for the pipelined variant: the fused producer is not a function of one array's element
struct ScanNotPipeable {};
// thrown by Codegen::scan when the function to apply to the results reads arrays
struct ScanPostNotFusable {};

// Everything the executor needs to launch a generated kernel.
struct KernelSource {
  std::string source;                 // full translation unit
  std::vector<ArraySlot> arrays;      // Env fields, in order (per array: leaf pointers, then extents)
  std::vector<ST> outLeaves;          // element leaves of Spec::Out
  int vec = 1;                        // Spec::V
  int group = 1;                      // Spec::G (scan: groups per wave)
  int words = 1;                      // 32-bit words of Spec::Elt (scan descriptors)
  int block = 256;                    // threads per workgroup of the main kernel
  bool commutative = false;
  bool streaming = false;             // has acc_*_stream entry points (non-temporal variant)
  bool xpose = false;                 // backpermute / transform of rank >= 2: has acc_map_xpose (tiles through LDS)
  bool scanRight = false;             // scan only: a right scan
  std::string pipeSlot;               // pipelined scan only: name of the array slot its loads move
  int rowsGroup = 1;                  // scan only: groups per wave of acc_scan_rows (small-tile variant)
  std::string permuteMode;            // permute only: "atomic", "cas", "lock", "store"
  bool permuteCount = false;          // permute only: has acc_permute_count (sum of a constant per source)
  bool permuteCountSet = false;       // permute only: has count_set (defaults of one constant, written with the counts)
  bool permuteTarget32 = false;       // permute only: has target32 (rank-1 destination, index widened from <= 32 bits)
};

class Codegen {
 public:
  // aenv[i] is the type of array variable with de Bruijn index i at this node
  explicit Codegen(std::vector<ArrayR> aenv) : aenv_(std::move(aenv)) {}

  // off: a permute with `const` as its combination over a product type goes through the
  // per-element locks, so that no element mixes two sources (Language.hs:786-790)
  bool fastPermuteConst = true;

  std::string addTemp(const ArrayR& r);  // returns slot name for a materialised operand

  KernelSource fold(const Sx& f, const Sx* seed, const Operand& src);
  KernelSource map(const TypeP& outElt, const Sx* f, const Operand& src);
  KernelSource zipWith(const TypeP& outElt, const Sx& f, const Operand& a, const Operand& b, int rank);
  KernelSource generate(const ArrayR& out, const Sx& f);
  KernelSource backpermute(int outRank, const Sx& p, const Sx* f, const TypeP& outElt, const Operand& src);
  // kind 0: scanl1/scanr1, 1: scanl/scanr, 2: scanl'/scanr' (seed required for 1 and 2)
  // small: the variant for short rows (256-thread workgroups)
  // variant 0: large tiles, 1: small tiles (short rows), 2: persistent pipeline for long rows of a plain array
  // (only where scanPipeable holds)
  // post (with its result type): a function applied to every result on its way to memory -- the
  // `map g` of `map g (scan f z xs)`, which then costs neither a launch nor an array of its own
  KernelSource scan(const Sx& f, const Sx* seed, const Operand& src, bool right, int kind, int variant = 0,
                    const Sx* post = nullptr, const TypeP& postElt = nullptr);
  static bool scanPipeable(const Operand& src, bool right);
  KernelSource foldSeg(const Sx& f, const Sx* seed, const Operand& src, const Operand& seg, ST segType);
  // freshInit: the literal every element of the defaults holds when they are `generate sh (\_ -> c)`
  // (the counting variant can then write defaults and counts together), else null
  KernelSource permute(const Sx& f, const ArrayR& dst, const Sx& p, const Operand& src, const Sx* freshInit = nullptr);
  KernelSource stencil(const std::vector<Sx>& patterns, const TypeP& outElt, const Sx& f,
                       const std::vector<Sx>& boundaries, const std::vector<Operand>& srcs);
  // rank-2 single-source stencil through LDS halo tiles
  KernelSource stencil2d(const Sx& pattern, const TypeP& outElt, const Sx& f, const Sx& boundary, const Operand& src);
  KernelSource stencil3d(const Sx& pattern, const TypeP& outElt, const Sx& f, const Sx& boundary, const Operand& src);
  KernelSource scalarKernel(const Sx& exp);  // evaluates a closed Exp with one thread

  // type of a closed scalar expression / result of a function, without emitting code
  TypeP typeOfExp(const Sx& e);

  struct Emit {
    std::string code;
    int ind = 2;
    void line(const std::string& s) { code.append(ind, ' ').append(s).append("\n"); }
  };
  using Env = std::vector<ValP>;  // scalar environment; back() has de Bruijn index 0

 private:
  friend struct CodegenImpl;
  std::vector<ArrayR> aenv_;
  std::map<std::string, ArraySlot> used_;
  std::vector<ArraySlot> temps_;
  int next_ = 0;

  std::string fresh() { return "v" + std::to_string(next_++); }
  const ArraySlot& slotForVar(int idx);
  const ArraySlot& slotByName(const std::string& name);

  ValP exp(const Sx& e, const Env& env, Emit& em);
  ValP applyFun(const Sx& f, const std::vector<ValP>& args, const Env& env, Emit& em);
  ValP prim(const std::string& name, const std::vector<ST>& tys, const ValP& arg, Emit& em);
  ValP bindLeaf(ST st, const std::string& ex, Emit& em);  // const T vN = ex;
  ValP readArray(const ArraySlot& s, const std::string& lin, Emit& em);
  ValP shapeOf(const ArraySlot& s);
  std::string toIndex(const ValP& sh, const ValP& ix, Emit& em);
  ValP fromIndex(int rank, const ValP& sh, const std::string& lin, Emit& em);
  // from_index / next_index over the result's extents, the index value (ix[0], ix[1], ..) and
  // the tail that marks a producer as taking the multi-dimensional index (map.hpp)
  std::string indexedFns(int rank, const ArraySlot& o);
  ValP indexedIx(int rank);
  std::string indexedTail(int rank);
  ValP operandLinear(const Operand& o, const std::string& lin, Emit& em);
  ValP operandIndex(const Operand& o, const ValP& ix, Emit& em);
  ValP operandShape(const Operand& o, Emit& em);
  ValP declareVars(const TypeP& t, Emit& em);                // uninitialised mutable variables
  void assign(const ValP& dst, const ValP& src, Emit& em);
  ValP copyToVars(const ValP& v, Emit& em);

  std::string eltStruct(const TypeP& t, const std::string& name);
  std::string outStruct(const std::vector<ST>& leaves);
  std::string envStruct(std::vector<ArraySlot>& order);
  ValP eltVal(const TypeP& t, const std::string& var);
  std::string returnElt(const ValP& v, Emit& em);
  bool isCommutative(const Sx& f, std::string* op = nullptr, ST* st = nullptr);
  KernelSource finish(const std::string& specBody, const TypeP& elt, const std::vector<ST>& outLeaves,
                      const std::string& skeleton, int vec, bool ownStore = false);
};

// taps a stencil pattern reaches on either side of the focus, per dimension (outermost first)
std::vector<int> stencilHaloOf(const Sx& pattern);
std::string literalText(ST st, const std::string& tok);
const std::string& deviceHeader(const std::string& name);  // embedded device/*.hpp text

}  // namespace acchip
