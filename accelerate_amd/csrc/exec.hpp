// Executor: walks the array-level term (the counterpart of evalOpenAcc,
// Interpreter.hs:175-259), one kernel launch per array node, host-driven control flow.
// A Program is prepared once (parse, type inference, code generation and hipRTC for every
// node: what `runN f` does at partial application) and executed many times.
#pragma once
#include <map>
#include <memory>
#include <vector>

#include "runtime.hpp"

namespace acchip {

struct Buffer {
  std::shared_ptr<Context> ctx;  // keeps the pool alive until the block has gone back to it
  void* p = nullptr;
  size_t bytes = 0;
  bool owned = false;
  ~Buffer() {
    if (owned && ctx) ctx->free(p);
  }
};
using BufferP = std::shared_ptr<Buffer>;

// A device-resident array: shape + one dense buffer per scalar leaf of the element type
// (struct-of-arrays, Array/Data.hs:95-119; row-major, Representation/Shape.hs:98-106).
struct DArray {
  ArrayR r;
  std::vector<int64_t> shape;
  std::vector<BufferP> bufs;
  // A rank-0 array of one integral leaf whose value the host computed alongside the device
  // (`unit e` with e made of index arithmetic and such arrays): loop counters and flags of
  // awhile / acond are then read here instead of from the device.
  bool hostKnown = false;
  int64_t hostValue = 0;
  bool onDevice = true;  // false: the buffer has not been written yet (Program::materialize)
  int64_t size() const {
    int64_t n = 1;
    for (int64_t d : shape) n = d <= 0 ? 0 : n * d;
    for (int64_t d : shape)
      if (d <= 0) return 0;
    return n;
  }
};
using DArrayP = std::shared_ptr<DArray>;

struct AVal;
using AValP = std::shared_ptr<AVal>;
struct AVal {
  enum K { Unit, Arr, Pair } k = Unit;
  DArrayP arr;
  AValP a, b;
};

struct ATy;
using ATyP = std::shared_ptr<ATy>;
struct ATy {
  enum K { Unit, Arr, Pair } k = Unit;
  ArrayR r;
  ATyP a, b;
};

// host-side scalar value (extents, predicates)
struct HVal;
using HValP = std::shared_ptr<HVal>;
struct HVal {
  enum K { Unit, Leaf, Pair } k = Unit;
  ST st = ST::I64;
  int64_t i = 0;   // integral leaves (any width, stored sign/zero-extended)
  double f = 0;    // floating leaves
  HValP a, b;
};

struct Plan {
  KernelP k, k2, k3;                             // k3: scans only, the pipelined kernel for long rows of a plain array
  std::vector<const Sx*> temps;                  // nested manifest operands, in slot order
  std::map<const Sx*, KernelP> scalarKernels;    // expressions evaluated by a one-thread kernel
  std::map<const Sx*, std::vector<const Sx*>> scalarTemps;
  std::string mode;
  ATyP ty;                                       // result type of the node
};

class Program {
 public:
  Program(Context& ctx, const char* text, size_t len);
  // args: one AVal per lambda of the program, in order; uses: arrays for (use ..) slots
  AValP run(const std::vector<AValP>& args, const std::vector<DArrayP>& uses);
  // The same for a program whose body is one scan over array variables or fused producers,
  // written into arrays the caller made (`dest`: the result array, or the pair (array, totals)
  // of scanl' / scanr'); tile descriptors and ticket live in the device's static scratch, so the
  // call allocates no device memory.  Throws when the program or its size does not qualify.
  void runInto(const std::vector<AValP>& args, const std::vector<DArrayP>& uses, const AValP& dest);

  std::vector<ATyP> argTypes;
  ATyP resultType;
  size_t kernelCount() const { return plans_.size(); }
  // cache keys of every kernel the program may launch (all variants of every node, scalar kernels), sorted, distinct
  std::vector<std::string> kernelKeys() const;

 private:
  Context& ctx_;
  Sx root_;
  const Sx* body_ = nullptr;
  std::vector<const Sx*> lams_;
  std::map<const Sx*, Plan> plans_;
  const std::vector<DArrayP>* uses_ = nullptr;
  // runInto: alloc() hands out the caller's arrays, in the order the node asks for its results,
  // and fails once they are used up
  bool noAlloc_ = false;
  std::vector<DArrayP> dest_;
  size_t destNext_ = 0;

  using TEnv = std::vector<ArrayR>;     // back() has de Bruijn index 0
  using AEnv = std::vector<DArrayP>;

  // preparation
  ATyP prepare(const Sx& n, TEnv& tenv);
  ATyP prepareFun(const Sx& f, TEnv& tenv, std::vector<ATyP>* params);
  Operand operandOf(const Sx& o, Codegen& cg, TEnv& tenv, Plan& plan);
  void prepareHostExp(const Sx& e, TEnv& tenv, Plan& plan);
  static std::vector<ArrayR> aenvOf(const TEnv& tenv);
  ATyP prepareScan(const Sx& n, TEnv& tenv, Plan& plan, const Sx* post, const TypeP& postElt);

  // execution
  AValP eval(const Sx& n, AEnv& aenv);
  AValP evalFun(const Sx& f, AEnv& aenv, const std::vector<AValP>& args);
  HValP hostExp(const Sx& e, const AEnv& aenv, const Plan& plan);
  std::vector<int64_t> hostShape(const Sx& e, const AEnv& aenv, const Plan& plan, int rank);
  std::vector<DArrayP> evalTemps(const std::vector<const Sx*>& temps, AEnv& aenv);
  std::vector<int64_t> operandExtent(const Sx& o, const AEnv& aenv, const Plan& plan, const std::vector<DArrayP>& temps,
                                     size_t& tempCursor);
  DArrayP alloc(const ArrayR& r, const std::vector<int64_t>& shape);
  // write a host-known scalar to its device buffer if that has not happened yet
  void materialize(DArray& a);
  void materializeAll(const AValP& v);
  std::vector<uint64_t> packArgs(const KernelSource& ks, const AEnv& aenv, const std::vector<DArrayP>& temps,
                                 const std::vector<int64_t>& outShape);
  static void packOut(std::vector<uint64_t>& args, const DArray& a);
  // does a launch of ks move so much more than the last-level cache holds that its
  // streaming variant pays?  (the whole of every array it reads, plus `more` bytes)
  bool streams(const KernelSource& ks, const AEnv& aenv, const std::vector<DArrayP>& temps, int64_t more);
  void launchMap(const KernelP& k, const AEnv& aenv, const std::vector<DArrayP>& temps, DArray& out);
};

}  // namespace acchip
