// Device context: one HIP stream, a size-bucketed device memory pool, and the kernel cache
// (SHA3-256 of the generated source -> loaded code object; memory, then disk, then hipRTC).
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <condition_variable>
#include <functional>
#include <future>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "codegen.hpp"
#include "scratch.hpp"

namespace acchip {

struct Kernel {
  std::string hash;
  std::string code;                 // code object (hsaco), complete once `ready` is
  hipModule_t module = nullptr;     // loaded lazily, on first launch
  std::map<std::string, hipFunction_t> fns;
  KernelSource meta;                // argument plan (source text dropped after compilation)
  // compilation in flight (valid only when hipRTC had to run).  Declared last: it is destroyed
  // first, and destroying the last reference to an async task waits for the worker, which
  // writes into `code`.
  std::shared_future<void> ready;
};
using KernelP = std::shared_ptr<Kernel>;

// Counters with the meaning of the reference's cbits/monitoring.c:26-32.
struct Stats {
  std::atomic<long long> bytesAllocated{0}, bytesCopiedToRemote{0}, bytesCopiedFromRemote{0}, bytesEvicted{0},
      kernelsCompiled{0}, kernelsFromDisk{0}, kernelsFromMemory{0}, launches{0}, poolHits{0}, poolMisses{0};
};

// Always owned by a std::shared_ptr: device buffers, programs and events keep their
// context alive, so handles may be released in any order (finalisers run in any order).
class Context : public std::enable_shared_from_this<Context> {
 public:
  // device < 0: a context that can generate and compile code but owns no GPU
  explicit Context(int device);
  ~Context();

  bool hasDevice() const { return device_ >= 0; }
  int device() const { return device_; }
  hipStream_t stream() const { return stream_; }

  // memory pool (counterpart of Array/Remote/Table.hs:170-211 + Nursery.hs:43-113):
  // requests are rounded up to 1 KiB chunks, freed blocks wait in per-size free lists and
  // are handed out again for the same rounded size; on exhaustion the free lists are
  // released and the request retried once; failure returns nullptr, never throws.
  void* malloc(size_t bytes);
  void free(void* p);
  void purge();
  size_t blockSize(void* p);
  void memInfo(size_t* total, size_t* avail);

  void poke(void* dev, const void* host, size_t bytes);   // H->D through pinned staging, stream-ordered
  void peek(void* host, const void* dev, size_t bytes);   // D->H, synchronises the stream
  void copy(void* dst, const void* src, size_t bytes);    // D->D
  void fill0(void* dev, size_t bytes);
  void sync();
  // A word of pinned host memory that kernels write when they meet what the reference reports
  // through boundsCheck (Error.hs:33-62; e.g. an empty segment under fold1Seg).  Kernels get
  // errorWord(); every call that waits for the stream (sync, peek) then raises the error.
  unsigned* errorWord();
  void raiseDeviceError();

  // Looks the kernel up (memory, then disk) or starts its compilation on a worker thread:
  // the kernels of a program compile side by side.  wait() returns when the code object is
  // there, and throws what the compiler reported.
  KernelP kernel(const KernelSource& ks);
  void wait(const KernelP& k);
  void launch(const KernelP& k, const char* fn, uint64_t grid, unsigned block, const std::vector<uint64_t>& args);

  // Where Atrace nodes deliver their message and the arrays they were given (the C ABI
  // installs the caller's callback here; the value is an AVal); empty: a line on stderr.
  std::function<void(const std::string& msg, const std::shared_ptr<void>& arrays)> traceSink;

  // persistent device scratch for single-pass scans (tile descriptors + ticket counter),
  // allocated and grown on demand
  ScanState& scanState(size_t descBytes);
  // Load the kernel's code object and look its entry points up now instead of at the first
  // launch, so that a later launch does no set-up work on the device.
  void preload(const KernelP& k, std::initializer_list<const char*> fns);

  Stats stats;
  std::string cacheDir;
  bool dumpCC = false, dumpExec = false, forceRecomp = false;

 private:
  int device_ = -1;
  hipStream_t stream_ = nullptr;
  std::mutex mu_;
  std::unordered_map<void*, size_t> live_;                  // block -> rounded size
  std::map<size_t, std::vector<void*>> nursery_;            // rounded size -> free blocks
  std::unordered_map<std::string, KernelP> kernels_;
  void* staging_ = nullptr;
  unsigned* errHost_ = nullptr;  // pinned, mapped: written by kernels, read here
  unsigned* errDev_ = nullptr;
  size_t stagingBytes_ = 0;
  ScanState scan_;
  void ensureLoaded(const KernelP& k);
  void* staging(size_t bytes);
};

void hipCheck(hipError_t e, const char* what);
std::string libraryDir();  // directory holding this shared library

}  // namespace acchip
