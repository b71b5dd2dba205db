// Device context: one HIP stream, a size-bucketed device memory pool, and the kernel cache
// (SHA3-256 of the generated source -> loaded code object; memory, then disk, then hipRTC).
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <condition_variable>
#include <functional>
#include <future>
#include <map>
#include <unordered_set>
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
  std::map<std::string, int> perCu;  // workgroups of an entry point that one CU holds at a time (asked once)
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
      kernelsCompiled{0}, kernelsFromDisk{0}, kernelsFromMemory{0}, launches{0}, poolHits{0}, poolMisses{0},
      arraysEvicted{0},
      rawAllocs{0},      // device or pinned host allocations of any kind the library asked the runtime for
      modulesLoaded{0};  // code objects loaded onto the device
};

// Launch-time choices that tests and tuning override.  Read from the environment once, when
// the context is made (ACCHIP_<NAME IN CAPITALS>), and changed afterwards only through set():
// no launch looks at the environment.
struct Knobs {
  long long stream_bytes = (long long)512 << 20;  // bytes a launch must move before the non-temporal variants are taken
  long long map_max_blocks = (long long)1 << 23;  // workgroups per launch of the map skeleton
  long long map_tiled = -1;         // -1: decide per launch, 0 / 1: never / always tile index-permuting producers
  long long fold_rows = -1;         // -1: decide per launch; 0 / 1: never / always the several-rows-per-workgroup fold; 2: always a few lanes per row
  long long fold_target = 2048;     // workgroups a fold aims at
  long long fold_staged = 1;        // 0: ordered folds never take the kernel that stages blocks of tiles in LDS
  long long scan_post = 1;          // 0: a map around a scan is always a launch of its own
  long long scan_ticketless = 1;    // 0: the tiles of a scan always take their numbers from the ticket counter
  long long foldseg_one_launch = 1; // 0: the ends that reach across tile borders are completed by a launch of their own
  long long fold_one_launch = 1;    // 0: a single row cut into chunks always takes the second launch (acc_fold_final)
  long long fold_max_blocks = (long long)1 << 24;  // workgroups per launch of the fold skeleton
  long long permute_parts = 128;    // LDS-fuls of destination the privatised permute accepts
  long long permute_count = 1;      // 0: never take the counting kernel
  long long permute_groups = 0;     // 0: decide per launch
  long long permute_partials = -1;  // -1 / 0 / 1: counters summed by a second launch
  long long permute_fresh = 1;      // 0: constant defaults are materialised also where the counting kernels could write them
  long long stencil_chain = 0;      // 0: decide per launch; tiles (rank 2) or planes (rank 3) per workgroup
  long long stencil_no2d = 0, stencil_no3d = 0;  // 1: rank-2 / rank-3 stencils through the generic skeleton
  long long pool_async = 1;         // 1: device blocks come from the stream-ordered allocator (hipMallocAsync), 0: hipMalloc
  long long scan_tiles = 0;         // 0: decide per launch, 1 large, 2 small, 3 rows, 4 pipelined (where the operand allows)
  long long scan_spin_limit = (long long)1 << 22;  // polls after which a tile stops waiting (seconds)
  long long scan_test_skew = 0;     // fault injection: the ticket base passed to the kernel lags by this much
  void fromEnv();
  bool set(const std::string& name, long long value);  // false: no such knob
  bool get(const std::string& name, long long& value) const;
};

// Always owned by a std::shared_ptr: device buffers, programs and events keep their
// context alive, so handles may be released in any order (finalisers run in any order).
class Context : public std::enable_shared_from_this<Context> {
 public:
  // device < 0: a context that can generate and compile code but owns no GPU
  explicit Context(int device);
  ~Context();

  bool hasDevice() const { return device_ >= 0; }
  // device == -2: no GPU, but host memory stands in for device memory, so that the memory
  // manager (pool, table, eviction) can be driven without one; programs still cannot run
  bool hasMemory() const { return device_ >= 0 || fakeMemory_; }
  int device() const { return device_; }
  int computeUnits();  // of the device (256 on MI355X); 256 for a context without one
  // workgroups of `block` threads of entry point fn that the device holds at the same time (0: unknown)
  int64_t residentGroups(const KernelP& k, const char* fn, unsigned block);
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

  // Array table (counterpart of Array/Remote/LRU.hs + Table.hs): host arrays, named by an id
  // the caller chooses (the reference's StableArray / Unique), and the device blocks that
  // mirror them.  An array in use (between tableUse and tableRelease) stays where it is; any
  // other may be evicted when memory runs out -- copied back to its host array first if the
  // device copy is the newer one (Dirty) -- and is uploaded again by the next tableUse.
  // Allocation ladder (Table.hs:194-211, LRU.hs:250-341): free list of the size class, the
  // device, the clean hook (the caller's garbage collector, whose finalisers call tableFree)
  // and the free list again, purge + the device, then eviction of the eldest unused arrays
  // one at a time, and only then failure.
  enum class Status { Clean, Dirty, Unmanaged, Evicted };
  bool tableMalloc(uint64_t id, void* host, size_t bytes, bool frozen);  // false: already known
  void* tableUse(uint64_t id);                 // nullptr: never allocated (LRU.withRemote -> Nothing)
  void tableRelease(uint64_t id);              // end of the use; work queued so far may still touch it
  void tableFree(uint64_t id);                 // the host array died
  void tableInsertUnmanaged(uint64_t id, void* dev);
  // a block of the pool (e.g. a program's result) becomes the device copy of host array `id`
  void tableAdopt(uint64_t id, void* host, size_t bytes, void* dev, bool clean);
  void tableReclaim();                         // LRU.reclaim: clean + purge
  int tableStatus(uint64_t id);                // -1 unknown, else a Status
  std::function<void()> cleanHook;

  void poke(void* dev, const void* host, size_t bytes);   // H->D through pinned staging, stream-ordered
  void peek(void* host, const void* dev, size_t bytes);   // D->H, synchronises the stream, raises what kernels reported
  void copyFromDevice(void* host, const void* dev, size_t bytes);  // the same without looking at the error word
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
  Knobs knobs;
  std::string cacheDir;
  // The reference's option word (cbits/flags.h:19-49); only the bits below change anything here.
  enum Flag : uint32_t {
    kInplace = 1u << 4, kFastMath = 1u << 5, kFastPermuteConst = 1u << 6, kForceRecomp = 1u << 7,
    kDumpGc = 1u << 18, kDumpCc = 1u << 20, kDumpExec = 1u << 23,
  };
  uint32_t flags = kInplace | kFastPermuteConst;
  bool flag(Flag f) const { return (flags & f) != 0; }

 private:
  int device_ = -1;
  int cus_ = 0;
  hipStream_t stream_ = nullptr;
  std::mutex mu_;
  std::unordered_map<void*, size_t> live_;                  // block -> rounded size
  std::unordered_set<void*> asyncBlocks_;                   // blocks that came from the stream-ordered allocator
  bool asyncPoolReady_ = false;
  std::map<size_t, std::vector<void*>> nursery_;            // rounded size -> free blocks
  std::unordered_map<std::string, KernelP> kernels_;
  unsigned* errHost_ = nullptr;  // pinned, mapped: written by kernels, read here
  unsigned* errDev_ = nullptr;
  // two pinned staging buffers: the host copies into / out of one while the other is on the wire
  std::mutex stagingMu_;
  void* staging_[2] = {nullptr, nullptr};
  hipEvent_t stagingDone_[2] = {nullptr, nullptr};
  ScanState scan_;
  void ensureLoaded(const KernelP& k);
  void ensureStaging();

  // raw device memory under the byte budget (ACCHIP_POOL_LIMIT; 0 = whatever the device has)
  bool fakeMemory_ = false;
  size_t limit_ = 0, rawBytes_ = 0;
  void* rawMalloc(size_t n);
  void rawFree(void* p, size_t n);
  void* poolMalloc(size_t bytes, bool mayEvict);

  struct Entry {
    void* dev = nullptr;
    size_t bytes = 0;       // of the host array
    void* host = nullptr;
    Status st = Status::Clean;
    int count = 0;          // uses in progress
    uint64_t stamp = 0;     // time of the last release
    hipEvent_t task = nullptr;  // recorded at the last release: work queued until then
  };
  std::mutex tableMu_;
  std::unordered_map<uint64_t, Entry> table_;
  uint64_t clock_ = 0;
  bool evictEldest();       // tableMu_ held
  bool taskDone(Entry& e);
};

void hipCheck(hipError_t e, const char* what);
std::string libraryDir();  // directory holding this shared library

}  // namespace acchip
