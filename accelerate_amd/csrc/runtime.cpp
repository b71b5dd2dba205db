#include "runtime.hpp"

#include <dlfcn.h>
#include <hip/hiprtc.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cctype>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>

#include "sha3.hpp"

namespace acchip {

void hipCheck(hipError_t e, const char* what) {
  if (e != hipSuccess) throw Error(std::string(what) + ": " + hipGetErrorString(e));
}

std::string libraryDir() {
  Dl_info info;
  if (dladdr((void*)&libraryDir, &info) && info.dli_fname) {
    std::string p = info.dli_fname;
    size_t k = p.rfind('/');
    return k == std::string::npos ? "." : p.substr(0, k);
  }
  return ".";
}

// Without fast-math a kernel computes what the scalar language says, operation by operation
// (no contraction into fused multiply-adds), which is what bit-wise parity with a CPU needs; with
// it the compiler may contract, reassociate and use reciprocals, as the reference's LLVM backends
// do under -ffast-math (cbits/flags.h:26), NaN and infinity still honoured.
static std::vector<const char*> compileOptions(bool fastMath) {
  std::vector<const char*> o = {"--offload-arch=gfx950", "-O3", "-std=c++17",
                                // packed fp32 instructions are kept out of generated code on this target
                                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  if (fastMath) {
    for (const char* x : {"-ffp-contract=fast", "-fno-math-errno", "-fno-trapping-math", "-fno-signed-zeros",
                          "-fassociative-math", "-freciprocal-math"})
      o.push_back(x);
  } else {
    o.push_back("-ffp-contract=off");
  }
  return o;
}

namespace {
struct KnobName {
  const char* name;
  long long Knobs::*field;
};
const KnobName kKnobs[] = {
    {"stream_bytes", &Knobs::stream_bytes},       {"map_max_blocks", &Knobs::map_max_blocks},
    {"map_tiled", &Knobs::map_tiled},             {"fold_rows", &Knobs::fold_rows},
    {"fold_target", &Knobs::fold_target},         {"fold_staged", &Knobs::fold_staged},         {"fold_max_blocks", &Knobs::fold_max_blocks},         {"permute_parts", &Knobs::permute_parts},
    {"permute_count", &Knobs::permute_count},     {"permute_groups", &Knobs::permute_groups},
    {"permute_partials", &Knobs::permute_partials}, {"permute_fresh", &Knobs::permute_fresh}, {"stencil_chain", &Knobs::stencil_chain},
    {"pool_async", &Knobs::pool_async}, {"fold_one_launch", &Knobs::fold_one_launch},
    {"foldseg_one_launch", &Knobs::foldseg_one_launch}, {"scan_ticketless", &Knobs::scan_ticketless}, {"scan_post", &Knobs::scan_post},
    {"stencil_no2d", &Knobs::stencil_no2d},       {"stencil_no3d", &Knobs::stencil_no3d},
    {"scan_tiles", &Knobs::scan_tiles},           {"scan_spin_limit", &Knobs::scan_spin_limit},
    {"scan_test_skew", &Knobs::scan_test_skew},
};
}  // namespace

bool Knobs::set(const std::string& name, long long value) {
  for (const KnobName& k : kKnobs)
    if (name == k.name) {
      this->*k.field = value;
      return true;
    }
  return false;
}

bool Knobs::get(const std::string& name, long long& value) const {
  for (const KnobName& k : kKnobs)
    if (name == k.name) {
      value = this->*k.field;
      return true;
    }
  return false;
}

void Knobs::fromEnv() {
  for (const KnobName& k : kKnobs) {
    std::string env = "ACCHIP_";
    for (const char* c = k.name; *c; ++c) env += (char)std::toupper((unsigned char)*c);
    const char* v = std::getenv(env.c_str());
    if (!v || !*v) continue;
    const std::string sv = v;
    if (sv == "large") this->*k.field = 1;  // ACCHIP_SCAN_TILES also takes the variants' names
    else if (sv == "small") this->*k.field = 2;
    else if (sv == "rows") this->*k.field = 3;
    else this->*k.field = std::atoll(v);
  }
}

Context::Context(int device) : device_(device) {
  knobs.fromEnv();
  const char* cd = std::getenv("ACCHIP_CACHE_DIR");
  cacheDir = cd ? cd : libraryDir() + "/kcache";
  const char* fl = std::getenv("ACCHIP_FLAGS");
  if (fl) {
    // names as the reference spells them after -f / -d (Debug/Internal/Flags.hs:70-105)
    static const struct { const char* name; uint32_t bit; } names[] = {
        {"inplace", kInplace}, {"fast-math", kFastMath}, {"fast-permute-const", kFastPermuteConst},
        {"force-recomp", kForceRecomp}, {"dump-gc", kDumpGc}, {"dump-cc", kDumpCc}, {"dump-exec", kDumpExec}};
    // tokens separated by blanks or commas; "-f" / "-d" in front as on the reference's command
    // line are accepted, "no-" clears the bit, unknown tokens are ignored
    const std::string f = std::string(fl) + " ";
    std::string tok;
    for (char ch : f) {
      if (ch != ' ' && ch != ',' && ch != '\t') {
        tok += ch;
        continue;
      }
      if (tok.size() > 2 && tok[0] == '-' && (tok[1] == 'f' || tok[1] == 'd')) tok = tok.substr(2);
      const bool no = tok.compare(0, 3, "no-") == 0;
      if (no) tok = tok.substr(3);
      for (const auto& nm : names)
        if (tok == nm.name) flags = no ? flags & ~nm.bit : flags | nm.bit;
      tok.clear();
    }
  }
  if (device_ == -2) {
    fakeMemory_ = true;
    device_ = -1;
  }
  if (const char* pl = std::getenv("ACCHIP_POOL_LIMIT")) limit_ = (size_t)std::strtoull(pl, nullptr, 0);
  if (device_ >= 0) {
    hipCheck(hipSetDevice(device_), "hipSetDevice");
    hipCheck(hipStreamCreateWithFlags(&stream_, hipStreamNonBlocking), "hipStreamCreate");
    staticScratchSetup(device_);  // address of the static scan scratch on this device
    (void)errorWord();            // pinned now: launches allocate nothing for it later
  }
}

int Context::computeUnits() {
  if (cus_ == 0) {
    cus_ = 256;
    if (device_ >= 0) {
      int v = 0;
      if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device_) == hipSuccess && v > 0) cus_ = v;
    }
  }
  return cus_;
}

Context::~Context() {
  for (auto& kv : kernels_) {
    try {
      wait(kv.second);  // a worker may still be writing into the kernel
    } catch (...) {
    }
  }
  if (device_ < 0) {
    purge();
    for (auto& kv : live_) rawFree(kv.first, kv.second);
    return;
  }
  (void)hipSetDevice(device_);
  (void)hipStreamSynchronize(stream_);
  for (auto& kv : kernels_)
    if (kv.second->module) (void)hipModuleUnload(kv.second->module);
  for (auto& kv : table_)
    if (kv.second.task) (void)hipEventDestroy(kv.second.task);
  purge();
  for (auto& kv : live_) rawFree(kv.first, kv.second);
  for (int b = 0; b < 2; ++b) {
    if (staging_[b]) (void)hipHostFree(staging_[b]);
    if (stagingDone_[b]) (void)hipEventDestroy(stagingDone_[b]);
  }
  if (errHost_) (void)hipHostFree(errHost_);
  if (scan_.desc) (void)hipFree(scan_.desc);
  if (scan_.ticket) (void)hipFree(scan_.ticket);
  (void)hipStreamSynchronize(stream_);  // the stream-ordered frees above
  (void)hipStreamDestroy(stream_);
}

// ------------------------------------------------------------------------------------
// memory

static const size_t kStagePiece = (size_t)32 << 20;

static size_t roundUp(size_t bytes) {
  const size_t chunk = 1024;  // remoteAllocationSize default (Array/Remote/Table.hs:180-190)
  if (bytes == 0) bytes = 1;
  return (bytes + chunk - 1) / chunk * chunk;
}

void* Context::rawMalloc(size_t n) {
  {
    std::lock_guard<std::mutex> g(mu_);
    if (limit_ && rawBytes_ + n > limit_) return nullptr;  // the budget stands in for a full device
    rawBytes_ += n;
  }
  void* p = nullptr;
  if (fakeMemory_) {
    p = std::malloc(n);
  } else {
    // Stream-ordered underneath (the reference's ladder, Array/Remote/Table.hs:194-211, sits on
    // top): a block freed behind queued work needs no synchronisation, the runtime's pool keeps
    // what is freed (release threshold = everything) and hands it out again in stream order.
    (void)hipSetDevice(device_);
    const bool async = knobs.pool_async != 0;
    if (async && !asyncPoolReady_) {
      hipMemPool_t mp = nullptr;
      if (hipDeviceGetDefaultMemPool(&mp, device_) == hipSuccess && mp) {
        uint64_t keep = ~(uint64_t)0;
        (void)hipMemPoolSetAttribute(mp, hipMemPoolAttrReleaseThreshold, &keep);
      }
      (void)hipGetLastError();
      asyncPoolReady_ = true;
    }
    const hipError_t e = async ? hipMallocAsync(&p, n, stream_) : hipMalloc(&p, n);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      p = nullptr;
    } else {
      stats.rawAllocs++;
      std::lock_guard<std::mutex> g(mu_);
      if (async) asyncBlocks_.insert(p);
    }
  }
  if (!p) {
    std::lock_guard<std::mutex> g(mu_);
    rawBytes_ -= n;
  }
  return p;
}

void Context::rawFree(void* p, size_t n) {
  bool async = false;
  {
    std::lock_guard<std::mutex> g(mu_);
    async = asyncBlocks_.erase(p) > 0;
    rawBytes_ -= n;
  }
  if (fakeMemory_) std::free(p);
  else if (async) (void)hipFreeAsync(p, stream_);   // ordered behind whatever the stream still does with the block
  else (void)hipFree(p);
}

void* Context::malloc(size_t bytes) { return poolMalloc(bytes, true); }

void* Context::poolMalloc(size_t bytes, bool mayEvict) {
  if (!hasMemory()) return nullptr;
  const size_t n = roundUp(bytes);
  auto fromNursery = [&]() -> void* {
    std::lock_guard<std::mutex> g(mu_);
    auto it = nursery_.find(n);
    if (it == nursery_.end() || it->second.empty()) return nullptr;
    void* p = it->second.back();
    it->second.pop_back();
    live_[p] = n;
    return p;
  };
  auto fresh = [&]() -> void* {
    void* p = rawMalloc(n);
    if (p) {
      stats.bytesAllocated += (long long)n;
      std::lock_guard<std::mutex> g(mu_);
      live_[p] = n;
    }
    return p;
  };
  if (void* p = fromNursery()) {
    stats.poolHits++;
    return p;
  }
  stats.poolMisses++;
  if (void* p = fresh()) return p;
  // the caller's collector may find dead host arrays, whose blocks then wait in the free lists
  if (cleanHook) {
    cleanHook();
    if (void* p = fromNursery()) return p;
  }
  // work queued on the stream may still use blocks waiting in the free lists: blocks of the
  // stream-ordered allocator are freed behind it, others only once the stream has drained
  if (device_ >= 0 && knobs.pool_async == 0) (void)hipStreamSynchronize(stream_);
  purge();
  if (void* p = fresh()) return p;
  // evict unused arrays of the table, eldest first, until the block fits or nothing is left
  while (mayEvict) {
    {
      std::lock_guard<std::mutex> g(tableMu_);
      if (!evictEldest()) break;
    }
    if (void* p = fromNursery()) return p;
    purge();
    if (void* p = fresh()) return p;
  }
  return nullptr;
}

void Context::free(void* p) {
  if (!p) return;
  std::lock_guard<std::mutex> g(mu_);
  auto it = live_.find(p);
  if (it == live_.end()) return;  // not ours (or freed twice): ignore, as the reference's table does
  nursery_[it->second].push_back(p);
  live_.erase(it);
}

void Context::purge() {
  std::map<size_t, std::vector<void*>> take;
  {
    std::lock_guard<std::mutex> g(mu_);
    take.swap(nursery_);
  }
  for (auto& kv : take)
    for (void* p : kv.second) {
      rawFree(p, kv.first);
      stats.bytesEvicted += (long long)kv.first;
    }
}

size_t Context::blockSize(void* p) {
  std::lock_guard<std::mutex> g(mu_);
  auto it = live_.find(p);
  return it == live_.end() ? 0 : it->second;
}

void Context::memInfo(size_t* total, size_t* avail) {
  *total = *avail = 0;
  if (!hasMemory()) return;
  if (device_ >= 0) {
    hipCheck(hipMemGetInfo(avail, total), "hipMemGetInfo");
    // what the stream-ordered allocator keeps for reuse is not in use
    hipMemPool_t mp = nullptr;
    uint64_t reserved = 0, used = 0;
    if (asyncPoolReady_ && hipDeviceGetDefaultMemPool(&mp, device_) == hipSuccess && mp &&
        hipMemPoolGetAttribute(mp, hipMemPoolAttrReservedMemCurrent, &reserved) == hipSuccess &&
        hipMemPoolGetAttribute(mp, hipMemPoolAttrUsedMemCurrent, &used) == hipSuccess && reserved > used)
      *avail += (size_t)(reserved - used);
    (void)hipGetLastError();
  }
  std::lock_guard<std::mutex> g(mu_);
  if (limit_) {
    *total = limit_;
    *avail = limit_ > rawBytes_ ? limit_ - rawBytes_ : 0;
  } else if (fakeMemory_) {
    *total = *avail = (size_t)1 << 40;
  }
  for (auto& kv : nursery_) *avail += kv.first * kv.second.size();  // reusable without asking the driver
}

// ------------------------------------------------------------------------------------
// array table

bool Context::taskDone(Entry& e) {
  if (!e.task) return true;
  const hipError_t r = hipEventQuery(e.task);
  if (r == hipErrorNotReady) {
    (void)hipGetLastError();
    return false;
  }
  return true;
}

// LRU.evictLRU (LRU.hs:273-337): the eldest array that nobody uses and whose last task has
// finished gives up its device block; a Dirty one is copied back to its host array first.
bool Context::evictEldest() {
  uint64_t best = 0;
  Entry* pick = nullptr;
  for (auto& kv : table_) {
    Entry& e = kv.second;
    if (e.count != 0 || !e.dev || (e.st != Status::Clean && e.st != Status::Dirty) || !taskDone(e)) continue;
    if (!pick || e.stamp < best) {
      pick = &e;
      best = e.stamp;
    }
  }
  if (!pick) return false;
  if (pick->st == Status::Dirty && pick->host) copyFromDevice(pick->host, pick->dev, pick->bytes);
  if (flag(kDumpGc))
    fprintf(stderr, "[acchip] gc: evict %zu bytes (%s)\n", pick->bytes, pick->st == Status::Dirty ? "copied back" : "clean");
  free(pick->dev);
  stats.arraysEvicted++;
  pick->dev = nullptr;
  pick->st = Status::Evicted;
  return true;
}

bool Context::tableMalloc(uint64_t id, void* host, size_t bytes, bool frozen) {
  if (!hasMemory()) throw Error("no device");
  {
    std::lock_guard<std::mutex> g(tableMu_);
    if (table_.count(id)) return false;
  }
  void* dev = poolMalloc(bytes, true);  // (not under the table's lock: eviction takes it)
  if (!dev) throw Error("Remote memory exhausted");
  std::lock_guard<std::mutex> g(tableMu_);
  Entry e;
  e.dev = dev;
  e.bytes = bytes;
  e.host = host;
  e.st = frozen ? Status::Clean : Status::Dirty;
  e.stamp = ++clock_;
  if (!table_.emplace(id, e).second) {  // someone else was quicker
    free(dev);
    return false;
  }
  return true;
}

void* Context::tableUse(uint64_t id) {
  {
    std::lock_guard<std::mutex> g(tableMu_);
    auto it = table_.find(id);
    if (it == table_.end()) return nullptr;
    Entry& e = it->second;
    ++e.count;  // from here on it cannot be evicted
    if (e.dev) return e.dev;
    if (e.st != Status::Evicted) throw Error("internal error: non-evicted array has been lost");
  }
  // evicted: a new block, filled from the host array, which holds the current contents
  // (withRemote / copyBack, LRU.hs:140-207)
  size_t bytes;
  void* host;
  {
    std::lock_guard<std::mutex> g(tableMu_);
    Entry& e = table_.at(id);
    bytes = e.bytes;
    host = e.host;
  }
  void* dev = poolMalloc(bytes, true);
  if (!dev) {
    std::lock_guard<std::mutex> g(tableMu_);
    --table_.at(id).count;
    throw Error("Remote memory exhausted");
  }
  if (host) poke(dev, host, bytes);
  std::lock_guard<std::mutex> g(tableMu_);
  Entry& e = table_.at(id);
  if (e.dev) {  // a concurrent use uploaded it meanwhile
    free(dev);
    return e.dev;
  }
  e.dev = dev;
  e.st = Status::Clean;
  return dev;
}

void Context::tableRelease(uint64_t id) {
  std::lock_guard<std::mutex> g(tableMu_);
  auto it = table_.find(id);
  if (it == table_.end()) return;
  Entry& e = it->second;
  if (e.count > 0) --e.count;
  e.stamp = ++clock_;
  if (device_ >= 0) {  // everything queued so far may still read or write the block
    if (!e.task) hipCheck(hipEventCreateWithFlags(&e.task, hipEventDisableTiming), "hipEventCreate");
    hipCheck(hipEventRecord(e.task, stream_), "hipEventRecord");
  }
}

void Context::tableFree(uint64_t id) {
  std::lock_guard<std::mutex> g(tableMu_);
  auto it = table_.find(id);
  if (it == table_.end()) return;
  Entry& e = it->second;
  if (e.dev && e.st != Status::Unmanaged) free(e.dev);  // to the free list of its size (one stream: reuse is ordered)
  if (e.task) (void)hipEventDestroy(e.task);
  table_.erase(it);
}

void Context::tableInsertUnmanaged(uint64_t id, void* dev) {
  std::lock_guard<std::mutex> g(tableMu_);
  Entry e;
  e.dev = dev;
  e.st = Status::Unmanaged;
  e.stamp = ++clock_;
  table_[id] = e;
}

void Context::tableAdopt(uint64_t id, void* host, size_t bytes, void* dev, bool clean) {
  if (blockSize(dev) < bytes) throw Error("table adopt: not a live block of this context's pool, or too small");
  std::lock_guard<std::mutex> g(tableMu_);
  if (table_.count(id)) throw Error("table adopt: the id is already in the table");
  Entry e;
  e.dev = dev;
  e.bytes = bytes;
  e.host = host;
  e.st = clean ? Status::Clean : Status::Dirty;
  e.stamp = ++clock_;
  table_.emplace(id, e);
}

void Context::tableReclaim() {
  if (cleanHook) cleanHook();
  if (device_ >= 0) (void)hipStreamSynchronize(stream_);
  purge();
}

int Context::tableStatus(uint64_t id) {
  std::lock_guard<std::mutex> g(tableMu_);
  auto it = table_.find(id);
  return it == table_.end() ? -1 : (int)it->second.st;
}

// ------------------------------------------------------------------------------------
// transfers

void Context::ensureStaging() {
  if (staging_[0]) return;
  for (int b = 0; b < 2; ++b) {
    hipCheck(hipHostMalloc(&staging_[b], kStagePiece, hipHostMallocDefault), "hipHostMalloc");
    stats.rawAllocs++;
    hipCheck(hipEventCreateWithFlags(&stagingDone_[b], hipEventDisableTiming), "hipEventCreate");
  }
}

// Pageable host memory goes through two pinned buffers of 32 MiB in turn: while one piece is
// on the wire the host copies the next one into (or the previous one out of) the other buffer.
void Context::poke(void* dev, const void* host, size_t bytes) {
  if (bytes == 0) return;
  if (fakeMemory_) {
    std::memcpy(dev, host, bytes);
    stats.bytesCopiedToRemote += (long long)bytes;
    return;
  }
  if (device_ < 0) throw Error("no device");
  std::lock_guard<std::mutex> g(stagingMu_);
  ensureStaging();
  const char* src = static_cast<const char*>(host);
  char* dst = static_cast<char*>(dev);
  int b = 0;
  bool used[2] = {false, false};
  for (size_t off = 0; off < bytes; off += kStagePiece, b ^= 1) {
    const size_t n = bytes - off < kStagePiece ? bytes - off : kStagePiece;
    if (used[b]) hipCheck(hipEventSynchronize(stagingDone_[b]), "hipEventSynchronize");  // its last copy has left
    std::memcpy(staging_[b], src + off, n);
    hipCheck(hipMemcpyAsync(dst + off, staging_[b], n, hipMemcpyHostToDevice, stream_), "hipMemcpyAsync(H2D)");
    hipCheck(hipEventRecord(stagingDone_[b], stream_), "hipEventRecord");
    used[b] = true;
  }
  for (int k = 0; k < 2; ++k)
    if (used[k]) hipCheck(hipEventSynchronize(stagingDone_[k]), "hipEventSynchronize");  // the buffers are free again
  stats.bytesCopiedToRemote += (long long)bytes;
}

void Context::peek(void* host, const void* dev, size_t bytes) {
  copyFromDevice(host, dev, bytes);
  raiseDeviceError();
}

// The copy alone: what eviction uses to write a Dirty block back.  An error that an earlier
// kernel left in the error word stays there for the next call that waits for the stream on the
// caller's behalf -- raised from inside an allocation it would come back as "out of memory".
void Context::copyFromDevice(void* host, const void* dev, size_t bytes) {
  if (bytes == 0) return;
  if (fakeMemory_) {
    std::memcpy(host, dev, bytes);
    stats.bytesCopiedFromRemote += (long long)bytes;
    return;
  }
  if (device_ < 0) throw Error("no device");
  {
    std::lock_guard<std::mutex> g(stagingMu_);
    ensureStaging();
    char* dst = static_cast<char*>(host);
    const char* src = static_cast<const char*>(dev);
    const size_t pieces = (bytes + kStagePiece - 1) / kStagePiece;
    auto len = [&](size_t k) { return bytes - k * kStagePiece < kStagePiece ? bytes - k * kStagePiece : kStagePiece; };
    auto start = [&](size_t k) {
      hipCheck(hipMemcpyAsync(staging_[k & 1], src + k * kStagePiece, len(k), hipMemcpyDeviceToHost, stream_), "hipMemcpyAsync(D2H)");
      hipCheck(hipEventRecord(stagingDone_[k & 1], stream_), "hipEventRecord");
    };
    start(0);
    for (size_t k = 0; k < pieces; ++k) {
      if (k + 1 < pieces) start(k + 1);  // the next piece travels while this one is copied out
      hipCheck(hipEventSynchronize(stagingDone_[k & 1]), "hipEventSynchronize");
      std::memcpy(dst + k * kStagePiece, staging_[k & 1], len(k));
    }
  }
  stats.bytesCopiedFromRemote += (long long)bytes;
}

void Context::copy(void* dst, const void* src, size_t bytes) {
  if (bytes == 0) return;
  hipCheck(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, stream_), "hipMemcpyAsync(D2D)");
}

void Context::fill0(void* dev, size_t bytes) {
  if (bytes == 0) return;
  hipCheck(hipMemsetAsync(dev, 0, bytes, stream_), "hipMemsetAsync");
}

void Context::sync() {
  if (device_ >= 0) hipCheck(hipStreamSynchronize(stream_), "hipStreamSynchronize");
  raiseDeviceError();
}

unsigned* Context::errorWord() {
  if (!errDev_) {
    hipCheck(hipHostMalloc((void**)&errHost_, 64, hipHostMallocMapped), "hipHostMalloc(error word)");
    stats.rawAllocs++;
    *errHost_ = 0;
    hipCheck(hipHostGetDevicePointer((void**)&errDev_, errHost_, 0), "hipHostGetDevicePointer");
  }
  return errDev_;
}

// call after the stream has been waited for
void Context::raiseDeviceError() {
  if (!errHost_) return;
  const unsigned code = __atomic_exchange_n(errHost_, 0u, __ATOMIC_ACQ_REL);
  if (code == 1) throw Error("empty segment");  // foldSegOp / fold1SegOp, Interpreter.hs:407, 424
  if (code == 2) throw Error("index out of bounds");  // permute target, Shape.hs:98-106
  if (code == 3) throw Error("internal error: a scan tile gave up waiting for its predecessors (ticket count out of step)");
  if (code == 4) throw Error("internal error: a permute update gave up waiting for its destination's lock");
  if (code == 5) throw Error("internal error: a counting permute relieved more counters than its list holds");
  if (code != 0) throw Error("a kernel reported error " + std::to_string(code));
}

ScanState& Context::scanState(size_t descBytes) {
  if (!scan_.ticket) {
    hipCheck(hipMalloc((void**)&scan_.ticket, 256), "hipMalloc(scan ticket)");
    stats.rawAllocs++;
    hipCheck(hipMemsetAsync(scan_.ticket, 0, 256, stream_), "hipMemsetAsync");
    scan_.ticketBase = 0;
  }
  if (descBytes > scan_.descBytes) {
    if (scan_.desc) {
      hipCheck(hipStreamSynchronize(stream_), "hipStreamSynchronize");
      (void)hipFree(scan_.desc);
    }
    size_t n = std::max(descBytes, (size_t)4 << 20);
    hipCheck(hipMalloc(&scan_.desc, n), "hipMalloc(scan descriptors)");
    stats.rawAllocs++;
    hipCheck(hipMemsetAsync(scan_.desc, 0, n, stream_), "hipMemsetAsync");
    scan_.descBytes = n;
    scan_.epoch = 0;
  }
  if (++scan_.epoch >= (1u << 30)) {  // wrapped: stale tags could alias, start over from a clean slate
    hipCheck(hipMemsetAsync(scan_.desc, 0, scan_.descBytes, stream_), "hipMemsetAsync");
    scan_.epoch = 1;
  }
  return scan_;
}

// ------------------------------------------------------------------------------------
// kernels

static bool readFile(const std::string& path, std::string& out) {
  std::ifstream f(path, std::ios::binary);
  if (!f) return false;
  out.assign(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
  return true;
}

static void writeFile(const std::string& path, const std::string& data) {
  static std::atomic<unsigned long> serial{0};  // several writers in one process get a file each
  std::string tmp = path + ".tmp" + std::to_string((long long)getpid()) + "." + std::to_string(serial++);
  {
    std::ofstream f(tmp, std::ios::binary);
    if (!f) return;
    f.write(data.data(), (std::streamsize)data.size());
    if (!f) return;
  }
  std::rename(tmp.c_str(), path.c_str());
}

static std::string compileHipRTC(const std::string& source, bool fastMath, std::string& log) {
  const std::vector<const char*> opts = compileOptions(fastMath);
  hiprtcProgram prog;
  if (hiprtcCreateProgram(&prog, source.c_str(), "acchip_kernel.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS)
    throw Error("hiprtcCreateProgram failed");
  hiprtcResult r = hiprtcCompileProgram(prog, (int)opts.size(), const_cast<const char**>(opts.data()));
  size_t ls = 0;
  hiprtcGetProgramLogSize(prog, &ls);
  log.assign(ls, '\0');
  if (ls) hiprtcGetProgramLog(prog, &log[0]);
  if (r != HIPRTC_SUCCESS) {
    hiprtcDestroyProgram(&prog);
    throw Error(std::string("hipRTC compilation failed: ") + hiprtcGetErrorString(r) + "\n" + log);
  }
  size_t cs = 0;
  hiprtcGetCodeSize(prog, &cs);
  std::string code(cs, '\0');
  hiprtcGetCode(prog, &code[0]);
  hiprtcDestroyProgram(&prog);
  return code;
}

// Extra preprocessor definitions for generated kernels (tuning experiments):
// ACCHIP_DEFINES="NAME=VALUE NAME2" becomes #define lines in front of the source, and so
// takes part in the cache key.
static std::string definesPrefix() {
  const char* d = std::getenv("ACCHIP_DEFINES");
  std::string out;
  if (!d) return out;
  std::string tok;
  for (const char* p = d;; ++p) {
    if (*p == ' ' || *p == '\0') {
      if (!tok.empty()) {
        size_t eq = tok.find('=');
        out += "#define " + (eq == std::string::npos ? tok : tok.substr(0, eq) + " " + tok.substr(eq + 1)) + "\n";
        tok.clear();
      }
      if (!*p) break;
    } else {
      tok += *p;
    }
  }
  return out;
}

// limits the hipRTC compilations that run at the same time
namespace {
std::mutex g_slotMu;
std::condition_variable g_slotCv;
int g_slotsFree = -1;
struct CompileSlot {
  CompileSlot() {
    std::unique_lock<std::mutex> l(g_slotMu);
    if (g_slotsFree < 0) {
      long n = sysconf(_SC_NPROCESSORS_ONLN);
      const char* e = std::getenv("ACCHIP_COMPILE_JOBS");
      if (e) n = std::atol(e);
      g_slotsFree = (int)std::max<long>(1, std::min<long>(n, 16));
    }
    g_slotCv.wait(l, [] { return g_slotsFree > 0; });
    --g_slotsFree;
  }
  ~CompileSlot() {
    {
      std::lock_guard<std::mutex> l(g_slotMu);
      ++g_slotsFree;
    }
    g_slotCv.notify_one();
  }
};
}  // namespace

KernelP Context::kernel(const KernelSource& ks0) {
  KernelSource ks = ks0;
  ks.source = definesPrefix() + ks0.source;
  std::string keyText = ks.source;
  const bool fastMath = flag(kFastMath);
  for (const char* o : compileOptions(fastMath)) keyText += std::string("\n//opt ") + o;
  int major = 0, minor = 0;
  hiprtcVersion(&major, &minor);
  keyText += "\n//hiprtc " + std::to_string(major) + "." + std::to_string(minor);
  std::string hash = sha3_256_hex(keyText);
  {
    std::lock_guard<std::mutex> g(mu_);
    auto it = kernels_.find(hash);
    if (it != kernels_.end()) {
      stats.kernelsFromMemory++;
      return it->second;
    }
  }
  auto k = std::make_shared<Kernel>();
  k->hash = hash;
  k->meta = ks;
  k->meta.source.clear();
  std::string path = cacheDir + "/" + hash + ".hsaco";
  if (flag(kDumpCc)) fprintf(stderr, "[acchip] kernel %s\n%s\n", hash.c_str(), ks.source.c_str());
  // a cached code object must at least look like one (an ELF image); anything else is compiled anew
  const bool fromDisk =
      !flag(kForceRecomp) && readFile(path, k->code) && k->code.size() > 64 && k->code.compare(0, 4, "\177ELF") == 0;
  // Two threads may miss on the same key: the one that enters the table first owns the
  // compilation, the other takes its kernel.  The worker is started under the lock, after the
  // entry is in the table, so no kernel with a worker attached is ever dropped.
  std::lock_guard<std::mutex> g(mu_);
  auto ins = kernels_.emplace(hash, k);
  if (!ins.second) {
    stats.kernelsFromMemory++;
    return ins.first->second;
  }
  if (fromDisk) {
    stats.kernelsFromDisk++;
  } else {
    // compile on a worker thread, at most as many at once as there are cores
    stats.kernelsCompiled++;
    const bool dump = flag(kDumpCc);
    const std::string dir = cacheDir;
    k->code.clear();
    Kernel* raw = k.get();  // kept alive by kernels_ until the context goes, which waits
    k->ready = std::async(std::launch::async, [raw, src = ks.source, path, dir, dump, fastMath]() {
                 CompileSlot slot;
                 std::string log;
                 raw->code = compileHipRTC(src, fastMath, log);
                 if (dump && !log.empty()) fprintf(stderr, "[acchip] hipRTC log:\n%s\n", log.c_str());
                 ::mkdir(dir.c_str(), 0777);
                 writeFile(path, raw->code);
               }).share();
  }
  return k;
}

void Context::wait(const KernelP& k) {
  if (k && k->ready.valid()) k->ready.get();
}

void Context::ensureLoaded(const KernelP& k) {
  if (k->module) return;
  wait(k);
  if (device_ < 0) throw Error("this context has no device: programs can be compiled but not executed");
  hipCheck(hipModuleLoadData(&k->module, k->code.data()), "hipModuleLoadData");
  stats.modulesLoaded++;
}

void Context::preload(const KernelP& k, std::initializer_list<const char*> fns) {
  if (!k || device_ < 0) return;
  std::lock_guard<std::mutex> g(mu_);
  ensureLoaded(k);
  for (const char* fn : fns) {
    if (k->fns.count(fn)) continue;
    hipFunction_t f;
    hipCheck(hipModuleGetFunction(&f, k->module, fn), fn);
    k->fns[fn] = f;
  }
}

int64_t Context::residentGroups(const KernelP& k, const char* fn, unsigned block) {
  if (device_ < 0) return 0;
  std::lock_guard<std::mutex> g(mu_);
  auto it = k->perCu.find(fn);
  if (it == k->perCu.end()) {
    ensureLoaded(k);
    hipFunction_t f;
    auto fi = k->fns.find(fn);
    if (fi == k->fns.end()) {
      hipCheck(hipModuleGetFunction(&f, k->module, fn), fn);
      k->fns[fn] = f;
    } else {
      f = fi->second;
    }
    int n = 0;
    if (hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&n, f, (int)block, 0) != hipSuccess) n = 0;
    it = k->perCu.emplace(fn, n).first;
  }
  int cus = cus_;
  if (cus == 0) {
    cus = 256;
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device_) == hipSuccess && v > 0) cus = v;
  }
  return (int64_t)it->second * cus;
}

void Context::launch(const KernelP& k, const char* fn, uint64_t grid, unsigned block, const std::vector<uint64_t>& args) {
  if (grid == 0) return;
  // a launch holds fewer than 2^32 threads; a count cut to 32 bits would leave part of the work undone
  if (grid > 0x7fffffffull || grid * block > 0xffffffffull)
    throw Error(std::string(fn) + ": " + std::to_string(grid) + " workgroups of " + std::to_string(block) +
                " threads exceed what one launch can hold");
  hipFunction_t f;
  {
    std::lock_guard<std::mutex> g(mu_);
    ensureLoaded(k);
    auto it = k->fns.find(fn);
    if (it == k->fns.end()) {
      hipCheck(hipModuleGetFunction(&f, k->module, fn), fn);
      k->fns[fn] = f;
    } else {
      f = it->second;
    }
  }
  size_t size = args.size() * sizeof(uint64_t);
  void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, (void*)args.data(), HIP_LAUNCH_PARAM_BUFFER_SIZE, &size,
                    HIP_LAUNCH_PARAM_END};
  if (flag(kDumpExec)) fprintf(stderr, "[acchip] launch %s<<<%llu,%u>>> %s (%zu arg bytes)\n", fn, (unsigned long long)grid, block, k->hash.substr(0, 12).c_str(), size);
  hipCheck(hipModuleLaunchKernel(f, (unsigned)grid, 1, 1, block, 1, 1, 0, stream_, nullptr, config), "hipModuleLaunchKernel");
  stats.launches++;
}

}  // namespace acchip
