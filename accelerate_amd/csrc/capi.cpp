// extern "C" boundary: see include/acchip.h for the contract of every entry point.
#include <cstring>
#include <new>

#include "../../include/acchip.h"
#include "exec.hpp"
#include "sha3.hpp"

using namespace acchip;

// Handles may be released in any order, also after acchip_shutdown: programs, arrays and
// events each hold a reference to the context, which goes away with the last of them.
struct acchip_ctx {
  std::shared_ptr<Context> ctx;
  explicit acchip_ctx(int device) : ctx(std::make_shared<Context>(device)) {}
};
struct acchip_program {
  std::shared_ptr<Context> keep;  // declared first: destroyed after prog
  Program prog;
  std::vector<std::string> keys;
  acchip_program(acchip_ctx* c, const char* t, size_t n) : keep(c->ctx), prog(*c->ctx, t, n), keys(prog.kernelKeys()) {}
};
struct acchip_array {
  AValP v;
  std::string eltText;
};
struct acchip_event {
  std::shared_ptr<Context> keep;
  hipEvent_t ev;
};

static thread_local std::string g_lastError;

static int fail(const std::exception& e) {
  g_lastError = e.what();
  const std::string& m = g_lastError;
  if (m.find("Remote memory exhausted") != std::string::npos) return ACCHIP_OUT_OF_MEMORY;
  if (m.find("no device") != std::string::npos) return ACCHIP_NO_DEVICE;
  if (m == "empty array" || m == "shape mismatch" || m == "empty segment descriptor" || m == "empty segment" ||
      m.compare(0, 19, "index out of bounds") == 0)
    return ACCHIP_BOUNDS;
  return ACCHIP_ERROR;
}
static int failMsg(const char* m) {
  g_lastError = m;
  return ACCHIP_ERROR;
}

#define ACCHIP_TRY try {
#define ACCHIP_END                                     \
  }                                                    \
  catch (const std::exception& e) { return fail(e); }  \
  catch (...) { return failMsg("unknown error"); }

extern "C" {

const char* acchip_last_error(void) { return g_lastError.c_str(); }

int acchip_init(int device, acchip_ctx** out) {
  ACCHIP_TRY
  if (!out) return failMsg("null output pointer");
  if (device >= 0) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || device >= n) {
      (void)hipGetLastError();
      g_lastError = "no device " + std::to_string(device) + " (HIP reports " + std::to_string(n) + " devices)";
      return ACCHIP_NO_DEVICE;
    }
  }
  *out = new acchip_ctx(device);
  return ACCHIP_OK;
  ACCHIP_END
}

void acchip_shutdown(acchip_ctx* ctx) { delete ctx; }

int acchip_mem_info(acchip_ctx* ctx, size_t* total, size_t* available) {
  ACCHIP_TRY
  ctx->ctx->memInfo(total, available);
  return ACCHIP_OK;
  ACCHIP_END
}

void* acchip_malloc(acchip_ctx* ctx, size_t bytes) {
  try {
    return ctx->ctx->malloc(bytes);
  } catch (...) {
    return nullptr;
  }
}
void acchip_free(acchip_ctx* ctx, void* p) {
  try {
    ctx->ctx->free(p);
  } catch (...) {
  }
}
void acchip_purge(acchip_ctx* ctx) {
  try {
    ctx->ctx->purge();
  } catch (...) {
  }
}

int acchip_poke(acchip_ctx* ctx, void* devptr, const void* host, size_t bytes) {
  ACCHIP_TRY
  ctx->ctx->poke(devptr, host, bytes);
  return ACCHIP_OK;
  ACCHIP_END
}
int acchip_peek(acchip_ctx* ctx, void* host, const void* devptr, size_t bytes) {
  ACCHIP_TRY
  ctx->ctx->peek(host, devptr, bytes);
  return ACCHIP_OK;
  ACCHIP_END
}

int acchip_table_malloc(acchip_ctx* ctx, uint64_t id, void* host, size_t bytes, int frozen, int* allocated) {
  ACCHIP_TRY
  const bool fresh = ctx->ctx->tableMalloc(id, host, bytes, frozen != 0);
  if (allocated) *allocated = fresh ? 1 : 0;
  return ACCHIP_OK;
  ACCHIP_END
}
int acchip_table_use(acchip_ctx* ctx, uint64_t id, void** devptr) {
  ACCHIP_TRY
  if (!devptr) return failMsg("null output pointer");
  *devptr = ctx->ctx->tableUse(id);
  return ACCHIP_OK;
  ACCHIP_END
}
int acchip_table_release(acchip_ctx* ctx, uint64_t id) {
  ACCHIP_TRY
  ctx->ctx->tableRelease(id);
  return ACCHIP_OK;
  ACCHIP_END
}
void acchip_table_free(acchip_ctx* ctx, uint64_t id) {
  try {
    ctx->ctx->tableFree(id);
  } catch (...) {
  }
}
int acchip_table_insert_unmanaged(acchip_ctx* ctx, uint64_t id, void* devptr) {
  ACCHIP_TRY
  ctx->ctx->tableInsertUnmanaged(id, devptr);
  return ACCHIP_OK;
  ACCHIP_END
}
int acchip_table_adopt(acchip_ctx* ctx, uint64_t id, void* host, size_t bytes, acchip_array* a, int leaf, int clean) {
  ACCHIP_TRY
  if (!a || a->v->k != AVal::Arr || leaf < 0 || leaf >= (int)a->v->arr->bufs.size())
    throw Error("table adopt: no such buffer");
  Buffer& b = *a->v->arr->bufs[leaf];
  // a buffer the handle does not own (wrapped, or adopted before through another handle) stays
  // where it is: the caller copies instead
  if (!b.owned || b.ctx != ctx->ctx) throw Error("table adopt: the array does not own this buffer");
  ctx->ctx->tableAdopt(id, host, bytes, b.p, clean != 0);
  b.owned = false;  // from here on the table frees the block
  return ACCHIP_OK;
  ACCHIP_END
}
void acchip_table_reclaim(acchip_ctx* ctx) {
  try {
    ctx->ctx->tableReclaim();
  } catch (...) {
  }
}
int acchip_table_status(acchip_ctx* ctx, uint64_t id) {
  try {
    return ctx->ctx->tableStatus(id);
  } catch (...) {
    return -1;
  }
}
int acchip_set_clean_hook(acchip_ctx* ctx, acchip_clean_fn fn, void* user) {
  ACCHIP_TRY
  if (!fn) ctx->ctx->cleanHook = nullptr;
  else ctx->ctx->cleanHook = [fn, user]() { fn(user); };
  return ACCHIP_OK;
  ACCHIP_END
}

int acchip_set_knob(acchip_ctx* ctx, const char* name, long long value) {
  ACCHIP_TRY
  if (!name || !ctx->ctx->knobs.set(name, value)) throw Error(std::string("no such knob: ") + (name ? name : "(null)"));
  return ACCHIP_OK;
  ACCHIP_END
}
int acchip_get_knob(acchip_ctx* ctx, const char* name, long long* value) {
  ACCHIP_TRY
  if (!name || !value || !ctx->ctx->knobs.get(name, *value)) throw Error(std::string("no such knob: ") + (name ? name : "(null)"));
  return ACCHIP_OK;
  ACCHIP_END
}
int acchip_set_flags(acchip_ctx* ctx, uint32_t bitfield) {
  ACCHIP_TRY
  ctx->ctx->flags = bitfield;
  return ACCHIP_OK;
  ACCHIP_END
}
uint32_t acchip_get_flags(acchip_ctx* ctx) { return ctx->ctx->flags; }

long long acchip_stat(acchip_ctx* ctx, const char* name) {
  Stats& s = ctx->ctx->stats;
  std::string n = name ? name : "";
  if (n == "bytes_allocated_remote") return s.bytesAllocated;
  if (n == "bytes_copied_to_remote") return s.bytesCopiedToRemote;
  if (n == "bytes_copied_from_remote") return s.bytesCopiedFromRemote;
  if (n == "bytes_evicted_from_remote") return s.bytesEvicted;
  if (n == "kernels_compiled") return s.kernelsCompiled;
  if (n == "kernels_from_disk") return s.kernelsFromDisk;
  if (n == "kernels_from_memory") return s.kernelsFromMemory;
  if (n == "launches") return s.launches;
  if (n == "pool_hits") return s.poolHits;
  if (n == "pool_misses") return s.poolMisses;
  if (n == "arrays_evicted") return s.arraysEvicted;
  if (n == "raw_allocs") return s.rawAllocs;
  if (n == "modules_loaded") return s.modulesLoaded;
  return -1;
}

// --- events ---------------------------------------------------------------------------

int acchip_event_record(acchip_ctx* ctx, acchip_event** out) {
  ACCHIP_TRY
  if (!ctx->ctx->hasDevice()) throw Error("no device");
  auto* e = new acchip_event{ctx->ctx, nullptr};
  hipError_t r = hipEventCreate(&e->ev);
  if (r == hipSuccess) r = hipEventRecord(e->ev, ctx->ctx->stream());
  if (r != hipSuccess) {
    delete e;
    hipCheck(r, "hipEventRecord");
  }
  *out = e;
  return ACCHIP_OK;
  ACCHIP_END
}
int acchip_event_query(acchip_event* ev, int* completed) {
  ACCHIP_TRY
  hipError_t r = hipEventQuery(ev->ev);
  if (r == hipSuccess) *completed = 1;
  else if (r == hipErrorNotReady) {
    (void)hipGetLastError();
    *completed = 0;
  } else hipCheck(r, "hipEventQuery");
  return ACCHIP_OK;
  ACCHIP_END
}
int acchip_event_sync(acchip_event* ev) {
  ACCHIP_TRY
  hipCheck(hipEventSynchronize(ev->ev), "hipEventSynchronize");
  return ACCHIP_OK;
  ACCHIP_END
}
int acchip_event_elapsed_ms(acchip_event* start, acchip_event* stop, float* ms) {
  ACCHIP_TRY
  hipCheck(hipEventElapsedTime(ms, start->ev, stop->ev), "hipEventElapsedTime");
  return ACCHIP_OK;
  ACCHIP_END
}
void acchip_event_destroy(acchip_event* ev) {
  if (!ev) return;
  (void)hipEventDestroy(ev->ev);
  delete ev;
}
int acchip_sync(acchip_ctx* ctx) {
  ACCHIP_TRY
  ctx->ctx->sync();
  return ACCHIP_OK;
  ACCHIP_END
}

// --- arrays ---------------------------------------------------------------------------

static acchip_array* wrapVal(AValP v) {
  auto* a = new acchip_array();
  a->v = std::move(v);
  if (a->v->k == AVal::Arr) a->eltText = typeStr(a->v->arr->r.elt);
  return a;
}

static DArrayP describe(int rank, const int64_t* shape, const char* elt) {
  if (rank < 0 || rank > ACCHIP_MAX_RANK) throw Error("array rank out of range");
  auto d = std::make_shared<DArray>();
  d->r.rank = rank;
  Sx t = parseSx(elt, std::strlen(elt));
  d->r.elt = parseType(t);
  for (int i = 0; i < rank; ++i) d->shape.push_back(shape[i]);
  return d;
}

int acchip_array_wrap(acchip_ctx* ctx, int rank, const int64_t* shape, const char* elt_type, void* const* buffers,
                      int n_buffers, acchip_array** out) {
  ACCHIP_TRY
  DArrayP d = describe(rank, shape, elt_type);
  auto leaves = typeLeaves(d->r.elt);
  if ((int)leaves.size() != n_buffers) throw Error("array_wrap: one buffer per scalar leaf of the element type is required");
  int64_t n = d->size();
  for (int i = 0; i < n_buffers; ++i) {
    auto b = std::make_shared<Buffer>();
    b->ctx = ctx->ctx;
    b->p = buffers[i];
    b->bytes = (size_t)n * stSize(leaves[i]);
    b->owned = false;
    if (!b->p && n > 0) throw Error("array_wrap: null device pointer");
    d->bufs.push_back(b);
  }
  auto v = std::make_shared<AVal>();
  v->k = AVal::Arr;
  v->arr = d;
  *out = wrapVal(v);
  return ACCHIP_OK;
  ACCHIP_END
}

int acchip_array_new(acchip_ctx* ctx, int rank, const int64_t* shape, const char* elt_type, acchip_array** out) {
  ACCHIP_TRY
  if (!ctx->ctx->hasMemory()) throw Error("no device");
  DArrayP d = describe(rank, shape, elt_type);
  int64_t n = d->size();
  for (ST st : typeLeaves(d->r.elt)) {
    auto b = std::make_shared<Buffer>();
    b->ctx = ctx->ctx;
    b->bytes = (size_t)n * stSize(st);
    b->p = ctx->ctx->malloc(b->bytes);
    if (!b->p) throw Error("Remote memory exhausted");
    b->owned = true;
    d->bufs.push_back(b);
  }
  auto v = std::make_shared<AVal>();
  v->k = AVal::Arr;
  v->arr = d;
  *out = wrapVal(v);
  return ACCHIP_OK;
  ACCHIP_END
}

int acchip_array_pair(acchip_array* a, acchip_array* b, acchip_array** out) {
  ACCHIP_TRY
  auto v = std::make_shared<AVal>();
  v->k = AVal::Pair;
  v->a = a->v;
  v->b = b->v;
  *out = wrapVal(v);
  return ACCHIP_OK;
  ACCHIP_END
}
int acchip_array_unit(acchip_array** out) {
  ACCHIP_TRY
  *out = wrapVal(std::make_shared<AVal>());
  return ACCHIP_OK;
  ACCHIP_END
}
int acchip_array_kind(const acchip_array* a) { return (int)a->v->k; }
int acchip_array_fst(const acchip_array* a, acchip_array** out) {
  ACCHIP_TRY
  if (a->v->k != AVal::Pair) throw Error("array_fst: not a pair");
  *out = wrapVal(a->v->a);
  return ACCHIP_OK;
  ACCHIP_END
}
int acchip_array_snd(const acchip_array* a, acchip_array** out) {
  ACCHIP_TRY
  if (a->v->k != AVal::Pair) throw Error("array_snd: not a pair");
  *out = wrapVal(a->v->b);
  return ACCHIP_OK;
  ACCHIP_END
}
int acchip_array_rank(const acchip_array* a) { return a->v->k == AVal::Arr ? a->v->arr->r.rank : -1; }
int acchip_array_shape(const acchip_array* a, int64_t* shape_out) {
  ACCHIP_TRY
  if (a->v->k != AVal::Arr) throw Error("array_shape: not a single array");
  for (size_t i = 0; i < a->v->arr->shape.size(); ++i) shape_out[i] = a->v->arr->shape[i];
  return ACCHIP_OK;
  ACCHIP_END
}
int acchip_array_num_buffers(const acchip_array* a) { return a->v->k == AVal::Arr ? (int)a->v->arr->bufs.size() : -1; }
void* acchip_array_buffer(const acchip_array* a, int leaf) {
  if (a->v->k != AVal::Arr || leaf < 0 || leaf >= (int)a->v->arr->bufs.size()) return nullptr;
  return a->v->arr->bufs[leaf]->p;
}
size_t acchip_array_buffer_bytes(const acchip_array* a, int leaf) {
  if (a->v->k != AVal::Arr || leaf < 0 || leaf >= (int)a->v->arr->bufs.size()) return 0;
  return a->v->arr->bufs[leaf]->bytes;
}
const char* acchip_array_elt_type(const acchip_array* a) { return a->eltText.c_str(); }
void acchip_array_release(acchip_array* a) { delete a; }

// --- programs -------------------------------------------------------------------------

int acchip_compile(acchip_ctx* ctx, const char* program_text, size_t length, acchip_program** out) {
  ACCHIP_TRY
  if (!program_text || !out) return failMsg("null argument");
  *out = new acchip_program(ctx, program_text, length);
  return ACCHIP_OK;
  ACCHIP_END
}
void acchip_program_release(acchip_program* p) { delete p; }
int acchip_program_arity(const acchip_program* p) { return (int)p->prog.argTypes.size(); }
int acchip_program_num_kernels(const acchip_program* p) { return (int)p->keys.size(); }
const char* acchip_program_kernel_key(const acchip_program* p, int k) {
  return k >= 0 && k < (int)p->keys.size() ? p->keys[k].c_str() : nullptr;
}

int acchip_sha3_256(const void* data, size_t length, uint8_t digest[32]) {
  ACCHIP_TRY
  sha3_256(data, length, digest);
  return ACCHIP_OK;
  ACCHIP_END
}

int acchip_set_trace(acchip_ctx* ctx, acchip_trace_fn fn, void* user) {
  ACCHIP_TRY
  if (!fn) {
    ctx->ctx->traceSink = nullptr;
  } else {
    ctx->ctx->traceSink = [fn, user](const std::string& msg, const std::shared_ptr<void>& arrays) {
      acchip_array* h = wrapVal(std::static_pointer_cast<AVal>(arrays));
      fn(user, msg.c_str(), h);
      delete h;
    };
  }
  return ACCHIP_OK;
  ACCHIP_END
}

int acchip_execute(acchip_ctx* ctx, acchip_program* p, acchip_array* const* args, int n_args,
                   acchip_array* const* uses, int n_uses, acchip_array** result) {
  ACCHIP_TRY
  if (!ctx->ctx->hasDevice()) throw Error("no device");
  if (p->keep != ctx->ctx) throw Error("program was compiled in a different context");
  std::vector<AValP> av;
  for (int i = 0; i < n_args; ++i) av.push_back(args[i]->v);
  std::vector<DArrayP> uv;
  for (int i = 0; i < n_uses; ++i) {
    if (uses[i]->v->k != AVal::Arr) throw Error("use slots take single arrays");
    uv.push_back(uses[i]->v->arr);
  }
  *result = wrapVal(p->prog.run(av, uv));
  return ACCHIP_OK;
  ACCHIP_END
}

int acchip_execute_into(acchip_ctx* ctx, acchip_program* p, acchip_array* const* args, int n_args,
                        acchip_array* const* uses, int n_uses, acchip_array* result) {
  ACCHIP_TRY
  if (!ctx->ctx->hasDevice()) throw Error("no device");
  if (p->keep != ctx->ctx) throw Error("program was compiled in a different context");
  if (!result) throw Error("acchip_execute_into: null result array");
  std::vector<AValP> av;
  for (int i = 0; i < n_args; ++i) av.push_back(args[i]->v);
  std::vector<DArrayP> uv;
  for (int i = 0; i < n_uses; ++i) {
    if (uses[i]->v->k != AVal::Arr) throw Error("use slots take single arrays");
    uv.push_back(uses[i]->v->arr);
  }
  p->prog.runInto(av, uv, result->v);
  return ACCHIP_OK;
  ACCHIP_END
}

}  // extern "C"
