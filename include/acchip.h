/* acchip -- C ABI of the MI355X (gfx950) execution backend for Accelerate programs.
 *
 * This is the boundary a `Data.Array.Accelerate.HIP` module binds with `foreign import
 * ccall`: it stands where the reference's own backend stands, below the optimiser
 * (`Trafo.convertAfun`) and behind `run / run1 / runN`
 * (src/Data/Array/Accelerate/Interpreter.hs:93-126).  Citations name the reference
 * interface each entry point replaces; paths are relative to
 * src/Data/Array/Accelerate/ of the reference.
 *
 * Conventions: every function that can fail returns 0 on success and a non-zero code on
 * failure, in which case acchip_last_error() describes the failure (thread-local
 * string).  No C++ exception crosses the boundary.  All handles are opaque.  Nothing in
 * this library falls back to a CPU implementation: without a GPU, programs can be
 * compiled (code generation + hipRTC for gfx950) but execution entry points fail.
 */
#ifndef ACCHIP_H
#define ACCHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ACCHIP_MAX_RANK 8

typedef struct acchip_ctx acchip_ctx;         /* device + stream + memory pool + kernel cache */
typedef struct acchip_program acchip_program; /* a prepared array function (result of runN f) */
typedef struct acchip_array acchip_array;     /* a device-resident array (or tuple of arrays) */
typedef struct acchip_event acchip_event;     /* a point in the context's stream */

/* error codes */
enum {
  ACCHIP_OK = 0,
  ACCHIP_ERROR = 1,          /* malformed program, type error, internal error: see last_error */
  ACCHIP_NO_DEVICE = 2,      /* the context owns no GPU */
  ACCHIP_OUT_OF_MEMORY = 3,  /* "Remote memory exhausted", Array/Remote/LRU.hs:250-341 */
  ACCHIP_BOUNDS = 4          /* a condition the reference reports via boundsCheck (Error.hs:33-62):
                                empty fold1, shape mismatch in reshape, empty segment descriptor */
};

const char* acchip_last_error(void);

/* --- context ---------------------------------------------------------------------- */

/* Create a context on HIP device `device` (one stream, default priority).  device = -1
 * creates a compile-only context.  device = -2 creates a compile-only context in which host
 * memory stands in for device memory, so that the memory manager below (pool, array table,
 * eviction) can be exercised without a GPU; it cannot run programs either.  Replaces the
 * implicit global state of the reference interpreter; a compiling backend creates this once
 * per process.  ACCHIP_POOL_LIMIT=<bytes> in the environment caps what a context takes from
 * its device, as if the device were that small. */
int acchip_init(int device, acchip_ctx** out);
/* Gives up the caller's handle.  Arrays, programs and events made in the context keep it
 * alive and may be released afterwards, in any order (GHC finalisers run in any order,
 * Array/Remote/Table.hs:116-128); the device resources go with the last of them. */
void acchip_shutdown(acchip_ctx* ctx);

/* totalRemoteMem / availableRemoteMem of class RemoteMemory (Array/Remote/Class.hs:47-73). */
int acchip_mem_info(acchip_ctx* ctx, size_t* total, size_t* available);

/* mallocRemote (Array/Remote/Class.hs:52-54): returns NULL when the device is exhausted
 * even after releasing the pool's free lists (Array/Remote/Table.hs:194-211); never
 * aborts.  Thread-safe; may be called from finaliser threads. */
void* acchip_malloc(acchip_ctx* ctx, size_t bytes);
/* freeRemote; the block returns to the pool's free list of its size class
 * (Array/Remote/Nursery.hs:43-113). */
void acchip_free(acchip_ctx* ctx, void* devptr);
/* Release every block waiting in the free lists (Table.purge, Table.hs:341-348). */
void acchip_purge(acchip_ctx* ctx);

/* pokeRemote / peekRemote (Array/Remote/Class.hs:56-62): host <-> device copies through
 * two pinned staging buffers in turn on the context's stream.  poke is stream-ordered and returns
 * once the host buffer may be reused; peek returns once the data is in `host`. */
int acchip_poke(acchip_ctx* ctx, void* devptr, const void* host, size_t bytes);
int acchip_peek(acchip_ctx* ctx, void* host, const void* devptr, size_t bytes);

/* --- array table: Array/Remote/LRU.hs (on top of Table.hs and Nursery.hs) ------------- */

/* The reference keeps, per host array, the device block that mirrors it, evicts the least
 * recently used ones when the device is full and uploads them again on their next use.  Here
 * the host array is named by an id the caller chooses (the reference's StableArray is the
 * array's Unique, Array/Unique.hs:48-51) and described by its pinned host address and size.
 *
 * acchip_table_malloc: LRU.malloc (LRU.hs:225-248).  Allocates the block if the id is new
 * (*allocated = 1) and is a no-op otherwise (*allocated = 0).  frozen != 0: the host copy
 * stays valid (Clean), so eviction just drops the block; otherwise the device copy is taken
 * to be the newer one (Dirty) and eviction copies it back to `host` first.  When memory runs
 * out the ladder of Table.hs:194-211 and LRU.hs:250-341 runs: free list, device, clean hook
 * + free list, purge + device, then eviction of the eldest arrays not in use, one by one;
 * ACCHIP_OUT_OF_MEMORY ("Remote memory exhausted") only when all of that fails. */
int acchip_table_malloc(acchip_ctx* ctx, uint64_t id, void* host, size_t bytes, int frozen, int* allocated);
/* LRU.withRemote (LRU.hs:140-207), split in two: acchip_table_use pins the array and yields
 * its device pointer, uploading the host copy again if it had been evicted (*devptr = NULL
 * with ACCHIP_OK: the id was never allocated -- withRemote's Nothing); acchip_table_release
 * ends the use, stamps the array as most recently used and remembers the point the stream
 * has reached (the `Task` of LRU.hs:105-110): the array cannot be evicted before that work
 * has finished. */
int acchip_table_use(acchip_ctx* ctx, uint64_t id, void** devptr);
int acchip_table_release(acchip_ctx* ctx, uint64_t id);
/* The host array died (the finaliser of Table.insert, Table.hs:247-265): its block goes to
 * the free list of its size.  Thread-safe; may be called from finaliser threads. */
void acchip_table_free(acchip_ctx* ctx, uint64_t id);
/* Table.insertUnmanaged (Table.hs:293-311): memory the caller owns; never evicted or freed. */
int acchip_table_insert_unmanaged(acchip_ctx* ctx, uint64_t id, void* devptr);
/* A buffer the library allocated (leaf `leaf` of a result of acchip_execute, or of an array made
 * by acchip_array_new) becomes the device copy of host array `id`: what a backend does when it
 * hands a result to the caller without copying it back at once, or after it has (the reference
 * keeps results in its table the same way, LRU.malloc followed by the kernel's writes).
 * clean != 0: `host` already holds the same data; otherwise the device copy is the newer one and
 * eviction writes it to `host`.  The handle stops owning the buffer and may be released; fails if
 * it does not own it (wrapped memory, or adopted before). */
int acchip_table_adopt(acchip_ctx* ctx, uint64_t id, void* host, size_t bytes, acchip_array* a, int leaf, int clean);
/* LRU.reclaim / Table.reclaim: run the clean hook and release the free lists. */
void acchip_table_reclaim(acchip_ctx* ctx);
/* -1: unknown id; 0 Clean, 1 Dirty, 2 Unmanaged, 3 Evicted (data Status, LRU.hs:81-86). */
int acchip_table_status(acchip_ctx* ctx, uint64_t id);
/* Table.clean (Table.hs:313-339) needs the caller's garbage collector: the hook is called when
 * the device is full, before anything is purged or evicted; a Haskell caller passes performGC,
 * whose finalisers then call acchip_table_free. */
typedef void (*acchip_clean_fn)(void* user);
int acchip_set_clean_hook(acchip_ctx* ctx, acchip_clean_fn fn, void* user);

/* Launch-time choices (kernel variant selection, thresholds) that tests and tuning override:
 * read from the environment once, when the context is made (ACCHIP_STREAM_BYTES, ACCHIP_SCAN_TILES,
 * ...: the name in capitals), and changed afterwards only here.  Names: stream_bytes,
 * map_max_blocks, map_tiled, fold_rows, fold_target, fold_max_blocks, permute_parts, permute_count, permute_groups,
 * permute_partials, permute_fresh, stencil_chain, stencil_no2d, stencil_no3d (these two take effect for programs
 * compiled afterwards), scan_tiles (0 automatic, 1 large, 2 small, 3 rows, 4 pipelined), scan_spin_limit,
 * scan_test_skew, scan_ticketless (0: the tiles of a scan always take their numbers from the counter),
 * scan_post (0: the function of a map around a scan is never applied by the scan itself; read by acchip_compile),
 * fold_staged (0: folds under operators that are not commutative never stage blocks of tiles in LDS),
 * fold_one_launch and foldseg_one_launch (0: the work that rides behind the main launch
 * takes a launch of its own), pool_async (0: plain hipMalloc / hipFree under the pool).  Fails for a name
 * it does not know.  No counterpart in the reference. */
int acchip_set_knob(acchip_ctx* ctx, const char* name, long long value);
int acchip_get_knob(acchip_ctx* ctx, const char* name, long long* value);
/* The reference's option word (cbits/flags.h:19-49: `__cmd_line_flags.bitfield`), of which a
 * backend honours: inplace (bit 4: off = permute always copies its defaults), fast_math (bit 5: on =
 * kernels compiled afterwards may contract and reassociate floating point), fast_permute_const
 * (bit 6: see below), force_recomp (bit 7), dump_gc (bit 18), dump_cc (bit 20), dump_exec (bit 23).
 * A context starts from the defaults of cbits/flags.c:37 (inplace and fast_permute_const on,
 * fast_math off for bit-wise parity) adjusted by the names in $ACCHIP_FLAGS (dump-cc, dump-exec,
 * dump-gc, force-recomp, fast-math, no-inplace, no-fast-permute-const).  fast_permute_const: a
 * permute whose combination ignores the old value (`const`) is written with plain stores; off, its
 * targets are taken to collide and the stores go through per-element locks, so that every element
 * holds one complete source value (Language.hs:786-790). */
int acchip_set_flags(acchip_ctx* ctx, uint32_t bitfield);
uint32_t acchip_get_flags(acchip_ctx* ctx);

/* Counters with the meaning of cbits/monitoring.c:26-32 plus kernel-cache statistics.
 * names: "bytes_allocated_remote", "bytes_copied_to_remote", "bytes_copied_from_remote",
 * "bytes_evicted_from_remote", "kernels_compiled", "kernels_from_disk",
 * "kernels_from_memory", "launches", "pool_hits", "pool_misses", "arrays_evicted".  Unknown
 * name: -1. */
long long acchip_stat(acchip_ctx* ctx, const char* name);

/* --- events: `Task` of Array/Remote/LRU.hs:105-110 --------------------------------- */

int acchip_event_record(acchip_ctx* ctx, acchip_event** out); /* record on the stream */
int acchip_event_query(acchip_event* ev, int* completed);     /* Task.completed */
int acchip_event_sync(acchip_event* ev);
int acchip_event_elapsed_ms(acchip_event* start, acchip_event* stop, float* ms);
void acchip_event_destroy(acchip_event* ev);
/* Wait for everything queued on the context's stream.  Conditions that only a kernel can see and
 * that the reference reports through boundsCheck (Error.hs:33-62; "empty segment" of fold1Seg,
 * Interpreter.hs:424; "index out of bounds" for a permute target outside the destination, which
 * is not written) are raised here and by acchip_peek, i.e. by the first call after the
 * offending launch that waits for the stream: it fails with that message. */
int acchip_sync(acchip_ctx* ctx);

/* --- arrays ------------------------------------------------------------------------ */

/* Describe an array whose buffers the caller owns (e.g. blocks its memory table got from
 * acchip_malloc): rank, extents (outermost first, row-major: Representation/Shape.hs:98-106)
 * element type as text ("f32", "(pair (pair unit i32) f32)", ...), and one device pointer
 * per scalar leaf of the element type in left-to-right order -- the struct-of-arrays
 * payload of Array/Data.hs:95-119.  A SIMD vector type `Vec n t` is one leaf, written
 * "v<n><t>" ("v3f32"); its buffer holds the n components of each element side by side
 * (Array/Data.hs:119,190).  The handle does not take ownership of the buffers. */
int acchip_array_wrap(acchip_ctx* ctx, int rank, const int64_t* shape, const char* elt_type,
                      void* const* buffers, int n_buffers, acchip_array** out);
/* Allocate an array from the pool (allocateArray + mallocRemote); owned by the handle. */
int acchip_array_new(acchip_ctx* ctx, int rank, const int64_t* shape, const char* elt_type, acchip_array** out);
/* Build / take apart tuples of arrays (Apair / Anil of the array-level language). */
int acchip_array_pair(acchip_array* a, acchip_array* b, acchip_array** out);
int acchip_array_unit(acchip_array** out);
int acchip_array_kind(const acchip_array* a);                 /* 0 unit, 1 array, 2 pair */
int acchip_array_fst(const acchip_array* a, acchip_array** out);
int acchip_array_snd(const acchip_array* a, acchip_array** out);
int acchip_array_rank(const acchip_array* a);
int acchip_array_shape(const acchip_array* a, int64_t* shape_out /* rank entries */);
int acchip_array_num_buffers(const acchip_array* a);
void* acchip_array_buffer(const acchip_array* a, int leaf);   /* device pointer of one leaf */
size_t acchip_array_buffer_bytes(const acchip_array* a, int leaf);
const char* acchip_array_elt_type(const acchip_array* a);     /* valid while the handle lives */
/* Drop a handle; buffers the library allocated return to the pool when the last handle
 * that shares them is released. */
void acchip_array_release(acchip_array* a);

/* --- programs ---------------------------------------------------------------------- */

/* Prepare an array function: parse the textual DelayedOpenAfun (Trafo/Delayed.hs:42-59;
 * one S-expression per constructor, de Bruijn indices as in AST/Idx.hs), infer types,
 * generate one kernel per array node and compile it for gfx950 (memory cache, then disk
 * cache keyed by SHA3-256 of the source as in Analysis/Hash.hs:107-111, then hipRTC).
 * This is everything `runN f` does at partial application (Interpreter.hs:110-118). */
int acchip_compile(acchip_ctx* ctx, const char* program_text, size_t length, acchip_program** out);
void acchip_program_release(acchip_program* p);
int acchip_program_arity(const acchip_program* p);
/* Number of distinct compiled kernels behind the program: every variant of every array node
 * (a scan has up to three: large tiles, small tiles, the pipelined kernel) and the one-thread
 * kernels that evaluate scalar expressions for the host. */
int acchip_program_num_kernels(const acchip_program* p);
/* Cache key of the program's k-th kernel, k = 0 .. num_kernels - 1 (sorted): the hexadecimal SHA3-256 of
 * its generated source, compile options and hipRTC version (the counterpart of the reference's
 * hashPreOpenAccWith, Analysis/Hash.hs:107-111, which names the kernels of accelerate-llvm's
 * cache).  NULL beyond the last kernel; valid while the program lives.  Profiles refer to
 * kernels by this key, so a figure measured on other code is recognised as stale. */
const char* acchip_program_kernel_key(const acchip_program* p, int k);

/* SHA3-256 digest used for kernel cache keys; same function as the reference's
 * Crypto.Hash.XKCP (src/Crypto/Hash/XKCP.hs:93-170, cbits/xkcp SHA3_256). */
int acchip_sha3_256(const void* data, size_t length, uint8_t digest[32]);

/* Atrace nodes (`atraceArray` and friends; Interpreter.hs:215, atraceOp :873-880): the
 * traced arrays are evaluated, the stream is synchronised, and the callback receives the
 * message and a handle to the arrays (a tuple handle for several), valid during the call
 * only, so that the caller can print them with its own Show instances; then the body
 * runs.  Without a callback (fn = NULL, the default) one line with the message and the
 * arrays' shapes goes to stderr. */
typedef void (*acchip_trace_fn)(void* user, const char* message, acchip_array* arrays);
int acchip_set_trace(acchip_ctx* ctx, acchip_trace_fn fn, void* user);

/* Apply a prepared function to device-resident arguments (the `go` closure returned by
 * runN, Interpreter.hs:118-126): args[i] is the i-th lambda's argument; uses[k] fills
 * `(use .. k)` nodes.  All work is queued on the context's stream; the result handle may
 * be passed to further calls without synchronising.  Results are owned by the library's
 * pool until released. */
int acchip_execute(acchip_ctx* ctx, acchip_program* p, acchip_array* const* args, int n_args,
                   acchip_array* const* uses, int n_uses, acchip_array** result);

/* No counterpart in the reference: a variant of acchip_execute for callers that cannot allocate
 * device memory (tight serving loops, harnesses that forbid hipMalloc).  It is NOT meant for
 * recording into a HIP graph: the ticket base and the epoch of a launch are kernel arguments that
 * the host advances per call, so a recorded launch replayed later would carry stale ones (every
 * tile would then refuse its ticket and report an error), and the context's stream is not
 * exposed for capture.  The program's body must be a single scan (any of the six) whose operand is an
 * array variable or a fused producer with a host-computable extent; `result` is an array the
 * caller made (acchip_array_wrap / acchip_array_new) with the type and extents of the
 * program's result -- for scanl' / scanr' the pair (array, totals) built with
 * acchip_array_pair.  The tile descriptors and the ticket counter that acchip_execute keeps in
 * pool memory live in a static device array of 1 MiB + 256 B per GPU instead (131072 descriptor
 * words: a scan may have at most 131072 / ceil(element bytes / 4) tiles, e.g. 2^28 Int64
 * elements in one row take 10923 tiles of two words, 2^28 Float32 elements 8192 tiles of one);
 * larger scans fail with an error and
 * nothing is launched.  The call performs no hipMalloc / hipFree and clears nothing with memset
 * nodes; code objects were loaded by acchip_compile.  All contexts on one GPU share the array:
 * calls of this entry point that overlap on one GPU (two streams, two threads) race. */
int acchip_execute_into(acchip_ctx* ctx, acchip_program* p, acchip_array* const* args, int n_args,
                        acchip_array* const* uses, int n_uses, acchip_array* result);

#ifdef __cplusplus
}
#endif
#endif /* ACCHIP_H */
