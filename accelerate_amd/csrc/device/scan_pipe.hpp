// Scans over long rows of a plain array (Interpreter.hs:427-474, right scans :513-560), as a pipeline inside
// persistent workgroups: one workgroup of 1024 threads per CU walks over tiles that it takes from
// the ticket counter, and the three things a tile needs from memory overlap with the phases
// that need nothing from it.
//
//  * The input of the next tile is on its way while the current one is scanned.  It travels
//    with direct global -> LDS loads (16 bytes per lane, no registers held while they fly);
//    a wave loads and later reads only its own stretch of the buffer, so the arrival is a
//    wait on the wave's own counter, not a barrier.
//  * The results of a tile leave while the *next* tile waits for its predecessors: a tile's
//    final values stay in registers for one iteration (G x 16 bytes per lane) and are stored
//    when the workgroup would otherwise idle in the look-back.
//  * Rows of the tile are dealt to the waves in turn (wave w holds rows w, w + 16, ...), so
//    that one load or store instruction of the workgroup covers 16 KiB of consecutive
//    addresses; all accesses carry the non-temporal hint.  A persistent copy of this shape
//    reaches 6.0 TB/s on MI355X against 5.3 for wave-contiguous rows without the hint.
//
// A right scan is the same walk over the row's mirror image: tile t of the walk lies t tiles from
// the row's end, a lane asks for the 16 bytes at the mirrored place (they arrive in its own
// stretch of the buffer all the same: the lane's offset into memory is free, its place in LDS is
// not), reads them back to front, and stores its results reversed.
//
// Order inside a tile: position = (g * 1024 + thread) * V + k.  Lane-local scan of the V
// elements, then the 1024 * G lane totals are raked through LDS by the whole workgroup (every
// thread scans G consecutive totals serially, one ordered wave scan joins the 64 chunks of a
// wave, every wave scans the 16 wave totals for itself), the prefixes go back through LDS.
// The rake area lies over the load buffer, which is free between the moment all waves hold
// their elements in registers and the moment the next tile's loads are sent.
//
// Look-back and descriptors are those of scan.hpp (acc_window, acc_publish).  Wave 0 polls;
// it sends its share of the next tile's loads and its stores only after the look-back, because
// a wave's memory operations complete in issue order and a poll would otherwise wait for them.
// The aggregate is published by the last wave for the same reason.  The pipeline takes the full
// tiles of every row; a row's last, partial tile is left to acc_scan_pipe_tail, a second launch
// with the same epoch and descriptors (a row's last tile has no successors, and by then all its
// predecessors have published their inclusive prefixes).
//
// Tickets: a workgroup takes the ticket of its next tile while it rakes the current one (the
// counter's round trip is then never waited for) and stops at the first one beyond the launch,
// so a launch of T tiles by B workgroups consumes exactly T + B tickets.  A workgroup works on
// its tickets in increasing order and every smaller ticket belongs to a workgroup that is
// running, so no tile ever waits for one that has not started.

#ifndef ACC_PIPE_SETTLE
#define ACC_PIPE_SETTLE 32    // s_sleep argument before the first poll of a tile (0: poll at once)
#endif

// 16 bytes per lane from global memory (wave-uniform address `g` + the lane's byte offset) to LDS
// at ldsBase + lane * 16 (ldsBase wave-uniform).  Written in assembly so that the compiler does
// not track it: the waits are placed by hand.
ACC_DEV void acc_dma16(const void* g, u32 laneOff, u32 ldsBase) {
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1 nt" ::"v"(laneOff), "s"(g), "s"(__builtin_amdgcn_readfirstlane((int)ldsBase)) : "memory");
}
// address = wave-uniform base + a lane's 32-bit byte offset: one register per lane serves every row of a tile
template <class T> ACC_DEV T* acc_at(T* base, u32 byteOff) { return (T*)((char*)base + byteOff); }
template <class T> ACC_DEV const T* acc_at(const T* base, u32 byteOff) { return (const T*)((const char*)base + byteOff); }
template <class T> ACC_DEV T* acc_back(T* base, u32 byteOff) { return (T*)((char*)base - byteOff); }
// wait until at most N of this wave's vector memory operations are outstanding (they complete in issue order)
template <int N> ACC_DEV void acc_wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
// workgroup barrier that orders LDS accesses only (a full fence would also wait for loads in flight)
ACC_DEV void acc_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
// The ticket counter's fetch-and-add in two halves: `send` issues it, `receive` waits for the
// answer.  Between the two the register named by `old` must not be touched (the compiler does not
// know that a load is pending on it, which is the point: it would wait at once).
ACC_DEV void acc_ticket_send(u64* counter, u64& old) {
  asm volatile("global_atomic_add_x2 %0, %1, %2, off sc0" : "=&v"(old) : "v"(counter), "v"(1ull) : "memory");
}
// N: vector memory operations the wave has issued since `send` (they complete in issue order)
template <int N> ACC_DEV void acc_ticket_receive(u64& old) { asm volatile("s_waitcnt vmcnt(%1)" : "+v"(old) : "n"(N) : "memory"); }
// a value that all lanes of the wave hold alike, moved to scalar registers
ACC_DEV i64 acc_uniform(i64 v) {
  const u32 lo = (u32)__builtin_amdgcn_readfirstlane((int)(u32)(u64)v), hi = (u32)__builtin_amdgcn_readfirstlane((int)(u32)((u64)v >> 32));
  return (i64)(((u64)hi << 32) | lo);
}

#ifndef ACC_PIPE_EARLY
#define ACC_PIPE_EARLY 1      // with the rake area over the load buffer: waves beyond it send the next loads early
#endif
#ifndef ACC_PIPE_WINDOW
#define ACC_PIPE_WINDOW 1     // predecessors a lane of the polling wave looks at per round trip (window = 64 x this)
#endif

// acc_window of scan.hpp over K * 64 predecessors per round trip: lane l looks at the tiles
// look - l - 64 j, j < K.  With one workgroup per CU and a tile per workgroup in flight, the nearest
// predecessor that has finished lies some 80 tiles back (256 tiles in flight, a quarter to a
// third of a tile's time between a tile's aggregate and its inclusive prefix), so a window of 64
// needs a second round trip for most tiles and one of 128 does not.
template <class S, int K>
ACC_DEV void acc_window_wide(const typename S::Env& env, const u64* rowDesc, i64 look, u64 epoch, u64 limit, u32* err,
                             typename S::Elt& r, int& nv, bool& terminal) {
  typedef typename S::Elt Elt;
  const int W = AccScanCfg<S>::W;
  const int lane = acc_lane();
  int st[K];   // 0 not yet, 1 aggregate, 2 inclusive prefix, 3 before the row
  Elt val[K];
  int first[K];  // per group of 64: lane of the first predecessor that ends the walk, or 64
  int groups = K;  // groups that take part, nearest first
  u64 polls = 0;
  for (;;) {
    bool ready = true;
    groups = K;
#pragma unroll
    for (int j = 0; j < K; ++j) {
      const i64 idx = look - lane - (i64)j * ACC_WAVE;
      st[j] = idx < 0 ? 3 : acc_try_read<Elt>(rowDesc + idx * W, val[j], epoch);
      if (st[j] == 1 && S::stops(val[j])) st[j] = 2;
    }
#pragma unroll
    for (int j = 0; j < K; ++j) {
      if (j < groups) {
        const u64 mEnd = __ballot(st[j] >= 2);
        const u64 mInv = __ballot(st[j] == 0);
        first[j] = mEnd ? __builtin_ctzll(mEnd) : ACC_WAVE;
        const u64 need = first[j] >= 63 ? ~0ull : ((2ull << first[j]) - 1);
        if (mInv & need) ready = false;
        if (first[j] < ACC_WAVE) groups = j + 1;  // the walk ends inside this group
      }
    }
    if (ready) break;
    if (++polls >= limit) {
      if (lane == 0) __hip_atomic_store(err, 3u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      nv = 0;
      terminal = true;
      return;
    }
    __builtin_amdgcn_s_sleep(ACC_SCAN_SLEEP);
  }
  terminal = first[groups - 1] < ACC_WAVE;
  nv = 0;
  bool have = false;
#pragma unroll
  for (int j = 0; j < K; ++j) {
    if (j < groups) {
      int cnt = ACC_WAVE;
      if (first[j] < ACC_WAVE) {
        const int stEnd = __shfl(st[j], first[j], ACC_WAVE);
        if (stEnd == 3) {
          if (S::kSeeded) {
            if (lane == first[j]) val[j] = S::seed(env);
            cnt = first[j] + 1;
          } else {
            cnt = first[j];
          }
        } else {
          cnt = first[j] + 1;
        }
      }
      // earlier tiles sit in higher lanes: fold them in from the left
      Elt v = val[j];
#pragma unroll
      for (int d = 1; d < ACC_WAVE; d <<= 1) {
        Elt o = acc_shfl_down(v, d);
        if (lane + d < cnt) v = S::combine(env, o, v);
      }
      if (cnt > 0) {
        r = have ? S::combine(env, v, r) : v;  // group j lies before the groups already joined
        have = true;
        nv += cnt;
      }
    }
  }
}

#ifndef ACC_PIPE_EXCL
#define ACC_PIPE_EXCL 1  // 0: scanl / scanl' / scanr' store their running values one position on (stores off the 16-byte grid)
#endif

extern "C" __global__ void __launch_bounds__(ACC_SCAN_BLOCK, ACC_SCAN_MINWAVES)
acc_scan_pipe(Spec::Env env, Spec::Out out, Spec::Out tot, ScanParams p) {
  typedef Spec S;
  typedef S::Elt Elt;
  typedef S::Raw Raw;        // what lies in the source array
  typedef S::RawOut RawOut;  // what goes to the result (the element's one scalar)
  typedef AccScanCfg<S> C;
  constexpr int V = C::V, G = C::G, W = C::W, NW = ACC_SCAN_WAVES;
  static_assert(sizeof(Raw) * V == 16 && sizeof(RawOut) == sizeof(Raw), "a lane's share of a row is 16 bytes, in and out");
  static_assert(ACC_SCAN_BLOCK == 1024, "the pipelined scan runs 16 waves");
  typedef RawOut RawRun __attribute__((ext_vector_type(V), aligned(sizeof(RawOut))));  // in memory: aligned like an element (scanl shifts by one)
  typedef Raw RawRow __attribute__((ext_vector_type(V)));                        // in LDS: 16-byte aligned

  __shared__ __attribute__((aligned(16))) unsigned char sh_buf[G * 16384];  // load buffer; the rake area lies over it
  __shared__ Elt sh_wtot[NW];
  __shared__ Elt sh_excl;
  __shared__ int sh_has_excl;
  __shared__ i64 sh_next;
  // The rake area has LDS of its own when the two fit side by side (the next tile's loads can
  // then be sent as soon as its ticket is known, in the middle of the rake); otherwise it lies
  // over the load buffer, and the loads wait until the prefixes have been read back.
  constexpr bool kSep = sizeof(sh_buf) + sizeof(Elt) * (G + 1) * ACC_SCAN_BLOCK + 1024 <= 160 * 1024;
  __shared__ Elt sh_rake[kSep ? (G + 1) * ACC_SCAN_BLOCK : 1];
  static_assert(kSep || sizeof(Elt) * (G + 1) * ACC_SCAN_BLOCK <= sizeof(sh_buf), "rake area must fit the load buffer");
  Elt* const rk = kSep ? sh_rake : (Elt*)sh_buf;
  // Waves whose part of the load buffer the rake area does not touch send the next tile's loads
  // in the middle of the rake, as soon as the tile's aggregate has been published (all waves but
  // the polling one when the rake area has LDS of its own); the others after the prefixes have
  // been read back.  Sending them before the aggregate is out delays every successor's look-back
  // (Float32, 112 B per lane: 409 us against 353).
  // scans whose result u is the running value u - 1 store each lane's results on the 16-byte grid (see where yprev is filled)
  // (scanr writes its running values at its elements' own positions already; scanr' does not)
  constexpr bool kExcl = ACC_PIPE_EXCL && S::kKind != 0 && !(S::kRight && S::kKind == 1);
  constexpr int kRakeBytes = (int)sizeof(Elt) * (G + 1) * ACC_SCAN_BLOCK;
  constexpr int kFirstEarly = kSep ? 1 : (ACC_PIPE_EARLY ? (kRakeBytes + G * 1024 - 1) / (G * 1024) : NW);

  const int tid = (int)threadIdx.x;
  const int lane = acc_lane();
  const int w = __builtin_amdgcn_readfirstlane(acc_wave());
  const bool early = w >= kFirstEarly;
  const i64 tpf = p.tpr_full;            // full tiles per row: the pipeline's share
  const i64 total = p.rows * tpf;
  const i64 n = p.n;
  const i64 m = S::kKind == 1 ? n + 1 : n;  // entries per output row
  const Raw* const inP = S::in_base(env);
  const u32 myLds = __builtin_amdgcn_readfirstlane((u32)(size_t)(__attribute__((address_space(3))) unsigned char*)sh_buf) + (u32)w * G * 1024u;
  const Raw* const myRows = (const Raw*)(sh_buf + (size_t)w * G * 1024);

  // Tickets are taken by a lane of wave 1 (wave 0 polls, and keeps its queue of memory operations
  // short), one tile ahead: the answer is needed when the next tile's loads are sent, after the rake.
  const bool ticketLane = tid == ACC_WAVE;
  if (ticketLane)
    sh_next = (i64)(__hip_atomic_fetch_add(p.ticket, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - p.ticket_base);
  acc_lds_barrier();
  i64 cur = acc_uniform(sh_next);
  acc_lds_barrier();  // read by all before it is written again
  if (cur < 0) {
    // the host's count of tickets is off: touch nothing
    if (tid == 0) __hip_atomic_store(p.err, 3u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    return;
  }
  if (cur >= total) return;

  // the lane's 16 bytes of row g lie at element (g * 1024 + tid) * V of the tile: g * 16 KiB + tid * 16 bytes
  const u32 laneOff = (u32)tid * 16u;
  constexpr bool R = S::kRight;
  // where the lane's 16 bytes of a row lie in memory, relative to the row's (mirrored: last) 16 KiB
  const u32 loadOff = R ? (u32)(ACC_SCAN_BLOCK - 1 - tid) * 16u : laneOff;
  auto sendLoads = [&](i64 gt) {
    const i64 row = gt / tpf, tile = gt - row * tpf;
    const Raw* src = R ? inP + row * n + (n - (tile + 1) * (i64)C::TILE) : inP + row * n + tile * (i64)C::TILE;
#pragma unroll
    for (int g = 0; g < G; ++g)
      acc_dma16(src + (i64)(R ? G - 1 - g : g) * ACC_SCAN_BLOCK * V, loadOff, myLds + (u32)g * 1024u);
  };

  // the tile whose results wait in registers
  Elt yprev[C::G][C::V];
  bool hasPrev = false;
  i64 prevOut = 0;      // output position of the previous tile's first value (right scans: of thread 0's first run of V)
  // rows [lo, hi) of it
  auto storePrev = [&](int lo, int hi) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if (g < lo || g >= hi) continue;
      RawRun r;
#pragma unroll
      for (int k = 0; k < V; ++k) r[R ? V - 1 - k : k] = S::to_raw(yprev[g][k]);
      if (R) __builtin_nontemporal_store(r, (RawRun*)acc_back(S::out_base(out) + prevOut - (i64)g * ACC_SCAN_BLOCK * V, laneOff));
      else __builtin_nontemporal_store(r, (RawRun*)acc_at(S::out_base(out) + prevOut + (i64)g * ACC_SCAN_BLOCK * V, laneOff));
    }
  };
  // The previous tile's values leave in three pieces (a store holds its wave until the memory
  // pipeline has taken the data): two after the aggregate has been published, between the last
  // phases of the rake, the rest while wave 0 looks back.  Wave 0 stores all of its rows after the
  // look-back, behind its share of the next tile's loads.
  constexpr int S1 = G / 4, S2 = G / 2;

  sendLoads(cur);
  bool tailStores = false;  // stores were issued behind the loads of `cur`

  for (;;) {
    const i64 row = cur / tpf;
    const i64 tile = cur - row * tpf;
    const i64 outBase = row * m;
    u64* rowDesc = p.desc + (u64)row * (u64)p.tpr * W;
    // the tile's elements are in LDS or on their way there; behind them only stores
    if (tailStores) {
      if (w == 0 || early) acc_wait_vm<G>();
      else acc_wait_vm<G - S2>();
    } else {
      acc_wait_vm<0>();
    }
    Elt x[C::G][C::V];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const RawRow r = *(const RawRow*)(myRows + (size_t)(g * ACC_WAVE + lane) * V);
      x[g][0] = S::from_raw(env, r[R ? V - 1 : 0]);
#pragma unroll
      for (int k = 1; k < V; ++k) x[g][k] = S::combine(env, x[g][k - 1], S::from_raw(env, r[R ? V - 1 - k : k]));
    }
    // ticket of the next tile; nothing looks at the counter's answer before the end of the rake,
    // so the round trip is not waited for
    u64 nextRaw;
    if (ticketLane) acc_ticket_send(p.ticket, nextRaw);
    if (!kSep) acc_lds_barrier();  // every wave holds its elements: the buffer becomes the rake area

    // rake: entry e = g * 1024 + tid, chunk e / G, a chunk takes G + 1 slots
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int e = g * ACC_SCAN_BLOCK + tid;
      rk[(e / G) * (G + 1) + e % G] = x[g][V - 1];
    }
    acc_lds_barrier();
    Elt c[C::G];
#pragma unroll
    for (int j = 0; j < G; ++j) c[j] = rk[tid * (G + 1) + j];
#pragma unroll
    for (int j = 1; j < G; ++j) c[j] = S::combine(env, c[j - 1], c[j]);
    Elt ts = acc_wave_scan<S>(env, c[G - 1], lane);
    const Elt chunkPre = acc_prev_lane(ts);  // everything of this wave before the lane's chunk (lane > 0)
    if (lane == ACC_WAVE - 1) sh_wtot[w] = ts;
    if (ticketLane) {
      acc_ticket_receive<0>(nextRaw);
      sh_next = (i64)(nextRaw - p.ticket_base);
    }
    acc_lds_barrier();
    const i64 nxt = acc_uniform(sh_next);
    const bool nextLoaded = nxt < total;
    // every wave scans the 16 wave totals for itself
    Elt wt = sh_wtot[lane & (NW - 1)];
    wt = acc_wave_scan<S>(env, wt, lane);
    const Elt tileAgg = acc_readlane(wt, NW - 1);
    const bool successors = tile + 1 < p.tpr;
    if (w == NW - 1 && lane == 0 && tile > 0 && successors) acc_publish<Elt>(rowDesc + tile * W, tileAgg, p.epoch, 1);
    {
      // exclusive prefixes of the chunk's entries go back in place
      Elt pre;
      bool hasPre = false;
      if (w > 0) {
        pre = acc_readlane(wt, w - 1);
        hasPre = true;
      }
      if (lane > 0) {
        pre = hasPre ? S::combine(env, pre, chunkPre) : chunkPre;
        hasPre = true;
      }
      if (hasPre) rk[tid * (G + 1)] = pre;
#pragma unroll
      for (int j = 1; j < G; ++j) rk[tid * (G + 1) + j] = hasPre ? S::combine(env, pre, c[j - 1]) : c[j - 1];
    }
    if (early && w != 0 && nextLoaded) sendLoads(nxt);
    if (hasPrev && w != 0) storePrev(0, S1);
    acc_lds_barrier();
    // (scanl, scanl' and scanr' write what lies before each position: the value in front of a lane's
    // run is this prefix, kept so that the run can be stored on the 16-byte grid, see below)
    Elt runPre[kExcl ? C::G : 1];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int e = g * ACC_SCAN_BLOCK + tid;
      if (e > 0) {
        const Elt pre = rk[(e / G) * (G + 1) + e % G];
        if (kExcl) runPre[g] = pre;
#pragma unroll
        for (int k = 0; k < V; ++k) x[g][k] = S::combine(env, pre, x[g][k]);
      }
    }
    if (hasPrev && w != 0) storePrev(S1, S2);
    if (!kSep) {
      acc_lds_barrier();  // the rake area has been read: the whole buffer may receive the next tile
      if (!early && w != 0 && nextLoaded) sendLoads(nxt);
    }
    if (w != 0 && hasPrev) storePrev(S2, G);

    // the tile's exclusive prefix: seed or nothing for the first tile of a row, look-back otherwise
    if (w == 0) {
      Elt excl;
      bool hasExcl = false;
      if (tile == 0) {
        if (S::kSeeded) {
          excl = S::seed(env);
          hasExcl = true;
        }
      } else {
        if (ACC_PIPE_SETTLE) __builtin_amdgcn_s_sleep(ACC_PIPE_SETTLE);
        i64 look = tile - 1;
        for (;;) {
          Elt r;
          int nv;
          bool term;
          acc_window_wide<S, ACC_PIPE_WINDOW>(env, rowDesc, look, p.epoch, p.spin_limit, p.err, r, nv, term);
          if (nv > 0) {
            excl = hasExcl ? S::combine(env, r, excl) : r;
            hasExcl = true;
          }
          if (term) break;
          look -= (i64)ACC_PIPE_WINDOW * ACC_WAVE;
        }
      }
      if (lane == 0) {
        if (successors) {
          Elt inc;
          acc_join<S>(env, hasExcl, excl, true, tileAgg, inc);
          acc_publish<Elt>(rowDesc + tile * W, inc, p.epoch, 2);
        }
        sh_excl = excl;
        sh_has_excl = hasExcl ? 1 : 0;
      }
    }
    acc_lds_barrier();
    if (w == 0) {
      asm volatile("" ::: "memory");  // the polling wave's own traffic stays behind its polls
      if (nextLoaded) sendLoads(nxt);
      if (hasPrev) storePrev(0, G);
    }
    tailStores = nextLoaded && hasPrev;
    const bool hasBase = __builtin_amdgcn_readfirstlane(sh_has_excl) != 0;
    const Elt base = sh_excl;
    // final values: kept for the next iteration, or written now where a position needs a test
    const i64 shift = S::kKind == 0 ? 0 : 1;
    // scan' keeps the row's total apart: the tile that holds it stores value by value -- unless the
    // results go out as `what lies before`, which never touches the position of the total
    const bool deferable = kExcl || S::kKind != 2 || tile + 1 < p.tpr;
    if (deferable && kExcl) {
      // scanl / scanl' / scanr': result u is everything before element u (in the scan's direction).  A lane's run of results is then
      // (what lies before its run, its first V - 1 running values) at the positions of its elements,
      // which are on the 16-byte grid; stored one position on, as the running values themselves,
      // every store straddled two 16-byte words (2^28 Int64: 749 against 714 us for scanl1).  The
      // base is there: these scans have a seed.
#pragma unroll
      for (int g = 0; g < G; ++g) {
        yprev[g][0] = g * ACC_SCAN_BLOCK + tid > 0 ? S::combine(env, base, runPre[g]) : base;
#pragma unroll
        for (int k = 1; k < V; ++k) yprev[g][k] = S::combine(env, base, x[g][k - 1]);
      }
      prevOut = R ? outBase + m - V - tile * (i64)C::TILE : outBase + tile * (i64)C::TILE;
      hasPrev = true;
      if (tile + 1 == tpf) {
        // the value behind the row's last full tile: the row's last result, or the first of its partial tile
        if (tid == ACC_SCAN_BLOCK - 1) {
          const Elt behind = S::combine(env, base, x[G - 1][V - 1]);
          const i64 u = (tile + 1) * (i64)C::TILE;
          if (S::kKind == 2 && u == n) S::store(tot, row, behind);  // scanl' / scanr': the row's total
          else S::store(out, outBase + (R ? m - 1 - u : u), behind);
        }
        tailStores = false;
      }
    } else if (deferable) {
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int k = 0; k < V; ++k) yprev[g][k] = hasBase ? S::combine(env, base, x[g][k]) : x[g][k];
      prevOut = R ? outBase + m - shift - V - tile * (i64)C::TILE : outBase + tile * (i64)C::TILE + shift;
      hasPrev = true;
    } else {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const i64 t0 = tile * (i64)C::TILE + ((i64)g * ACC_SCAN_BLOCK + tid) * V;
#pragma unroll
        for (int k = 0; k < V; ++k) {
          const Elt y = hasBase ? S::combine(env, base, x[g][k]) : x[g][k];
          const i64 u = t0 + k + 1;
          if (u == n) S::store(tot, row, y);
          else S::store(out, outBase + (R ? m - 1 - u : u), y);
        }
      }
      hasPrev = false;
      tailStores = false;  // more than the counted stores lie behind the loads: wait for all
    }
    if (S::kKind != 0 && tile == 0 && tid == 0) {
      S::store(out, outBase + (R ? m - 1 : 0), S::seed(env));
      tailStores = false;
    }
    cur = nxt;
    if (cur >= total) break;
  }
  if (hasPrev) storePrev(0, G);
}

// The last tile of every row when the row is not a whole number of tiles: one workgroup per row,
// launched after acc_scan_pipe with the same parameters.
extern "C" __global__ void __launch_bounds__(ACC_SCAN_BLOCK, ACC_SCAN_MINWAVES)
acc_scan_pipe_tail(Spec::Env env, Spec::Out out, Spec::Out tot, ScanParams p) {
  typedef Spec S;
  typedef S::Elt Elt;
  const int W = AccScanCfg<S>::W;
  const i64 row = blockIdx.x;
  const i64 tile = p.tpr_full;
  const i64 n = p.n;
  const i64 m = S::kKind == 1 ? n + 1 : n;
  const i64 inBase = row * n, outBase = row * m;
  u64* rowDesc = p.desc + (u64)row * (u64)p.tpr * W;
  auto load = [&](i64 t) -> Elt { return S::in_linear(env, inBase + (S::kRight ? n - 1 - t : t)); };
  auto store = [&](i64 t, const Elt& y) {
    if (S::kKind == 0) {
      S::store(out, outBase + (S::kRight ? n - 1 - t : t), y);
    } else {
      const i64 u = t + 1;
      if (S::kKind == 2 && u == n) S::store(tot, row, y);
      else S::store(out, outBase + (S::kRight ? m - 1 - u : u), y);
    }
  };
  auto storeRun = [&](i64 t0, const Elt* y) {
    const i64 shift = S::kKind == 0 ? 0 : 1;
    if (!S::kRight) {
      S::store_run(out, outBase + t0 + shift, y);
    } else {
      Elt z[S::V];
#pragma unroll
      for (int k = 0; k < S::V; ++k) z[k] = y[S::V - 1 - k];
      S::store_run(out, outBase + (m - 1 - shift) - (t0 + S::V - 1), z);
    }
  };
  acc_scan_tile<S>(env, rowDesc, p.tpr, tile, n, p.epoch, p.spin_limit, p.err, load, store, storeRun, false, false);
}
