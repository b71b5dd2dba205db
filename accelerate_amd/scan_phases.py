"""Per-phase time stamps of the pipelined scan kernel (acc_scan_pipe), tile by tile.

The kernel that the library generates for `scanl1 (+)` is rebuilt as a standalone program with a
time stamp (s_memrealtime, 100 MHz) written by thread 0 of every workgroup at the border of
every phase of every tile, plus the number of polls and look-back windows the tile needed:

  python -m accelerate_amd.scan_phases build i64        # here: accelerate_amd/build/scan_phases_i64
  accelerate_amd/build/scan_phases_i64 28 stamps.txt    # on the GPU: 2^28 elements, checks the result
  python -m accelerate_amd.scan_phases summary stamps.txt

The device code is the library's own (csrc/device/scan.hpp, scan_pipe.hpp and the Spec the code
generator emits), with the stamps put in by text substitution at the places named below; `build`
fails when one of those places is no longer found, so the tool cannot silently measure other code.
Stamps: 0 top of the iteration, 1 the tile's loads have arrived, 2 rake done (prefixes read back),
3 next loads sent / first stores issued, 4 look-back done, 5 exclusive prefix broadcast, 6 end.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
DEV = os.path.join(HERE, "csrc", "device")
OUT = os.path.join(HERE, "build")

# (text in scan_pipe.hpp, what it becomes); every one must match exactly once
PIPE_STAMPS = [
    ("  for (;;) {\n    const i64 row = cur / tpf;",
     "  for (;;) {\n    u64* lab_stamps = p.stamps; const i64 lab_tile = cur; STAMP(0);\n    const i64 row = cur / tpf;"),
    ("    Elt x[C::G][C::V];\n#pragma unroll\n    for (int g = 0; g < G; ++g) {\n      const RawRow r",
     "    STAMP(1);\n    Elt x[C::G][C::V];\n#pragma unroll\n    for (int g = 0; g < G; ++g) {\n      const RawRow r"),
    ("    if (hasPrev && w != 0) storePrev(S1, S2);\n", "    if (hasPrev && w != 0) storePrev(S1, S2);\n    STAMP(2);\n"),
    ("    // the tile's exclusive prefix: seed or nothing", "    STAMP(3);\n    // the tile's exclusive prefix: seed or nothing"),
    ("      if (lane == 0) {\n        if (successors) {\n          Elt inc;", "      STAMP(4);\n      if (lane == 0) {\n        if (successors) {\n          Elt inc;"),
    ("    const bool hasBase = __builtin_amdgcn_readfirstlane(sh_has_excl) != 0;",
     "    STAMP(5);\n    const bool hasBase = __builtin_amdgcn_readfirstlane(sh_has_excl) != 0;"),
    ("    cur = nxt;\n    if (cur >= total) break;\n  }\n  if (hasPrev) storePrev(0, G);",
     "    STAMP(6);\n    if (tid == 0 && lab_stamps) { lab_stamps[lab_tile * 8 + 7] = blockIdx.x | ((u64)lab_polls << 16) | ((u64)lab_windows << 40); "
     "lab_polls = 0; lab_windows = 0; }\n    cur = nxt;\n    if (cur >= total) break;\n  }\n  if (hasPrev) storePrev(0, G);"),
]
SCAN_STAMPS = [
    ("  i64 tpr_full;", "  i64 tpr_full;\n  u64* stamps;"),
    ("template <class S> struct AccScanCfg",
     "#define STAMP(k) do { if (threadIdx.x == 0 && lab_stamps) lab_stamps[lab_tile * 8 + (k)] = __builtin_amdgcn_s_memrealtime(); } while (0)\n"
     "__shared__ unsigned lab_polls, lab_windows;\ntemplate <class S> struct AccScanCfg"),
]
PIPE_COUNTS = [
    ("    if (ready) break;\n    if (++polls >= limit) {", "    if (lane == 0) ++lab_polls;\n    if (ready) break;\n    if (++polls >= limit) {"),
    ("  terminal = first[groups - 1] < ACC_WAVE;", "  if (lane == 0) ++lab_windows;\n  terminal = first[groups - 1] < ACC_WAVE;"),
]

HOST = r'''
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <vector>
#include <algorithm>
#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); exit(1);} } while (0)
typedef @ELT@ HostElt;
int main(int argc, char** argv) {
  const int lg = argc > 1 ? atoi(argv[1]) : 28;
  const char* path = argc > 2 ? argv[2] : nullptr;
  const long n = 1L << lg;
  typedef AccScanCfg<Spec> C;
  const long tile = C::TILE, full = n / tile, tiles = (n + tile - 1) / tile;
  if (full < 1) { printf("too short for the pipelined kernel\n"); return 1; }
  std::vector<HostElt> h(n);
  unsigned s = 12345;
  for (long i = 0; i < n; ++i) { s = s * 1664525u + 1013904223u; h[i] = (HostElt)((int)(s >> 20) % 2001 - 1000) / (sizeof(HostElt) == 4 ? 1000.0f : 1); }
  HostElt *in, *out;
  CK(hipMalloc(&in, n * sizeof(HostElt))); CK(hipMalloc(&out, n * sizeof(HostElt)));
  CK(hipMemcpy(in, h.data(), n * sizeof(HostElt), hipMemcpyHostToDevice));
  u64 *desc, *ticket, *stamps = nullptr;
  u32* err;
  CK(hipMalloc(&desc, tiles * C::W * 8 + 64)); CK(hipMemset(desc, 0, tiles * C::W * 8));
  CK(hipMalloc(&ticket, 256)); CK(hipMemset(ticket, 0, 256));
  CK(hipHostMalloc(&err, 64)); *err = 0;
  if (path) { CK(hipMalloc(&stamps, tiles * 64)); CK(hipMemset(stamps, 0, tiles * 64)); }
  Env env{}; env.a0_0 = (const HostElt*)in; env.a0_d0 = n;
  Out o{}; o.o0 = out;
  ScanParams p{};
  p.rows = 1; p.n = n; p.tpr = tiles; p.tpr_full = full; p.desc = desc; p.ticket = ticket; p.spin_limit = 1 << 22; p.err = err; p.stamps = stamps;
  int cus = 0; CK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0));
  const long groups = std::min<long>(full, cus);
  u64 base = 0, epoch = 1;
  auto launch = [&] {
    p.ticket_base = base; p.epoch = epoch;
    hipLaunchKernelGGL(acc_scan_pipe, dim3((unsigned)groups), dim3(ACC_SCAN_BLOCK), 0, 0, env, o, o, p);
    if (full < tiles) hipLaunchKernelGGL(acc_scan_pipe_tail, dim3(1), dim3(ACC_SCAN_BLOCK), 0, 0, env, o, o, p);
    base += full + groups; ++epoch;
  };
  for (int i = 0; i < 3; ++i) launch();
  hipEvent_t a, b;
  CK(hipEventCreate(&a)); CK(hipEventCreate(&b));
  CK(hipEventRecord(a));
  const int K = 10;
  for (int i = 0; i < K; ++i) launch();
  CK(hipEventRecord(b));
  CK(hipDeviceSynchronize());
  float ms; CK(hipEventElapsedTime(&ms, a, b));
  ms /= K;
  std::vector<HostElt> r(n);
  CK(hipMemcpy(r.data(), out, n * sizeof(HostElt), hipMemcpyDeviceToHost));
  long bad = 0; double acc = 0; HostElt run = 0;
  for (long i = 0; i < n; ++i) {
    if (sizeof(HostElt) == 8) { run += h[i]; if (r[i] != run) ++bad; }
    else { acc += h[i]; if (std::fabs((double)r[i] - acc) > 1e-4 * (i + 1)) ++bad; }
  }
  printf("n=2^%d tiles=%ld: %.1f us per launch (stamps compiled in), %.2f TB/s, err=%u, mismatches=%ld\n", lg, tiles, ms * 1e3,
         2.0 * n * sizeof(HostElt) / ms / 1e9, *err, bad);
  if (path) {
    std::vector<u64> st(tiles * 8);
    CK(hipMemcpy(st.data(), stamps, tiles * 64, hipMemcpyDeviceToHost));
    u64 t0 = ~0ull;
    for (long t = 0; t < full; ++t) t0 = std::min(t0, st[t * 8]);
    FILE* f = fopen(path, "w");
    for (long t = 0; t < full; ++t) {
      fprintf(f, "%ld", t);
      for (int k = 0; k < 8; ++k) fprintf(f, " %llu", (unsigned long long)(k < 7 ? st[t * 8 + k] - t0 : st[t * 8 + k]));
      fprintf(f, "\n");
    }
    fclose(f);
  }
  return bad != 0 || *err != 0;
}
'''


def _patch(text, pairs, what):
    for old, new in pairs:
        if text.count(old) != 1:
            raise SystemExit("scan_phases: %s no longer contains exactly once:\n%s" % (what, old))
        text = text.replace(old, new)
    return text


def build(ty="i64"):
    """Writes and compiles accelerate_amd/build/scan_phases_<ty>; returns its path."""
    root = os.path.dirname(HERE)
    env = dict(os.environ, ACCHIP_FLAGS="dump-cc force-recomp", ACCHIP_CACHE_DIR=os.path.join(OUT, "scan_phases_cache"))
    code = ("import sys\nsys.path.insert(0, %r)\nfrom accelerate_amd import hip, programs as P, ir as A\n"
            "hip.Context(-1).compile(P.scanl1_sum(A.%s))\n" % (root, ty))
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True)
    units = [u[u.index("\n") + 1:] for u in r.stderr.split("[acchip] kernel ")[1:]]
    units = [u for u in units if "acc_scan_pipe(" in u]
    if not units:
        raise SystemExit("scan_phases: the program has no pipelined kernel\n" + r.stderr[-2000:])
    spec = units[0][:units[0].index("// Scan skeleton:")]          # prelude + generated Spec
    scan = _patch(open(os.path.join(DEV, "scan.hpp")).read(), SCAN_STAMPS, "scan.hpp")
    pipe = _patch(open(os.path.join(DEV, "scan_pipe.hpp")).read(), PIPE_STAMPS + PIPE_COUNTS, "scan_pipe.hpp")
    os.makedirs(OUT, exist_ok=True)
    src = os.path.join(OUT, "scan_phases_%s.hip" % ty)
    with open(src, "w") as f:
        f.write("#include <hip/hip_runtime.h>\n" + spec + scan + pipe + HOST.replace("@ELT@", "long long" if ty == "i64" else "float"))
    exe = os.path.join(OUT, "scan_phases_%s" % ty)
    cmd = ["/opt/rocm/bin/hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-Xclang", "-target-feature",
           "-Xclang", "-packed-fp32-ops", "-o", exe, src]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise SystemExit("scan_phases: hipcc failed\n" + "\n".join(l for l in r.stderr.splitlines() if "error" in l)[:4000])
    return exe


def summary(path):
    """Markdown summary of a stamps file."""
    import numpy as np
    a = np.loadtxt(path, dtype=np.uint64).astype(np.int64)
    t = a[:, 1:8] / 100.0                       # us since the launch's first stamp
    wg, polls, wins = a[:, 8] & 0xffff, (a[:, 8] >> 16) & 0xffffff, a[:, 8] >> 40
    n = len(t)
    names = ["wait for the tile's loads", "lane scans + rake", "next loads sent, stores begun", "look-back", "other waves' stores, broadcast", "final values"]
    lines = ["tiles %d, workgroups %d, %.1f us from the first stamp to the last" % (n, int(wg.max()) + 1, t[:, 6].max() - t[:, 0].min()), "",
             "| tiles | " + " | ".join(names) + " | per tile |", "|---|" + "---|" * (len(names) + 1)]
    for lo, hi, lab in ((0, 256, "first 256"), (n // 2 - 500, n // 2 + 500, "middle 1000"), (n - 256, n, "last 256")):
        d = np.diff(t[lo:hi], axis=1).mean(axis=0)
        lines.append("| %s | " % lab + " | ".join("%.2f" % v for v in d) + " | %.2f |" % (t[lo:hi, 6] - t[lo:hi, 0]).mean())
    mid = slice(512, n - 512)
    lb = np.diff(t[mid], axis=1)[:, 3]
    lines += ["", "look-back (us): p10 %.2f, p50 %.2f, p90 %.2f, p99 %.2f; polls per tile %.2f (p90 %d), windows per tile %.2f"
              % (*np.percentile(lb, [10, 50, 90, 99]), polls[mid].mean(), np.percentile(polls[mid], 90), wins[mid].mean())]
    raked, start, done = t[:, 2], t[:, 3], t[:, 4]
    late = np.array([max(0.0, raked[max(0, k - 32):k].max() - start[k]) for k in range(1000, n - 1000)])
    dist = []
    for k in range(1000, n - 1000, 7):
        j = k - 1
        while j > 0 and done[j] > start[k]:
            j -= 1
        dist.append(k - j)
    lines += ["when a tile starts to poll, the slowest rake of its 32 nearest predecessors ends %.2f us later (p90 %.2f); "
              "the nearest predecessor that has finished its look-back is %d tiles back (p90 %d)"
              % (late.mean(), np.percentile(late, 90), int(np.median(dist)), int(np.percentile(dist, 90)))]
    order = np.sum(np.diff(t[:, 0]) < 0)
    lines += ["%d of %d tiles start before the tile with the number below theirs" % (order, n)]
    return "\n".join(lines)


if __name__ == "__main__":
    if len(sys.argv) >= 2 and sys.argv[1] == "build":
        print(build(sys.argv[2] if len(sys.argv) > 2 else "i64"))
    elif len(sys.argv) >= 3 and sys.argv[1] == "summary":
        print(summary(sys.argv[2]))
    else:
        sys.exit(__doc__)
