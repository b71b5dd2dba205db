"""Build libacchip.so in-tree.

The host side (parser, code generator, executor, C ABI) is C++; the device side is the
set of skeleton headers under csrc/device/, embedded into the library as text and
compiled for gfx950 at run time by hipRTC together with the generated scalar code.
Usage: python -m accelerate_amd.build
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libacchip.so")
HOST_SOURCES = ["codegen.cpp", "runtime.cpp", "exec.cpp", "capi.cpp"]


def _embed_device_headers(out_path):
    dev = os.path.join(CSRC, "device")
    names = sorted(f for f in os.listdir(dev) if f.endswith(".hpp"))
    parts = ['#include <map>\n#include <string>\n#include "../csrc/codegen.hpp"\nnamespace acchip {\n',
             "const std::string& deviceHeader(const std::string& name) {\n",
             "  static const std::map<std::string, std::string> table = {\n"]
    for n in names:
        text = open(os.path.join(dev, n)).read()
        assert ')ACCHIP"' not in text
        # string literals are limited in length by some compilers: split into pieces
        pieces = [text[i:i + 8000] for i in range(0, len(text), 8000)] or [""]
        lit = "\n".join('R"ACCHIP(%s)ACCHIP"' % p for p in pieces)
        parts.append('    {"%s", std::string(%s)},\n' % (n, lit))
    parts.append("  };\n  auto it = table.find(name);\n")
    parts.append('  if (it == table.end()) throw Error("unknown device header " + name);\n  return it->second;\n}\n}\n')
    os.makedirs(os.path.dirname(out_path), exist_ok=True)
    with open(out_path, "w") as f:
        f.write("".join(parts))


def build(verbose=True):
    gen = os.path.join(HERE, "build", "device_embed.cpp")
    _embed_device_headers(gen)
    # The library holds host code only (the device code is compiled by hipRTC at run time),
    # so the host compiler builds it against the HIP runtime and hipRTC.
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cxx = os.environ.get("CXX", "g++")
    # ... except scratch.hip, which holds a static device array and is compiled by hipcc
    hipcc = os.path.join(rocm, "bin", "hipcc")
    obj = os.path.join(HERE, "build", "scratch.o")
    hcmd = [hipcc, "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-c",
            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
            "-o", obj, os.path.join(CSRC, "scratch.hip")]
    if verbose:
        print(" ".join(hcmd), flush=True)
    subprocess.run(hcmd, check=True, stderr=None if verbose else subprocess.DEVNULL)
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function",
           "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(rocm, "include"),
           "-o", LIB] + [os.path.join(CSRC, s) for s in HOST_SOURCES] + [
               gen, obj, "-L" + os.path.join(rocm, "lib"), "-Wl,-rpath," + os.path.join(rocm, "lib"),
               "-lamdhip64", "-lhiprtc", "-pthread", "-ldl"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    build()
    print("built", LIB)
    sys.exit(0)
