"""Term texts that arrive damaged: every golden term with one random edit (cut short, a byte
replaced, a stretch removed, a stray parenthesis, two bytes swapped) must either still make a
program or be refused with an error the caller can read.  Nothing may abort the process: the
reference's front end never sends such text, a foreign caller's bug might."""
from __future__ import annotations

import ctypes as C
import os
import random

import pytest

from accelerate_amd import hip

TERMS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "terms")


def _mangle(rng, t):
    kind = rng.randrange(5)
    if kind == 0:
        return t[: rng.randrange(len(t) + 1)]
    a = rng.randrange(len(t))
    if kind == 1:
        return t[:a] + bytes([rng.randrange(256)]) + t[a + 1:]
    if kind == 2:
        return t[:a] + t[a + rng.randrange(16):]
    if kind == 3:
        return t[:a] + rng.choice([b"(", b")"]) + t[a:]
    b = rng.randrange(len(t))
    u = bytearray(t)
    u[a], u[b] = u[b], u[a]
    return bytes(u)


def test_damaged_terms_are_refused_or_compiled(tmp_path, monkeypatch):
    monkeypatch.setenv("ACCHIP_CACHE_DIR", str(tmp_path))  # programs that survive the edit are not worth keeping
    ctx = hip.Context(-1)
    L = hip.lib()
    rng = random.Random(20240611)
    refused = accepted = 0
    for name in sorted(os.listdir(TERMS)):
        with open(os.path.join(TERMS, name), "rb") as f:
            text = f.read()
        bad = _mangle(rng, text)
        h = C.c_void_p()
        rc = L.acchip_compile(ctx._h, bad, len(bad), C.byref(h))  # the bytes as they are, through the C ABI
        if rc == 0:
            accepted += 1
            L.acchip_program_release(h)
        else:
            assert L.acchip_last_error()
            refused += 1
    ctx.close()
    assert refused > 10 * accepted > 0
