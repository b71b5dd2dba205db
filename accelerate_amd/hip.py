"""`run`, `run1`, `runN` over libacchip.so -- the Python face of the backend's entry points.

Mirrors the interface of the reference backend module (Interpreter.hs:31-42, 93-126):
`runN(f)` prepares an array function once (all code generation and compilation happens
here, like the bang-pattern idiom `let !go = runN f`), and the returned callable applies
it to arrays.  Everything goes through the C ABI declared in include/acchip.h; this
module only moves numpy data in and out and never computes a result itself.  There is no
CPU fallback: without the shared library or without a GPU, calls fail.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from . import ir

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libacchip.so")

NP = {"i8": np.int8, "i16": np.int16, "i32": np.int32, "i64": np.int64,
      "u8": np.uint8, "u16": np.uint16, "u32": np.uint32, "u64": np.uint64,
      "f16": np.float16, "f32": np.float32, "f64": np.float64}


class AccError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(msg)
        self.code = code


_lib = None


def lib():
    """Load the shared library (built by accelerate_amd.build); fails loudly if absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise AccError(1, "libacchip.so is not built: run `python -m accelerate_amd.build`")
    L = C.CDLL(LIB_PATH)
    vp, i64p = C.c_void_p, C.POINTER(C.c_int64)
    sigs = {
        "acchip_last_error": (C.c_char_p, []),
        "acchip_init": (C.c_int, [C.c_int, C.POINTER(vp)]),
        "acchip_shutdown": (None, [vp]),
        "acchip_mem_info": (C.c_int, [vp, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
        "acchip_malloc": (vp, [vp, C.c_size_t]),
        "acchip_free": (None, [vp, vp]),
        "acchip_purge": (None, [vp]),
        "acchip_poke": (C.c_int, [vp, vp, vp, C.c_size_t]),
        "acchip_peek": (C.c_int, [vp, vp, vp, C.c_size_t]),
        "acchip_stat": (C.c_longlong, [vp, C.c_char_p]),
        "acchip_table_malloc": (C.c_int, [vp, C.c_uint64, vp, C.c_size_t, C.c_int, C.POINTER(C.c_int)]),
        "acchip_table_use": (C.c_int, [vp, C.c_uint64, C.POINTER(vp)]),
        "acchip_table_release": (C.c_int, [vp, C.c_uint64]),
        "acchip_table_free": (None, [vp, C.c_uint64]),
        "acchip_table_insert_unmanaged": (C.c_int, [vp, C.c_uint64, vp]),
        "acchip_table_reclaim": (None, [vp]),
        "acchip_table_adopt": (C.c_int, [vp, C.c_uint64, vp, C.c_size_t, vp, C.c_int, C.c_int]),
        "acchip_table_status": (C.c_int, [vp, C.c_uint64]),
        "acchip_set_clean_hook": (C.c_int, [vp, vp, vp]),
        "acchip_set_knob": (C.c_int, [vp, C.c_char_p, C.c_longlong]),
        "acchip_get_knob": (C.c_int, [vp, C.c_char_p, C.POINTER(C.c_longlong)]),
        "acchip_set_flags": (C.c_int, [vp, C.c_uint32]),
        "acchip_get_flags": (C.c_uint32, [vp]),
        "acchip_event_record": (C.c_int, [vp, C.POINTER(vp)]),
        "acchip_event_query": (C.c_int, [vp, C.POINTER(C.c_int)]),
        "acchip_event_sync": (C.c_int, [vp]),
        "acchip_event_elapsed_ms": (C.c_int, [vp, vp, C.POINTER(C.c_float)]),
        "acchip_event_destroy": (None, [vp]),
        "acchip_sync": (C.c_int, [vp]),
        "acchip_array_wrap": (C.c_int, [vp, C.c_int, i64p, C.c_char_p, C.POINTER(vp), C.c_int, C.POINTER(vp)]),
        "acchip_array_new": (C.c_int, [vp, C.c_int, i64p, C.c_char_p, C.POINTER(vp)]),
        "acchip_array_pair": (C.c_int, [vp, vp, C.POINTER(vp)]),
        "acchip_array_unit": (C.c_int, [C.POINTER(vp)]),
        "acchip_array_kind": (C.c_int, [vp]),
        "acchip_array_fst": (C.c_int, [vp, C.POINTER(vp)]),
        "acchip_array_snd": (C.c_int, [vp, C.POINTER(vp)]),
        "acchip_array_rank": (C.c_int, [vp]),
        "acchip_array_shape": (C.c_int, [vp, i64p]),
        "acchip_array_num_buffers": (C.c_int, [vp]),
        "acchip_array_buffer": (vp, [vp, C.c_int]),
        "acchip_array_buffer_bytes": (C.c_size_t, [vp, C.c_int]),
        "acchip_array_elt_type": (C.c_char_p, [vp]),
        "acchip_array_release": (None, [vp]),
        "acchip_compile": (C.c_int, [vp, C.c_char_p, C.c_size_t, C.POINTER(vp)]),
        "acchip_program_release": (None, [vp]),
        "acchip_program_arity": (C.c_int, [vp]),
        "acchip_program_num_kernels": (C.c_int, [vp]),
        "acchip_program_kernel_key": (C.c_char_p, [vp, C.c_int]),
        "acchip_sha3_256": (C.c_int, [vp, C.c_size_t, C.c_char_p]),
        "acchip_set_trace": (C.c_int, [vp, vp, vp]),
        "acchip_execute": (C.c_int, [vp, vp, C.POINTER(vp), C.c_int, C.POINTER(vp), C.c_int, C.POINTER(vp)]),
        "acchip_execute_into": (C.c_int, [vp, vp, C.POINTER(vp), C.c_int, C.POINTER(vp), C.c_int, vp]),
    }
    for name, (res, args) in sigs.items():
        fn = getattr(L, name)
        fn.restype, fn.argtypes = res, args
    L._declared = sorted(sigs)
    _lib = L
    return L


def _check(rc):
    if rc != 0:
        raise AccError(rc, lib().acchip_last_error().decode(errors="replace"))


def _leaves(ty):
    return ir.tleaves(_parse_type(ty) if isinstance(ty, str) and ty.startswith("(") else ty)


def _parse_type(text):
    toks = text.replace("(", " ( ").replace(")", " ) ").split()

    def rd(pos):
        if toks[pos] == "(":
            out, pos = [], pos + 1
            while toks[pos] != ")":
                x, pos = rd(pos)
                out.append(x)
            return tuple(out), pos + 1
        return toks[pos], pos + 1
    return rd(0)[0]


TRACE_FN = C.CFUNCTYPE(None, C.c_void_p, C.c_char_p, C.c_void_p)
CLEAN_FN = C.CFUNCTYPE(None, C.c_void_p)


class Context:
    """One device, one stream, one memory pool, one kernel cache (acchip_init)."""

    def __init__(self, device=0):
        self._h = C.c_void_p()
        _check(lib().acchip_init(device, C.byref(self._h)))
        self.device = device

    def close(self):
        if self._h:
            lib().acchip_shutdown(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_trace(self, fn):
        """fn(message, arrays) receives what Atrace nodes report (arrays already copied to the
        host); None restores the default, a line on stderr."""
        if fn is None:
            self._trace_cb = None
            _check(lib().acchip_set_trace(self._h, None, None))
            return

        def cb(_user, msg, handle):
            view = DeviceArray(self, C.c_void_p(handle))
            try:
                fn(msg.decode(errors="replace"), view.to_host())
            finally:
                view._h = C.c_void_p()     # the library owns the handle

        self._trace_cb = TRACE_FN(cb)      # keep the thunk alive while it is installed
        _check(lib().acchip_set_trace(self._h, C.cast(self._trace_cb, C.c_void_p), None))

    # memory --------------------------------------------------------------------------
    def mem_info(self):
        t, a = C.c_size_t(), C.c_size_t()
        _check(lib().acchip_mem_info(self._h, C.byref(t), C.byref(a)))
        return t.value, a.value

    def malloc(self, nbytes):
        return lib().acchip_malloc(self._h, nbytes)

    def free(self, p):
        lib().acchip_free(self._h, p)

    def purge(self):
        lib().acchip_purge(self._h)

    def stat(self, name):
        return lib().acchip_stat(self._h, name.encode())

    # array table (Array/Remote/LRU.hs): host arrays named by an id, mirrored on the device
    def table_malloc(self, ident, host, frozen=False):
        """host: a C-contiguous numpy array the caller keeps alive until table_free."""
        fresh = C.c_int()
        _check(lib().acchip_table_malloc(self._h, ident, host.ctypes.data, host.nbytes, int(frozen), C.byref(fresh)))
        return bool(fresh.value)

    def table_use(self, ident):
        p = C.c_void_p()
        _check(lib().acchip_table_use(self._h, ident, C.byref(p)))
        return p.value

    def table_release(self, ident):
        _check(lib().acchip_table_release(self._h, ident))

    def table_free(self, ident):
        lib().acchip_table_free(self._h, ident)

    def table_status(self, ident):
        return lib().acchip_table_status(self._h, ident)

    def table_adopt(self, ident, host, array, leaf=0, clean=False):
        _check(lib().acchip_table_adopt(self._h, ident, host.ctypes.data, host.nbytes, array._h, leaf, int(clean)))

    def table_reclaim(self):
        lib().acchip_table_reclaim(self._h)

    # bits of the reference's option word that this backend honours (cbits/flags.h:19-49)
    FLAG_INPLACE, FLAG_FAST_MATH, FLAG_FAST_PERMUTE_CONST, FLAG_FORCE_RECOMP = 1 << 4, 1 << 5, 1 << 6, 1 << 7
    FLAG_DUMP_GC, FLAG_DUMP_CC, FLAG_DUMP_EXEC = 1 << 18, 1 << 20, 1 << 23

    def set_knob(self, name, value):
        """Override one launch-time choice (see acchip_set_knob); returns the previous value."""
        old = self.knob(name)
        _check(lib().acchip_set_knob(self._h, name.encode(), int(value)))
        return old

    def knob(self, name):
        v = C.c_longlong(0)
        _check(lib().acchip_get_knob(self._h, name.encode(), C.byref(v)))
        return v.value

    @property
    def flags(self):
        return lib().acchip_get_flags(self._h)

    @flags.setter
    def flags(self, bitfield):
        _check(lib().acchip_set_flags(self._h, int(bitfield) & 0xFFFFFFFF))

    def set_clean_hook(self, fn):
        if fn is None:
            self._clean_cb = None
            _check(lib().acchip_set_clean_hook(self._h, None, None))
            return
        self._clean_cb = CLEAN_FN(lambda _user: fn())
        _check(lib().acchip_set_clean_hook(self._h, C.cast(self._clean_cb, C.c_void_p), None))

    def poke(self, devptr, host):
        _check(lib().acchip_poke(self._h, devptr, host.ctypes.data, host.nbytes))

    def peek(self, host, devptr):
        _check(lib().acchip_peek(self._h, host.ctypes.data, devptr, host.nbytes))

    def sync(self):
        _check(lib().acchip_sync(self._h))

    def event(self):
        return Event(self)

    # arrays --------------------------------------------------------------------------
    def to_device(self, data, aty):
        """numpy array (or list of arrays, one per leaf of a tuple element type) -> DeviceArray."""
        rank, ety = int(aty[1]), aty[2]
        lv = ir.tleaves(ety)
        parts = list(data) if isinstance(data, (list, tuple)) else [data]
        if len(parts) != len(lv):
            raise ValueError("one numpy array per scalar leaf of the element type")
        # a SIMD vector leaf carries its components in one more, innermost numpy dimension
        vecs = [ir.vec_of(t) for t in lv]
        parts = [np.asarray(p, dtype=NP[v[1] if v else t], order="C") for p, t, v in zip(parts, lv, vecs)]  # keeps rank 0
        shape = (parts[0].shape[:-1] if vecs[0] else parts[0].shape) if parts else ()
        if len(shape) != rank:
            raise ValueError("array of rank %d passed where rank %d is declared" % (len(shape), rank))
        h = C.c_void_p()
        shp = (C.c_int64 * max(1, rank))(*shape)
        _check(lib().acchip_array_new(self._h, rank, shp, ir.render(ety).encode(), C.byref(h)))
        arr = DeviceArray(self, h)
        for k, p in enumerate(parts):
            if p.nbytes:
                _check(lib().acchip_poke(self._h, lib().acchip_array_buffer(h, k), p.ctypes.data, p.nbytes))
        return arr

    def empty(self, shape, aty):
        """An uninitialised device array of the given extents (acchip_array_new)."""
        rank, ety = int(aty[1]), aty[2]
        if len(shape) != rank:
            raise ValueError("array of rank %d asked for where rank %d is declared" % (len(shape), rank))
        h = C.c_void_p()
        shp = (C.c_int64 * max(1, rank))(*shape)
        _check(lib().acchip_array_new(self._h, rank, shp, ir.render(ety).encode(), C.byref(h)))
        return DeviceArray(self, h)

    def pair(self, a, b):
        h = C.c_void_p()
        _check(lib().acchip_array_pair(a._h, b._h, C.byref(h)))
        return DeviceArray(self, h)

    def compile(self, program):
        return Program(self, program)


class Event:
    def __init__(self, ctx):
        self._h = C.c_void_p()
        _check(lib().acchip_event_record(ctx._h, C.byref(self._h)))

    def sync(self):
        _check(lib().acchip_event_sync(self._h))

    def done(self):
        d = C.c_int()
        _check(lib().acchip_event_query(self._h, C.byref(d)))
        return bool(d.value)

    def elapsed_ms(self, later):
        ms = C.c_float()
        _check(lib().acchip_event_elapsed_ms(self._h, later._h, C.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if self._h:
                lib().acchip_event_destroy(self._h)
        except Exception:
            pass


class DeviceArray:
    """Handle to a device-resident array or tuple of arrays (acchip_array)."""

    def __init__(self, ctx, handle):
        self.ctx, self._h = ctx, handle

    @property
    def kind(self):
        return lib().acchip_array_kind(self._h)

    @property
    def shape(self):
        r = lib().acchip_array_rank(self._h)
        s = (C.c_int64 * max(1, r))()
        _check(lib().acchip_array_shape(self._h, s))
        return tuple(s[i] for i in range(r))

    @property
    def elt_type(self):
        return _parse_type(lib().acchip_array_elt_type(self._h).decode())

    def parts(self):
        a, b = C.c_void_p(), C.c_void_p()
        _check(lib().acchip_array_fst(self._h, C.byref(a)))
        _check(lib().acchip_array_snd(self._h, C.byref(b)))
        return DeviceArray(self.ctx, a), DeviceArray(self.ctx, b)

    def to_host(self):
        """Copy back: a numpy array, a list of them for tuple elements, or nested pairs."""
        k = self.kind
        if k == 0:
            return ()
        if k == 2:
            a, b = self.parts()
            return (a.to_host(), b.to_host())
        shape = self.shape
        outs = []
        for i, t in enumerate(ir.tleaves(self.elt_type)):
            v = ir.vec_of(t)
            out = np.empty(tuple(shape) + (v[0],), NP[v[1]]) if v else np.empty(shape, NP[t])
            if out.nbytes:
                _check(lib().acchip_peek(self.ctx._h, out.ctypes.data, lib().acchip_array_buffer(self._h, i), out.nbytes))
            outs.append(out)
        return outs[0] if len(outs) == 1 else outs

    def release(self):
        if self._h:
            lib().acchip_array_release(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


def _lhs_type(lhs):
    if lhs[0] in ("single", "wild"):
        return lhs[1]
    return ("pair", _lhs_type(lhs[1]), _lhs_type(lhs[2]))


class Program:
    """A prepared array function: acchip_compile at construction, acchip_execute per call."""

    def __init__(self, ctx, program):
        self.ctx = ctx
        self.text = program.text() if isinstance(program, ir.Node) else str(program)
        self._h = C.c_void_p()
        raw = self.text.encode()
        _check(lib().acchip_compile(ctx._h, raw, len(raw), C.byref(self._h)))
        # the library accepted the text, so it is well formed: read the argument types off it
        sx = _parse_type(self.text)
        if isinstance(sx, tuple) and sx and sx[0] == "acchip-ir":
            sx = sx[2]
        self.arg_types = []
        while isinstance(sx, tuple) and sx and sx[0] == "alam":
            self.arg_types.append(_lhs_type(sx[1]))
            sx = sx[2]

    @property
    def num_kernels(self):
        return lib().acchip_program_num_kernels(self._h)

    @property
    def kernel_keys(self):
        """Cache keys (hex SHA3-256) of the program's kernels, sorted."""
        out, k = [], 0
        while True:
            key = lib().acchip_program_kernel_key(self._h, k)
            if key is None:
                return out
            out.append(key.decode())
            k += 1

    def _arg(self, ty, v, keep):
        if isinstance(v, DeviceArray):
            return v
        if ty == "unit":
            h = C.c_void_p()
            _check(lib().acchip_array_unit(C.byref(h)))
            d = DeviceArray(self.ctx, h)
        elif ty[0] == "array":
            d = self.ctx.to_device(v, ty)
        else:
            a, b = self._arg(ty[1], v[0], keep), self._arg(ty[2], v[1], keep)
            h = C.c_void_p()
            _check(lib().acchip_array_pair(a._h, b._h, C.byref(h)))
            d = DeviceArray(self.ctx, h)
        keep.append(d)
        return d

    def execute(self, *args, uses=()):
        """Device arrays in, device array out; nothing is synchronised."""
        if len(args) != len(self.arg_types):
            raise TypeError("program takes %d arguments" % len(self.arg_types))
        keep = []
        hs = [self._arg(t, a, keep) for t, a in zip(self.arg_types, args)]
        av = (C.c_void_p * max(1, len(hs)))(*[h._h for h in hs])
        uv = (C.c_void_p * max(1, len(uses)))(*[u._h for u in uses])
        res = C.c_void_p()
        _check(lib().acchip_execute(self.ctx._h, self._h, av, len(hs), uv, len(uses), C.byref(res)))
        return DeviceArray(self.ctx, res)

    def execute_into(self, result, *args, uses=()):
        """acchip_execute_into: a single-scan program written into `result`, a DeviceArray the
        caller made; allocates no device memory."""
        if len(args) != len(self.arg_types):
            raise TypeError("program takes %d arguments" % len(self.arg_types))
        if not all(isinstance(a, DeviceArray) for a in args):
            raise TypeError("execute_into takes device arrays")
        av = (C.c_void_p * max(1, len(args)))(*[a._h for a in args])
        uv = (C.c_void_p * max(1, len(uses)))(*[u._h for u in uses])
        _check(lib().acchip_execute_into(self.ctx._h, self._h, av, len(args), uv, len(uses), result._h))
        return result

    def __call__(self, *args, uses=()):
        """numpy in, numpy out (the `go` closure of runN)."""
        return self.execute(*args, uses=uses).to_host()

    def __del__(self):
        try:
            if self._h:
                lib().acchip_program_release(self._h)
        except Exception:
            pass


_default_ctx = None


def default_context():
    global _default_ctx
    if _default_ctx is None:
        _default_ctx = Context(0)
    return _default_ctx


def runN(f, ctx=None):
    """Prepare an array function; the result is applied to arrays (Interpreter.hs:110-126)."""
    return Program(ctx or default_context(), f)


run1 = runN


def run(acc, ctx=None, uses=()):
    """Run a closed array program (Interpreter.hs:93-101)."""
    return Program(ctx or default_context(), acc)(uses=uses)
