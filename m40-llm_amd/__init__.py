"""m40llm decode hot path on MI355X: Python view of the C-ABI library.

The package holds the HIP kernels + C ABI (``csrc/``), the C++ host layer that mirrors the
reference's decode / batch-plan / KV-config / selection-telemetry modules (``host/``) and this
thin ctypes binding, which is what the parity tests and the benchmark call through.  There is no
CPU fallback: loading fails loudly when the native library is missing.
"""
from __future__ import annotations

import ctypes as C
import os
import re

import numpy as np

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
HEADER = os.path.join(ROOT, "include", "m40llm.h")
NATIVE_LIB = os.path.join(PKG, "lib", "libm40llm_native.so")
HOST_LIB = os.path.join(PKG, "lib", "libm40llm_host.so")
HOST_HEADER = os.path.join(ROOT, "include", "m40llm_host.h")


class NativeLibraryMissing(RuntimeError):
    pass


def _ctype_of(decl: str):
    d = decl.strip()
    if "*" in d:
        return C.c_char_p if d.replace(" ", "") == "constchar*" else C.c_void_p
    base = d.replace("const", "").strip().split()
    ty = base[0] if base else ""
    return {"size_t": C.c_size_t, "uint32_t": C.c_uint32, "uint64_t": C.c_uint64, "int": C.c_int,
            "float": C.c_float, "void": None, "int32_t": C.c_int32, "int64_t": C.c_int64, "double": C.c_double}.get(ty, C.c_void_p)


def parse_header(path: str):
    """Returns {name: (restype, [argtypes])} for every prototype in a C header."""
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    protos = {}
    for m in re.finditer(r"([A-Za-z_][\w\s\*]*?)\b((?:m40llm|m40host)_\w+)\s*\(([^;{}]*?)\)\s*;", text, flags=re.S):
        ret, name, args = m.group(1).strip(), m.group(2), m.group(3).strip()
        if ret.startswith("typedef"):
            continue
        argtypes = []
        if args and args != "void":
            for a in args.split(","):
                a = a.strip()
                # drop the parameter name when present
                mm = re.match(r"^(.*?[\*\s])([A-Za-z_]\w*)$", a)
                ty = mm.group(1) if (mm and mm.group(1).strip() not in ("const", "")) else a
                argtypes.append(_ctype_of(ty))
        protos[name] = (_ctype_of(ret) if ret != "void" else None, argtypes)
    return protos


_native = None
_host = None


def _bind(lib, protos):
    for name, (res, args) in protos.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args


def native() -> C.CDLL:
    """The C-ABI library with argument types taken from include/m40llm.h."""
    global _native
    if _native is None:
        if not os.path.exists(NATIVE_LIB):
            raise NativeLibraryMissing(
                f"{NATIVE_LIB} is not built; run `python -c 'import __graft_entry__ as g; g.build()'`")
        lib = C.CDLL(NATIVE_LIB, mode=C.RTLD_GLOBAL)
        _bind(lib, parse_header(HEADER))
        _native = lib
    return _native


def host() -> C.CDLL:
    """The C++ host layer (decode loop, batch plan, KV config, selection telemetry, model step)."""
    global _host
    if _host is None:
        native()
        if not os.path.exists(HOST_LIB):
            raise NativeLibraryMissing(f"{HOST_LIB} is not built")
        lib = C.CDLL(HOST_LIB, mode=C.RTLD_GLOBAL)
        _bind(lib, parse_header(HOST_HEADER))
        _host = lib
    return _host


def build(verbose: bool = False):
    from importlib import import_module
    mod = import_module(__name__ + "._build")
    return mod.build_all(verbose)


class M40Error(RuntimeError):
    def __init__(self, fn: str, code: int):
        super().__init__(f"{fn} failed with code {code}")
        self.fn, self.code = fn, code


def check(code: int, fn: str = "m40llm call"):
    if code != 0:
        raise M40Error(fn, code)


# -------------------------------------------------------------------------------------------
# Small object wrappers used by tests and the benchmark.  They mirror the shape of the
# reference's Rust wrappers (CudaContext / DeviceBuffer / KVCache in src/cuda.rs): every method
# is one C-ABI call plus error-code translation.
# -------------------------------------------------------------------------------------------
class DeviceBuffer:
    def __init__(self, ctx: "Context", nbytes: int):
        self.ctx, self.nbytes = ctx, int(nbytes)
        p = C.c_void_p()
        check(ctx.lib.m40llm_device_malloc(ctx.h, max(self.nbytes, 1), C.byref(p)), "m40llm_device_malloc")
        self.ptr = p.value

    def free(self):
        if self.ptr:
            self.ctx.lib.m40llm_device_free(self.ctx.h, self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    def upload(self, arr: np.ndarray, offset: int = 0):
        arr = np.ascontiguousarray(arr)
        assert offset + arr.nbytes <= self.nbytes
        if arr.nbytes:
            check(self.ctx.lib.m40llm_memcpy_h2d(self.ctx.h, self.ptr + offset, arr.ctypes.data, arr.nbytes),
                  "m40llm_memcpy_h2d")
        return self

    def download(self, dtype, shape, offset: int = 0) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert offset + out.nbytes <= self.nbytes
        if out.nbytes:
            check(self.ctx.lib.m40llm_memcpy_d2h(self.ctx.h, out.ctypes.data, self.ptr + offset, out.nbytes),
                  "m40llm_memcpy_d2h")
        return out


class Context:
    def __init__(self, device_id: int = 0):
        self.lib = native()
        self.h = self.lib.m40llm_create_context(device_id)
        if not self.h:
            raise M40Error("m40llm_create_context", -1)

    def close(self):
        if self.h:
            self.lib.m40llm_destroy_context(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def alloc(self, nbytes: int) -> DeviceBuffer:
        return DeviceBuffer(self, nbytes)

    def to_device(self, arr: np.ndarray) -> DeviceBuffer:
        arr = np.ascontiguousarray(arr)
        return DeviceBuffer(self, arr.nbytes).upload(arr)

    def sync(self, kind: int = 1):
        check(self.lib.m40llm_stream_synchronize(self.h, kind), "m40llm_stream_synchronize")

    def wait(self, waiting: int, signal: int):
        check(self.lib.m40llm_stream_wait_for_stream(self.h, waiting, signal), "m40llm_stream_wait_for_stream")

    # events ---------------------------------------------------------------------------
    def event(self):
        e = C.c_void_p()
        check(self.lib.m40llm_cuda_event_create(self.h, C.byref(e)), "m40llm_cuda_event_create")
        return e.value

    def record(self, ev, kind: int = 1):
        check(self.lib.m40llm_cuda_event_record(self.h, ev, kind), "m40llm_cuda_event_record")

    def elapsed_ms(self, start, stop) -> float:
        ms = C.c_float()
        check(self.lib.m40llm_cuda_event_elapsed_sync(self.h, start, stop, C.byref(ms)),
              "m40llm_cuda_event_elapsed_sync")
        return float(ms.value)

    def event_destroy(self, ev):
        self.lib.m40llm_cuda_event_destroy(ev)


class KVCache:
    def __init__(self, ctx: Context, max_seq_len, max_batch, kv_heads, head_dim, compressed=None):
        """compressed: None, or dict(recent_window, block_size, top_blocks, representatives=0,
        representative_policy=0, exact_old_backing=2)"""
        self.ctx = ctx
        self.max_seq_len, self.max_batch, self.kv_heads, self.head_dim = max_seq_len, max_batch, kv_heads, head_dim
        self.compressed = compressed
        if compressed is None:
            self.h = ctx.lib.m40llm_kvcache_create(ctx.h, max_seq_len, max_batch, kv_heads, head_dim)
        else:
            c = compressed
            self.h = ctx.lib.m40llm_kvcache_create_compressed(
                ctx.h, max_seq_len, max_batch, kv_heads, head_dim, c["recent_window"], c["block_size"],
                c.get("top_blocks", 8), c.get("representatives", 0), c.get("representative_policy", 0),
                c.get("exact_old_backing", 2))
        if not self.h:
            raise M40Error("m40llm_kvcache_create", -1)

    def destroy(self):
        if self.h:
            self.ctx.lib.m40llm_kvcache_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass

    def read_token(self, seq, token):
        n = self.kv_heads * self.head_dim
        k = np.empty(n, dtype=np.uint16)
        v = np.empty(n, dtype=np.uint16)
        check(self.ctx.lib.m40llm_kvcache_debug_read_token(self.ctx.h, self.h, seq, token, k.ctypes.data,
                                                           v.ctypes.data), "m40llm_kvcache_debug_read_token")
        return k, v

    def read_raw(self, which, dtype, shape, offset=0):
        out = np.empty(shape, dtype=dtype)
        check(self.ctx.lib.m40llm_ext_kvcache_debug_read_raw(self.ctx.h, self.h, which, offset, out.nbytes,
                                                             out.ctypes.data), "m40llm_ext_kvcache_debug_read_raw")
        return out
