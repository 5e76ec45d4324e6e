"""`Device` interface and `HipDevice`, the MI355X device behind the C-ABI library.

`Device` mirrors the reference trait (src/core/ir.rs:126-143): `execute`, `get_tensor`,
`ir_callback`, `dot_prod_shape`.  The reference hands `execute` an already lowered kernel
procedure; here the device receives the IR procedure plus the keep list and does its own
lowering behind the C ABI (`adhip_execute`), which is the part of the reference this
backend replaces (src/kernel/*, src/devices/opencl/*).

There is no CPU fallback: if `libadhip.so` is missing or no GPU is present, constructing a
`HipDevice` raises.
"""
from __future__ import annotations

import ctypes
import os
from typing import Dict, Iterable, List, Optional

import numpy as np

from . import ir as IR
from .core import ValueData

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB_NAME = "libadhip.so"


def library_path() -> str:
    """Location of the in-tree shared library built by `adhip.build.build_library()`."""
    return os.environ.get("ADHIP_LIBRARY", os.path.join(os.path.dirname(_PKG_DIR), "csrc", _LIB_NAME))


class Device:
    """The reference's `Device` trait."""

    def execute(self, proc: IR.IRProcedure, dep_ids: Iterable[str]) -> None:
        raise NotImplementedError

    def get_tensor(self, id: str) -> ValueData:
        raise NotImplementedError

    def ir_callback(self, irb: IR.IRBase) -> None:
        pass

    def dot_prod_shape(self, a: List[int], b: List[int]) -> List[int]:
        return [a[0], b[-1]]


_lib = None


def load_library(path: Optional[str] = None) -> ctypes.CDLL:
    """dlopen the C-ABI library and declare the prototypes of include/adhip.h."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or library_path()
    if not os.path.exists(p):
        raise RuntimeError(
            f"{p} not found: build it first (python -c 'import __graft_entry__ as g; g.build()'); "
            "there is no CPU fallback for the device path")
    lib = ctypes.CDLL(p, mode=ctypes.RTLD_GLOBAL)
    c = ctypes
    vp, sz, i32 = c.c_void_p, c.c_size_t, c.c_int
    lib.adhip_create.argtypes = [i32, c.POINTER(vp)]
    lib.adhip_create.restype = i32
    lib.adhip_destroy.argtypes = [vp]
    lib.adhip_destroy.restype = None
    lib.adhip_execute.argtypes = [vp, c.c_char_p, sz, c.POINTER(c.c_char_p), sz]
    lib.adhip_execute.restype = i32
    lib.adhip_get_tensor.argtypes = [vp, c.c_char_p, c.POINTER(c.POINTER(c.c_float)),
                                     c.POINTER(c.POINTER(c.c_uint64)), c.POINTER(sz)]
    lib.adhip_get_tensor.restype = i32
    lib.adhip_last_error.argtypes = [vp]
    lib.adhip_last_error.restype = c.c_char_p
    lib.adhip_dot_prod_shape.argtypes = [c.POINTER(c.c_uint64), sz, c.POINTER(c.c_uint64), sz,
                                         c.POINTER(c.c_uint64)]
    lib.adhip_dot_prod_shape.restype = i32
    lib.adhip_program_create.argtypes = [vp, c.c_char_p, sz, c.POINTER(c.c_char_p), sz, c.POINTER(vp)]
    lib.adhip_program_create.restype = i32
    for name in ("adhip_program_upload", "adhip_program_run", "adhip_program_enqueue", "adhip_program_enqueue_noalloc",
                 "adhip_program_sync", "adhip_program_readback"):
        getattr(lib, name).argtypes = [vp]
        getattr(lib, name).restype = i32
    lib.adhip_program_destroy.argtypes = [vp]
    lib.adhip_program_destroy.restype = None
    lib.adhip_program_set_profiling.argtypes = [vp, i32]
    lib.adhip_program_set_profiling.restype = i32
    lib.adhip_program_kernel_count.argtypes = [vp]
    lib.adhip_program_kernel_count.restype = i32
    lib.adhip_program_kernel_stat.argtypes = [vp, i32, c.c_char_p, sz, c.POINTER(c.c_uint64),
                                              c.POINTER(c.c_double), c.POINTER(c.c_double),
                                              c.POINTER(c.c_double)]
    lib.adhip_program_kernel_stat.restype = i32
    lib.adhip_program_kernel_source.argtypes = [vp, i32]
    lib.adhip_program_kernel_source.restype = c.c_char_p
    lib.adhip_program_describe.argtypes = [vp]
    lib.adhip_program_describe.restype = c.c_char_p
    lib.adhip_lower_describe.argtypes = [c.c_char_p, sz, c.POINTER(c.c_char_p), sz, c.c_char_p, sz]
    lib.adhip_lower_describe.restype = i32
    lib.adhip_version.argtypes = []
    lib.adhip_version.restype = c.c_char_p
    if path is None:
        _lib = lib
    return lib


def _dep_array(dep_ids):
    ids = sorted(d for d in dep_ids if d != "")
    arr = (ctypes.c_char_p * max(1, len(ids)))()
    for i, d in enumerate(ids):
        arr[i] = d.encode("utf-8")
    return arr, len(ids)


class KernelStat:
    def __init__(self, name, launches, total_ms, bytes_per_launch, flops_per_launch):
        self.name = name
        self.launches = launches
        self.total_ms = total_ms
        self.bytes_per_launch = bytes_per_launch
        self.flops_per_launch = flops_per_launch

    @property
    def avg_ms(self):
        return self.total_ms / self.launches if self.launches else 0.0

    def __repr__(self):
        return (f"KernelStat({self.name!r}, launches={self.launches}, avg_ms={self.avg_ms:.4f}, "
                f"bytes={self.bytes_per_launch:.0f}, flops={self.flops_per_launch:.0f})")


class Program:
    """A lowered program whose buffers stay resident on the GPU: create → upload → run (any
    number of times) → readback.  `HipDevice.execute` is exactly that sequence, once."""

    def __init__(self, dev: "HipDevice", proc: IR.IRProcedure, dep_ids: Iterable[str]):
        self._dev = dev
        self._lib = dev._lib
        blob, self._keepalive = IR.serialize(proc)
        self._blob = blob
        arr, n = _dep_array(dep_ids)
        h = ctypes.c_void_p()
        rc = self._lib.adhip_program_create(dev._ctx, blob, len(blob), arr, n, ctypes.byref(h))
        if rc != 0:
            raise RuntimeError("adhip_program_create failed: " + dev.last_error())
        self._h = h

    def _call(self, name):
        rc = getattr(self._lib, name)(self._h)
        if rc != 0:
            raise RuntimeError(f"{name} failed: " + self._dev.last_error())

    def upload(self):
        self._call("adhip_program_upload")

    def run(self):
        self._call("adhip_program_run")

    def enqueue(self):
        """Queue one run without waiting for it; `sync()` waits for everything queued."""
        self._call("adhip_program_enqueue")

    def enqueue_noalloc(self):
        """`enqueue()` with the program's temporaries in the library's static device array: allocates nothing."""
        self._call("adhip_program_enqueue_noalloc")

    def sync(self):
        self._call("adhip_program_sync")

    def readback(self):
        self._call("adhip_program_readback")

    def set_profiling(self, on: bool):
        self._lib.adhip_program_set_profiling(self._h, 1 if on else 0)

    def kernel_stats(self) -> List[KernelStat]:
        out = []
        n = self._lib.adhip_program_kernel_count(self._h)
        buf = ctypes.create_string_buffer(256)
        for i in range(n):
            launches = ctypes.c_uint64()
            ms, by, fl = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
            self._lib.adhip_program_kernel_stat(self._h, i, buf, 256, ctypes.byref(launches),
                                                ctypes.byref(ms), ctypes.byref(by), ctypes.byref(fl))
            out.append(KernelStat(buf.value.decode(), launches.value, ms.value, by.value, fl.value))
        return out

    def kernel_source(self, i: int) -> str:
        s = self._lib.adhip_program_kernel_source(self._h, i)
        return s.decode() if s else ""

    def describe(self) -> str:
        s = self._lib.adhip_program_describe(self._h)
        return s.decode() if s else ""

    def close(self):
        if self._h:
            self._lib.adhip_program_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class HipDevice(Device):
    """MI355X device: IR in, kept tensors out, everything in between behind `libadhip.so`."""

    def __init__(self, ordinal: int = 0, library: Optional[str] = None):
        self._lib = load_library(library)
        ctx = ctypes.c_void_p()
        rc = self._lib.adhip_create(ordinal, ctypes.byref(ctx))
        if rc != 0 or not ctx:
            raise RuntimeError("adhip_create failed (no HIP device?); there is no CPU fallback")
        self._ctx = ctx

    def last_error(self) -> str:
        s = self._lib.adhip_last_error(self._ctx)
        return s.decode() if s else ""

    def execute(self, proc: IR.IRProcedure, dep_ids: Iterable[str]) -> None:
        blob, keepalive = IR.serialize(proc)
        arr, n = _dep_array(dep_ids)
        rc = self._lib.adhip_execute(self._ctx, blob, len(blob), arr, n)
        del keepalive
        if rc != 0:
            raise RuntimeError("adhip_execute failed: " + self.last_error())

    def execute_serialized(self, blob: bytes, dep_ids: Iterable[str]) -> None:
        """`execute` for a procedure that `ir.serialize` has already turned into the wire format (the caller keeps
        the payload arrays alive): what one `adhip_execute` call costs without the Python serialiser in front."""
        arr, n = _dep_array(dep_ids)
        rc = self._lib.adhip_execute(self._ctx, blob, len(blob), arr, n)
        if rc != 0:
            raise RuntimeError("adhip_execute failed: " + self.last_error())

    def compile(self, proc: IR.IRProcedure, dep_ids: Iterable[str]) -> Program:
        return Program(self, proc, dep_ids)

    def get_tensor(self, id: str) -> ValueData:
        data = ctypes.POINTER(ctypes.c_float)()
        dims = ctypes.POINTER(ctypes.c_uint64)()
        ndim = ctypes.c_size_t()
        rc = self._lib.adhip_get_tensor(self._ctx, id.encode("utf-8"), ctypes.byref(data),
                                        ctypes.byref(dims), ctypes.byref(ndim))
        if rc == 1:
            return ValueData.none()
        if rc != 0:
            raise RuntimeError("adhip_get_tensor failed: " + self.last_error())
        dim = [int(dims[i]) for i in range(ndim.value)]
        n = int(np.prod(dim)) if dim else 1
        arr = np.ctypeslib.as_array(data, shape=(n,)).copy() if n else np.zeros(0, np.float32)
        return ValueData(dim, arr, id, False)

    def dot_prod_shape(self, a, b):
        A = (ctypes.c_uint64 * len(a))(*a)
        B = (ctypes.c_uint64 * len(b))(*b)
        out = (ctypes.c_uint64 * 2)()
        self._lib.adhip_dot_prod_shape(A, len(a), B, len(b), out)
        return [int(out[0]), int(out[1])]

    def close(self):
        if getattr(self, "_ctx", None):
            self._lib.adhip_destroy(self._ctx)
            self._ctx = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def lower_describe(proc: IR.IRProcedure, dep_ids: Iterable[str], library: Optional[str] = None) -> str:
    """Run the lowering only (no GPU needed) and return a text description of the kernels,
    buffers and control structure it produced."""
    lib = load_library(library)
    blob, keepalive = IR.serialize(proc)
    arr, n = _dep_array(dep_ids)
    cap = 1 << 22
    buf = ctypes.create_string_buffer(cap)
    rc = lib.adhip_lower_describe(blob, len(blob), arr, n, buf, cap)
    del keepalive
    if rc != 0:
        raise RuntimeError("lowering failed: " + buf.value.decode())
    return buf.value.decode()
