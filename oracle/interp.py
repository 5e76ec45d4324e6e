"""TEST INFRASTRUCTURE ONLY -- the CPU oracle for the device path.

`OracleDevice` implements the same `Device` interface as the product's `HipDevice`, but runs
the IR on the host the way the reference's backend would: one operation at a time in program
order, every intermediate stored, views resolved against the source buffer at the time of use,
host-evaluated If (`== 1.0`) / While (`!= 0.0`), stop at `EX`, read back the kept ids.  It is
imported only by tests/, `__graft_entry__.smoke()` and bench.py's `cpu_baseline` leg; the
product package never imports it.

What each part follows in the reference (read as text; the reference is Rust + OpenCL C and
cannot be built or run in this image):
  * per-command shape rules ............ src/kernel/trackers/shape.rs:14-111
  * constants inlined, never allocated . src/kernel/trackers/constant.rs:15-56
  * view chains back to a source id .... src/kernel/trackers/kernel.rs:76-232,
                                         src/kernel/helper/shape.rs:13-76
  * arithmetic of each kernel .......... src/devices/opencl/kernels/{unary,binary,reduce,dotprod}.rs
                                         (restated in C in oracle/ref_kernels.c)
  * control flow and read-back ......... src/devices/opencl/device.rs:62-146

Where the reference is defective the evident intent is followed (it coincides with
numpy/torch semantics): Concat and Index work; the reduce tree covers every element for any
reduce size; `const += const` adds; Permute uses `out[i] = in[p[i]]`.

Pinned by (tests/test_oracle_kats.py, tests/test_oracle_math.py):
  * every known-answer vector in the reference's own tests (nn, grd, eq, ctrl x4, ct, norm x2,
    everything), driven through the same front end the product uses;
  * closed forms: tree-sum and sequential-k dot against float64 sums, bit-exact integer cases,
    permute/view/index/concat against brute-force index arithmetic written independently of numpy's
    reshape/transpose.
  * `Max` (an extension: declared, never implemented by the reference): brute-force loops over small matrices
    including NaN, infinities and signed zeros.
Parity unpinned: the exact last-ulp behaviour of exp2/log2/sin of whichever OpenCL runtime the
reference ran on (libm's float functions are used here), and random initial weights (`randn`
draws from an unseeded generator in the reference).
"""
from __future__ import annotations

import ctypes
import os
import sys
from typing import Dict, Iterable, List, Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PKG = os.path.join(os.path.dirname(_HERE), "autodiff-ir-rust_amd")
if _PKG not in sys.path:
    sys.path.insert(0, _PKG)

from adhip import ir as IR  # noqa: E402
from adhip.core import ValueData  # noqa: E402
from adhip.device import Device  # noqa: E402

_f32p = ctypes.POINTER(ctypes.c_float)
_clib = None


def build_c_kernels() -> str:
    """Compile oracle/ref_kernels.c (gcc + OpenMP) and return the library path."""
    import subprocess
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return os.path.join(_HERE, "liboracle_kernels.so")


def c_kernels() -> ctypes.CDLL:
    global _clib
    if _clib is None:
        path = os.path.join(_HERE, "liboracle_kernels.so")
        if not os.path.exists(path):
            build_c_kernels()
        lib = ctypes.CDLL(path)
        i64 = ctypes.c_int64
        lib.ref_dot.argtypes = [_f32p, i64, i64, _f32p, i64, i64, _f32p, i64, i64, i64]
        lib.ref_reduce_sum.argtypes = [_f32p, i64, i64, _f32p, i64, i64]
        lib.ref_unary.argtypes = [ctypes.c_int, _f32p, _f32p, i64]
        lib.ref_binary.argtypes = [ctypes.c_int, _f32p, i64, _f32p, i64, _f32p, i64]
        lib.ref_num_threads.restype = ctypes.c_int
        _clib = lib
    return _clib


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(_f32p)


def ref_dot(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """[m,k] x [k,n], one accumulator per output, k ascending (dotprod.rs:23-53)."""
    a = np.asarray(a, dtype=np.float32)
    b = np.asarray(b, dtype=np.float32)
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    out = np.empty((m, n), dtype=np.float32)
    if m * n == 0:
        return out
    if k == 0:
        out[:] = 0
        return out
    isz = 4
    c_kernels().ref_dot(_ptr(a), a.strides[0] // isz, a.strides[1] // isz,
                        _ptr(b), b.strides[0] // isz, b.strides[1] // isz, _ptr(out), m, k, n)
    return out


def ref_reduce_sum(a: np.ndarray) -> np.ndarray:
    """[vec,red] -> [vec], pairwise halving tree over zero-padded lanes (reduce.rs:29-63)."""
    a = np.asarray(a, dtype=np.float32)
    vec, red = a.shape
    out = np.zeros(vec, dtype=np.float32)
    if vec == 0 or red == 0:
        return out
    isz = 4
    c_kernels().ref_reduce_sum(_ptr(a), a.strides[0] // isz, a.strides[1] // isz, _ptr(out), vec, red)
    return out


def ref_reduce_max(a: np.ndarray) -> np.ndarray:
    """[vec,red] -> [vec], the largest element of every row.  The reference only declares this reduction
    (`ReduceOp::Max`, src/kernel/kernel_decl.rs:75-78; "add max, min", src/core/ir.rs:49) and has no kernel for it,
    so there is no algorithm of its to restate: the result is order-independent (maximum is associative and
    commutative and rounds nothing) and is taken with C's `fmax` rule, which OpenCL C's `fmax`/`max` share: a NaN
    operand is ignored unless both are NaN.  Pinned by brute force in tests/test_oracle_math.py."""
    a = np.asarray(a, dtype=np.float32)
    return np.fmax.reduce(a, axis=1).astype(np.float32)


_UNARY_OPS = {IR.T_EXP2: 0, IR.T_LOG2: 1, IR.T_SIN: 2, IR.T_RECIP: 4, IR.T_SQRT: 5,
              IR.T_EQUAL_ZERO: 6, IR.T_MORE_ZERO: 7, IR.T_LESS_ZERO: 8}


def ref_binary(mul: bool, a, b, shape) -> np.ndarray:
    """res[g] = a[g] (+|*) b[g]; either operand may be an inline constant (binary.rs:3-14)."""
    n = int(np.prod(shape)) if len(shape) else 1
    out = np.empty(n, dtype=np.float32)
    if n == 0:
        return out

    def prep(x):
        if np.ndim(x) == 0:
            return np.full(1, x, dtype=np.float32), 0
        x = np.asarray(x, dtype=np.float32)
        if x.size != n:
            x = np.broadcast_to(x, shape)
        return np.ascontiguousarray(x).reshape(-1), 1

    (pa, sa), (pb, sb) = prep(a), prep(b)
    c_kernels().ref_binary(1 if mul else 0, _ptr(pa), sa, _ptr(pb), sb, _ptr(out), n)
    return out


def ref_unary(tag: int, a: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty_like(a)
    if a.size:
        c_kernels().ref_unary(_UNARY_OPS[tag], _ptr(a), _ptr(out), a.size)
    return out


class _Exit(Exception):
    pass


class OracleDevice(Device):
    """Reference-semantics interpreter (see module docstring)."""

    def __init__(self):
        self.result: Dict[str, np.ndarray] = {}
        self.result_shape: Dict[str, List[int]] = {}
        self.op_count = 0
        self.max_terms = 1   # most terms any single Sum or DotProduct of the last program added up

    # -- Device interface ---------------------------------------------------------------
    def execute(self, proc: IR.IRProcedure, dep_ids: Iterable[str]) -> None:
        self.result.clear()
        self.result_shape.clear()
        self.max_terms = 1
        self.buf: Dict[str, np.ndarray] = {}      # id -> flat f32 buffer
        self.shape: Dict[str, List[int]] = {}     # id -> logical shape (shape tracker)
        self.const: Dict[str, np.float32] = {}    # id -> inline constant
        self.alias: Dict[str, tuple] = {}         # id -> data command back to another id
        # a view of a view of ... is resolved recursively (_value); the caller side spells a slice of n lines as n
        # Index commands joined by a chain of n - 1 Concats, so chains run to thousands of links on larger tensors
        limit = sys.getrecursionlimit()
        sys.setrecursionlimit(max(limit, 20000))
        try:
            self._execute(proc, dep_ids)
        finally:
            sys.setrecursionlimit(limit)

    def _execute(self, proc: IR.IRProcedure, dep_ids: Iterable[str]) -> None:
        try:
            self._run(proc)
        except _Exit:
            pass
        for d in dep_ids:
            if d == "":
                continue
            if d in self.buf or d in self.alias or d in self.const:
                arr = np.ascontiguousarray(self._value(d), dtype=np.float32)
                self.result[d] = arr.reshape(-1).copy()
                self.result_shape[d] = list(self.shape[d])

    def get_tensor(self, id: str) -> ValueData:
        if id in self.result:
            return ValueData(self.result_shape[id], self.result[id], id, False)
        return ValueData.none()

    # -- value lookup -------------------------------------------------------------------
    def _value(self, id: str) -> np.ndarray:
        """Logical value of an id *now*: buffers by content, views by applying their data command
        to the current value of what they view (kernel.rs:76-232), constants filled to shape."""
        if id in self.const:
            return np.full(self.shape[id], self.const[id], dtype=np.float32)
        if id in self.alias:
            a = self.alias[id]
            kind = a[0]
            if kind == "view":
                return np.reshape(self._value(a[1]), a[2])
            if kind == "index":
                return np.take(self._value(a[1]), a[2], axis=a[3])
            if kind == "permute":
                return np.transpose(self._value(a[1]), a[2])
            if kind == "broadcast":
                src = self._value(a[1])
                tgt = list(src.shape)
                tgt[a[2]] = a[3]
                return np.broadcast_to(src, tgt)
            if kind == "concat":
                return np.concatenate([self._value(a[1]), self._value(a[2])], axis=a[3])
            raise AssertionError(kind)
        return self.buf[id].reshape(self.shape[id])

    def _operand(self, id: str):
        """Operand of an element-wise kernel: constants stay scalars (inlined literals)."""
        if id in self.const:
            return self.const[id]
        return self._value(id)

    def _store(self, id: str, shape, arr: np.ndarray) -> None:
        self.alias.pop(id, None)
        self.const.pop(id, None)
        self.shape[id] = list(shape)
        self.buf[id] = np.ascontiguousarray(arr, dtype=np.float32).reshape(-1)
        self.op_count += 1

    # -- execution ----------------------------------------------------------------------
    def _run(self, proc: IR.IRProcedure) -> None:
        for cmd in proc.main:
            t = cmd.tag
            if t == IR.T_EX:
                raise _Exit()
            if t == IR.T_IF:
                ran = False
                for cond, p in cmd.conditions:
                    if self._value(cond).reshape(-1)[0] == np.float32(1.0):
                        self._run(p)
                        ran = True
                        break
                if not ran and cmd.else_proc is not None:
                    self._run(cmd.else_proc)
            elif t == IR.T_WHILE:
                while self._value(cmd.conditional_var).reshape(-1)[0] != np.float32(0.0):
                    self._run(cmd.block)
            else:
                self._step(cmd)

    def _step(self, cmd) -> None:
        t = cmd.tag
        if t == IR.T_HEADING:
            return
        if t == IR.T_CREATE_MAT:
            self._store(cmd.id, cmd.dim, np.array(cmd.contents, dtype=np.float32, copy=True))
        elif t == IR.T_CREATE_CONSTANT:
            self.alias.pop(cmd.id, None)
            self.buf.pop(cmd.id, None)
            self.const[cmd.id] = np.float32(cmd.contents)
            self.shape[cmd.id] = list(cmd.dim)
        elif t in (IR.T_ELW_MULTIPLY, IR.T_ELW_ADD):
            a, b = self._operand(cmd.a), self._operand(cmd.b)
            shape = self.shape[cmd.a]                     # shape.rs:31-32: result takes a's shape
            self._store(cmd.res, shape, ref_binary(t == IR.T_ELW_MULTIPLY, a, b, shape))
        elif t in (IR.T_ELW_MULTIPLY_EQ, IR.T_ELW_ADD_EQ):
            if cmd.s in self.const and cmd.o in self.const:   # folded, no kernel (elw.rs:41-43)
                if t == IR.T_ELW_MULTIPLY_EQ:
                    self.const[cmd.s] = np.float32(self.const[cmd.s] * self.const[cmd.o])
                else:
                    self.const[cmd.s] = np.float32(self.const[cmd.s] + self.const[cmd.o])
                return
            s, o = self._operand(cmd.s), self._operand(cmd.o)
            shape = self.shape[cmd.o] if cmd.s in self.const else self.shape[cmd.s]
            self._store(cmd.s, shape, ref_binary(t == IR.T_ELW_MULTIPLY_EQ, s, o, shape))
        elif t in _UNARY_OPS:
            a = self._value(cmd.a)
            self._store(cmd.res, self.shape[cmd.a], ref_unary(t, a))
        elif t == IR.T_SUM:
            a = self._value(cmd.a)
            assert a.ndim == 2, "Sum needs a 2-D operand"
            self.max_terms = max(self.max_terms, int(a.shape[-1]))
            self._store(cmd.res, list(a.shape[:-1]), ref_reduce_sum(a))
        elif t == IR.T_MAX:
            a = self._value(cmd.a)
            assert a.ndim == 2 and a.shape[1] > 0, "Max needs a 2-D operand with a non-empty last dim"
            self._store(cmd.res, list(a.shape[:-1]), ref_reduce_max(a))
        elif t == IR.T_DOT_PRODUCT:
            a, b = self._value(cmd.a), self._value(cmd.b)
            assert a.ndim == 2 and b.ndim == 2 and a.shape[1] == b.shape[0]
            self.max_terms = max(self.max_terms, int(a.shape[1]))
            self._store(cmd.res, [a.shape[0], b.shape[1]], ref_dot(a, b))
        elif t == IR.T_CONTIGIOUS:
            self._store(cmd.res, self.shape[cmd.a], self._value(cmd.a))
        elif t == IR.T_VIEW:
            self._alias(cmd.res, ("view", cmd.a, list(cmd.target_dim)), list(cmd.target_dim))
        elif t == IR.T_INDEX:
            sh = list(self.shape[cmd.a])
            del sh[cmd.dim]
            self._alias(cmd.res, ("index", cmd.a, cmd.index, cmd.dim), sh)
        elif t == IR.T_PERMUTE:
            sa = self.shape[cmd.a]
            self._alias(cmd.res, ("permute", cmd.a, list(cmd.p)), [sa[i] for i in cmd.p])
        elif t == IR.T_BROADCAST:
            sh = list(self.shape[cmd.a])
            sh[cmd.dim] = cmd.r
            self._alias(cmd.res, ("broadcast", cmd.a, cmd.dim, cmd.r), sh)
        elif t == IR.T_CONCAT:
            sh = list(self.shape[cmd.a])
            sh[cmd.dim] += self.shape[cmd.b][cmd.dim]
            self._alias(cmd.res, ("concat", cmd.a, cmd.b, cmd.dim), sh)
        else:
            raise ValueError(f"unknown IR command {cmd!r}")

    def _alias(self, id, rec, shape):
        self.buf.pop(id, None)
        self.const.pop(id, None)
        self.alias[id] = rec
        self.shape[id] = list(shape)
