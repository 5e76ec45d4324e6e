"""IR data model and wire format.

Mirrors the reference's program representation: the 26 `IRCmds` variants
(reference src/core/ir.rs:8-105), the nested `IRProcedure` (ir.rs:109-112) and the
`IRBase` builder with its id generator and temp-procedure stack (src/ir/base.rs:6-61).

`serialize()` flattens a nested procedure into the little-endian byte stream that the
C-ABI entry point `adhip_execute` parses.  `CreateMat` payloads are passed by host
pointer (borrowed for the duration of the call), everything else by value.
"""
from __future__ import annotations

import struct
from dataclasses import dataclass, field
from typing import List, Optional, Tuple

import numpy as np

WIRE_MAGIC = b"ADIR"
WIRE_VERSION = 1

# tag numbers of the wire format, in the order of the reference enum (ir.rs:8-105)
T_CREATE_MAT, T_CREATE_CONSTANT = 0, 1
T_ELW_MULTIPLY, T_ELW_ADD, T_ELW_MULTIPLY_EQ, T_ELW_ADD_EQ = 2, 3, 4, 5
T_EQUAL_ZERO, T_MORE_ZERO, T_LESS_ZERO = 6, 7, 8
T_SUM, T_DOT_PRODUCT = 9, 10
T_VIEW, T_INDEX, T_CONCAT, T_PERMUTE, T_BROADCAST, T_CONTIGIOUS = 11, 12, 13, 14, 15, 16
T_EXP2, T_LOG2, T_SIN, T_RECIP, T_SQRT = 17, 18, 19, 20, 21
T_WHILE, T_IF, T_EX, T_HEADING = 22, 23, 24, 25
# not in the reference's enum: the reduction it declares (`ReduceOp::Max`, kernel_decl.rs:75-78) but never emits
T_MAX = 26


class IRCmd:
    """Base class of all IR commands."""
    tag = -1


@dataclass
class CreateMat(IRCmd):
    contents: np.ndarray  # float32, row-major, flat
    dim: List[int]
    id: str
    tag = T_CREATE_MAT


@dataclass
class CreateConstant(IRCmd):
    contents: float
    id: str
    dim: List[int]
    tag = T_CREATE_CONSTANT


@dataclass
class ElwMultiply(IRCmd):
    a: str
    b: str
    res: str
    tag = T_ELW_MULTIPLY


@dataclass
class ElwAdd(IRCmd):
    a: str
    b: str
    res: str
    tag = T_ELW_ADD


@dataclass
class ElwMultiplyEq(IRCmd):
    s: str
    o: str
    tag = T_ELW_MULTIPLY_EQ


@dataclass
class ElwAddEq(IRCmd):
    s: str
    o: str
    tag = T_ELW_ADD_EQ


@dataclass
class EqualZero(IRCmd):
    a: str
    res: str
    tag = T_EQUAL_ZERO


@dataclass
class MoreZero(IRCmd):
    a: str
    res: str
    tag = T_MORE_ZERO


@dataclass
class LessZero(IRCmd):
    a: str
    res: str
    tag = T_LESS_ZERO


@dataclass
class Sum(IRCmd):
    a: str
    res: str
    tag = T_SUM


@dataclass
class Max(IRCmd):
    """Largest element of every row of a 2-D tensor (same operand rules as `Sum`); NaN only where a whole row is NaN."""
    a: str
    res: str
    tag = T_MAX


@dataclass
class DotProduct(IRCmd):
    a: str
    b: str
    res: str
    tag = T_DOT_PRODUCT


@dataclass
class View(IRCmd):
    a: str
    target_dim: List[int]
    res: str
    tag = T_VIEW


@dataclass
class Index(IRCmd):
    a: str
    index: int
    dim: int
    res: str
    tag = T_INDEX


@dataclass
class Concat(IRCmd):
    a: str
    b: str
    dim: int
    res: str
    tag = T_CONCAT


@dataclass
class Permute(IRCmd):
    a: str
    p: List[int]
    res: str
    tag = T_PERMUTE


@dataclass
class Broadcast(IRCmd):
    a: str
    dim: int
    r: int
    res: str
    tag = T_BROADCAST


@dataclass
class Contigious(IRCmd):
    a: str
    res: str
    tag = T_CONTIGIOUS


@dataclass
class Exp2(IRCmd):
    a: str
    res: str
    tag = T_EXP2


@dataclass
class Log2(IRCmd):
    a: str
    res: str
    tag = T_LOG2


@dataclass
class Sin(IRCmd):
    a: str
    res: str
    tag = T_SIN


@dataclass
class Recip(IRCmd):
    a: str
    res: str
    tag = T_RECIP


@dataclass
class Sqrt(IRCmd):
    a: str
    res: str
    tag = T_SQRT


@dataclass
class While(IRCmd):
    conditional_var: str
    block: "IRProcedure"
    tag = T_WHILE


@dataclass
class If(IRCmd):
    conditions: List[Tuple[str, "IRProcedure"]]
    else_proc: Optional["IRProcedure"]
    tag = T_IF


@dataclass
class EX(IRCmd):
    tag = T_EX


@dataclass
class Heading(IRCmd):
    cmt: str
    tag = T_HEADING


@dataclass
class IRProcedure:
    """A list of commands with an id; nested through While/If (ir.rs:109-112)."""
    id: str
    main: List[IRCmd] = field(default_factory=list)

    def push(self, cmd: IRCmd) -> None:
        self.main.append(cmd)

    def __iter__(self):
        return iter(self.main)

    def __len__(self):
        return len(self.main)

    def walk(self):
        """Yield every command of this procedure and of all nested ones, in program order."""
        for cmd in self.main:
            yield cmd
            if isinstance(cmd, While):
                yield from cmd.block.walk()
            elif isinstance(cmd, If):
                for _, p in cmd.conditions:
                    yield from p.walk()
                if cmd.else_proc is not None:
                    yield from cmd.else_proc.walk()


def unique_id_idx(idx: int) -> str:
    """Spreadsheet-column style ids a..z, aa.. (src/ir/base.rs:19-33)."""
    alphabet = "abcdefghijklmnopqrstuvwxyz"
    base = len(alphabet)
    out = []
    while idx >= base:
        out.append(alphabet[idx % base])
        idx //= base
        idx -= 1
    out.append(alphabet[idx])
    return "".join(reversed(out))


class IRBase:
    """IR builder: id counters, the main procedure and a stack of open nested blocks
    (src/ir/base.rs:6-61)."""

    def __init__(self) -> None:
        self.id = 0
        self.proc_id = 0
        self.proc = IRProcedure("main")
        self.temp_proc: List[IRProcedure] = []

    def unique_id(self) -> str:
        res = unique_id_idx(self.id)
        self.id += 1
        return res

    def unique_id_proc(self) -> str:
        res = unique_id_idx(self.proc_id)
        self.proc_id += 1
        return res

    def create_temp_proc(self) -> None:
        self.temp_proc.append(IRProcedure(self.unique_id_proc()))

    def return_temp_proc(self) -> IRProcedure:
        if not self.temp_proc:
            raise RuntimeError("Unwrapping procedure but none")
        return self.temp_proc.pop()

    def add_cmd(self, cmd: IRCmd) -> None:
        if self.temp_proc:
            self.temp_proc[-1].push(cmd)
        else:
            self.proc.push(cmd)


# --------------------------------------------------------------------------------------
# wire format
# --------------------------------------------------------------------------------------

_ENCODED: dict = {}   # string -> its length-prefixed UTF-8 form (ids repeat all over a program)
_DIMS_STRUCT: dict = {}   # rank -> struct for "<I rank Q..."


def _s(out: bytearray, s: str) -> None:
    b = _ENCODED.get(s)
    if b is None:
        e = s.encode("utf-8")
        if len(_ENCODED) > 200000:
            _ENCODED.clear()
        b = _ENCODED[s] = struct.pack("<I", len(e)) + e
    out += b


def _dims(out: bytearray, dims) -> None:
    n = len(dims)
    st = _DIMS_STRUCT.get(n)
    if st is None:
        st = _DIMS_STRUCT[n] = struct.Struct("<I%dQ" % n)
    out += st.pack(n, *[int(d) for d in dims])


_THREE_IDS = frozenset((T_ELW_MULTIPLY, T_ELW_ADD, T_DOT_PRODUCT))
_TWO_IDS_SO = frozenset((T_ELW_MULTIPLY_EQ, T_ELW_ADD_EQ))
_TWO_IDS_AR = frozenset((T_EQUAL_ZERO, T_MORE_ZERO, T_LESS_ZERO, T_SUM, T_MAX, T_CONTIGIOUS,
                         T_EXP2, T_LOG2, T_SIN, T_RECIP, T_SQRT))
_PACK_QQ = struct.Struct("<QQ").pack
_PACK_Q = struct.Struct("<Q").pack
_PACK_I = struct.Struct("<I").pack
_PACK_F = struct.Struct("<f").pack


def _proc(out: bytearray, proc: IRProcedure, keepalive: list, offsets: Optional[list] = None) -> None:
    _s(out, proc.id)
    out += _PACK_I(len(proc.main))
    for cmd in proc.main:
        t = cmd.tag
        out.append(t)
        if t in _THREE_IDS:
            _s(out, cmd.a); _s(out, cmd.b); _s(out, cmd.res)
        elif t in _TWO_IDS_AR:
            _s(out, cmd.a); _s(out, cmd.res)
        elif t in _TWO_IDS_SO:
            _s(out, cmd.s); _s(out, cmd.o)
        elif t == T_CREATE_MAT:
            arr = cmd.contents
            if not (isinstance(arr, np.ndarray) and arr.dtype == np.float32 and arr.ndim == 1 and arr.flags.c_contiguous):
                arr = np.ascontiguousarray(arr, dtype=np.float32).reshape(-1)
            keepalive.append(arr)
            _s(out, cmd.id)
            _dims(out, cmd.dim)
            if offsets is not None:
                offsets.append(len(out))
            out += _PACK_QQ(arr.ctypes.data if arr.size else 0, arr.size)
        elif t == T_CREATE_CONSTANT:
            out += _PACK_F(np.float32(cmd.contents))
            _s(out, cmd.id)
            _dims(out, cmd.dim)
        elif t == T_VIEW:
            _s(out, cmd.a); _dims(out, cmd.target_dim); _s(out, cmd.res)
        elif t == T_INDEX:
            _s(out, cmd.a); out += _PACK_QQ(cmd.index, cmd.dim); _s(out, cmd.res)
        elif t == T_CONCAT:
            _s(out, cmd.a); _s(out, cmd.b); out += _PACK_Q(cmd.dim); _s(out, cmd.res)
        elif t == T_PERMUTE:
            _s(out, cmd.a); _dims(out, cmd.p); _s(out, cmd.res)
        elif t == T_BROADCAST:
            _s(out, cmd.a); out += _PACK_QQ(cmd.dim, cmd.r); _s(out, cmd.res)
        elif t == T_WHILE:
            _s(out, cmd.conditional_var)
            _proc(out, cmd.block, keepalive, offsets)
        elif t == T_IF:
            out += _PACK_I(len(cmd.conditions))
            for cond, p in cmd.conditions:
                _s(out, cond)
                _proc(out, p, keepalive, offsets)
            out.append(1 if cmd.else_proc is not None else 0)
            if cmd.else_proc is not None:
                _proc(out, cmd.else_proc, keepalive, offsets)
        elif t == T_EX:
            pass
        elif t == T_HEADING:
            _s(out, cmd.cmt)
        else:
            raise ValueError(f"unknown IR command {cmd!r}")


def serialize(proc: IRProcedure, payload_offsets: Optional[list] = None):
    """Return (bytes, keepalive).  `keepalive` holds the float32 arrays whose addresses are
    embedded in the stream; the caller must keep it alive until `adhip_execute` returns.
    `payload_offsets`, when given, receives the byte offset of every CreateMat pointer field (the only
    bytes of the stream that differ from run to run)."""
    out = bytearray()
    out += WIRE_MAGIC
    out += struct.pack("<I", WIRE_VERSION)
    keepalive: list = []
    _proc(out, proc, keepalive, payload_offsets)
    return bytes(out), keepalive


def format_ir(proc: IRProcedure, indent: int = 0) -> str:
    """Plain-text dump of a procedure (the reference has a coloured one, src/ir/debug.rs:85-186)."""
    pad = "    " * indent
    lines = []
    for cmd in proc.main:
        if isinstance(cmd, CreateMat):
            lines.append(f"{pad}{cmd.id} = mat(dim={cmd.dim})")
        elif isinstance(cmd, CreateConstant):
            lines.append(f"{pad}{cmd.id} = const({cmd.contents}, dim={cmd.dim})")
        elif isinstance(cmd, While):
            lines.append(f"{pad}while ({cmd.conditional_var} != 0) {{")
            lines.append(format_ir(cmd.block, indent + 1))
            lines.append(f"{pad}}}")
        elif isinstance(cmd, If):
            for i, (c, p) in enumerate(cmd.conditions):
                lines.append(f"{pad}{'if' if i == 0 else 'else if'} ({c} == 1) {{")
                lines.append(format_ir(p, indent + 1))
                lines.append(f"{pad}}}")
            if cmd.else_proc is not None:
                lines.append(f"{pad}else {{")
                lines.append(format_ir(cmd.else_proc, indent + 1))
                lines.append(f"{pad}}}")
        elif isinstance(cmd, EX):
            lines.append(f"{pad}EXIT")
        elif isinstance(cmd, Heading):
            lines.append(f"{pad}# {cmd.cmt}")
        else:
            d = dict(cmd.__dict__)
            res = d.pop("res", None)
            args = ", ".join(f"{k}={v}" for k, v in d.items())
            name = type(cmd).__name__
            lines.append(f"{pad}{res} = {name}({args})" if res is not None else f"{pad}{name}({args})")
    return "\n".join(l for l in lines if l != "")
