"""`autodiff::*` entry points: tensor creation, device selection, control-flow builders
and `execute()` (reference src/core/autodiff.rs:21-135, src/core/control.rs:12-111).

Usage mirrors the reference:

    autodiff.set_device(HipDevice())
    x = autodiff.tensor([...], [2, 5])
    y = net.f(x); y.forward(); y.backward()
    autodiff.execute()
    y.val().get()
"""
from __future__ import annotations

from typing import Callable, Optional

import numpy as np

from . import ir as IR
from .core import (STATE, Tensor, TensorNode, Value, ValueData, add_to_dep, concat, constant,
                   dot, ir_b_add, is_harsh)

__all__ = [
    "tensor", "scalar", "constant", "ones", "zeros", "empty", "fill", "randn", "set_device",
    "add_heading", "execute", "print_and_exec", "eager_dep_opt", "ir_if", "ir_if_else",
    "ir_while", "ir_for", "concat", "dot", "seed",
]

_rng = np.random.default_rng()


def seed(s: int) -> None:
    """Seed the generator behind `randn`.  The reference draws from an unseeded thread RNG
    (autodiff.rs:75-80), so no result of the reference depends on particular draws."""
    global _rng
    _rng = np.random.default_rng(s)


def tensor(data, dim) -> Tensor:
    dim = [int(d) for d in dim]
    arr = np.asarray(data, dtype=np.float32).reshape(-1)
    if arr.size != int(np.prod(dim)):
        raise ValueError("# of values doesn't match dim size when calling from_vec")
    v = Value.new(arr, dim)
    if not is_harsh():
        add_to_dep(v.id)
    return Tensor(TensorNode(v, None))


def scalar(val: float) -> Tensor:
    return tensor([val], [1])


def fill(val: float, dim) -> Tensor:
    return tensor(np.full(int(np.prod(dim)), val, dtype=np.float32), dim)


def ones(dim) -> Tensor:
    return fill(1.0, dim)


def zeros(dim) -> Tensor:
    return fill(0.0, dim)


def empty() -> Tensor:
    return Tensor(TensorNode(Value.empty(), None))


def randn(dim) -> Tensor:
    return tensor(_rng.standard_normal(int(np.prod(dim)), dtype=np.float32), dim)


def set_device(device) -> None:
    """Install a device and reset the IR builder and the keep list (autodiff.rs:82-97).
    Unlike the reference's process-global flag, eager-dependency mode is also reset here so
    that consecutive programs in one process do not inherit it."""
    STATE.irb = IR.IRBase()
    STATE.device = device
    STATE.dep_tracker = set()
    STATE.harsh = False


def add_heading(cmt: str) -> None:
    ir_b_add(IR.Heading(cmt=cmt))


def eager_dep_opt() -> None:
    """Only ids marked with `Value.keep()` are read back (autodiff.rs:131-133)."""
    STATE.harsh = True


def _run(debug: bool) -> None:
    ir_b_add(IR.EX())
    dev = STATE.device
    if dev is None:
        raise RuntimeError("Can't unpack device")
    dev.ir_callback(STATE.irb)
    # The reference runs its IR clean-up passes here (DCE, CSE, constant hoisting;
    # src/ir/optimize.rs:8-44).  They do not change results; the device's own lowering
    # performs dead-code elimination and common-subexpression merging.
    if debug:
        print(IR.format_ir(STATE.irb.proc))
    dev.execute(STATE.irb.proc, set(STATE.dep_tracker))


def execute() -> None:
    _run(False)


def print_and_exec() -> None:
    _run(True)


# ---- control flow (src/core/control.rs) ------------------------------------------------


def ir_if(expr: Callable[[], Tensor], func: Callable[[], None]) -> None:
    v = expr().forward()
    add_to_dep(v.id)
    if v.dim != [1]:
        raise RuntimeError("If expression must have dim of [1]")
    STATE.irb.create_temp_proc()
    func()
    if_block = STATE.irb.return_temp_proc()
    ir_b_add(IR.If(conditions=[(v.id, if_block)], else_proc=None))


def ir_if_else(expr: Callable[[], Tensor], func: Callable[[], None], func_else: Callable[[], None]) -> None:
    v = expr().forward()
    add_to_dep(v.id)
    if v.dim != [1]:
        raise RuntimeError("Expr must return a boolean")
    STATE.irb.create_temp_proc()
    func()
    if_block = STATE.irb.return_temp_proc()
    STATE.irb.create_temp_proc()
    func_else()
    else_block = STATE.irb.return_temp_proc()
    ir_b_add(IR.If(conditions=[(v.id, if_block)], else_proc=else_block))


def ir_while(var: Tensor, func: Callable[[], None]) -> None:
    """while (var != 0) { func() }.  The body is traced once; the predicate is re-forwarded at
    the end of the body, re-defining its ids inside the block (control.rs:75-92)."""
    v = var.forward()
    add_to_dep(v.id)
    if v.dim != [1]:
        raise RuntimeError("Expr must return a boolean.")
    STATE.irb.create_temp_proc()
    func()
    r = var.forward()
    main_func = STATE.irb.return_temp_proc()
    ir_b_add(IR.While(conditional_var=r.id, block=main_func))


def ir_for(r: range, func: Callable[[Tensor], None]) -> None:
    """A while loop over a device-resident scalar counter (control.rs:97-111)."""
    assert r.step == 1
    x = scalar(float(r.start))
    x_end = constant(float(r.stop), [1])
    result = x.less_than(x_end)

    def body():
        nonlocal x
        func(x)
        x += 1.0

    ir_while(result, body)
