"""Front-end graph: the caller of the device path.

A Python counterpart of the reference's user-facing graph layer, kept to what the device
path needs in order to be driven exactly like the reference drives it: `Tensor` handles
over mutable graph nodes, `Value{dim,id}`, `ValueData`, the global IR builder / device /
dependency ("keep") list, and every node type's `forward` (emit IR) and `backward`
(build and forward small gradient graphs).

Reference files followed: src/core/{node,tensor,value,constant,dependency,value_data}.rs,
src/graph/ops/{ops,func,sum,dot_product,equality}.rs,
src/graph/data/{view,permute,broadcast,index,concat,contigious,repeat}.rs.
"""
from __future__ import annotations

import math
from typing import Callable, List, Optional, Sequence

import numpy as np

from . import ir as IR

# --------------------------------------------------------------------------------------
# global state (reference: statics IRB, DEVICE, DEP_TRACKER, HARSH_DEP_LIST;
# src/core/ir.rs:121-122, src/core/dependency.rs:4-5)
# --------------------------------------------------------------------------------------


class _State:
    irb: Optional[IR.IRBase] = None
    device = None
    dep_tracker: Optional[set] = None
    harsh: bool = False


STATE = _State()


def _irb() -> IR.IRBase:
    if STATE.irb is None:
        raise RuntimeError("Can't unpack IRBuilder (call autodiff.set_device first)")
    return STATE.irb


def ir_b_add(cmd: IR.IRCmd) -> None:
    _irb().add_cmd(cmd)


def ir_b_id() -> str:
    return _irb().unique_id()


def add_to_dep(id: str) -> None:
    if STATE.dep_tracker is None:
        raise RuntimeError("Can't unpack dep tracker")
    STATE.dep_tracker.add(id)


def is_harsh() -> bool:
    return STATE.harsh


# --------------------------------------------------------------------------------------
# ValueData / Value
# --------------------------------------------------------------------------------------


class ValueData:
    """Host copy of a kept tensor (src/core/value_data.rs:6-47)."""

    def __init__(self, dim, data, id, is_none=False):
        self.dim = list(dim)
        self.data = data
        self.id = id
        self.is_none = is_none

    @staticmethod
    def none() -> "ValueData":
        return ValueData([], np.zeros(0, dtype=np.float32), "", True)

    def round(self, num_digits: int) -> "ValueData":
        # (x * 10^n).round() / 10^n in f32; Rust's round() is half-away-from-zero
        mult = np.float32(10.0) ** np.int32(num_digits)
        x = self.data.astype(np.float32) * np.float32(mult)
        r = np.where(x >= 0, np.floor(x + np.float32(0.5)), np.ceil(x - np.float32(0.5))).astype(np.float32)
        return ValueData(self.dim, (r / np.float32(mult)).astype(np.float32), self.id, self.is_none)

    def numpy(self) -> np.ndarray:
        return np.asarray(self.data, dtype=np.float32).reshape(self.dim)

    def __repr__(self):
        if self.is_none:
            return "None"
        return f"ValueData(id={self.id!r}, dim={self.dim}, data={self.data!r})"


class Value:
    """`Value{dim,id}`: a handle to a value the program computes (src/core/value.rs:11-99)."""

    def __init__(self, dim, id):
        self.dim = list(dim)
        self.id = id

    def clone(self) -> "Value":
        return Value(self.dim, self.id)

    @staticmethod
    def new(data, dim) -> "Value":
        id = ir_b_id()
        arr = np.ascontiguousarray(np.asarray(data, dtype=np.float32).reshape(-1))
        ir_b_add(IR.CreateMat(contents=arr, dim=list(dim), id=id))
        return Value(dim, id)

    @staticmethod
    def fill(val: float, dim) -> "Value":
        n = int(np.prod(dim)) if len(dim) else 1
        return Value.new(np.full(n, val, dtype=np.float32), dim)

    @staticmethod
    def ones(dim) -> "Value":
        return Value.fill(1.0, dim)

    @staticmethod
    def zeros(dim) -> "Value":
        return Value.fill(0.0, dim)

    @staticmethod
    def empty() -> "Value":
        return Value([], "")

    def to_node(self) -> "Tensor":
        return Tensor(ValueNode(self.clone()))

    def to_node_with_grad(self) -> "Tensor":
        return Tensor(TensorNode(self.clone(), None))

    def get(self) -> ValueData:
        if STATE.device is None:
            raise RuntimeError("Can't unpack device")
        return STATE.device.get_tensor(self.id)

    def keep(self) -> None:
        add_to_dep(self.id)

    def __repr__(self):
        return f"Value(id={self.id!r}, dim={self.dim})"


# --------------------------------------------------------------------------------------
# Node base + Tensor handle
# --------------------------------------------------------------------------------------


class _BackwardSession:
    """One reverse sweep.  The reference propagates a gradient the moment a node receives it (node.rs:62-71 and every
    `backward` in src/graph), so a value with k consumers runs its whole upstream backward k times and the program grows
    exponentially with the depth of re-use (one transformer encoder layer: 4800 matrix products instead of 46).  Here the
    contributions a node receives are summed first and its `backward` runs once, consumers before producers: the same
    gradient, a program linear in the size of the graph."""

    def __init__(self, root: "Node"):
        # nodes in an order in which every node comes before the nodes it reads (reverse post-order of a DFS
        # along the handles a node holds)
        order, seen, stack = [], set(), [(root, False)]
        while stack:
            node, done = stack.pop()
            if done:
                order.append(node)
                continue
            if id(node) in seen:
                continue
            seen.add(id(node))
            stack.append((node, True))
            for child in _child_nodes(node):
                if id(child) not in seen:
                    stack.append((child, False))
        order.reverse()
        self.order = order
        self.known = seen
        self.pending = {}

    def receive(self, node: "Node", grad: "Value") -> None:
        have = self.pending.get(id(node))
        self.pending[id(node)] = grad if have is None else (have.to_node() + grad.to_node()).forward()

    def run(self) -> None:
        for node in self.order:
            grad = self.pending.pop(id(node), None)
            if grad is not None:
                node._backward_impl(grad)


def _child_nodes(node):
    out = []
    for v in vars(node).values():
        if isinstance(v, Tensor):
            out.append(v.n)
        elif isinstance(v, (list, tuple)):
            out.extend(t.n for t in v if isinstance(t, Tensor))
    return out


_SESSION: Optional[_BackwardSession] = None


class Node:
    """`NodeTrait` (src/core/node.rs:6-35)."""

    def __init_subclass__(cls, **kw):
        super().__init_subclass__(**kw)
        impl = cls.__dict__.get("backward")
        if impl is not None:
            # what the subclass wrote is the node's own rule; the public `backward` hands the gradient to the
            # running sweep, which calls the rule once with the sum of everything the node received
            cls._backward_impl = impl

            def backward(self, grad, _impl=impl):
                if _SESSION is not None and id(self) in _SESSION.known:
                    _SESSION.receive(self, grad)
                else:
                    _impl(self, grad)
            cls.backward = backward

    def forward(self) -> Value:
        raise NotImplementedError

    def backward(self, grad: Value) -> None:
        raise NotImplementedError

    def dim(self) -> List[int]:
        raise NotImplementedError

    def val(self) -> Optional[Value]:
        raise NotImplementedError

    def grad(self) -> Value:
        raise RuntimeError("Calling .grad() on a non-tensor node")

    def reset_grad(self) -> None:
        raise RuntimeError("Calling .reset_grad() on a non-tensor node")

    def is_const(self) -> bool:
        return False

    def deep_copy(self) -> "Node":
        import copy
        return copy.copy(self)  # shallow: children stay shared handles, like Rust's derive(Clone)


def _as_i32_list(d):
    return [int(x) for x in d]


class Tensor:
    """Handle over a replaceable graph node (`Rc<RefCell<Box<dyn NodeTrait>>>`,
    src/core/node.rs:39-106).  Copies of the handle share the node; `+=`-style operators
    replace the node in place so every holder sees the update."""

    __array_priority__ = 1000  # so numpy scalars defer to our reflected operators

    def __init__(self, node: Node):
        self.n = node

    # -- handle semantics -------------------------------------------------------------
    def clone(self) -> "Tensor":
        return self

    def replace(self, node: Node) -> None:
        self.n = node

    def deep_copy(self) -> "Tensor":
        return Tensor(self.n.deep_copy())

    # -- NodeTrait passthrough --------------------------------------------------------
    def forward(self) -> Value:
        return self.n.forward()

    def backward(self) -> None:
        # start autograd with a materialised matrix of ones (node.rs:62-71)
        global _SESSION
        dim = self.dim()
        if _SESSION is not None:
            raise RuntimeError("backward() called while another backward sweep is running")
        _SESSION = _BackwardSession(self.n)
        try:
            self.n.backward(Value.ones(dim))
            _SESSION.run()
        finally:
            _SESSION = None

    def dim(self) -> List[int]:
        return self.n.dim()

    def val(self) -> Optional[Value]:
        return self.n.val()

    def grad(self) -> Value:
        return self.n.grad()

    def reset_grad(self) -> None:
        self.n.reset_grad()

    def detach(self) -> "Tensor":
        self.forward()
        v = self.val()
        if v is None:
            raise RuntimeError("Forward process went wrong")
        return v.to_node()

    def detach_grad(self) -> "Tensor":
        self.forward()
        v = self.val()
        if v is None:
            raise RuntimeError("Forward process went wrong")
        return v.to_node_with_grad()

    def is_const(self) -> bool:
        return self.n.is_const()

    # -- binary operators (src/graph/ops/ops.rs) --------------------------------------
    def __add__(self, other):
        return _binary(AddNode, self, other)

    def __radd__(self, other):
        return _binary(AddNode, other, self)

    def __mul__(self, other):
        return _binary(MultiplyNode, self, other)

    def __rmul__(self, other):
        return _binary(MultiplyNode, other, self)

    def __neg__(self):
        return -1.0 * self  # ops.rs:250-255

    def __sub__(self, other):
        if isinstance(other, Tensor):
            return self + -1.0 * other  # ops.rs:258-264
        return self + (-1.0) * float(other)  # ops.rs:274-280 (folds on the host)

    def __rsub__(self, other):
        return float(other) + -1.0 * self  # ops.rs:266-272

    def __truediv__(self, other):
        if isinstance(other, Tensor):
            return self * other.recip()  # ops.rs:301-307
        return self * (1.0 / float(other))  # ops.rs:317-323

    def __rtruediv__(self, other):
        return float(other) * self.recip()  # ops.rs:309-315

    def __iadd__(self, other):
        _op_equal(AddNode, self, other)
        return self

    def __imul__(self, other):
        _op_equal(MultiplyNode, self, other)
        return self

    def __isub__(self, other):
        if isinstance(other, Tensor):
            _op_equal(AddNode, self, -1.0 * other)
        elif isinstance(other, Value):
            _op_equal(AddNode, self, -1.0 * other.to_node())
        else:
            # The reference's `Tensor -= f32` adds the scalar (ops.rs:288-291); the evident
            # intent is to subtract, which is what is done here.
            _op_equal(AddNode, self, -float(other))
        return self

    def __itruediv__(self, other):
        if isinstance(other, Tensor):
            _op_equal(MultiplyNode, self, other.recip())
        elif isinstance(other, Value):
            _op_equal(MultiplyNode, self, other.to_node().recip())
        else:
            _op_equal(MultiplyNode, self, 1.0 / float(other))
        return self

    # -- unary functions (src/graph/ops/func.rs) --------------------------------------
    def exp2(self):
        return Tensor(UnaryNode(self, "exp2"))

    def log2(self):
        return Tensor(UnaryNode(self, "log2"))

    def sin(self):
        return Tensor(UnaryNode(self, "sin"))

    def recip(self):
        return Tensor(UnaryNode(self, "recip"))

    def sqrt(self):
        return Tensor(UnaryNode(self, "sqrt"))

    def cos(self):
        return (np.float32(math.pi / 2) - self).sin()  # func.rs:100-102

    def exp(self):
        mult_const = np.float32(1.0) / np.log(np.float32(2.0))  # func.rs:104-107
        return (self * mult_const).exp2()

    def ln(self):
        return self.log2() * np.log(np.float32(2.0))  # func.rs:109-112

    def pow2(self):
        return self * self  # func.rs:114-117

    def pow3(self):
        return self.pow2() * self

    def pow(self, p: "Tensor"):
        return (p * self.log2()).exp2()

    def powf(self, p: float):
        if p == 2.0:
            return self.pow2()
        if p == 3.0:
            return self.pow3()
        return (float(p) * self.log2()).exp2()

    def sigmoid(self):
        return 1.0 / (1.0 + (-self).exp())  # src/nn/activations/sigmoid.rs:22-26

    def relu(self):
        return self * self.more_than(constant(0.0, self.dim()))

    def softmax(self, dim: int):
        """exp(x - max) / sum(exp(x - max)) along `dim`.  The reference writes `x.exp() / x.exp().sum(dim)`
        (src/nn/activations/softmax.rs:28-30): its sum loses `dim` and is broadcast back by the trailing-dim rule, so
        element (i, j) of a square matrix is divided by the sum of row j and any other shape fails to broadcast, and
        exp overflows beyond x = 88.  The evident intent is followed: normalise along `dim`, with the maximum along
        `dim` subtracted first.  The maximum carries no gradient: a shift of the argument cancels in the quotient."""
        d = len(self.dim()) + dim if dim < 0 else dim
        keep = list(self.dim())
        keep[d] = 1   # the reduced dim kept with extent 1 (a vector's reduction has one element, not rank 0)
        m = self.max(d).stop_grad().view(keep)
        e = (self - m).exp()
        return e / e.sum(d).view(keep)

    # -- comparisons (src/graph/ops/equality.rs) --------------------------------------
    def equal(self, b: "Tensor"):
        return Tensor(CompareNode(self - b, "equal"))

    def more_than(self, b: "Tensor"):
        return Tensor(CompareNode(self - b, "more"))

    def less_than(self, b: "Tensor"):
        return Tensor(CompareNode(self - b, "less"))

    def all(self):
        x = self
        total_val = int(np.prod(self.dim()))
        for _ in x.dim():
            x = x.sum(0)
        return x.equal(constant(float(total_val), [1]))

    # -- reductions (src/graph/ops/sum.rs:51-119) -------------------------------------
    def sum(self, dim: int):
        p_dim = len(self.dim())
        dim = p_dim + dim if dim < 0 else dim
        permute_to = list(range(p_dim))
        permute_to[-1] = dim
        permute_to[dim] = p_dim - 1
        node = self.permute(permute_to)
        new_dim = node.dim()
        node = node.view([-1, new_dim[-1]])
        node = Tensor(SumNode(node))
        new_dim = new_dim[:-1]
        node = node.view(list(new_dim))
        permute_to = permute_to[:dim] + permute_to[dim + 1:]
        return node.permute(permute_to)

    def max(self, dim: int):
        """Largest element along `dim`: the decomposition of `sum` (permute the dim last, view as 2-D, reduce, view
        and permute back) around the `Max` command.  The reference declares this reduction and never emits it
        (src/kernel/kernel_decl.rs:75-78, "add max, min" in src/core/ir.rs:49)."""
        p_dim = len(self.dim())
        dim = p_dim + dim if dim < 0 else dim
        permute_to = list(range(p_dim))
        permute_to[-1] = dim
        permute_to[dim] = p_dim - 1
        node = self.permute(permute_to)
        new_dim = node.dim()
        node = node.view([-1, new_dim[-1]])
        node = Tensor(MaxNode(node))
        new_dim = new_dim[:-1]
        node = node.view(list(new_dim))
        permute_to = permute_to[:dim] + permute_to[dim + 1:]
        return node.permute(permute_to)

    def stop_grad(self):
        """The same value, as a constant of the backward pass (nothing is propagated to what it was computed from)."""
        return Tensor(StopGradNode(self))

    def mean(self, dim: int):
        p_dim = self.dim()
        d = len(p_dim) + dim if dim < 0 else dim
        return self.sum(dim) / float(p_dim[d])

    def var(self, dim: int, correction: int):
        a = (self - self.mean(dim).unsqueeze(dim)).pow2()
        p_dim = self.dim()
        d = len(p_dim) + dim if dim < 0 else dim
        return a.sum(dim) / float(p_dim[d] - correction)

    # -- data movement (src/graph/data/*.rs) ------------------------------------------
    def view(self, target_dim: Sequence[int]):
        target_dim = list(target_dim) if len(target_dim) else [1]
        source_dim = self.dim()
        target_dim = handle_minus_dim(source_dim, target_dim)
        if target_dim != source_dim:
            return Tensor(ViewNode(self, target_dim))
        return self

    def flatten(self):
        return self.view([int(np.prod(self.dim()))])

    def unsqueeze(self, dim: int):
        p_dim = len(self.dim())
        dim = p_dim + dim + 1 if dim < 0 else dim
        new_dim = list(self.dim())
        new_dim.insert(dim, 1)
        return self.view(new_dim)

    def squeeze(self, dim: int):
        if len(self.dim()) <= 1:
            return self
        new_dim = list(self.dim())
        assert new_dim[dim] == 1, "Squeeze dim must be one"
        del new_dim[dim]
        return self.view(new_dim)

    def permute(self, p: Sequence[int]):
        p = list(p)
        if all(i == v for i, v in enumerate(p)):
            return self
        return Tensor(PermuteNode(self, p))

    def t(self):
        assert len(self.dim()) == 2, "Transpose only supprots 2D matrix"
        return Tensor(PermuteNode(self, [1, 0]))

    def broadcast(self, dim: int, r: int):
        target_dim = list(self.dim())
        dim = len(target_dim) + dim if dim < 0 else dim
        target_dim[dim] = r
        return make_broadcast_node(self, target_dim)

    def i(self, i: int, dim: int):
        p_dim = self.dim()
        dim = len(p_dim) + dim if dim < 0 else dim
        assert dim < len(p_dim), "invalid dimension!"
        assert i < p_dim[dim], "invalid index!"
        return Tensor(IndexNode(self, i, dim))

    def r(self, rng: range, dim: int):
        # per-index Index + unsqueeze + chained Concat (index.rs:84-89)
        return concat([self.i(i, dim).unsqueeze(dim) for i in rng], dim)

    def contigious(self):
        return Tensor(ContigiousNode(self))

    def repeat(self, f: Callable[["Tensor", int], "Tensor"], length: int, dim: int):
        return concat([f(self, i).unsqueeze(dim) for i in range(length)], dim)


# --------------------------------------------------------------------------------------
# leaf nodes
# --------------------------------------------------------------------------------------


class TensorNode(Node):
    """User tensor with an accumulated gradient (src/core/tensor.rs:8-53)."""

    def __init__(self, v: Value, gd: Optional[Value]):
        self.v = v
        self.gd = gd

    def forward(self):
        return self.v.clone()

    def backward(self, grad: Value):
        if self.gd is not None:
            # The reference accumulates in place into the id it adopted on the first call (tensor.rs:22-35).  That id
            # is the very gradient value other nodes were handed too (an AddNode passes one value to both parents),
            # so the in-place `+=` also changes what they see: d(v*v)/dx for v = x + w comes out 1.5 times too large.
            # The evident intent is a sum per leaf, so the accumulation goes to a fresh id here and the shared value
            # stays untouched.
            total = (self.gd.to_node() + grad.to_node()).forward()
            if not is_harsh() and STATE.dep_tracker is not None:
                STATE.dep_tracker.discard(self.gd.id)
            self.gd = total
            if not is_harsh():
                self.gd.keep()
        else:
            self.gd = grad.clone()
            if not is_harsh():
                self.gd.keep()

    def dim(self):
        return list(self.v.dim)

    def val(self):
        return self.v.clone()

    def grad(self):
        if self.gd is None:
            raise RuntimeError("Must run backwards before calling grad()")
        return self.gd.clone()

    def reset_grad(self):
        self.gd = None


class ValueNode(Node):
    """A computed value re-entering the graph as a constant leaf (src/core/value.rs:104-130)."""

    def __init__(self, v: Value):
        self.v = v

    def forward(self):
        return self.v.clone()

    def backward(self, grad):
        pass

    def dim(self):
        return list(self.v.dim)

    def val(self):
        return self.v.clone()


class ConstantNode(Node):
    """Scalar constant with a nominal dim; never allocated (src/core/constant.rs:5-57)."""

    def __init__(self, content: float, dim):
        self.content = float(np.float32(content))
        self._dim = list(dim)
        self._val: Optional[Value] = None

    def forward(self):
        if self._val is not None:
            return self._val
        id = ir_b_id()
        ir_b_add(IR.CreateConstant(contents=self.content, id=id, dim=list(self._dim)))
        self._val = Value(self._dim, id)
        return self._val

    def backward(self, grad):
        pass

    def dim(self):
        return list(self._dim)

    def val(self):
        return self._val

    def is_const(self):
        return True


def constant(val: float, dim) -> Tensor:
    return Tensor(ConstantNode(val, dim))


# --------------------------------------------------------------------------------------
# binary ops (create_op! macro, src/graph/ops/ops.rs:7-219)
# --------------------------------------------------------------------------------------


class _BinaryNode(Node):
    ir_cls = None
    ir_eq_cls = None

    def __init__(self, left: Tensor, right: Tensor, is_op_equal: bool):
        self.left = left
        self.right = right
        self._val: Optional[Value] = None
        self.is_op_equal = is_op_equal

    def forward(self):
        v = self.val()
        if v is not None:
            return v
        left = self.left.forward()
        right = self.right.forward()
        if self.is_op_equal:
            ir_b_add(self.ir_eq_cls(s=left.id, o=right.id))
            res = Value(left.dim, left.id)
        else:
            id = self._val.id if self._val is not None else ir_b_id()
            ir_b_add(self.ir_cls(a=left.id, b=right.id, res=id))
            res = Value(left.dim, id)
        self._val = res
        return res.clone()

    def dim(self):
        return self.right.dim() if self.left.is_const() else self.left.dim()

    def val(self):
        if self.left.val() is None or self.right.val() is None:
            return None
        return self._val

    def grad(self):
        if self.is_op_equal:
            return self.left.grad()
        raise RuntimeError("Calling .grad() on a non-tensor node")

    def reset_grad(self):
        if self.is_op_equal:
            self.left.reset_grad()
        else:
            raise RuntimeError("Calling .reset_grad() on a non-tensor node")


class AddNode(_BinaryNode):
    ir_cls = IR.ElwAdd
    ir_eq_cls = IR.ElwAddEq

    def backward(self, grad: Value):
        assert self.left.val() is not None, "l forward"
        assert self.right.val() is not None, "r forward"
        self.left.n.backward(grad.clone())
        self.right.n.backward(grad.clone())


class MultiplyNode(_BinaryNode):
    ir_cls = IR.ElwMultiply
    ir_eq_cls = IR.ElwMultiplyEq

    def backward(self, grad: Value):
        l = self.left.val()
        r = self.right.val()
        assert l is not None, "l forward"
        assert r is not None, "r forward"
        self.left.n.backward((r.to_node() * grad.to_node()).forward())
        self.right.n.backward((l.to_node() * grad.to_node()).forward())


def _binary(cls, a, b) -> Tensor:
    if isinstance(a, Tensor) and isinstance(b, Tensor):
        x, y = try_broadcast(a, b)
    elif isinstance(a, Tensor):
        x, y = try_broadcast(a, constant(float(b), a.dim()))
    else:
        x, y = try_broadcast(constant(float(a), b.dim()), b)
    return Tensor(cls(x, y, False))


def _op_equal(cls, self_t: Tensor, rhs) -> None:
    s_clone = self_t.deep_copy()
    if isinstance(rhs, Value):
        rhs = rhs.to_node()
    elif not isinstance(rhs, Tensor):
        rhs = constant(float(rhs), self_t.dim())
    a, b = try_broadcast(s_clone, rhs)
    self_t.replace(cls(a, b, True))


# --------------------------------------------------------------------------------------
# unary functions (create_func! macro, src/graph/ops/func.rs:6-98)
# --------------------------------------------------------------------------------------

_UNARY_IR = {"exp2": IR.Exp2, "log2": IR.Log2, "sin": IR.Sin, "recip": IR.Recip, "sqrt": IR.Sqrt}


class UnaryNode(Node):
    def __init__(self, parent: Tensor, fn: str):
        self.parent = parent
        self.fn = fn
        self._val: Optional[Value] = None

    def forward(self):
        v = self.val()
        if v is not None:
            return v
        a = self.parent.forward()
        id = self._val.id if self._val is not None else ir_b_id()
        ir_b_add(_UNARY_IR[self.fn](a=a.id, res=id))
        self._val = Value(a.dim, id)
        return self._val.clone()

    def dim(self):
        return self.parent.dim()

    def backward(self, grad: Value):
        v = self.parent.val()
        assert v is not None, "parent val invalid at unary func"
        g = grad.to_node()
        if self.fn == "exp2":
            out = g * np.log(np.float32(2.0)) * v.to_node().exp2()  # func.rs:72-76
        elif self.fn == "log2":
            out = g * v.to_node().recip() * np.log2(np.float32(math.e))  # func.rs:78-82
        elif self.fn == "recip":
            out = g * (-1.0 / v.to_node().pow2())  # func.rs:84-87
        elif self.fn == "sqrt":
            out = g * (1.0 / (2.0 * v.to_node().sqrt()))  # func.rs:89-92
        else:
            out = g * v.to_node().cos()  # func.rs:94-97
        self.parent.n.backward(out.forward())

    def val(self):
        if self.parent.val() is None:
            return None
        return self._val


_CMP_IR = {"equal": IR.EqualZero, "more": IR.MoreZero, "less": IR.LessZero}


class CompareNode(Node):
    """`x.equal(b)` etc.: a comparison of (a-b) with zero, no gradient
    (src/graph/ops/equality.rs:3-78)."""

    def __init__(self, parent: Tensor, kind: str):
        self.parent = parent
        self.kind = kind
        self._val: Optional[Value] = None

    def forward(self):
        v = self.val()
        if v is not None:
            return v
        a = self.parent.forward()
        id = self._val.id if self._val is not None else ir_b_id()
        ir_b_add(_CMP_IR[self.kind](a=a.id, res=id))
        self._val = Value(a.dim, id)
        return self._val.clone()

    def dim(self):
        return self.parent.dim()

    def backward(self, grad):
        pass

    def val(self):
        if self.parent.val() is None:
            return None
        return self._val

    def grad(self):
        return Value.zeros(self.dim())


# --------------------------------------------------------------------------------------
# sum / dot
# --------------------------------------------------------------------------------------


class SumNode(Node):
    """2-D sum over the last dim (src/graph/ops/sum.rs:3-49)."""

    def __init__(self, parent: Tensor):
        self.parent = parent
        self._val: Optional[Value] = None

    def forward(self):
        v = self.val()
        if v is not None:
            return v
        a = self.parent.forward()
        assert len(self.parent.dim()) == 2, "Reduce (sum) node needs dim=2"
        id = self._val.id if self._val is not None else ir_b_id()
        ir_b_add(IR.Sum(a=a.id, res=id))
        self._val = Value(a.dim[:-1], id)
        return self._val.clone()

    def dim(self):
        return self.parent.dim()[:-1]

    def backward(self, grad: Value):
        repeat_n = self.parent.dim()[-1]
        self.parent.n.backward(grad.to_node().unsqueeze(-1).broadcast(-1, repeat_n).forward())

    def val(self):
        if self.parent.val() is None:
            return None
        return self._val


class MaxNode(Node):
    """2-D maximum over the last dim: the `Max` command.  Backward: the gradient goes to the positions that hold the
    maximum, in equal shares when several do."""

    def __init__(self, parent: Tensor):
        self.parent = parent
        self._val: Optional[Value] = None

    def forward(self):
        v = self.val()
        if v is not None:
            return v
        a = self.parent.forward()
        assert len(self.parent.dim()) == 2, "Reduce (max) node needs dim=2"
        id = self._val.id if self._val is not None else ir_b_id()
        ir_b_add(IR.Max(a=a.id, res=id))
        self._val = Value(a.dim[:-1], id)
        return self._val.clone()

    def dim(self):
        return self.parent.dim()[:-1]

    def backward(self, grad: Value):
        n = self.parent.dim()[-1]
        m = self._val.to_node().unsqueeze(-1).broadcast(-1, n)
        at_max = self.parent.equal(m)
        share = at_max / Tensor(SumNode(at_max)).unsqueeze(-1).broadcast(-1, n)
        self.parent.n.backward((grad.to_node().unsqueeze(-1).broadcast(-1, n) * share).forward())

    def val(self):
        if self.parent.val() is None:
            return None
        return self._val


class StopGradNode(Node):
    """Passes its parent's value through and ends the backward pass there."""

    def __init__(self, parent: Tensor):
        self.parent = parent

    def forward(self):
        return self.parent.forward()

    def dim(self):
        return self.parent.dim()

    def backward(self, grad: Value):
        return None

    def val(self):
        return self.parent.val()


class DotProductNode(Node):
    """2-D x 2-D matrix product (src/graph/ops/dot_product.rs:6-86)."""

    def __init__(self, left: Tensor, right: Tensor):
        self.left = left
        self.right = right
        self._val: Optional[Value] = None

    def forward(self):
        v = self.val()
        if v is not None:
            return v
        left = self.left.forward()
        right = self.right.forward()
        assert len(left.dim) == 2, "A must be a 2d array"
        assert len(right.dim) == 2, "B must be a 2d array"
        assert left.dim[1] == right.dim[0], "A's second dimension must equal B's first dimension"
        id = self._val.id if self._val is not None else ir_b_id()
        ir_b_add(IR.DotProduct(a=left.id, b=right.id, res=id))
        self._val = Value([left.dim[0], right.dim[-1]], id)
        return self._val.clone()

    def dim(self):
        return [self.left.dim()[0], self.right.dim()[-1]]

    def backward(self, grad: Value):
        g_node = grad.to_node()
        self.left.n.backward(dot(g_node, self.right.t()).forward())
        self.right.n.backward(dot(self.left.t(), g_node).forward())

    def val(self):
        if self.left.val() is None or self.right.val() is None:
            return None
        return self._val


def dot(a: Tensor, b: Tensor) -> Tensor:
    return Tensor(DotProductNode(a, b))


# --------------------------------------------------------------------------------------
# data movement nodes
# --------------------------------------------------------------------------------------


def handle_minus_dim(source_dim, input_dim):
    input_dim = _as_i32_list(input_dim)
    if -1 in input_dim:
        idx = input_dim.index(-1)
        total_size = int(np.prod(source_dim))
        inp_size = -int(np.prod(input_dim))
        assert total_size % inp_size == 0, "Can't fill in -1"
        ret = list(input_dim)
        ret[idx] = total_size // inp_size
        return ret
    return list(input_dim)


def c_view(p: Value, target_dim, id: Optional[str]) -> Value:
    assert int(np.prod(target_dim)) == int(np.prod(p.dim)), "Target dim must be same size as input dim"
    id = id if id is not None else ir_b_id()
    ir_b_add(IR.View(a=p.id, target_dim=list(target_dim), res=id))
    return Value(target_dim, id)


class ViewNode(Node):
    def __init__(self, parent: Tensor, target_dim):
        self.parent = parent
        self.target_dim = list(target_dim)
        self._val: Optional[Value] = None

    def forward(self):
        # The reference returns its cached value without looking at the parent (view.rs:18-20), so a
        # predicate whose chain contains a view (every `.all()` does) is never refreshed when
        # `ir_while` re-forwards it.  Like every other node, the view is re-emitted here (with the
        # same id) when something below it was invalidated.
        v = self.val()
        if v is not None:
            return v.clone()
        p = self.parent.forward()
        self._val = c_view(p, self.target_dim, self._val.id if self._val is not None else None)
        return self._val.clone()

    def dim(self):
        return list(self.target_dim)

    def backward(self, grad: Value):
        self.parent.n.backward(c_view(grad, self.parent.dim(), None))

    def val(self):
        if self.parent.val() is None:
            return None
        return self._val


def c_permute(a: Value, permute, id: Optional[str]) -> Value:
    assert len(permute) == len(a.dim), "Permute dimension mismatch"
    for i in permute:
        if i >= len(a.dim):
            raise RuntimeError("Permute index out of bounds")
    if all(i == v for i, v in enumerate(permute)):
        return a.clone()
    id = id if id is not None else ir_b_id()
    ir_b_add(IR.Permute(a=a.id, p=list(permute), res=id))
    return Value([a.dim[permute[i]] for i in range(len(a.dim))], id)


class PermuteNode(Node):
    def __init__(self, parent: Tensor, permute):
        self.parent = parent
        self.permute = list(permute)
        self._val: Optional[Value] = None

    def forward(self):
        v = self.val()
        if v is not None:
            return v
        p_val = self.parent.forward()
        self._val = c_permute(p_val, self.permute, self._val.id if self._val is not None else None)
        return self._val.clone()

    def dim(self):
        c_dim = self.parent.dim()
        return [c_dim[self.permute[i]] for i in range(len(c_dim))]

    def backward(self, grad: Value):
        inverse = [0] * len(self.permute)
        for i, p in enumerate(self.permute):
            inverse[p] = i
        self.parent.n.backward(c_permute(grad, inverse, None))

    def val(self):
        if self.parent.val() is None:
            return None
        return self._val


class BroadcastNode(Node):
    def __init__(self, parent: Tensor, repeat: int, dim: int):
        self.parent = parent
        self.repeat = repeat
        self._dim = dim
        self._val: Optional[Value] = None

    def forward(self):
        v = self.val()
        if v is not None:
            return v
        p = self.parent.forward()
        id = self._val.id if self._val is not None else ir_b_id()
        ir_b_add(IR.Broadcast(a=p.id, dim=self._dim, r=self.repeat, res=id))
        r_dim = list(p.dim)
        r_dim[self._dim] = self.repeat
        self._val = Value(r_dim, id)
        return self._val.clone()

    def dim(self):
        p_dim = self.parent.dim()
        p_dim[self._dim] = self.repeat
        return p_dim

    def backward(self, grad: Value):
        # The reference hands the parent the summed gradient with the broadcast dim dropped
        # (broadcast.rs:28-32), which only works when the parent is the left-padding view.  The dim is
        # put back (a free view) so any parent sees a gradient of its own shape.
        g = grad.to_node().sum(self._dim).view(self.parent.dim())
        self.parent.n.backward(g.forward())

    def val(self):
        if self.parent.val() is None:
            return None
        return self._val


def is_broadcastable(dim_a, dim_b) -> bool:
    la, lb = len(dim_a), len(dim_b)
    if la == 0 or lb == 0:
        return False
    for i in range(max(la, lb)):
        if i >= la or i >= lb:
            return True
        x, y = dim_a[la - i - 1], dim_b[lb - i - 1]
        if x != y and x != 1 and y != 1:
            return False
    return True


def make_broadcast_node(n: Tensor, target_dim) -> Tensor:
    n_dim = list(n.dim())
    assert len(target_dim) >= len(n_dim), "Wrong broadcasted node"
    n_dim = [1] * (len(target_dim) - len(n_dim)) + n_dim
    ret_n = n.view(n_dim)
    for i in range(len(target_dim)):
        if target_dim[i] != n_dim[i]:
            assert n_dim[i] == 1, "Can't broadcast to target dim"
            ret_n = Tensor(BroadcastNode(ret_n, target_dim[i], i))
    return ret_n


def try_broadcast(a: Tensor, b: Tensor):
    """src/graph/data/broadcast.rs:145-190."""
    if len(a.dim()) == 0 and len(b.dim()) > 0:
        a = a.unsqueeze(0)
    if len(b.dim()) == 0 and len(a.dim()) > 0:
        b = b.unsqueeze(0)
    if a.dim() == b.dim():
        return a, b
    if a.is_const() or b.is_const():
        return a, b
    if is_broadcastable(a.dim(), b.dim()):
        la, lb = len(a.dim()), len(b.dim())
        if la == lb:
            is_a_broadcast = sum(a.dim()) < sum(b.dim())
        else:
            is_a_broadcast = la < lb
        if is_a_broadcast:
            return make_broadcast_node(a, b.dim()), b
        return a, make_broadcast_node(b, a.dim())
    raise RuntimeError(f"Cannot broadcast {a.dim()} to {b.dim()}")


class IndexNode(Node):
    def __init__(self, parent: Tensor, idx: int, dim: int):
        self.parent = parent
        self.idx = idx
        self._dim = dim
        self._val: Optional[Value] = None

    def forward(self):
        v = self.val()
        if v is not None:
            return v
        p = self.parent.forward()
        id = self._val.id if self._val is not None else ir_b_id()
        ir_b_add(IR.Index(a=p.id, index=self.idx, dim=self._dim, res=id))
        d = list(p.dim)
        del d[self._dim]
        self._val = Value(d, id)
        return self._val.clone()

    def dim(self):
        d = self.parent.dim()
        del d[self._dim]
        return d

    def backward(self, grad: Value):
        # zeros before, the gradient slice, zeros after, concatenated on the indexed dim.
        # The reference sizes the trailing block from dim 0 and unsqueezes at 0
        # (index.rs:44,51), which is only right for dim == 0; the general form is used here
        # and coincides with the reference wherever the reference is right.
        i_dim = self.parent.dim()
        first = list(i_dim)
        first[self._dim] = self.idx
        second = list(i_dim)
        second[self._dim] = i_dim[self._dim] - self.idx - 1
        first_zero = Value.zeros(first).to_node()
        second_zero = Value.zeros(second).to_node()
        grad_n = grad.to_node()
        self.parent.n.backward(
            concat([first_zero, grad_n.unsqueeze(self._dim), second_zero], self._dim).forward())

    def val(self):
        if self.parent.val() is None:
            return None
        return self._val


class ConcatNode(Node):
    def __init__(self, nodes: List[Tensor], dim: int):
        self.nodes = list(nodes)
        self._dim = dim
        self._val: Optional[Value] = None

    def forward(self):
        v = self.val()
        if v is not None:
            return v
        values = [n.forward() for n in self.nodes]
        self._val = c_concat(values, self._dim, self._val.id if self._val is not None else None)
        return self._val.clone()

    def dim(self):
        d = self.nodes[0].dim()
        for n in self.nodes[1:]:
            d[self._dim] += n.dim()[self._dim]
        return d

    def backward(self, grad: Value):
        c = 0
        for n in self.nodes:
            d_interest = n.dim()[self._dim]
            g = grad.to_node().r(range(c, c + d_interest), self._dim).forward()
            n.n.backward(g)
            c += d_interest

    def val(self):
        for n in self.nodes:
            if n.val() is None:
                return None
        return self._val


def concat(nodes: List[Tensor], dim: int) -> Tensor:
    assert len(nodes) > 0, "Empty concat tensor"
    n_dim = len(nodes[0].dim())
    dim = n_dim + dim if dim < 0 else dim
    return Tensor(ConcatNode(nodes, dim))


def c_concat(nodes: List[Value], dim: int, id: Optional[str]) -> Value:
    """Chained two-operand `Concat` commands (concat.rs:75-118)."""
    first_dim = None
    for v in nodes:
        if first_dim is None:
            first_dim = list(v.dim)
        else:
            f_d, i_d = list(first_dim), list(v.dim)
            assert len(f_d) == len(i_d), "Dimensions are not equal at concat"
            del f_d[dim]
            del i_d[dim]
            assert f_d == i_d, "Dim misaligned at concat"
    prev = nodes[0].id
    total_d = list(nodes[0].dim)
    last_id = id if id is not None else ir_b_id()
    for i in range(1, len(nodes)):
        new_id = last_id if i == len(nodes) - 1 else ir_b_id()
        ir_b_add(IR.Concat(a=prev, b=nodes[i].id, dim=dim, res=new_id))
        prev = new_id
        total_d[dim] += nodes[i].dim[dim]
    return Value(total_d, prev)


class ContigiousNode(Node):
    def __init__(self, parent: Tensor):
        self.parent = parent
        self._val: Optional[Value] = None

    def forward(self):
        v = self.val()
        if v is not None:
            return v
        p = self.parent.forward()
        id = self._val.id if self._val is not None else ir_b_id()
        ir_b_add(IR.Contigious(a=p.id, res=id))
        self._val = Value(p.dim, id)
        return self._val.clone()

    def dim(self):
        return self.parent.dim()

    def backward(self, grad: Value):
        self.parent.n.backward(grad)

    def val(self):
        if self.parent.val() is None:
            return None
        return self._val
