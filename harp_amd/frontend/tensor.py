"""Lazy tensors: operations build a graph, `realize()` runs it on the default
device.

Host-side mirror of the reference's `src/tensor/`: `tensor.rs:58-160`
(constructors), `ops.rs` (elementwise `:21-160`, reductions `:178-245`,
views `:336-450`, `scale`/`ones_like`/`zeros_like` `:699-725`),
`realize.rs` (`realize` `:134-247`, `to_vec` `:268-298`, `set_data`
`:322-359`, constant buffers for nodes named ones/zeros/scalar `:391-421`).
Reference behaviours kept as they are: `scale(f)` multiplies by a tensor of
ones and ignores `f`; `mean` returns `sum`; `pow` is `exp(ln(x))`.
"""

from __future__ import annotations

from collections import OrderedDict
from typing import Dict, List, Optional, Sequence

import numpy as np

from . import graph as G
from .ast import DType, F32
from .device import allocate_buffer_on_default_device, has_default_device
from .executor import ExecutionError, execute_graph

_NP = {"f32": np.float32, "f64": np.float64, "i32": np.int32, "i64": np.int64,
       "u8": np.uint8, "bool": np.uint8, "i8": np.int8, "i16": np.int16,
       "u16": np.uint16, "u32": np.uint32, "u64": np.uint64, "f16": np.float16}

# set_data() registers buffers here so any graph that uses the input can find
# them (INPUT_BUFFER_CACHE, realize.rs:30-31); values keep their node alive.
_INPUT_BUFFER_CACHE: Dict[int, tuple] = {}


class Tensor:
    def __init__(self, graph: G.GraphNode):
        self.graph = graph
        self.buffer = None
        self._requires_grad = False
        self._grad: Optional["Tensor"] = None

    # -- constructors -------------------------------------------------------
    @staticmethod
    def from_graph(graph: G.GraphNode) -> "Tensor":
        return Tensor(graph)

    @staticmethod
    def input(shape: Sequence[int], dtype: DType = F32) -> "Tensor":
        return Tensor(G.input(list(shape), dtype))

    @staticmethod
    def named_input(name: str, shape: Sequence[int], dtype: DType = F32) -> "Tensor":
        return Tensor(G.named_input(name, list(shape), dtype))

    @staticmethod
    def zeros(shape, dtype: DType = F32) -> "Tensor":
        return Tensor(G.zeros(list(shape), dtype))

    @staticmethod
    def ones(shape, dtype: DType = F32) -> "Tensor":
        return Tensor(G.ones(list(shape), dtype))

    @staticmethod
    def ones_like(other: "Tensor") -> "Tensor":
        return Tensor(G.ones(other.shape(), other.dtype()))

    @staticmethod
    def zeros_like(other: "Tensor") -> "Tensor":
        return Tensor(G.zeros(other.shape(), other.dtype()))

    @staticmethod
    def scalar(_value=0.0, dtype: DType = F32) -> "Tensor":
        """A rank-0 constant node.  The value is not recorded (tensor.rs:332-337): realize
        fills every synthesised constant that is not `zeros` with 1.0 (realize.rs:391-421)."""
        return Tensor(G.scalar(dtype))

    @staticmethod
    def from_shape_data(shape: Sequence[int], data) -> "Tensor":
        """Checks that `data` has the shape's element count and returns a plain input: the
        reference does not attach the data either (tensor.rs:186-200); call set_data()."""
        n = 1
        for d in shape:
            n *= int(d)
        if len(data) != n:
            raise ValueError(f"Data length {len(data)} doesn't match shape {list(shape)} (numel={n})")
        return Tensor.input(shape)

    @staticmethod
    def from_numpy(arr: np.ndarray) -> "Tensor":
        """Convenience: input + set_data (needs a default device)."""
        dt = {v: k for k, v in _NP.items() if k != "bool"}[arr.dtype.type]
        t = Tensor.input(arr.shape, DType(dt))
        t.set_data(arr)
        return t

    # -- accessors ------------------------------------------------------------
    def shape(self) -> List[int]:
        return [int(e.evaluate()) for e in self.graph.shape()]

    def ndim(self) -> int:
        return self.graph.ndim()

    def dtype(self) -> DType:
        return self.graph.dtype

    def numel(self) -> int:
        n = 1
        for s in self.shape():
            n *= s
        return n

    def with_name(self, name: str) -> "Tensor":
        return Tensor(self.graph.with_name(name))

    # -- elementwise --------------------------------------------------------------
    def add(self, o): return Tensor(self.graph + o.graph)
    def mul(self, o): return Tensor(self.graph * o.graph)
    def sub(self, o): return Tensor(self.graph - o.graph)
    def div(self, o): return Tensor(self.graph / o.graph)
    __add__, __mul__, __sub__, __truediv__ = add, mul, sub, div

    def maximum(self, o): return Tensor(self.graph.maximum(o.graph))
    def minimum(self, o): return Tensor(self.graph.minimum(o.graph))
    def neg(self): return Tensor(-self.graph)
    __neg__ = neg
    def recip(self): return Tensor(self.graph.recip())
    def sqrt(self): return Tensor(self.graph.sqrt())
    def ln(self): return Tensor(self.graph.ln())
    def log2(self): return Tensor(self.graph.log2())
    def exp(self): return Tensor(self.graph.exp())
    def exp2(self): return Tensor(self.graph.exp2())
    def sin(self): return Tensor(self.graph.sin())
    def cos(self): return Tensor(self.graph.cos())
    def floor(self): return Tensor(self.graph.floor())
    def abs(self): return Tensor(self.graph.abs())
    def square(self): return self.mul(self)
    def pow(self, _exp: float): return self.ln().exp()

    def lt(self, o): return Tensor(self.graph.lt(o.graph))
    def gt(self, o): return Tensor(self.graph.gt(o.graph))
    def le(self, o): return Tensor(self.graph.le(o.graph))
    def ge(self, o): return Tensor(self.graph.ge(o.graph))
    def eq(self, o): return Tensor(self.graph.eq_node(o.graph))
    def ne(self, o): return Tensor(self.graph.ne_node(o.graph))

    def where_cond(self, cond, other):
        return Tensor(self.graph.where_cond(cond.graph, other.graph))

    def cast(self, dtype: DType): return Tensor(self.graph.cast(dtype))

    def scale(self, _factor: float) -> "Tensor":
        return self.mul(Tensor.ones_like(self))

    def scale_exact(self, factor: float) -> "Tensor":
        """x * factor as a literal in the map (not in the reference, whose `scale`
        ignores the factor).  The result is dense: a unary op keeps its operand's view
        (ops.rs:255-274) and the lowerer stores through that view, which for a slice of a
        larger buffer (the gradient of a padded input) indexes past a result sized by its
        shape -- neither the reference's backend-c nor the oracle checks that."""
        from .ast import AstNode
        from .grad import _dense_unary
        return Tensor(_dense_unary(self.graph, lambda x: AstNode.mul(x, AstNode.const_f32(factor))))

    # -- reductions (the reduced axis is squeezed away) ------------------------------
    def _check_axis(self, axis):
        if not 0 <= axis < self.ndim():
            raise IndexError(f"Axis {axis} out of bounds for {self.ndim()}D tensor")

    def sum(self, axis):
        self._check_axis(axis)
        return Tensor(self.graph.sum(axis).squeeze(axis))

    def max(self, axis):
        self._check_axis(axis)
        return Tensor(self.graph.max(axis).squeeze(axis))

    def min(self, axis):
        self._check_axis(axis)
        return Tensor(self.graph.min(axis).squeeze(axis))

    def prod(self, axis):
        self._check_axis(axis)
        return Tensor(self.graph.prod(axis).squeeze(axis))

    def mean(self, axis): return self.sum(axis)

    def cumsum(self, axis): return Tensor(self.graph.cumsum(axis))
    def cumprod(self, axis): return Tensor(self.graph.cumprod(axis))
    def cummax(self, axis): return Tensor(self.graph.cummax(axis))

    # -- views ---------------------------------------------------------------------------
    def unsqueeze(self, axis): return Tensor(self.graph.unsqueeze(axis))
    def squeeze(self, axis): return Tensor(self.graph.squeeze(axis))
    def permute(self, axes): return Tensor(self.graph.permute(list(axes)))
    def contiguous(self): return Tensor(self.graph.contiguous())
    def expand(self, axis, size): return Tensor(self.graph.expand(axis, size))

    def t(self):
        n = self.ndim()
        axes = list(range(n))
        axes[n - 2], axes[n - 1] = axes[n - 1], axes[n - 2]
        return self.permute(axes)

    def reshape(self, shape):
        n = 1
        for s in shape:
            n *= s
        if n != self.numel():
            raise ValueError(f"Cannot reshape tensor of {self.numel()} elements to {n} elements")
        return Tensor(self.graph.reshape(list(shape)))

    def flatten(self): return self.reshape([self.numel()])

    def pad(self, padding): return Tensor(self.graph.pad(list(padding), "zero"))

    def unfold(self, axes, sizes, strides, dilations):
        return Tensor(self.graph.unfold(axes, sizes, strides, dilations))

    def unfold_1d(self, kernel_size, stride, dilation):
        """[N,C,L] -> [N,C,L_out,K] (ops.rs:592-598)."""
        return self.unfold([2], [kernel_size], [stride], [dilation])

    def unfold_2d(self, kernel_size, stride, dilation):
        """[N,C,H,W] -> [N,C,H_out,W_out,kH,kW] (ops.rs:566-580)."""
        return self.unfold([2, 3], list(kernel_size), list(stride), list(dilation))

    def unfold_3d(self, kernel_size, stride, dilation):
        """[N,C,D,H,W] -> [N,C,D_out,H_out,W_out,kD,kH,kW] (ops.rs:611-624)."""
        return self.unfold([2, 3, 4], list(kernel_size), list(stride), list(dilation))

    def fold(self, output_shape, axes, sizes, strides, dilations):
        return Tensor(self.graph.fold(output_shape, axes, sizes, strides, dilations))

    # -- autograd (src/tensor/autograd.rs:83-340) ------------------------------------------------
    def requires_grad_(self, flag: bool = True) -> "Tensor":
        self._requires_grad = bool(flag)
        return self

    def requires_grad(self) -> bool:
        return self._requires_grad

    def grad(self) -> Optional["Tensor"]:
        return self._grad

    def set_grad(self, grad: "Tensor") -> None:
        self._grad = grad

    def zero_grad(self) -> None:
        self._grad = None

    def accumulate_grad(self, grad: "Tensor") -> None:
        """Adds to the stored gradient graph, or stores the first one (autograd.rs:200-209)."""
        self._grad = grad if self._grad is None else Tensor(self._grad.graph + grad.graph)

    def try_buffer(self):
        """The realized buffer or None (realize.rs:97-104)."""
        return self.buffer

    def detach(self) -> "Tensor":
        t = Tensor(self.graph)
        t.buffer = self.buffer
        return t

    def backward(self):
        raise ExecutionError("NoParams: backward() requires explicit parameters. Use "
                             "backward_with_params([tensor1, tensor2, ...]) instead.")

    def backward_with_params(self, params: Sequence["Tensor"], exact: bool = None) -> None:
        """Builds the gradient graphs and stores them on the parameters; nothing
        runs until a gradient is realized.  `exact=True` uses mathematically correct
        VJPs instead of the reference's rules as written."""
        from .grad import backward as compute_backward
        from . import config
        if exact is None:
            exact = config.EXACT
        if not params:
            raise ExecutionError("NoParams: No parameters provided for backward pass.")
        res = compute_backward(self.graph, [p.graph for p in params], exact=exact)
        for p in params:
            g = res.get(p.graph)
            if g is not None:
                p.set_grad(Tensor(g))

    # -- realisation -------------------------------------------------------------------------
    def is_realized(self) -> bool:
        return self.buffer is not None

    def set_data(self, data) -> None:
        if not has_default_device():
            raise ExecutionError("NoDevice")
        arr = np.ascontiguousarray(np.asarray(data, dtype=_NP[self.dtype().name]))
        if arr.size != self.numel():
            raise ExecutionError(f"ShapeMismatch: Data size {arr.size} doesn't match "
                                 f"tensor size {self.numel()}")
        buf = allocate_buffer_on_default_device(self.shape(), self.dtype())
        if hasattr(buf, "write_array"):
            buf.write_array(arr)                       # straight from the array's memory
        else:
            buf.write_from_host(arr.tobytes())
        _INPUT_BUFFER_CACHE[id(self.graph)] = (self.graph, buf.clone_buffer())
        self.buffer = buf

    def set_buffer(self, buf) -> None:
        """Binds an input tensor to a buffer that is already on the device (the realized buffer
        of another tensor of this size).  Not in the reference, whose only way to give an input
        its data is `set_data` from host memory."""
        if not self.graph.is_external():
            raise ExecutionError("NotAnInput: set_buffer() needs an input tensor")
        want = self.numel() * np.dtype(_NP[self.dtype().name]).itemsize
        if buf is None or buf.byte_len() != want:
            raise ExecutionError(f"ShapeMismatch: buffer of {None if buf is None else buf.byte_len()} bytes "
                                 f"for a tensor of {want}")
        _INPUT_BUFFER_CACHE[id(self.graph)] = (self.graph, buf)
        self.buffer = buf

    def realize(self) -> "Tensor":
        if self.is_realized():
            return self
        if not has_default_device():
            raise ExecutionError("NoDevice")
        g = self.graph
        if g.is_external():
            hit = _INPUT_BUFFER_CACHE.get(id(g))
            if hit is None:
                raise ExecutionError("MissingInput: Input tensor has no data. "
                                     "Call set_data() first.")
            self.buffer = hit[1].clone_buffer()
            return self
        input_buffers = {}
        constant_inputs = {}
        for node in G.collect_inputs([g]):
            hit = _INPUT_BUFFER_CACHE.get(id(node))
            if hit is not None:
                input_buffers[id(node)] = hit[1].clone_buffer()
                continue
            const = _create_constant_buffer(node)
            if const is None:
                raise ExecutionError(f"MissingInput: Input tensor "
                                     f"'{node.name or hex(id(node))}' has no data. "
                                     f"Call set_data() first.")
            input_buffers[id(node)] = const
            constant_inputs[id(node)] = "zeros" if node.name == "zeros" else "ones"
        res = execute_graph([g], input_buffers, constant_inputs=constant_inputs)
        if not res or res[0] is None:
            raise ExecutionError("Internal: No output buffer returned from execution")
        self.buffer = res[0]
        return self

    def to_numpy(self) -> np.ndarray:
        """Flat array of the buffer's elements (to_vec, realize.rs:268-298)."""
        if not self.is_realized():
            raise ExecutionError("NotRealized")
        raw = self.buffer.read_to_host()
        return np.frombuffer(raw, dtype=_NP[self.dtype().name]).copy()

    def to_vec(self) -> list:
        return self.to_numpy().tolist()

    def clear_buffer(self) -> None:
        self.buffer = None


def realize_many(tensors: Sequence[Tensor]) -> None:
    """Realizes several tensors with one `execute_graph` call (`execute_graph` takes a slice
    of roots, executor.rs:149-152), so work they share is done once."""
    todo = [t for t in tensors if not t.is_realized() and not t.graph.is_external()]
    for t in tensors:
        if t.graph.is_external():
            t.realize()
    if not todo:
        return
    if not has_default_device():
        raise ExecutionError("NoDevice")
    roots = [t.graph for t in todo]
    input_buffers, constant_inputs = {}, {}
    for node in G.collect_inputs(roots):
        hit = _INPUT_BUFFER_CACHE.get(id(node))
        if hit is not None:
            input_buffers[id(node)] = hit[1].clone_buffer()
            continue
        const = _create_constant_buffer(node)
        if const is None:
            raise ExecutionError(f"MissingInput: Input tensor '{node.name or hex(id(node))}' "
                                 f"has no data. Call set_data() first.")
        input_buffers[id(node)] = const
        constant_inputs[id(node)] = "zeros" if node.name == "zeros" else "ones"
    res = execute_graph(roots, input_buffers, constant_inputs=constant_inputs)
    for t, b in zip(todo, res):
        if b is None:
            raise ExecutionError("Internal: No output buffer returned from execution")
        t.buffer = b


_CONSTANT_BUFFERS: "OrderedDict[tuple, object]" = OrderedDict()
_CONSTANT_BUFFERS_MAX = 32


def _create_constant_buffer(node: G.GraphNode):
    """Buffer for a ones / zeros tensor (realize.rs:391-421).  The filled buffers are kept per
    device, shape and value: a training loop asks for the same ones every step, and the
    executor only ever reads them (it clones its inputs)."""
    fill = {"ones": 1.0, "zeros": 0.0, "scalar": 1.0}.get(node.name)
    if fill is None:
        return None
    shape = [int(e.evaluate()) for e in node.shape()]
    from .device import get_default_device
    dev = get_default_device()
    key = (id(dev.device) if dev is not None else None, tuple(shape), node.dtype.name, fill)
    hit = _CONSTANT_BUFFERS.get(key)
    if hit is not None:
        _CONSTANT_BUFFERS.move_to_end(key)
        return hit
    buf = allocate_buffer_on_default_device(shape, node.dtype)
    if fill != 0.0:                                   # a fresh buffer is zero-filled already
        n = 1
        for s in shape:
            n *= s
        buf.write_from_host(np.full(n, fill, dtype=_NP[node.dtype.name]).tobytes())
    _CONSTANT_BUFFERS[key] = buf
    while len(_CONSTANT_BUFFERS) > _CONSTANT_BUFFERS_MAX:
        _CONSTANT_BUFFERS.popitem(last=False)
    return buf
