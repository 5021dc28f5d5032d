"""StableHLO text emitter with reverse-mode autodiff.

The five benchmark programs have to reach ``PJRT_Client_Compile`` as StableHLO,
and no JAX is installed next to this package, so the programs are traced by this
small builder instead.  It prints the textual forms that ``jax.jit(f).lower(...)
.as_text()`` prints (pretty forms where StableHLO has one, the generic
``"stablehlo.op"(...) <{...}>`` form for gather/scatter/case) and its VJP rules
emit what JAX's transpose rules emit for the same primitive (convolution input
and filter gradients as convolutions with lhs/rhs dilation and swapped dimension
numbers, gather gradient as scatter-add, broadcast gradient as reduce, ...).

The reference receives exactly this kind of module at
src/pjrt_plugin/pjrt_client.cc:179-257 (format "mlir", bytecode or text).
"""
from __future__ import annotations

import math
import struct
from typing import Callable, Dict, List, Optional, Sequence, Tuple, Union

import numpy as np

# ----------------------------------------------------------------------------
# element types
# ----------------------------------------------------------------------------
FLOAT_TYPES = ("f32", "bf16", "f16", "f64")
INT_TYPES = ("i8", "i16", "i32", "i64", "ui8", "ui16", "ui32", "ui64")
_NP = {
    "f32": np.float32, "f64": np.float64, "f16": np.float16, "i1": np.bool_,
    "i8": np.int8, "i16": np.int16, "i32": np.int32, "i64": np.int64,
    "ui8": np.uint8, "ui16": np.uint16, "ui32": np.uint32, "ui64": np.uint64,
}


def ttype(shape: Sequence[int], dtype: str) -> str:
    if len(shape) == 0:
        return f"tensor<{dtype}>"
    return "tensor<" + "x".join(str(int(d)) for d in shape) + f"x{dtype}>"


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even float32 -> bfloat16 bit pattern (uint16)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + (0x7FFF + ((u >> 16) & 1))) >> 16
    r = np.where(nan, (u >> 16) | 0x40, r)
    return r.astype(np.uint16)


_SPECIAL_HEX = {  # (nan, +inf, -inf) bit patterns as MLIR prints them for each float type
    "f32": ("0x7FC00000", "0x7F800000", "0xFF800000"),
    "bf16": ("0x7FC0", "0x7F80", "0xFF80"),
    "f16": ("0x7E00", "0x7C00", "0xFC00"),
    "f64": ("0x7FF8000000000000", "0x7FF0000000000000", "0xFFF0000000000000"),
}


def _fmt_float(x: float, dtype: str = "f32") -> str:
    if math.isnan(x):
        return _SPECIAL_HEX[dtype][0]
    if math.isinf(x):
        return _SPECIAL_HEX[dtype][1 if x > 0 else 2]
    return "%.9e" % x


class Val:
    """One SSA value of the module under construction."""

    __slots__ = ("b", "name", "shape", "dtype", "block")
    __array_priority__ = 1000

    def __init__(self, b: "Builder", name: str, shape, dtype: str, block):
        self.b = b
        self.name = name
        self.shape = tuple(int(d) for d in shape)
        self.dtype = dtype
        self.block = block

    @property
    def type(self) -> str:
        return ttype(self.shape, self.dtype)

    @property
    def ndim(self) -> int:
        return len(self.shape)

    @property
    def size(self) -> int:
        n = 1
        for d in self.shape:
            n *= d
        return n

    # arithmetic sugar with numpy-style broadcasting
    def __add__(self, o): return self.b.add(self, o)
    def __radd__(self, o): return self.b.add(o, self)
    def __sub__(self, o): return self.b.sub(self, o)
    def __rsub__(self, o): return self.b.sub(o, self)
    def __mul__(self, o): return self.b.mul(self, o)
    def __rmul__(self, o): return self.b.mul(o, self)
    def __truediv__(self, o): return self.b.div(self, o)
    def __rtruediv__(self, o): return self.b.div(o, self)
    def __neg__(self): return self.b.neg(self)

    def astype(self, dt): return self.b.convert(self, dt)
    def reshape(self, *s):
        if len(s) == 1 and isinstance(s[0], (tuple, list)):
            s = tuple(s[0])
        return self.b.reshape(self, s)

    def __repr__(self):
        return f"Val({self.name}: {self.type})"


class _Node:
    __slots__ = ("ins", "outs", "vjp")

    def __init__(self, ins, outs, vjp):
        self.ins, self.outs, self.vjp = ins, outs, vjp


class _Block:
    _uid = 0

    def __init__(self, indent: int):
        _Block._uid += 1
        self.uid = _Block._uid
        self.lines: List[str] = []
        self.tape: List[_Node] = []
        self.indent = indent


class Builder:
    """Builds one module with a public @main."""

    def __init__(self, name: str = "jit_step"):
        self.module_name = name
        self._n = 0
        self._blocks: List[_Block] = []
        self._main_args: List[Val] = []
        self._arg_alias: Dict[str, int] = {}
        self._main_block = _Block(2)
        self._blocks.append(self._main_block)
        self._results: List[Val] = []
        self._const_cache = {}
        self._wanted = None   # names that need a cotangent during grad(); None = all

    def _want(self, v: "Val") -> bool:
        return self._wanted is None or v.name in self._wanted

    # ------------------------------------------------------------------ util
    @property
    def _blk(self) -> _Block:
        return self._blocks[-1]

    def _fresh(self, prefix="") -> str:
        self._n += 1
        return f"%{prefix}{self._n}"

    def _emit(self, line: str):
        self._blk.lines.append("  " * self._blk.indent + line)

    def _new(self, shape, dtype, prefix="") -> Val:
        return Val(self, self._fresh(prefix), shape, dtype, self._blk)

    def _record(self, ins, outs, vjp):
        if vjp is not None:
            self._blk.tape.append(_Node(list(ins), list(outs), vjp))

    def arg(self, shape, dtype="f32", alias_output: Optional[int] = None) -> Val:
        """Entry-function argument; `alias_output=k` marks it donated to result k (`tf.aliasing_output`, what
        jax.jit(..., donate_argnums=...) lowers to)."""
        v = Val(self, f"%arg{len(self._main_args)}", shape, dtype, self._main_block)
        self._main_args.append(v)
        if alias_output is not None:
            self._arg_alias[v.name] = int(alias_output)
        return v

    def donate(self, arg: Val, output_index: int):
        """Marks an existing argument as donated to result `output_index`."""
        self._arg_alias[arg.name] = int(output_index)

    def ret(self, *vals: Val):
        self._results = list(vals)

    # --------------------------------------------------------------- literals
    def constant(self, value, dtype: Optional[str] = None, shape=None) -> Val:
        """Splat scalar (optionally broadcast to `shape`) or dense ndarray."""
        if isinstance(value, Val):
            return value
        if isinstance(value, np.ndarray) and value.ndim > 0:
            arr = value
            if dtype is None:
                dtype = {v: k for k, v in _NP.items()}[arr.dtype.type]
            v = self._new(arr.shape, dtype, "cst_")
            if dtype == "bf16":
                raw = f32_to_bf16_bits(arr.astype(np.float32)).tobytes()
            else:
                raw = np.ascontiguousarray(arr.astype(_NP[dtype])).tobytes()
            if arr.size <= 16 and dtype not in ("bf16",):
                flat = arr.reshape(-1)
                if dtype in FLOAT_TYPES:
                    elems = [_fmt_float(float(x), dtype) for x in flat]
                elif dtype == "i1":
                    elems = ["true" if x else "false" for x in flat]
                else:
                    elems = [str(int(x)) for x in flat]

                def nest(shape, it):
                    if len(shape) == 1:
                        return "[" + ", ".join(next(it) for _ in range(shape[0])) + "]"
                    return "[" + ", ".join(nest(shape[1:], it) for _ in range(shape[0])) + "]"
                lit = nest(arr.shape, iter(elems))
            else:
                lit = '"0x' + raw.hex().upper() + '"'
            self._emit(f"{v.name} = stablehlo.constant dense<{lit}> : {v.type}")
            return v
        if isinstance(value, np.ndarray):
            value = value.item()
        if dtype is None:
            dtype = "f32" if isinstance(value, float) else ("i1" if isinstance(value, bool) else "i32")
        key = (self._blk.uid, dtype, repr(value))
        sc = self._const_cache.get(key)
        if sc is None:
            sc = self._new((), dtype, "cst_")
            if dtype in FLOAT_TYPES:
                lit = _fmt_float(float(value), dtype)
            elif dtype == "i1":
                lit = "true" if value else "false"
            else:
                lit = str(int(value))
            self._emit(f"{sc.name} = stablehlo.constant dense<{lit}> : {sc.type}")
            self._const_cache[key] = sc
        if shape is None or len(shape) == 0:
            return sc
        return self.broadcast_in_dim(sc, shape, ())

    def zeros(self, shape, dtype="f32"):
        return self.constant(0.0 if dtype in FLOAT_TYPES else 0, dtype, shape)

    def full_like(self, x: Val, value):
        return self.constant(float(value) if x.dtype in FLOAT_TYPES else value, x.dtype, x.shape)

    def iota(self, shape, dim: int, dtype="i32") -> Val:
        v = self._new(shape, dtype)
        self._emit(f"{v.name} = stablehlo.iota dim = {dim} : {v.type}")
        return v

    # ------------------------------------------------------------ broadcasting
    def _lift(self, a, b):
        """numpy-style broadcast of two operands (python scalars allowed)."""
        if not isinstance(a, Val) and not isinstance(b, Val):
            raise TypeError("need at least one Val")
        if not isinstance(a, Val):
            a = self.constant(float(a) if b.dtype in FLOAT_TYPES else a, b.dtype)
        if not isinstance(b, Val):
            b = self.constant(float(b) if a.dtype in FLOAT_TYPES else b, a.dtype)
        if a.dtype != b.dtype:
            raise TypeError(f"dtype mismatch {a} vs {b}")
        if a.shape == b.shape:
            return a, b
        shape = tuple(np.broadcast_shapes(a.shape, b.shape))
        return self._bcast_np(a, shape), self._bcast_np(b, shape)

    def _bcast_np(self, x: Val, shape) -> Val:
        if x.shape == tuple(shape):
            return x
        off = len(shape) - x.ndim
        if any(d == 1 and shape[off + i] != 1 for i, d in enumerate(x.shape)):
            keep = [i for i, d in enumerate(x.shape) if not (d == 1 and shape[off + i] != 1)]
            x = self.reshape(x, [x.shape[i] for i in keep])
            dims = [off + i for i in keep]
        else:
            dims = [off + i for i in range(x.ndim)]
        return self.broadcast_in_dim(x, shape, dims)

    def broadcast_in_dim(self, x: Val, shape, dims) -> Val:
        shape = tuple(int(s) for s in shape)
        dims = tuple(int(d) for d in dims)
        v = self._new(shape, x.dtype)
        self._emit(f"{v.name} = stablehlo.broadcast_in_dim {x.name}, dims = [{', '.join(map(str, dims))}] : ({x.type}) -> {v.type}")

        def vjp(g):
            red = [i for i in range(len(shape)) if i not in dims]
            gx = self.reduce_sum(g, red) if red else g
            # operand dims of size 1 that were expanded
            exp = [k for k, d in enumerate(dims) if x.shape[k] == 1 and shape[d] != 1]
            if exp:
                gx = self.reduce_sum(gx, exp)
            if gx.shape != x.shape:
                gx = self.reshape(gx, x.shape)
            return [gx]
        self._record([x], [v], vjp)
        return v

    # ------------------------------------------------------------- elementwise
    def _binary(self, op, a, b, vjp_fn=None) -> Val:
        a, b = self._lift(a, b)
        v = self._new(a.shape, a.dtype)
        self._emit(f"{v.name} = stablehlo.{op} {a.name}, {b.name} : {v.type}")
        if vjp_fn is not None and a.dtype in FLOAT_TYPES:
            self._record([a, b], [v], lambda g: vjp_fn(g, a, b, v))
        return v

    def add(self, a, b): return self._binary("add", a, b, lambda g, a, b, v: [g, g])
    def sub(self, a, b): return self._binary("subtract", a, b, lambda g, a, b, v: [g, self.neg(g)])
    def mul(self, a, b): return self._binary("multiply", a, b, lambda g, a, b, v: [self.mul(g, b), self.mul(g, a)])

    def div(self, a, b):
        return self._binary("divide", a, b, lambda g, a, b, v: [self.div(g, b), self.neg(self.div(self.mul(g, v), b))])

    def maximum(self, a, b):
        def vjp(g, a, b, v):
            m = self.compare(a, b, "GT")
            z = self.full_like(g, 0.0)
            return [self.select(m, g, z), self.select(m, z, g)]
        return self._binary("maximum", a, b, vjp)

    def minimum(self, a, b):
        def vjp(g, a, b, v):
            m = self.compare(a, b, "LT")
            z = self.full_like(g, 0.0)
            return [self.select(m, g, z), self.select(m, z, g)]
        return self._binary("minimum", a, b, vjp)

    def power(self, a, b): return self._binary("power", a, b)
    def remainder(self, a, b): return self._binary("remainder", a, b)
    def and_(self, a, b): return self._binary("and", a, b)
    def or_(self, a, b): return self._binary("or", a, b)
    def xor(self, a, b): return self._binary("xor", a, b)
    def shift_left(self, a, b): return self._binary("shift_left", a, b)
    def shift_right_logical(self, a, b): return self._binary("shift_right_logical", a, b)

    def _unary(self, op, x: Val, vjp_fn=None) -> Val:
        v = self._new(x.shape, x.dtype)
        self._emit(f"{v.name} = stablehlo.{op} {x.name} : {v.type}")
        if vjp_fn is not None and x.dtype in FLOAT_TYPES:
            self._record([x], [v], lambda g: [vjp_fn(g, x, v)])
        return v

    def neg(self, x): return self._unary("negate", x, lambda g, x, v: self.neg(g))
    def exp(self, x): return self._unary("exponential", x, lambda g, x, v: self.mul(g, v))
    def log(self, x): return self._unary("log", x, lambda g, x, v: self.div(g, x))
    def sqrt(self, x): return self._unary("sqrt", x, lambda g, x, v: self.div(g, self.mul(v, 2.0)))
    def rsqrt(self, x): return self._unary("rsqrt", x, lambda g, x, v: self.mul(g, self.mul(self.div(v, x), -0.5)))
    def tanh(self, x): return self._unary("tanh", x, lambda g, x, v: self.mul(g, self.sub(1.0, self.mul(v, v))))
    def logistic(self, x): return self._unary("logistic", x, lambda g, x, v: self.mul(g, self.mul(v, self.sub(1.0, v))))
    def abs(self, x): return self._unary("abs", x, lambda g, x, v: self.mul(g, self.sign(x)))
    def sign(self, x): return self._unary("sign", x)
    def floor(self, x): return self._unary("floor", x)
    def not_(self, x): return self._unary("not", x)

    def compare(self, a, b, direction: str, kind: Optional[str] = None) -> Val:
        a, b = self._lift(a, b)
        if kind is None:
            kind = "FLOAT" if a.dtype in FLOAT_TYPES else ("UNSIGNED" if a.dtype.startswith("ui") or a.dtype == "i1" else "SIGNED")
        v = self._new(a.shape, "i1")
        self._emit(f"{v.name} = stablehlo.compare  {direction}, {a.name}, {b.name},  {kind} : ({a.type}, {b.type}) -> {v.type}")
        return v

    def select(self, p: Val, a, b) -> Val:
        a, b = self._lift(a, b)
        if p.shape != a.shape:
            p = self._bcast_np(p, a.shape)
        v = self._new(a.shape, a.dtype)
        self._emit(f"{v.name} = stablehlo.select {p.name}, {a.name}, {b.name} : {p.type}, {v.type}")
        if a.dtype in FLOAT_TYPES:
            def vjp(g):
                z = self.full_like(g, 0.0)
                return [None, self.select(p, g, z), self.select(p, z, g)]
            self._record([p, a, b], [v], vjp)
        return v

    def clamp(self, lo, x: Val, hi) -> Val:
        lo = self.constant(lo, x.dtype) if not isinstance(lo, Val) else lo
        hi = self.constant(hi, x.dtype) if not isinstance(hi, Val) else hi
        v = self._new(x.shape, x.dtype)
        self._emit(f"{v.name} = stablehlo.clamp {lo.name}, {x.name}, {hi.name} : ({lo.type}, {x.type}, {hi.type}) -> {v.type}")
        return v

    def convert(self, x: Val, dtype: str) -> Val:
        if x.dtype == dtype:
            return x
        v = self._new(x.shape, dtype)
        self._emit(f"{v.name} = stablehlo.convert {x.name} : ({x.type}) -> {v.type}")
        if x.dtype in FLOAT_TYPES and dtype in FLOAT_TYPES:
            self._record([x], [v], lambda g: [self.convert(g, x.dtype)])
        return v

    def bitcast_convert(self, x: Val, dtype: str) -> Val:
        v = self._new(x.shape, dtype)
        self._emit(f"{v.name} = stablehlo.bitcast_convert {x.name} : ({x.type}) -> {v.type}")
        return v

    def stop_gradient(self, x: Val) -> Val:
        """Identity for values, cuts the tape (JAX prints nothing for it either)."""
        return Val(self, x.name, x.shape, x.dtype, x.block)

    # ------------------------------------------------------------ shape ops
    def reshape(self, x: Val, shape) -> Val:
        shape = tuple(int(s) for s in shape)
        if shape == x.shape:
            return x
        v = self._new(shape, x.dtype)
        assert v.size == x.size, (x.shape, shape)
        self._emit(f"{v.name} = stablehlo.reshape {x.name} : ({x.type}) -> {v.type}")
        self._record([x], [v], lambda g: [self.reshape(g, x.shape)])
        return v

    def transpose(self, x: Val, perm) -> Val:
        perm = tuple(int(p) for p in perm)
        if perm == tuple(range(x.ndim)):
            return x
        v = self._new([x.shape[p] for p in perm], x.dtype)
        self._emit(f"{v.name} = stablehlo.transpose {x.name}, dims = [{', '.join(map(str, perm))}] : ({x.type}) -> {v.type}")
        inv = [0] * len(perm)
        for i, p in enumerate(perm):
            inv[p] = i
        self._record([x], [v], lambda g: [self.transpose(g, inv)])
        return v

    def reverse(self, x: Val, dims) -> Val:
        v = self._new(x.shape, x.dtype)
        self._emit(f"{v.name} = stablehlo.reverse {x.name}, dims = [{', '.join(map(str, dims))}] : {v.type}")
        self._record([x], [v], lambda g: [self.reverse(g, dims)])
        return v

    def slice(self, x: Val, start, limit, strides=None) -> Val:
        strides = list(strides) if strides is not None else [1] * x.ndim
        shape = [max(0, -(-(l - s) // st)) for s, l, st in zip(start, limit, strides)]
        v = self._new(shape, x.dtype)
        parts = []
        for s, l, st in zip(start, limit, strides):
            parts.append(f"{s}:{l}" if st == 1 else f"{s}:{l}:{st}")
        self._emit(f"{v.name} = stablehlo.slice {x.name} [{', '.join(parts)}] : ({x.type}) -> {v.type}")

        def vjp(g):
            lo = list(start)
            hi = [x.shape[i] - (start[i] + (shape[i] - 1) * strides[i] + 1) if shape[i] > 0 else x.shape[i] - start[i] for i in range(x.ndim)]
            interior = [st - 1 for st in strides]
            return [self.pad(g, 0.0, lo, hi, interior)]
        self._record([x], [v], vjp)
        return v

    def pad(self, x: Val, value, low, high, interior=None) -> Val:
        interior = list(interior) if interior is not None else [0] * x.ndim
        pv = value if isinstance(value, Val) else self.constant(float(value) if x.dtype in FLOAT_TYPES else value, x.dtype)
        shape = []
        for d, lo, hi, it in zip(x.shape, low, high, interior):
            shape.append(lo + hi + d + max(d - 1, 0) * it)
        v = self._new(shape, x.dtype)
        f = lambda a: ", ".join(str(int(t)) for t in a)
        self._emit(f"{v.name} = stablehlo.pad {x.name}, {pv.name}, low = [{f(low)}], high = [{f(high)}], interior = [{f(interior)}] : ({x.type}, {pv.type}) -> {v.type}")

        def vjp(g):
            st = [it + 1 for it in interior]
            lim = [lo + (d - 1) * s + 1 if d > 0 else lo for d, lo, s in zip(x.shape, low, st)]
            return [self.slice(g, list(low), lim, st), None]
        self._record([x, pv], [v], vjp)
        return v

    def concatenate(self, xs: Sequence[Val], dim: int) -> Val:
        shape = list(xs[0].shape)
        shape[dim] = sum(x.shape[dim] for x in xs)
        v = self._new(shape, xs[0].dtype)
        self._emit(f"{v.name} = stablehlo.concatenate {', '.join(x.name for x in xs)}, dim = {dim} : ({', '.join(x.type for x in xs)}) -> {v.type}")

        def vjp(g):
            out, off = [], 0
            for x in xs:
                st = [0] * g.ndim
                li = list(g.shape)
                st[dim] = off
                li[dim] = off + x.shape[dim]
                out.append(self.slice(g, st, li))
                off += x.shape[dim]
            return out
        self._record(list(xs), [v], vjp)
        return v

    def dynamic_slice(self, x: Val, starts: Sequence[Val], sizes) -> Val:
        v = self._new(sizes, x.dtype)
        names = ", ".join([x.name] + [s.name for s in starts])
        types = ", ".join([x.type] + [s.type for s in starts])
        self._emit(f"{v.name} = stablehlo.dynamic_slice {names}, sizes = [{', '.join(map(str, sizes))}] : ({types}) -> {v.type}")

        def vjp(g):
            z = self.zeros(x.shape, x.dtype)
            return [self.dynamic_update_slice(z, g, starts)] + [None] * len(starts)
        self._record([x] + list(starts), [v], vjp)
        return v

    def dynamic_update_slice(self, x: Val, upd: Val, starts: Sequence[Val]) -> Val:
        v = self._new(x.shape, x.dtype)
        names = ", ".join([x.name, upd.name] + [s.name for s in starts])
        types = ", ".join([x.type, upd.type] + [s.type for s in starts])
        self._emit(f"{v.name} = stablehlo.dynamic_update_slice {names} : ({types}) -> {v.type}")
        return v

    # ------------------------------------------------------------ reductions
    def _reduce(self, x: Val, dims, op: str, init) -> Val:
        dims = sorted(int(d) % max(x.ndim, 1) for d in dims)
        shape = [d for i, d in enumerate(x.shape) if i not in dims]
        c = self.constant(init, x.dtype)
        v = self._new(shape, x.dtype)
        self._emit(f"{v.name} = stablehlo.reduce({x.name} init: {c.name}) applies stablehlo.{op} across dimensions = [{', '.join(map(str, dims))}] : ({x.type}, {c.type}) -> {v.type}")
        return v

    def _expand_back(self, r: Val, x: Val, dims) -> Val:
        dims = sorted(int(d) % max(x.ndim, 1) for d in dims)
        keep = [i for i in range(x.ndim) if i not in dims]
        return self.broadcast_in_dim(r, x.shape, keep)

    def reduce_sum(self, x: Val, dims) -> Val:
        init = 0.0 if x.dtype in FLOAT_TYPES else 0
        v = self._reduce(x, dims, "add", init)
        self._record([x], [v], lambda g: [self._expand_back(g, x, dims)])
        return v

    def reduce_max(self, x: Val, dims) -> Val:
        init = float("-inf") if x.dtype in FLOAT_TYPES else int(np.iinfo(_NP[x.dtype]).min)
        v = self._reduce(x, dims, "maximum", init)

        def vjp(g):
            m = self.compare(x, self._expand_back(v, x, dims), "EQ")
            mf = self.convert(m, x.dtype)
            cnt = self._expand_back(self.reduce_sum(mf, dims), x, dims)
            return [self.div(self.mul(self._expand_back(g, x, dims), mf), cnt)]
        self._record([x], [v], vjp)
        return v

    def reduce_min(self, x: Val, dims) -> Val:
        init = float("inf") if x.dtype in FLOAT_TYPES else int(np.iinfo(_NP[x.dtype]).max)
        return self._reduce(x, dims, "minimum", init)

    def mean(self, x: Val, dims) -> Val:
        n = 1
        for d in dims:
            n *= x.shape[d]
        return self.div(self.reduce_sum(x, dims), float(n))

    def argmax(self, x: Val, dim: int, index_dtype="i32") -> Val:
        """Two-operand reduce in the shape JAX prints for jnp.argmax."""
        idx = self.iota(x.shape, dim, index_dtype)
        ninf = self.constant(float("-inf"), x.dtype)
        zero = self.constant(0, index_dtype)
        shape = [d for i, d in enumerate(x.shape) if i != dim]
        name = self._fresh()
        rt_v, rt_i = ttype(shape, x.dtype), ttype(shape, index_dtype)
        sv, si = ttype((), x.dtype), ttype((), index_dtype)
        ind = "  " * self._blk.indent
        n0 = self._n
        a, bq, c, d = (f"%arg_r{n0}_{k}" for k in range(4))
        t = [f"%r{n0}_{k}" for k in range(9)]
        self._emit(f"{name}:2 = stablehlo.reduce({x.name} init: {ninf.name}), ({idx.name} init: {zero.name}) across dimensions = [{dim}] : ({x.type}, {idx.type}, {sv}, {si}) -> ({rt_v}, {rt_i})")
        self._emit(f" reducer({a}: {sv}, {c}: {sv}) ({bq}: {si}, {d}: {si})  {{")
        body = [
            f"{t[0]} = stablehlo.compare  GT, {a}, {c},  FLOAT : ({sv}, {sv}) -> tensor<i1>",
            f"{t[1]} = stablehlo.compare  NE, {a}, {a},  FLOAT : ({sv}, {sv}) -> tensor<i1>",
            f"{t[2]} = stablehlo.or {t[0]}, {t[1]} : tensor<i1>",
            f"{t[3]} = stablehlo.compare  EQ, {a}, {c},  FLOAT : ({sv}, {sv}) -> tensor<i1>",
            f"{t[4]} = stablehlo.compare  LT, {bq}, {d},  SIGNED : ({si}, {si}) -> tensor<i1>",
            f"{t[5]} = stablehlo.and {t[3]}, {t[4]} : tensor<i1>",
            f"{t[6]} = stablehlo.or {t[2]}, {t[5]} : tensor<i1>",
            f"{t[7]} = stablehlo.select {t[2]}, {a}, {c} : tensor<i1>, {sv}",
            f"{t[8]} = stablehlo.select {t[6]}, {bq}, {d} : tensor<i1>, {si}",
            f"stablehlo.return {t[7]}, {t[8]} : {sv}, {si}",
        ]
        for ln in body:
            self._blk.lines.append(ind + "  " + ln)
        self._emit("}")
        return Val(self, name + "#1", shape, index_dtype, self._blk)

    # ---------------------------------------------------------- contractions
    def dot_general(self, a: Val, b: Val, contract: Tuple[Sequence[int], Sequence[int]],
                    batch: Tuple[Sequence[int], Sequence[int]] = ((), ()), out_dtype: Optional[str] = None) -> Val:
        (ca, cb), (ba, bb) = contract, batch
        ca, cb, ba, bb = list(ca), list(cb), list(ba), list(bb)
        fa = [i for i in range(a.ndim) if i not in ca and i not in ba]
        fb = [i for i in range(b.ndim) if i not in cb and i not in bb]
        shape = [a.shape[i] for i in ba] + [a.shape[i] for i in fa] + [b.shape[i] for i in fb]
        od = out_dtype or a.dtype
        v = self._new(shape, od)
        f = lambda t: ", ".join(map(str, t))
        s = f"{v.name} = stablehlo.dot_general {a.name}, {b.name}, "
        if ba:
            s += f"batching_dims = [{f(ba)}] x [{f(bb)}], "
        s += f"contracting_dims = [{f(ca)}] x [{f(cb)}], precision = [DEFAULT, DEFAULT] : ({a.type}, {b.type}) -> {v.type}"
        self._emit(s)

        def vjp(g):
            nb, nfa, nfb = len(ba), len(fa), len(fb)
            # g dims: [batch..., fa..., fb...]
            g_b = list(range(nb))
            g_fa = list(range(nb, nb + nfa))
            g_fb = list(range(nb + nfa, nb + nfa + nfb))
            # dA = g . b over fb  -> dims [batch, fa, cb(order of cb)] then permute to a's layout
            da = db = None
            if self._want(a):
                da = self.dot_general(g, b, (g_fb, fb), (g_b, bb), out_dtype=a.dtype)
                cur = ba + fa + ca  # which a-dim each result dim represents
                perm = [cur.index(i) for i in range(a.ndim)]
                da = self.transpose(da, perm)
            if self._want(b):
                # dB = a . g over fa -> dims [batch, ca-ordered, fb]
                db = self.dot_general(a, g, (fa, g_fa), (ba, g_b), out_dtype=b.dtype)
                curb = bb + cb + fb
                permb = [curb.index(i) for i in range(b.ndim)]
                db = self.transpose(db, permb)
            return [da, db]
        if a.dtype in FLOAT_TYPES:
            self._record([a, b], [v], vjp)
        return v

    def matmul(self, a: Val, b: Val) -> Val:
        return self.dot_general(a, b, ([a.ndim - 1], [0]))

    def conv(self, lhs: Val, rhs: Val, *, strides=None, padding=None, lhs_dilation=None,
             rhs_dilation=None, dn=("b01f", "01io", "b01f"), feature_group_count=1, batch_group_count=1) -> Val:
        """General N-d convolution; dimension numbers as strings like 'b01f','01io','b01f' (spatial dims are digits)."""
        ls, rs, os_ = dn
        nsp = len(ls) - 2
        strides = tuple(strides) if strides is not None else (1,) * nsp
        padding = tuple(tuple(p) for p in padding) if padding is not None else ((0, 0),) * nsp
        lhs_dilation = tuple(lhs_dilation) if lhs_dilation is not None else (1,) * nsp
        rhs_dilation = tuple(rhs_dilation) if rhs_dilation is not None else (1,) * nsp
        lb, lf = ls.index("b"), ls.index("f")
        ri, ro = rs.index("i"), rs.index("o")
        ob, of = os_.index("b"), os_.index("f")
        lsp = [ls.index(str(d)) for d in range(nsp)]
        rsp = [rs.index(str(d)) for d in range(nsp)]
        osp = [os_.index(str(d)) for d in range(nsp)]
        if nsp == 2:
            l0, l1, r0, r1 = lsp[0], lsp[1], rsp[0], rsp[1]
        out_sp = []
        for d in range(nsp):
            isz, ksz = lhs.shape[lsp[d]], rhs.shape[rsp[d]]
            din = (isz - 1) * lhs_dilation[d] + 1 if isz > 0 else 0
            dk = (ksz - 1) * rhs_dilation[d] + 1 if ksz > 0 else 0
            padded = din + padding[d][0] + padding[d][1]
            out_sp.append(0 if padded < dk else (padded - dk) // strides[d] + 1)
        shape = [0] * (nsp + 2)
        shape[ob] = lhs.shape[lb] // batch_group_count
        shape[of] = rhs.shape[ro]
        for d in range(nsp):
            shape[osp[d]] = out_sp[d]
        v = self._new(shape, lhs.dtype)

        def fmt(s):
            return "[" + ", ".join(s) + "]"
        f2 = lambda t: "[" + ", ".join(str(int(q)) for q in t) + "]"
        pads = "[" + ", ".join(f"[{int(p[0])}, {int(p[1])}]" for p in padding) + "]"
        self._emit(
            f"{v.name} = stablehlo.convolution({lhs.name}, {rhs.name}) dim_numbers = {fmt(ls)}x{fmt(rs)}->{fmt(os_)}, "
            f"window = {{stride = {f2(strides)}, pad = {pads}, lhs_dilate = {f2(lhs_dilation)}, rhs_dilate = {f2(rhs_dilation)}}} "
            f"{{batch_group_count = {batch_group_count} : i64, feature_group_count = {feature_group_count} : i64, "
            f"precision_config = [#stablehlo<precision DEFAULT>, #stablehlo<precision DEFAULT>]}} : ({lhs.type}, {rhs.type}) -> {v.type}")

        def vjp(g):
            assert nsp == 2 and feature_group_count == 1 and batch_group_count == 1 and tuple(lhs_dilation) == (1, 1)
            in_sp = (lhs.shape[l0], lhs.shape[l1])
            k_sp = (rhs.shape[r0], rhs.shape[r1])
            # --- input gradient: conv(g dilated by stride, reversed kernel with i<->o swapped)
            pad_in = []
            for d in range(2):
                dk = (k_sp[d] - 1) * rhs_dilation[d] + 1
                lo = dk - 1 - padding[d][0]
                out_d = (out_sp[d] - 1) * strides[d] + 1
                hi = in_sp[d] + dk - 1 - out_d - lo
                pad_in.append((lo, hi))
            dx = dw = None
            if self._want(lhs):
                rev = self.reverse(rhs, sorted([r0, r1]))
                rs_t = rs.replace("i", "#").replace("o", "i").replace("#", "o")
                dx = self.conv(g, rev, strides=(1, 1), padding=pad_in, lhs_dilation=strides, rhs_dilation=rhs_dilation,
                               dn=(os_, rs_t, ls))
            if not self._want(rhs):
                return [dx, None]
            # --- filter gradient: conv(lhs with b<->f, g with b->i, f->o), window stride = rhs_dilation,
            #     rhs dilation = stride; output dims named so the result lands in rhs layout
            pad_w = []
            for d in range(2):
                dk = (k_sp[d] - 1) * rhs_dilation[d] + 1
                out_d = (out_sp[d] - 1) * strides[d] + 1
                hi = out_d + dk - 1 - in_sp[d] - padding[d][0]
                pad_w.append((padding[d][0], hi))
            ls_t = ls.replace("b", "#").replace("f", "b").replace("#", "f")
            g_as_rhs = os_.replace("b", "i").replace("f", "o")
            out_as = rs.replace("i", "b").replace("o", "f")
            dw = self.conv(lhs, g, strides=rhs_dilation, padding=pad_w, lhs_dilation=(1, 1), rhs_dilation=strides,
                           dn=(ls_t, g_as_rhs, out_as))
            return [dx, dw]
        self._record([lhs, rhs], [v], vjp)
        return v

    # -------------------------------------------------------- gather / scatter
    def gather(self, operand: Val, indices: Val, *, offset_dims, collapsed_slice_dims, start_index_map,
               index_vector_dim, slice_sizes, operand_batching_dims=(), start_indices_batching_dims=(),
               indices_are_sorted=False) -> Val:
        batch_shape = [d for i, d in enumerate(indices.shape) if i != index_vector_dim]
        off_sizes = [s for i, s in enumerate(slice_sizes) if i not in collapsed_slice_dims and i not in operand_batching_dims]
        rank = len(batch_shape) + len(off_sizes)
        shape, bi, oi = [], 0, 0
        for d in range(rank):
            if d in offset_dims:
                shape.append(off_sizes[oi]); oi += 1
            else:
                shape.append(batch_shape[bi]); bi += 1
        v = self._new(shape, operand.dtype)
        f = lambda t: ", ".join(map(str, t))
        dn = f"offset_dims = [{f(offset_dims)}], collapsed_slice_dims = [{f(collapsed_slice_dims)}], "
        if operand_batching_dims:
            dn += f"operand_batching_dims = [{f(operand_batching_dims)}], start_indices_batching_dims = [{f(start_indices_batching_dims)}], "
        dn += f"start_index_map = [{f(start_index_map)}], index_vector_dim = {index_vector_dim}"
        self._emit(
            f'{v.name} = "stablehlo.gather"({operand.name}, {indices.name}) <{{dimension_numbers = #stablehlo.gather<{dn}>, '
            f"indices_are_sorted = {'true' if indices_are_sorted else 'false'}, slice_sizes = array<i64: {f(slice_sizes)}>}}> : "
            f"({operand.type}, {indices.type}) -> {v.type}")

        def vjp(g):
            z = self.zeros(operand.shape, operand.dtype)
            return [self.scatter(z, indices, g, update_window_dims=offset_dims, inserted_window_dims=collapsed_slice_dims,
                                 scatter_dims_to_operand_dims=start_index_map, index_vector_dim=index_vector_dim,
                                 input_batching_dims=operand_batching_dims,
                                 scatter_indices_batching_dims=start_indices_batching_dims, body="add",
                                 indices_are_sorted=indices_are_sorted), None]
        if operand.dtype in FLOAT_TYPES:
            self._record([operand, indices], [v], vjp)
        return v

    def scatter(self, operand: Val, indices: Val, updates: Val, *, update_window_dims, inserted_window_dims,
                scatter_dims_to_operand_dims, index_vector_dim, body="add", input_batching_dims=(),
                scatter_indices_batching_dims=(), indices_are_sorted=False, unique_indices=False) -> Val:
        v = self._new(operand.shape, operand.dtype)
        f = lambda t: ", ".join(map(str, t))
        dn = f"update_window_dims = [{f(update_window_dims)}], inserted_window_dims = [{f(inserted_window_dims)}], "
        if input_batching_dims:
            dn += f"input_batching_dims = [{f(input_batching_dims)}], scatter_indices_batching_dims = [{f(scatter_indices_batching_dims)}], "
        dn += f"scatter_dims_to_operand_dims = [{f(scatter_dims_to_operand_dims)}], index_vector_dim = {index_vector_dim}"
        st = ttype((), operand.dtype)
        n0 = self._n
        a0, a1, r = f"%sarg{n0}_0", f"%sarg{n0}_1", f"%sres{n0}"
        ind = "  " * self._blk.indent
        self._emit(
            f'{v.name} = "stablehlo.scatter"({operand.name}, {indices.name}, {updates.name}) <{{indices_are_sorted = '
            f"{'true' if indices_are_sorted else 'false'}, scatter_dimension_numbers = #stablehlo.scatter<{dn}>, "
            f"unique_indices = {'true' if unique_indices else 'false'}}}> ({{")
        self._blk.lines.append(f"{ind}^bb0({a0}: {st}, {a1}: {st}):")
        if body == "set":
            self._blk.lines.append(f"{ind}  stablehlo.return {a1} : {st}")
        else:
            opn = {"add": "add", "mul": "multiply", "min": "minimum", "max": "maximum", "sub": "subtract"}[body]
            self._blk.lines.append(f"{ind}  {r} = stablehlo.{opn} {a0}, {a1} : {st}")
            self._blk.lines.append(f"{ind}  stablehlo.return {r} : {st}")
        self._emit(f"}}) : ({operand.type}, {indices.type}, {updates.type}) -> {v.type}")
        return v

    def _window_attr_text(self, window, strides, padding, base_dilation=None, window_dilation=None):
        rank = len(window)
        f = lambda t: ", ".join(map(str, t))
        arr = lambda t: f"array<i64: {f(t)}>" if len(t) else "array<i64>"
        pad = [[int(a), int(b)] for a, b in padding]
        attrs = []
        if base_dilation is not None:
            attrs.append(f"base_dilations = {arr(base_dilation)}")
        if any(a or b for a, b in pad):
            rows = ", ".join("[" + f(p) + "]" for p in pad)
            attrs.append(f"padding = dense<[{rows}]> : tensor<{rank}x2xi64>")
        if window_dilation is not None:
            attrs.append(f"window_dilations = {arr(window_dilation)}")
        attrs.append(f"window_dimensions = {arr(window)}")
        attrs.append(f"window_strides = {arr(strides)}")
        return ", ".join(attrs)

    def reduce_window(self, x: Val, init, kind: str, window, strides=None, padding=None, base_dilation=None, window_dilation=None) -> Val:
        """`lax.reduce_window` with an add / max / min / mul reducer, printed in the generic form JAX uses."""
        rank = len(x.shape)
        strides = list(strides) if strides is not None else [1] * rank
        padding = [tuple(p) for p in padding] if padding is not None else [(0, 0)] * rank
        bd = list(base_dilation) if base_dilation is not None else [1] * rank
        wdl = list(window_dilation) if window_dilation is not None else [1] * rank
        out = []
        for d in range(rank):
            dil = (x.shape[d] - 1) * bd[d] + 1 if x.shape[d] > 0 else 0
            span = (window[d] - 1) * wdl[d] + 1
            out.append(max(0, (dil + padding[d][0] + padding[d][1] - span) // strides[d] + 1))
        iv = init if isinstance(init, Val) else self.constant(init, x.dtype)
        v = self._new(out, x.dtype)
        st = ttype((), x.dtype)
        n0 = self._n
        a0, a1, r = f"%warg{n0}_0", f"%warg{n0}_1", f"%wres{n0}"
        ind = "  " * self._blk.indent
        opn = {"add": "add", "max": "maximum", "min": "minimum", "mul": "multiply"}[kind]
        self._emit(f'{v.name} = "stablehlo.reduce_window"({x.name}, {iv.name}) <{{{self._window_attr_text(window, strides, padding, base_dilation, window_dilation)}}}> ({{')
        self._blk.lines.append(f"{ind}^bb0({a0}: {st}, {a1}: {st}):")
        self._blk.lines.append(f"{ind}  {r} = stablehlo.{opn} {a0}, {a1} : {st}")
        self._blk.lines.append(f"{ind}  stablehlo.return {r} : {st}")
        self._emit(f"}}) : ({x.type}, {st}) -> {v.type}")
        return v

    def select_and_scatter(self, operand: Val, source: Val, init, window, strides, padding=None, direction="GE") -> Val:
        """The op JAX emits for the gradient of max (GE) / min (LE) pooling."""
        rank = len(operand.shape)
        padding = [tuple(p) for p in padding] if padding is not None else [(0, 0)] * rank
        iv = init if isinstance(init, Val) else self.constant(init, operand.dtype)
        v = self._new(operand.shape, operand.dtype)
        st = ttype((), operand.dtype)
        n0 = self._n
        ind = "  " * self._blk.indent
        self._emit(f'{v.name} = "stablehlo.select_and_scatter"({operand.name}, {source.name}, {iv.name}) <{{{self._window_attr_text(window, strides, padding)}}}> ({{')
        self._blk.lines.append(f"{ind}^bb0(%ssa{n0}: {st}, %ssb{n0}: {st}):")
        self._blk.lines.append(f"{ind}  %ssc{n0} = stablehlo.compare  {direction}, %ssa{n0}, %ssb{n0},  FLOAT : ({st}, {st}) -> tensor<i1>")
        self._blk.lines.append(f"{ind}  stablehlo.return %ssc{n0} : tensor<i1>")
        self._blk.lines.append(f"{ind}}}, {{")
        self._blk.lines.append(f"{ind}^bb0(%ssd{n0}: {st}, %sse{n0}: {st}):")
        self._blk.lines.append(f"{ind}  %ssf{n0} = stablehlo.add %ssd{n0}, %sse{n0} : {st}")
        self._blk.lines.append(f"{ind}  stablehlo.return %ssf{n0} : {st}")
        self._emit(f"}}) : ({operand.type}, {source.type}, {st}) -> {v.type}")
        return v

    def sort(self, operands: Sequence[Val], dimension: int = -1, num_keys: int = 1, descending: bool = False, is_stable: bool = True,
             comparator: Optional[Callable] = None) -> List[Val]:
        """`lax.sort` as JAX lowers it: a lexicographic comparator over the first `num_keys` operands (floats in
        total order, so NaNs sort last), or a caller-built `comparator(b, lhs, rhs) -> i1 Val` over scalar block arguments."""
        operands = list(operands)
        rank = operands[0].ndim
        dimension = dimension % rank if rank else 0
        name = self._fresh()
        n0 = self._n
        ind = self._blk.indent
        self._emit(f'{name}:{len(operands)} = "stablehlo.sort"({", ".join(o.name for o in operands)}) <{{dimension = {dimension} : i64, is_stable = {"true" if is_stable else "false"}}}> ({{')
        blk = _Block(ind + 1)
        self._blocks.append(blk)
        lhs = [Val(self, f"%sl{n0}_{k}", (), o.dtype, blk) for k, o in enumerate(operands)]
        rhs = [Val(self, f"%sr{n0}_{k}", (), o.dtype, blk) for k, o in enumerate(operands)]
        hdr = ", ".join(f"{a.name}: {a.type}, {b_.name}: {b_.type}" for a, b_ in zip(lhs, rhs))
        if comparator is not None:
            res = comparator(self, lhs, rhs)
        else:
            res = None
            for k in reversed(range(num_keys)):
                a, c = lhs[k], rhs[k]
                kind = "TOTALORDER" if a.dtype in FLOAT_TYPES else None
                first = self.compare(a, c, "GT" if descending else "LT", kind)
                if res is None:
                    res = first
                else:
                    res = self.or_(first, self.and_(self.compare(a, c, "EQ", kind), res))
        self._emit(f"stablehlo.return {res.name} : {res.type}")
        self._blocks.pop()
        self._blk.lines.append("  " * (ind + 1) + f"^bb0({hdr}):")
        self._blk.lines.extend(blk.lines)
        ts = ", ".join(o.type for o in operands)
        self._emit(f"}}) : ({ts}) -> ({ts})")
        return [Val(self, f"{name}#{k}", o.shape, o.dtype, self._blk) for k, o in enumerate(operands)]

    def top_k(self, x: Val, k: int):
        """`lax.top_k`: (values, i32 indices) of the k largest entries along the last dim."""
        name = self._fresh()
        shape = tuple(x.shape[:-1]) + (int(k),)
        self._emit(f"{name}:2 = chlo.top_k({x.name}, k = {int(k)}) : {x.type} -> ({ttype(shape, x.dtype)}, {ttype(shape, 'i32')})")
        return Val(self, f"{name}#0", shape, x.dtype, self._blk), Val(self, f"{name}#1", shape, "i32", self._blk)

    def custom_call(self, target: str, operands: Sequence[Val], result_types: Sequence[Tuple[Sequence[int], str]], backend_config: str = ""):
        """`mlir.custom_call(call_target_name=..., backend_config=...)` as jax prints it: the fused-op primitives of the
        reference's Python layer lower to this (src/jax_plugins/mps/ops.py:81-88 and its siblings).  Returns one Val
        per result."""
        name = self._fresh()
        types = [ttype(tuple(int(d) for d in shape), dt) for shape, dt in result_types]
        quoted = backend_config.replace("\\", "\\\\").replace('"', '\\22')        # MLIR prints a quote inside a string as \22
        lhs = name if len(types) == 1 else f"{name}:{len(types)}"
        res = types[0] if len(types) == 1 else "(" + ", ".join(types) + ")"
        self._emit(f"{lhs} = stablehlo.custom_call @{target}({', '.join(o.name for o in operands)}) "
                   f"{{api_version = 2 : i32, backend_config = \"{quoted}\"}} : ({', '.join(o.type for o in operands)}) -> {res}")
        if len(types) == 1:
            return [Val(self, name, tuple(result_types[0][0]), result_types[0][1], self._blk)]
        return [Val(self, f"{name}#{k}", tuple(shape), dt, self._blk) for k, (shape, dt) in enumerate(result_types)]

    def rng_bit_generator(self, state: Val, shape, dtype="ui32", algorithm="DEFAULT"):
        """`jax.random.bits` under the rbg / unsafe_rbg PRNG implementations: (new state, bits)."""
        name = self._fresh()
        shape = tuple(int(x) for x in shape)
        self._emit(f"{name}:2 = stablehlo.rng_bit_generator {state.name}, algorithm = {algorithm} : ({state.type}) -> ({state.type}, {ttype(shape, dtype)})")
        return Val(self, f"{name}#0", state.shape, state.dtype, self._blk), Val(self, f"{name}#1", shape, dtype, self._blk)

    def take_rows(self, table: Val, idx: Val) -> Val:
        """`jnp.take(table, idx, axis=0)` in the default (fill) mode: negative
        indices wrap, then rows outside [0, n) read as NaN (the mask JAX adds
        around the clamping gather)."""
        n = table.shape[0]
        lt = self.compare(idx, 0, "LT")
        wrapped = self.select(lt, self.add(idx, n), idx)
        iv = self.reshape(wrapped, list(idx.shape) + [1])
        g = self.gather(table, iv, offset_dims=[idx.ndim], collapsed_slice_dims=[0], start_index_map=[0],
                        index_vector_dim=idx.ndim, slice_sizes=[1] + list(table.shape[1:]))
        ok = self.and_(self.compare(wrapped, 0, "GE"), self.compare(wrapped, n - 1, "LE"))
        okb = self.broadcast_in_dim(ok, g.shape, list(range(idx.ndim)))
        if table.dtype in FLOAT_TYPES:
            return self.select(okb, g, self.full_like(g, float("nan")))
        return g

    # ------------------------------------------------------------ control flow
    def while_loop(self, init: Sequence[Val], cond_fn: Callable, body_fn: Callable) -> List[Val]:
        name = self._fresh()
        n0 = self._n
        iter_names = [f"%iterArg_{n0}_{k}" for k in range(len(init))]
        hdr = ", ".join(f"{n} = {v.name}" for n, v in zip(iter_names, init))
        self._emit(f"{name}:{len(init)} = stablehlo.while({hdr}) : {', '.join(v.type for v in init)}")
        ind = self._blk.indent
        results = []
        for part, fn in (("cond", cond_fn), ("do", body_fn)):
            blk = _Block(ind + 1)
            self._blocks.append(blk)
            args = [Val(self, n, v.shape, v.dtype, blk) for n, v in zip(iter_names, init)]
            out = fn(*args)
            if isinstance(out, Val):
                out = [out]
            out = list(out)
            self._emit(f"stablehlo.return {', '.join(o.name for o in out)} : {', '.join(o.type for o in out)}")
            self._blocks.pop()
            self._emit((" cond {" if part == "cond" else " } do {"))
            self._blk.lines.extend(blk.lines)
        self._emit(" }")
        for k, v in enumerate(init):
            results.append(Val(self, f"{name}#{k}", v.shape, v.dtype, self._blk))
        return results

    def case(self, index: Val, branches: Sequence[Callable], out_types: Sequence[Tuple[Sequence[int], str]]) -> List[Val]:
        name = self._fresh()
        self._emit(f'{name}:{len(out_types)} = "stablehlo.case"({index.name}) ({{')
        ind = self._blk.indent
        for bi, fn in enumerate(branches):
            blk = _Block(ind + 1)
            self._blocks.append(blk)
            out = fn()
            if isinstance(out, Val):
                out = [out]
            self._emit(f"stablehlo.return {', '.join(o.name for o in out)} : {', '.join(o.type for o in out)}")
            self._blocks.pop()
            self._blk.lines.extend(blk.lines)
            if bi + 1 < len(branches):
                self._emit("}, {")
        ts = ", ".join(ttype(s, d) for s, d in out_types)
        self._emit(f"}}) : ({index.type}) -> ({ts})")
        return [Val(self, f"{name}#{k}", s, d, self._blk) for k, (s, d) in enumerate(out_types)]

    # ---------------------------------------------------------------- autodiff
    def grad(self, y: Val, xs: Sequence[Val], seed: Optional[Val] = None) -> List[Val]:
        """Cotangents of scalar (or seeded) `y` with respect to `xs`, within the current block."""
        ct = {y.name: seed if seed is not None else self.constant(1.0, y.dtype, y.shape)}
        tape = list(self._blk.tape)
        needed, fwd = self._reachable(tape, xs, y)
        saved, self._wanted = self._wanted, fwd
        try:
            ct = self._backprop(tape, needed, ct)
        finally:
            self._wanted = saved
        out = []
        for x in xs:
            g = ct.get(x.name)
            out.append(g if g is not None else self.zeros(x.shape, x.dtype))
        return out

    def _backprop(self, tape, needed, ct):
        for node in reversed(tape):
            if id(node) not in needed:
                continue
            gs = [ct.get(o.name) for o in node.outs]
            if all(g is None for g in gs):
                continue
            g = gs[0]
            res = node.vjp(g)
            for inp, gi in zip(node.ins, res):
                if gi is None or inp.dtype not in FLOAT_TYPES:
                    continue
                if inp.name in ct:
                    ct[inp.name] = self.add(ct[inp.name], gi)
                else:
                    ct[inp.name] = gi
        return ct

    @staticmethod
    def _reachable(tape, xs, y):
        """Nodes that lie on a path from some x to y."""
        fwd = {x.name for x in xs}
        on_fwd = set()
        for node in tape:
            if any(i.name in fwd for i in node.ins):
                on_fwd.add(id(node))
                for o in node.outs:
                    fwd.add(o.name)
        bwd = {y.name}
        keep = set()
        for node in reversed(tape):
            if any(o.name in bwd for o in node.outs) and id(node) in on_fwd:
                keep.add(id(node))
                for i in node.ins:
                    bwd.add(i.name)
        return keep, fwd

    # -------------------------------------------------------------------- text
    def text(self) -> str:
        args = ", ".join(f"{a.name}: {a.type}" + (f" {{tf.aliasing_output = {self._arg_alias[a.name]} : i32}}" if a.name in self._arg_alias else "")
                         for a in self._main_args)
        if len(self._results) == 1:
            rts = f"({self._results[0].type} {{jax.result_info = \"result\"}})"
        else:
            rts = "(" + ", ".join(f"{r.type} {{jax.result_info = \"result[{i}]\"}}" for i, r in enumerate(self._results)) + ")"
        out = [f"module @{self.module_name} attributes {{mhlo.num_partitions = 1 : i32, mhlo.num_replicas = 1 : i32}} {{",
               f"  func.func public @main({args}) -> {rts} {{"]
        out.extend(self._main_block.lines)
        out.append(f"    return {', '.join(r.name for r in self._results)} : {', '.join(r.type for r in self._results)}")
        out.append("  }")
        out.append("}")
        return "\n".join(out) + "\n"

    @property
    def arg_types(self):
        return [(a.shape, a.dtype) for a in self._main_args]

    @property
    def result_types(self):
        return [(r.shape, r.dtype) for r in self._results]


# ----------------------------------------------------------------------------
# nn helpers written the way jax.nn / flax write them
# ----------------------------------------------------------------------------
def relu(b: Builder, x: Val) -> Val:
    return b.maximum(x, 0.0)


def log_softmax(b: Builder, x: Val, axis: int = -1) -> Val:
    axis = axis % x.ndim
    m = b.stop_gradient(b.reduce_max(x, [axis]))
    sh = b.sub(x, b._expand_back(m, x, [axis]))
    lse = b.log(b.reduce_sum(b.exp(sh), [axis]))
    return b.sub(sh, b._expand_back(lse, x, [axis]))


def softmax(b: Builder, x: Val, axis: int = -1) -> Val:
    axis = axis % x.ndim
    m = b.stop_gradient(b.reduce_max(x, [axis]))
    e = b.exp(b.sub(x, b._expand_back(m, x, [axis])))
    return b.div(e, b._expand_back(b.reduce_sum(e, [axis]), x, [axis]))


def one_hot(b: Builder, labels: Val, n: int, dtype="f32") -> Val:
    shape = list(labels.shape) + [n]
    io = b.iota(shape, len(shape) - 1, labels.dtype)
    lb = b.broadcast_in_dim(labels, shape, list(range(labels.ndim)))
    return b.convert(b.compare(lb, io, "EQ"), dtype)


def softmax_cross_entropy_int(b: Builder, logits: Val, labels: Val) -> Val:
    lp = log_softmax(b, logits)
    oh = one_hot(b, labels, logits.shape[-1], logits.dtype)
    per = b.neg(b.reduce_sum(b.mul(oh, lp), [logits.ndim - 1]))
    return b.mean(per, list(range(per.ndim)))


def gelu_tanh(b: Builder, x: Val) -> Val:
    c = math.sqrt(2.0 / math.pi)
    x3 = b.mul(b.mul(x, x), x)
    inner = b.mul(b.add(x, b.mul(x3, 0.044715)), c)
    return b.mul(b.mul(x, 0.5), b.add(b.tanh(inner), 1.0))


def layer_norm(b: Builder, x: Val, scale: Val, bias: Val, eps: float) -> Val:
    """flax.nnx.LayerNorm: statistics in f32 as E[x], E[x^2]; var = max(0, E[x^2]-E[x]^2)."""
    ax = x.ndim - 1
    xf = b.convert(x, "f32")
    mean = b.mean(xf, [ax])
    mean2 = b.mean(b.mul(xf, xf), [ax])
    var = b.maximum(b.sub(mean2, b.mul(mean, mean)), 0.0)
    y = b.sub(xf, b._expand_back(mean, xf, [ax]))
    mul = b.rsqrt(b.add(var, eps))
    y = b.mul(y, b._expand_back(mul, xf, [ax]))
    y = b.convert(y, x.dtype)
    y = b.mul(y, b.broadcast_in_dim(scale, x.shape, [ax]))
    return b.add(y, b.broadcast_in_dim(bias, x.shape, [ax]))
