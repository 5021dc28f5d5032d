"""CPU oracle: a numpy interpreter for the StableHLO subset on the hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product path may import this file; it
is the checker that the HIP path is compared with (tests/, the smoke entry and
the cpu_baseline leg of the benchmark).

It restates, op by op, what the reference's handlers compute
(`/root/reference/src/pjrt_plugin/ops/*.cc`); the arithmetic itself lives in the
third-party MLX library (pinned commit a025496c8f6da9d599e2010019ea5ee328c2d119,
not vendored in the reference), so every function here follows the StableHLO
specification for the op and the edge-case rules spelled out at the reference's
call sites (cited per function).  Contractions and float reductions accumulate in
float64 by default so that the oracle is a tighter truth than any f32 ordering;
`accum="f32"` switches them to float32 BLAS for the timed CPU baseline.

Pins (tests/test_oracle_*.py): literal gather/scatter/control-flow cases of the
reference's own tests, torch-CPU conv2d / conv_transpose2d and brute-force loops
for convolution, numpy einsum for dot_general, closed forms for while/case,
IEEE special cases for shifts/remainder/sign/round.  bf16 results are pinned only
by the rounding rule (round-to-nearest-even of the f32 result) — the reference
holds no bf16 expectation ("parity unpinned" by the reference for bf16).  Also
parity unpinned: which zero maximum / minimum return for two zeros of different
sign (MLX's published element rule restated; no test of the reference holds the case).
"""
from __future__ import annotations

import math
import re
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

# ----------------------------------------------------------------------------
# types
# ----------------------------------------------------------------------------
_NP = {
    "f32": np.float32, "f64": np.float64, "f16": np.float16, "bf16": np.float32,
    "i1": np.bool_, "i8": np.int8, "i16": np.int16, "i32": np.int32, "i64": np.int64,
    "ui8": np.uint8, "ui16": np.uint16, "ui32": np.uint32, "ui64": np.uint64,
}
FLOATS = ("f32", "f64", "f16", "bf16")


def round_bf16(a: np.ndarray) -> np.ndarray:
    """float32 values rounded to the nearest bfloat16 (ties to even), kept as float32."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    r = (u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))) & np.uint32(0xFFFF0000)
    r = np.where(nan, u | np.uint32(0x00400000), r).astype(np.uint32)
    return r.view(np.float32).reshape(a.shape)


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    return (round_bf16(a).view(np.uint32) >> np.uint32(16)).astype(np.uint16)


class TType:
    __slots__ = ("shape", "dtype")

    def __init__(self, shape, dtype):
        self.shape = tuple(shape)
        self.dtype = dtype

    def __repr__(self):
        return f"tensor<{'x'.join(map(str, self.shape + (self.dtype,)))}>"


class Op:
    __slots__ = ("name", "results", "operands", "attrs", "regions", "in_types", "out_types")

    def __init__(self):
        self.name = ""
        self.results: List[str] = []
        self.operands: List[str] = []
        self.attrs: Dict[str, object] = {}
        self.regions: List["Region"] = []
        self.in_types: List[TType] = []
        self.out_types: List[TType] = []


class Region:
    __slots__ = ("args", "arg_types", "ops")

    def __init__(self):
        self.args: List[str] = []
        self.arg_types: List[TType] = []
        self.ops: List[Op] = []


class Func:
    def __init__(self, name):
        self.name = name
        self.body = Region()
        self.result_types: List[TType] = []


# ----------------------------------------------------------------------------
# parser (recursive descent over characters; independent of the C++ front end)
# ----------------------------------------------------------------------------
class _P:
    def __init__(self, text: str):
        self.s = text
        self.i = 0
        self.n = len(text)

    def err(self, msg):
        ln = self.s.count("\n", 0, self.i) + 1
        raise SyntaxError(f"stablehlo text line {ln}: {msg}: ...{self.s[self.i:self.i + 60]!r}")

    def ws(self):
        s, n = self.s, self.n
        while self.i < n:
            c = s[self.i]
            if c in " \t\r\n":
                self.i += 1
            elif c == "/" and s.startswith("//", self.i):
                j = s.find("\n", self.i)
                self.i = n if j < 0 else j
            else:
                break

    def skip_loc(self):
        """`loc(...)` after an op, an argument or a signature is debug information."""
        save = self.i
        self.ws()
        if self.s.startswith("loc(", self.i):
            self.i += 3
            self.raw_until_balanced_paren()
        else:
            self.i = save

    def raw_until_balanced_paren(self):
        depth = 0
        while self.i < self.n:
            c = self.s[self.i]
            if c == '"':
                self.string()
                continue
            if c == "(":
                depth += 1
            elif c == ")":
                depth -= 1
                if depth == 0:
                    self.i += 1
                    return
            self.i += 1
        self.err("unbalanced parentheses")

    def skip_alias_lines(self):
        """`#loc3 = loc(...)` definitions outside functions."""
        while True:
            self.ws()
            if self.i >= self.n or self.s[self.i] != "#":
                return
            depth = 0
            while self.i < self.n:
                c = self.s[self.i]
                if c == '"':
                    self.string()
                    continue
                if c in "([{<":
                    depth += 1
                elif c in ")]}>":
                    depth -= 1
                elif c == "\n" and depth <= 0:
                    break
                self.i += 1

    def symbol(self) -> str:
        self.ws()
        if self.i < self.n and self.s[self.i] == '"':
            return self.string()
        return self.ident()

    def peek(self, lit: str) -> bool:
        self.ws()
        return self.s.startswith(lit, self.i)

    def eat(self, lit: str) -> bool:
        self.ws()
        if self.s.startswith(lit, self.i):
            self.i += len(lit)
            return True
        return False

    def expect(self, lit: str):
        if not self.eat(lit):
            self.err(f"expected {lit!r}")

    _ident = re.compile(r"[A-Za-z_][A-Za-z0-9_.$]*")
    _ssa = re.compile(r"%[A-Za-z0-9_.$]+(#[0-9]+)?")
    _num = re.compile(r"[-+]?(0x[0-9A-Fa-f]+|[0-9]+(\.[0-9]*)?([eE][-+]?[0-9]+)?|inf|nan)")

    def ident(self) -> str:
        self.ws()
        m = self._ident.match(self.s, self.i)
        if not m:
            self.err("identifier expected")
        self.i = m.end()
        return m.group(0)

    def try_ident(self) -> Optional[str]:
        self.ws()
        m = self._ident.match(self.s, self.i)
        if not m:
            return None
        self.i = m.end()
        return m.group(0)

    def ssa(self) -> str:
        self.ws()
        m = self._ssa.match(self.s, self.i)
        if not m:
            self.err("SSA value expected")
        self.i = m.end()
        return m.group(0)

    def string(self) -> str:
        self.ws()
        if self.s[self.i] != '"':
            self.err("string expected")
        j = self.i + 1
        out = []
        while self.s[j] != '"':
            if self.s[j] == "\\":
                pair = self.s[j + 1:j + 3]
                if len(pair) == 2 and all(ch in "0123456789abcdefABCDEF" for ch in pair):    # MLIR prints a quote as \22
                    out.append(chr(int(pair, 16)))
                    j += 3
                    continue
                out.append({"n": "\n", "t": "\t"}.get(self.s[j + 1], self.s[j + 1]))
                j += 2
            else:
                out.append(self.s[j])
                j += 1
        self.i = j + 1
        return "".join(out)

    def integer(self) -> int:
        self.ws()
        m = re.compile(r"[-+]?[0-9]+").match(self.s, self.i)
        if not m:
            self.err("integer expected")
        self.i = m.end()
        return int(m.group(0))

    def int_list(self, open_="[", close="]") -> List[int]:
        self.expect(open_)
        out = []
        if self.eat(close):
            return out
        while True:
            out.append(self.integer())
            if self.eat(close):
                return out
            self.expect(",")

    def type(self) -> TType:
        self.ws()
        if self.eat("tensor<"):
            j = self.s.index(">", self.i)
            body = self.s[self.i:j]
            self.i = j + 1
            parts = body.split("x")
            dims = []
            k = 0
            while k < len(parts) - 1 and re.fullmatch(r"[0-9]+", parts[k]):
                dims.append(int(parts[k]))
                k += 1
            dt = "x".join(parts[k:]).strip()
            if "," in dt:
                dt = dt.split(",")[0].strip()
            return TType(dims, dt)
        if self.eat("!stablehlo.token"):
            return TType((), "token")
        t = self.ident()  # bare scalar element type (i32, f32 ...) in attributes
        return TType((), t)

    def type_list_paren(self) -> List[TType]:
        out = []
        self.expect("(")
        if self.eat(")"):
            return out
        while True:
            out.append(self.type())
            self.skip_attr_dict()
            if self.eat(")"):
                return out
            self.expect(",")

    def skip_attr_dict(self):
        if self.peek("{"):
            self.attr_dict()

    # ---- attributes
    def attr_value(self):
        self.ws()
        s = self.s
        c = s[self.i]
        if c == '"':
            v = self.string()
            if self.eat(":"):
                self.type()
            return v
        if c == "[":
            self.i += 1
            out = []
            if self.eat("]"):
                return out
            while True:
                out.append(self.attr_value())
                if self.eat("]"):
                    return out
                self.expect(",")
        if c == "{":
            return self.attr_dict()
        if c == "#":
            return self.hash_attr()
        if c == "@":
            self.i += 1
            return "@" + self.symbol()
        if s.startswith("dense<", self.i):
            return self.dense()
        if s.startswith("array<", self.i):
            self.i += 6
            self.ident()
            out = []
            if self.eat(">"):
                return out
            self.expect(":")
            while True:
                out.append(self.integer() if not (self.peek("true") or self.peek("false")) else (self.ident() == "true"))
                if self.eat(">"):
                    return out
                self.expect(",")
        if s.startswith("true", self.i):
            self.i += 4
            return True
        if s.startswith("false", self.i):
            self.i += 5
            return False
        if s.startswith("unit", self.i):
            self.i += 4
            return True
        m = self._num.match(s, self.i)
        if m:
            self.i = m.end()
            tok = m.group(0)
            isf = any(ch in tok for ch in ".eE") and not tok.lower().startswith(("0x", "-0x")) or tok in ("inf", "nan")
            v = float(tok) if isf else int(tok, 0)
            self._eat_scalar_type_suffix()
            return v
        if s.startswith("tensor<", self.i):
            return self.type()
        idn = self.try_ident()
        if idn is not None:
            return idn
        self.err("attribute value expected")

    def _eat_scalar_type_suffix(self):
        """`1 : i64` is a typed literal; `dim = 0 : (tensor<...>)` is not (the colon starts the op's type)."""
        save = self.i
        if self.eat(":"):
            self.ws()
            m = re.compile(r"(i|ui|si|f|bf)[0-9]+\b|index\b").match(self.s, self.i)
            if m:
                self.i = m.end()
            else:
                self.i = save

    def hash_attr(self):
        """#stablehlo.gather<...>, #stablehlo<precision DEFAULT>, #stablehlo.conv<...> ..."""
        self.expect("#")
        name = self.ident()
        if not self.eat("<"):
            return ("#" + name, None)
        if name == "stablehlo":
            kind = self.ident()
            val = self.ident() if not self.peek(">") else None
            self.expect(">")
            return ("#" + kind, val)
        d = {}
        if name == "stablehlo.conv":
            raw = self.raw_until_balanced(">")
            return ("#stablehlo.conv", raw)
        while not self.eat(">"):
            k = self.ident()
            self.expect("=")
            d[k] = self.attr_value()
            self.eat(",")
        return ("#" + name, d)

    def raw_until_balanced(self, close):
        depth = 0
        j = self.i
        while True:
            c = self.s[j]
            if c in "<[({":
                depth += 1
            elif c == ">" and j > 0 and self.s[j - 1] == "-":
                pass                      # the arrow of a convolution's dimension numbers
            elif c in ">])}":
                if depth == 0 and c == close:
                    break
                depth -= 1
            j += 1
        raw = self.s[self.i:j]
        self.i = j + 1
        return raw

    def attr_dict(self) -> Dict[str, object]:
        self.expect("{")
        d = {}
        if self.eat("}"):
            return d
        while True:
            self.ws()
            k = self.string() if self.s[self.i] == '"' else self.ident()
            if self.eat("="):
                d[k] = self.attr_value()
            else:
                d[k] = True
            if self.eat("}"):
                return d
            self.expect(",")

    def dense(self):
        """dense<...> : tensor<...> -> numpy array (bf16 kept as rounded float32)."""
        self.expect("dense<")
        self.ws()
        start = self.i
        if self.s[self.i] == '"':
            payload = ("hex", self.string())
            self.expect(">")
        else:
            raw = self.raw_until_balanced(">")
            payload = ("lit", raw)
        self.expect(":")
        t = self.type()
        return _dense_to_numpy(payload, t)

    # ---- module structure
    def module(self) -> Dict[str, Func]:
        funcs = {}
        self.skip_alias_lines()
        wrapped = False
        if self.eat("module"):
            wrapped = True
            if self.eat("@"):
                self.ident()
            if self.eat("attributes"):
                self.module_attributes = self.attr_dict()
            self.expect("{")
        self.skip_alias_lines()
        while True:
            self.ws()
            if self.i >= self.n:
                break
            if wrapped and self.eat("}"):
                self.skip_loc()
                break
            self.skip_alias_lines()
            if self.i >= self.n:
                break
            f = self.func()
            funcs[f.name] = f
        return funcs

    def func(self) -> Func:
        self.expect("func.func")
        self.ws()
        if self.peek("public") or self.peek("private"):
            self.ident()
        self.expect("@")
        f = Func(self.symbol())
        self.expect("(")
        if not self.eat(")"):
            while True:
                f.body.args.append(self.ssa())
                self.expect(":")
                f.body.arg_types.append(self.type())
                self.skip_attr_dict()
                self.skip_loc()
                if self.eat(")"):
                    break
                self.expect(",")
        if self.eat("->"):
            if self.peek("("):
                f.result_types = self.type_list_paren()
            else:
                f.result_types = [self.type()]
        if self.eat("attributes"):
            self.attr_dict()
        self.expect("{")
        self.block_ops(f.body)
        self.expect("}")
        self.skip_loc()
        return f

    def block_ops(self, region: Region):
        """Parse ops until the closing brace of the enclosing region (not consumed)."""
        while True:
            self.ws()
            if self.peek("}"):
                return
            region.ops.append(self.op())

    def region(self) -> Region:
        """{ [^bb0(args):] ops }"""
        r = Region()
        self.expect("{")
        self.ws()
        if self.eat("^"):
            self.ident()
            if self.eat("("):
                if not self.eat(")"):
                    while True:
                        r.args.append(self.ssa())
                        self.expect(":")
                        r.arg_types.append(self.type())
                        self.skip_loc()
                        if self.eat(")"):
                            break
                        self.expect(",")
            self.expect(":")
        self.block_ops(r)
        self.expect("}")
        return r

    def op(self) -> Op:
        op = Op()
        self.ws()
        nres = 1
        listed = False
        if self.s[self.i] == "%":
            m = re.compile(r"%[A-Za-z0-9_.$]+").match(self.s, self.i)
            base = m.group(0)
            self.i = m.end()
            if self.eat(":"):
                nres = self.integer()
            end_decl = self.i
            explicit = ":" in self.s[m.end():end_decl]
            op.results = [base] if (nres == 1 and not explicit) else [f"{base}#{k}" for k in range(nres)]
            # `%a, %b = op`: one name per result (or per run of results with `%a:2`)
            while self.eat(","):
                listed = True
                self.ws()
                m = re.compile(r"%[A-Za-z0-9_.$]+").match(self.s, self.i)
                nm = m.group(0)
                self.i = m.end()
                if self.eat(":"):
                    c = self.integer()
                    op.results += [f"{nm}#{k}" for k in range(c)]
                else:
                    op.results.append(nm)
            self.expect("=")
            has_res = True
        else:
            has_res = False
        self.ws()
        if self.s[self.i] == '"':
            op.name = self.string()
            self.generic_op(op)
        else:
            op.name = self.ident()
            if op.name in ("return", "func.return", "stablehlo.return"):
                op.name = "return"
                if not self.peek("}"):
                    self.ws()
                    if self.s[self.i] == "%":
                        op.operands = self.ssa_list()
                        self.expect(":")
                        op.in_types = self.types_bare()
            elif op.name in ("call", "func.call"):
                op.name = "call"
                self.expect("@")
                op.attrs["callee"] = self.symbol()
                self.expect("(")
                op.operands = [] if self.peek(")") else self.ssa_list()
                self.expect(")")
                self.skip_attr_dict()
                self.expect(":")
                op.in_types = self.type_list_paren()
                self.expect("->")
                op.out_types = self.type_list_paren() if self.peek("(") else [self.type()]
            else:
                self.pretty_op(op)
        if has_res and not listed and nres == 1 and len(op.out_types) > 1:
            op.results = [f"{op.results[0]}#{k}" for k in range(len(op.out_types))]
        self.skip_loc()
        return op

    def ssa_list(self) -> List[str]:
        out = [self.ssa()]
        while True:
            save = self.i
            if not self.eat(","):
                break
            self.ws()
            if self.i >= self.n or self.s[self.i] != "%":
                self.i = save
                break
            out.append(self.ssa())
        return out

    def types_bare(self) -> List[TType]:
        out = [self.type()]
        while self.eat(","):
            out.append(self.type())
        return out

    def fn_type(self, op: Op):
        """(in types) -> out types   |   type (same for operands and result)"""
        if self.peek("("):
            op.in_types = self.type_list_paren()
            self.expect("->")
            op.out_types = self.type_list_paren() if self.peek("(") else [self.type()]
        else:
            t = self.type()
            op.in_types = [t] * len(op.operands)
            op.out_types = [t]
            if self.eat("->"):      # chlo's pretty form: `type -> type`
                op.out_types = self.type_list_paren() if self.peek("(") else [self.type()]

    def generic_op(self, op: Op):
        self.expect("(")
        op.operands = [] if self.peek(")") else self.ssa_list()
        self.expect(")")
        if self.eat("<"):
            op.attrs.update(self.attr_dict())
            self.expect(">")
        if self.peek("("):
            self.expect("(")
            while True:
                op.regions.append(self.region())
                if not self.eat(","):
                    break
            self.expect(")")
        if self.peek("{"):
            op.attrs.update(self.attr_dict())
        self.expect(":")
        op.in_types = self.type_list_paren()
        self.expect("->")
        op.out_types = self.type_list_paren() if self.peek("(") else [self.type()]
        self._normalize_generic(op)

    @staticmethod
    def _normalize_generic(op: Op):
        """Attribute names and shapes of the generic op form -> the ones the pretty forms produce (what the op_*
        methods read).  Mirrors the table of the generic StableHLO assembly: each op's attribute dictionary."""
        a = op.attrs
        n = op.name[len("stablehlo."):] if op.name.startswith("stablehlo.") else op.name

        def enum(v):
            return v[1] if isinstance(v, tuple) and isinstance(v[0], str) and v[0].startswith("#") else v

        def ints(v):
            if isinstance(v, tuple) and len(v) == 2 and isinstance(v[0], np.ndarray):
                return [int(x) for x in np.asarray(v[0]).reshape(-1)]
            if isinstance(v, np.ndarray):
                return [int(x) for x in v.reshape(-1)]
            return list(v)

        def move(old, new, conv=lambda v: v):
            if old in a:
                a[new] = conv(a.pop(old))
        for k in ("comparison_direction", "compare_type", "rng_algorithm"):
            if k in a:
                a[k] = enum(a[k])
        if n in ("return", "func.return"):
            op.name = "return"
        elif n in ("call", "func.call"):
            op.name = "call"
            a["callee"] = str(a["callee"]).lstrip("@")
        elif n == "broadcast_in_dim":
            move("broadcast_dimensions", "dims", ints)
        elif n == "transpose":
            move("permutation", "dims", ints)
        elif n == "reverse":
            move("dimensions", "dims", ints)
        elif n == "concatenate":
            move("dimension", "dim")
        elif n == "dynamic_slice":
            move("slice_sizes", "sizes", ints)
        elif n == "pad":
            move("edge_padding_low", "low", ints)
            move("edge_padding_high", "high", ints)
            move("interior_padding", "interior", ints)
        elif n in ("slice", "reduce", "gather", "sort", "reduce_window", "select_and_scatter"):
            for k in ("start_indices", "limit_indices", "strides", "dimensions", "slice_sizes", "window_dimensions", "window_strides",
                      "base_dilations", "window_dilations"):
                if k in a:
                    a[k] = ints(a[k])
            if n in ("reduce_window", "select_and_scatter") and "padding" in a and not isinstance(a["padding"], tuple):
                a["padding"] = (np.asarray(ints(a["padding"]), dtype=np.int64).reshape(-1, 2), None)
        elif n == "dot_general" and "dot_dimension_numbers" in a:
            d = a.pop("dot_dimension_numbers")[1] or {}
            a["batching_dims"] = (ints(d.get("lhs_batching_dimensions", [])), ints(d.get("rhs_batching_dimensions", [])))
            a["contracting_dims"] = (ints(d.get("lhs_contracting_dimensions", [])), ints(d.get("rhs_contracting_dimensions", [])))
        elif n == "convolution" and "dimension_numbers" in a:
            raw = a.pop("dimension_numbers")[1]
            groups = re.findall(r"\[([^\]]*)\]", raw)
            a["dim_numbers"] = tuple([t.strip() for t in g.split(",")] for g in groups)
            nsp = len(a["dim_numbers"][0]) - 2
            win = {}
            if "window_strides" in a:
                win["stride"] = ints(a.pop("window_strides"))
            if "padding" in a:
                win["pad"] = np.asarray(ints(a.pop("padding")), dtype=np.int64).reshape(nsp, 2).tolist()
            if "lhs_dilation" in a:
                win["lhs_dilate"] = ints(a.pop("lhs_dilation"))
            if "rhs_dilation" in a:
                win["rhs_dilate"] = ints(a.pop("rhs_dilation"))
            if "window_reversal" in a:
                win["reverse"] = [bool(x) for x in ints(a.pop("window_reversal"))]
            a["window"] = win

    def pretty_op(self, op: Op):
        n = op.name
        short = n[len("stablehlo."):] if n.startswith("stablehlo.") else n
        if short == "constant":
            self.skip_attr_dict()
            op.attrs["value"] = self.dense()
            a = op.attrs["value"]
            op.out_types = [a[1]]
            op.attrs["value"] = a[0]
            return
        if short == "iota":
            self.expect("dim")
            self.expect("=")
            op.attrs["iota_dimension"] = self.integer()
            self.expect(":")
            op.out_types = [self.type()]
            return
        if short == "compare":
            op.attrs["comparison_direction"] = self.ident()
            self.expect(",")
            op.operands = [self.ssa()]
            self.expect(",")
            op.operands.append(self.ssa())
            if self.eat(","):
                op.attrs["compare_type"] = self.ident()
            self.expect(":")
            self.fn_type(op)
            return
        if short == "reduce":
            return self.reduce_op(op)
        if short == "while":
            return self.while_op(op)
        if short == "convolution":
            return self.conv_op(op)
        if short == "custom_call":
            self.expect("@")
            op.attrs["call_target_name"] = self.ident()
            self.expect("(")
            op.operands = [] if self.peek(")") else self.ssa_list()
            self.expect(")")
            if self.peek("{"):
                op.attrs.update(self.attr_dict())
            self.expect(":")
            self.fn_type(op)
            return
        if op.name == "chlo.top_k":
            self.expect("(")
            op.operands = self.ssa_list()
            self.expect(",")
            self.expect("k")
            self.expect("=")
            op.attrs["k"] = self.integer()
            self.expect(")")
            self.expect(":")
            op.in_types = [self.type()]
            self.expect("->")
            op.out_types = self.type_list_paren()
            return
        if short == "rng_bit_generator":
            op.operands = self.ssa_list()
            self.expect(",")
            self.expect("algorithm")
            self.expect("=")
            op.attrs["rng_algorithm"] = self.ident()
            self.expect(":")
            self.fn_type(op)
            return
        if short == "optimization_barrier":
            op.operands = self.ssa_list() if self.peek("%") else []
            self.expect(":")
            ts = self.types_bare()
            op.in_types = ts
            op.out_types = ts
            return
        if short == "composite":
            op.attrs["name"] = self.string()
            self.ws()
            op.operands = self.ssa_list() if self.s[self.i] == "%" else []
            if self.peek("{"):
                op.attrs.update(self.attr_dict())
            self.expect(":")
            self.fn_type(op)
            return
        if short == "reduce_precision":
            op.operands = self.ssa_list()
            self.expect(",")
            self.expect("format")
            self.expect("=")
            self.ws()
            m = re.compile(r"e(\d+)m(\d+)").match(self.s, self.i)
            if not m:
                self.err("expected a format of the form e<exponent bits>m<mantissa bits>")
            self.i = m.end()
            op.attrs["exponent_bits"], op.attrs["mantissa_bits"] = int(m.group(1)), int(m.group(2))
            self.skip_attr_dict()
            self.expect(":")
            self.fn_type(op)
            return
        # generic pretty: operands, then keyword attrs, then type
        self.ws()
        if self.s[self.i] == "%":
            op.operands = self.ssa_list()
        if short == "slice":
            self.expect("[")
            st, li, sr = [], [], []
            if not self.eat("]"):
                while True:
                    st.append(self.integer())
                    self.expect(":")
                    li.append(self.integer())
                    sr.append(self.integer() if self.eat(":") else 1)
                    if self.eat("]"):
                        break
                    self.expect(",")
            op.attrs.update(start_indices=st, limit_indices=li, strides=sr)
        while self.eat(","):
            k = self.ident()
            self.expect("=")
            if k in ("batching_dims", "contracting_dims"):
                a = self.int_list()
                self.expect("x")
                bb = self.int_list()
                op.attrs[k] = (a, bb)
            else:
                op.attrs[k] = self.attr_value()
        if self.peek("{"):
            op.attrs.update(self.attr_dict())
        self.expect(":")
        if short == "select" and not self.peek("("):
            tp = self.type()
            self.expect(",")
            tv = self.type()
            op.in_types = [tp, tv, tv]
            op.out_types = [tv]
        else:
            self.fn_type(op)

    def reduce_op(self, op: Op):
        # stablehlo.reduce(%x init: %c), (%y init: %d) [applies stablehlo.add] across dimensions = [..] : (..) -> ..
        ins, inits = [], []
        while True:
            self.expect("(")
            ins.append(self.ssa())
            self.expect("init:")
            inits.append(self.ssa())
            self.expect(")")
            if not self.eat(","):
                break
        op.operands = ins + inits
        applies = None
        if self.eat("applies"):
            applies = self.ident()
        self.expect("across")
        self.expect("dimensions")
        self.expect("=")
        op.attrs["dimensions"] = self.int_list()
        self.skip_attr_dict()
        self.expect(":")
        self.fn_type(op)
        if applies is not None:
            r = Region()
            st = TType((), op.out_types[0].dtype)
            r.args = ["%__a", "%__b"]
            r.arg_types = [st, st]
            o = Op()
            o.name = applies
            o.results = ["%__r"]
            o.operands = ["%__a", "%__b"]
            o.in_types = [st, st]
            o.out_types = [st]
            rt = Op()
            rt.name = "return"
            rt.operands = ["%__r"]
            r.ops = [o, rt]
            op.regions = [r]
        else:
            self.expect("reducer")
            r = Region()
            pairs = []
            while self.eat("("):
                a = self.ssa(); self.expect(":"); ta = self.type(); self.expect(",")
                b_ = self.ssa(); self.expect(":"); tb = self.type(); self.expect(")")
                pairs.append((a, ta, b_, tb))
            r.args = [p[0] for p in pairs] + [p[2] for p in pairs]
            r.arg_types = [p[1] for p in pairs] + [p[3] for p in pairs]
            self.expect("{")
            self.block_ops(r)
            self.expect("}")
            op.regions = [r]

    def while_op(self, op: Op):
        self.expect("(")
        names = []
        if not self.eat(")"):
            while True:
                names.append(self.ssa())
                self.expect("=")
                op.operands.append(self.ssa())
                if self.eat(")"):
                    break
                self.expect(",")
        if self.eat(":"):
            ts = self.types_bare()
        else:
            ts = []
        op.in_types = ts
        op.out_types = ts
        if self.eat("attributes"):
            self.attr_dict()
        self.expect("cond")
        cond = Region()
        cond.args, cond.arg_types = list(names), list(ts)
        self.expect("{")
        self.block_ops(cond)
        self.expect("}")
        self.expect("do")
        body = Region()
        body.args, body.arg_types = list(names), list(ts)
        self.expect("{")
        self.block_ops(body)
        self.expect("}")
        op.regions = [cond, body]

    def conv_op(self, op: Op):
        self.expect("(")
        op.operands = self.ssa_list()
        self.expect(")")
        self.expect("dim_numbers")
        self.expect("=")

        def spec():
            self.expect("[")
            out = []
            while True:
                self.ws()
                m = re.compile(r"[a-z0-9]+").match(self.s, self.i)
                out.append(m.group(0))
                self.i = m.end()
                if self.eat("]"):
                    return out
                self.expect(",")
        l = spec(); self.expect("x"); r = spec(); self.expect("->"); o = spec()
        op.attrs["dim_numbers"] = (l, r, o)
        self.expect(",")
        self.expect("window")
        self.expect("=")
        self.expect("{")
        win = {}
        while not self.eat("}"):
            k = self.ident()
            self.expect("=")
            win[k] = self.attr_value()
            self.eat(",")
        op.attrs["window"] = win
        if self.peek("{"):
            op.attrs.update(self.attr_dict())
        self.expect(":")
        self.fn_type(op)


def _dense_to_numpy(payload, t: TType):
    kind, raw = payload
    dt = t.dtype
    n = int(np.prod(t.shape)) if t.shape else 1
    if kind == "hex":
        b = bytes.fromhex(raw[2:])
        if dt == "bf16":
            a = bf16_bits_to_f32(np.frombuffer(b, dtype=np.uint16))
        elif dt == "i1":
            a = np.frombuffer(b, dtype=np.uint8).astype(np.bool_)
        else:
            a = np.frombuffer(b, dtype=_NP[dt])
        if a.size == 1 and n != 1:
            a = np.full(n, a[0])
        return (a.reshape(t.shape).copy(), t)
    toks = re.findall(r"[^\s,\[\]]+", raw)

    def conv(tok):
        if tok == "true":
            return True
        if tok == "false":
            return False
        if dt in FLOATS:
            if tok.lower().startswith("0x"):
                bits = int(tok, 16)
                if dt == "f32":
                    return np.array([bits], dtype=np.uint32).view(np.float32)[0]
                if dt == "bf16":
                    return bf16_bits_to_f32(np.array([bits], dtype=np.uint16))[0]
                if dt == "f64":
                    return np.array([bits], dtype=np.uint64).view(np.float64)[0]
                if dt == "f16":
                    return np.array([bits], dtype=np.uint16).view(np.float16)[0]
            return float(tok)
        return int(tok, 0)
    vals = [conv(tk) for tk in toks]
    if dt in FLOATS:
        a = np.array(vals, dtype=np.float64).astype(_NP[dt])
        if dt == "bf16":
            a = round_bf16(a)
    else:
        a = np.array([int(v) for v in vals], dtype=object)
        a = np.array([v & ((1 << 64) - 1) if dt == "ui64" else v for v in vals]).astype(_NP[dt])
    if a.size == 1 and n != 1:
        a = np.full(n, a.reshape(-1)[0], dtype=a.dtype)
    return (a.reshape(t.shape), t)


def parse(text: str) -> Dict[str, Func]:
    return _P(text).module()


def parse_with_attributes(text: str):
    """The functions of a module and the attribute dictionary written after `module @name attributes`."""
    p = _P(text)
    funcs = p.module()
    return funcs, getattr(p, "module_attributes", {})


# ----------------------------------------------------------------------------
# interpreter
# ----------------------------------------------------------------------------
def _cast_result(a: np.ndarray, t: TType, keep_shape: bool = False) -> np.ndarray:
    a = np.asarray(a)
    if t.dtype == "token":
        return np.asarray(a, dtype=np.float32).reshape(())
    want = _NP[t.dtype]
    if a.dtype != want:
        a = a.astype(want)
    if t.dtype == "bf16":
        a = round_bf16(a)
    if a.shape != t.shape and not keep_shape:
        a = a.reshape(t.shape)
    return a


def _boundary_type(t: TType):
    """Type of an argument or result of main as a caller sees it: a token travels as an f32 scalar."""
    return ((), "f32") if t.dtype == "token" else (t.shape, t.dtype)


class Oracle:
    def __init__(self, text: str, accum: str = "f64", round_intermediates: bool = True):
        """`round_intermediates=False` keeps bf16-typed intermediate results unrounded (float32 carriers of the
        float64 arithmetic): the value the program's formulas define, against which the rounding noise of any
        bf16 evaluation order can be measured.  Arguments and dense constants keep their bf16 values."""
        self.funcs, self.module_attributes = parse_with_attributes(text)
        self.accum = np.float64 if accum == "f64" else np.float32
        self.round_intermediates = round_intermediates
        self.main = self.funcs["main"]

    # -- public
    def run(self, *args: np.ndarray, pinned: Optional[Dict[int, np.ndarray]] = None) -> List[np.ndarray]:
        """Evaluate main.  `pinned` maps an output index of main to an array that replaces that value at the point
        where the program defines it, so everything computed from it afterwards uses the given array (a checker's
        aid: two float32 evaluations of a ReLU network take different branches at the few activations that lie
        within rounding noise of zero, and gradients can only be compared element by element once both sides use
        the same branch decisions).  The values the oracle itself computed there are kept in `self.replaced`."""
        f = self.main
        assert len(args) == len(f.body.args), (len(args), len(f.body.args))
        vals = [_cast_result(np.asarray(a), t) for a, t in zip(args, f.body.arg_types)]
        self._pinned, self.replaced = {}, {}
        if pinned:
            ret = [op for op in f.body.ops if op.name == "return"][-1]
            self._pinned = {ret.operands[k]: (k, np.asarray(v)) for k, v in pinned.items()}
        try:
            return self._run_region(f.body, vals, {})
        finally:
            self._pinned = {}

    @property
    def arg_types(self):
        return [_boundary_type(t) for t in self.main.body.arg_types]

    @property
    def result_types(self):
        return [_boundary_type(t) for t in self.main.result_types]

    # -- engine
    def _run_region(self, region: Region, args, outer_env, vectorized: bool = False) -> List[np.ndarray]:
        env = dict(outer_env)
        for n, v in zip(region.args, args):
            env[n] = v
        for op in region.ops:
            if op.name == "return":
                return [env[o] for o in op.operands]
            ins = [env[o] for o in op.operands]
            outs = self._eval(op, ins, env)
            if not isinstance(outs, (list, tuple)):
                outs = [outs]
            for name, val, t in zip(op.results, outs, op.out_types):
                if not self.round_intermediates and t.dtype == "bf16":
                    val = np.asarray(val, dtype=np.float32)
                    env[name] = val if (vectorized or val.shape == t.shape) else val.reshape(t.shape)
                else:
                    env[name] = _cast_result(val, t, keep_shape=vectorized)
                if name.endswith("#0") and len(op.results) == 1:
                    env[name[:-2]] = env[name]
                if getattr(self, "_pinned", None) and region is self.main.body:
                    for alias in (name, name[:-2] if name.endswith("#0") else name):
                        if alias in self._pinned and alias in env:
                            k, given = self._pinned[alias]
                            assert given.shape == env[alias].shape, (alias, given.shape, env[alias].shape)
                            self.replaced.setdefault(k, env[alias])
                            env[alias] = given.astype(env[alias].dtype)
        return []

    def _eval(self, op: Op, ins, env):
        n = op.name
        if n.startswith("stablehlo."):
            n = n[10:]
        elif n.startswith("chlo."):
            n = "chlo_" + n[5:]
        fn = getattr(self, "op_" + n, None)
        if fn is None:
            raise NotImplementedError(f"oracle: unsupported op {op.name}")
        return fn(op, ins, env)

    # ------------------------------------------------------------------
    # elementwise (reference: ops/arithmetic.cc:535-607)
    # ------------------------------------------------------------------
    @staticmethod
    def _f(op):
        return op.out_types[0].dtype in FLOATS

    def _un(self, op, ins, f):
        x = ins[0]
        dt = op.out_types[0].dtype
        if dt in ("bf16", "f16"):
            return f(x.astype(np.float32))
        with np.errstate(all="ignore"):
            return f(x)

    def op_add(self, op, ins, env):
        a, b = ins
        if a.dtype == np.bool_:
            return a | b
        with np.errstate(all="ignore"):
            return a + b

    def op_subtract(self, op, ins, env):
        with np.errstate(all="ignore"):
            return ins[0] - ins[1]

    def op_multiply(self, op, ins, env):
        a, b = ins
        if a.dtype == np.bool_:
            return a & b
        with np.errstate(all="ignore"):
            return a * b

    def op_divide(self, op, ins, env):
        """Float: IEEE divide.  Integer: truncation toward zero (arithmetic.cc:496-513)."""
        a, b = ins
        with np.errstate(all="ignore"):
            if a.dtype.kind == "f":
                return a / b
            bz = np.where(b == 0, 1, b)
            if a.dtype.kind == "u":
                q = a // bz
                return np.where(b == 0, np.iinfo(a.dtype).max, q).astype(a.dtype)
            # magnitudes as unsigned 64-bit numbers (the most negative value has no signed magnitude), the sign put
            # back in wrapping arithmetic: the most negative value divided by -1 is itself
            mag = lambda v: np.where(v < 0, ~v.astype(np.int64).astype(np.uint64) + np.uint64(1), v.astype(np.int64).astype(np.uint64))
            q = mag(a) // mag(bz)
            q = np.where((a < 0) != (b < 0), ~q + np.uint64(1), q).astype(np.int64)
            return np.where(b == 0, -1, q).astype(a.dtype)

    def op_remainder(self, op, ins, env):
        """C-style remainder: sign follows the dividend (arithmetic.cc:46-83)."""
        a, b = ins
        with np.errstate(all="ignore"):
            if a.dtype.kind == "f":
                return np.fmod(a, b)
            bz = np.where(b == 0, 1, b)
            r = np.fmod(a, bz)
            return np.where(b == 0, a, r).astype(a.dtype)

    def op_maximum(self, op, ins, env):
        a, b = ins
        if a.dtype == np.bool_:
            return a | b
        if a.dtype.kind != "f":
            return np.maximum(a, b)
        # NaN-propagating, as in StableHLO.  The reference hands the op to mlx::core::maximum (arithmetic.cc:573), whose
        # published element rule is "x if x is NaN, else x > y ? x : y": of two equal operands (the two zeros) the second
        # is returned, which is what tells +0 from -0 in the result.
        with np.errstate(all="ignore"):
            return np.where(np.isnan(a), a, np.where(a > b, a, b)).astype(a.dtype)

    def op_minimum(self, op, ins, env):
        a, b = ins
        if a.dtype == np.bool_:
            return a & b
        if a.dtype.kind != "f":
            return np.minimum(a, b)
        with np.errstate(all="ignore"):   # mlx::core::minimum: x if x is NaN, else x < y ? x : y (arithmetic.cc:575)
            return np.where(np.isnan(a), a, np.where(a < b, a, b)).astype(a.dtype)

    def op_power(self, op, ins, env):
        a, b = ins
        with np.errstate(all="ignore"):
            if a.dtype.kind == "f":
                return np.power(a.astype(np.float64), b.astype(np.float64))
            out = np.ones_like(a)
            base, e = a.copy(), b.copy()
            neg = e < 0 if e.dtype.kind == "i" else np.zeros(e.shape, bool)
            e = np.where(neg, 0, e)
            for _ in range(64):
                out = np.where((e & 1) == 1, out * base, out)
                base = base * base
                e = e >> 1
            special = np.where(a == 1, 1, np.where(a == -1, np.where((b & 1) == 1, -1, 1), 0)) if a.dtype.kind == "i" else np.where(a == 1, 1, 0)
            return np.where(neg, special, out).astype(a.dtype)

    def op_atan2(self, op, ins, env): return np.arctan2(ins[0].astype(np.float64), ins[1].astype(np.float64))
    def op_and(self, op, ins, env): return ins[0] & ins[1]
    def op_or(self, op, ins, env): return ins[0] | ins[1]
    def op_xor(self, op, ins, env): return ins[0] ^ ins[1]

    def op_not(self, op, ins, env):
        x = ins[0]
        return ~x

    @staticmethod
    def _bits(dt):
        return np.dtype(dt).itemsize * 8

    def op_shift_left(self, op, ins, env):
        """Shift amounts >= bit width give 0 (mlx_executable.cc:293-301)."""
        a, b = ins
        w = self._bits(a.dtype)
        ub = b.astype(np.uint64)
        ok = ub < w
        u = a.view(np.dtype(f"u{a.dtype.itemsize}"))
        r = (u << np.where(ok, ub, 0).astype(u.dtype)).astype(u.dtype)
        return np.where(ok, r, 0).astype(u.dtype).view(a.dtype)

    def op_shift_right_logical(self, op, ins, env):
        a, b = ins
        w = self._bits(a.dtype)
        ub = b.astype(np.uint64)
        ok = ub < w
        u = a.view(np.dtype(f"u{a.dtype.itemsize}"))
        r = (u >> np.where(ok, ub, 0).astype(u.dtype)).astype(u.dtype)
        return np.where(ok, r, 0).astype(u.dtype).view(a.dtype)

    def op_shift_right_arithmetic(self, op, ins, env):
        """Out-of-range shift fills with the sign bit (arithmetic.cc:119-143)."""
        a, b = ins
        w = self._bits(a.dtype)
        ub = b.astype(np.uint64)
        sh = np.minimum(ub, w - 1).astype(a.dtype)
        return a >> sh

    def op_popcnt(self, op, ins, env):
        a = ins[0]
        u = a.view(np.dtype(f"u{a.dtype.itemsize}")).astype(np.uint64)
        c = np.zeros(a.shape, np.uint64)
        for k in range(self._bits(a.dtype)):
            c += (u >> np.uint64(k)) & np.uint64(1)
        return c.astype(a.dtype)

    def op_count_leading_zeros(self, op, ins, env):
        a = ins[0]
        w = self._bits(a.dtype)
        u = a.view(np.dtype(f"u{a.dtype.itemsize}")).astype(np.uint64)
        c = np.full(a.shape, w, np.int64)
        for k in range(w):
            c = np.where((u >> np.uint64(k)) != 0, w - 1 - k, c)
        return c.astype(a.dtype)

    def op_negate(self, op, ins, env):
        with np.errstate(all="ignore"):
            return -ins[0]

    def op_abs(self, op, ins, env):
        with np.errstate(all="ignore"):
            return np.abs(ins[0])

    def _f64un(self, op, ins, f):
        x = ins[0].astype(np.float64)
        with np.errstate(all="ignore"):
            return f(x)

    def op_exponential(self, op, ins, env): return self._f64un(op, ins, np.exp)
    def op_exponential_minus_one(self, op, ins, env): return self._f64un(op, ins, np.expm1)
    def op_log(self, op, ins, env): return self._f64un(op, ins, np.log)
    def op_log_plus_one(self, op, ins, env): return self._f64un(op, ins, np.log1p)
    def op_sqrt(self, op, ins, env): return self._un(op, ins, np.sqrt)
    def op_cbrt(self, op, ins, env): return self._f64un(op, ins, np.cbrt)
    def op_rsqrt(self, op, ins, env): return self._f64un(op, ins, lambda x: 1.0 / np.sqrt(x))
    def op_tanh(self, op, ins, env): return self._f64un(op, ins, np.tanh)
    def op_tan(self, op, ins, env): return self._f64un(op, ins, np.tan)
    def op_sine(self, op, ins, env): return self._f64un(op, ins, np.sin)
    def op_cosine(self, op, ins, env): return self._f64un(op, ins, np.cos)
    def op_logistic(self, op, ins, env): return self._f64un(op, ins, lambda x: 1.0 / (1.0 + np.exp(-x)))
    def op_floor(self, op, ins, env): return self._un(op, ins, np.floor)
    def op_ceil(self, op, ins, env): return self._un(op, ins, np.ceil)
    def op_round_nearest_even(self, op, ins, env): return self._un(op, ins, np.rint)

    def op_round_nearest_afz(self, op, ins, env):
        """Half away from zero as the reference computes it, sign(x) * floor(|x| + 0.5) in the operand type
        (arithmetic.cc:316-327).  The sum is rounded to the type before the floor, so the formula differs from an exact
        rounding at the predecessor of 0.5 (the sum rounds to 1) and at odd integers from 2^(significand bits - 1) on
        (the sum rounds to the even neighbour)."""
        dt = op.out_types[0].dtype

        def f(x):
            s = np.abs(x) + x.dtype.type(0.5)
            if dt == "bf16":
                s = round_bf16(s)
            elif dt == "f16":
                s = s.astype(np.float16).astype(np.float32)
            return np.where(np.isfinite(x), np.sign(x) * np.floor(s), x)
        return self._un(op, ins, f)

    def op_is_finite(self, op, ins, env): return np.isfinite(ins[0])

    def op_sign(self, op, ins, env):
        """NaN stays NaN, -0 stays -0 (arithmetic.cc:517-531)."""
        x = ins[0]
        if x.dtype.kind == "f":
            with np.errstate(all="ignore"):
                return np.where(np.isnan(x), x, np.where(x == 0, x, np.sign(x)))
        return np.sign(x)

    def op_erf(self, op, ins, env):
        from scipy import special
        return special.erf(ins[0].astype(np.float64))
    op_chlo_erf = op_erf

    # chlo unary ops, also spelled custom_call @mhlo.<name> (reference: ops/control_flow.cc:53-63)
    def op_chlo_erf_inv(self, op, ins, env):
        from scipy import special
        return special.erfinv(ins[0].astype(np.float64))
    def op_chlo_asin(self, op, ins, env): return self._f64un(op, ins, np.arcsin)
    def op_chlo_acos(self, op, ins, env): return self._f64un(op, ins, np.arccos)
    def op_chlo_atan(self, op, ins, env): return self._f64un(op, ins, np.arctan)
    def op_chlo_sinh(self, op, ins, env): return self._f64un(op, ins, np.sinh)
    def op_chlo_cosh(self, op, ins, env): return self._f64un(op, ins, np.cosh)
    def op_chlo_asinh(self, op, ins, env): return self._f64un(op, ins, np.arcsinh)
    def op_chlo_acosh(self, op, ins, env): return self._f64un(op, ins, np.arccosh)
    def op_chlo_atanh(self, op, ins, env): return self._f64un(op, ins, np.arctanh)

    def op_clamp(self, op, ins, env):
        lo, x, hi = ins
        return np.minimum(np.maximum(x, lo), hi)

    def op_select(self, op, ins, env):
        p, a, b = ins
        return np.where(p, a, b)

    def op_compare(self, op, ins, env):
        """EQ/NE/LT/LE/GT/GE; TOTALORDER compares the sign-magnitude key (arithmetic.cc:239-313)."""
        a, b = ins
        d = op.attrs["comparison_direction"]
        if op.attrs.get("compare_type") == "TOTALORDER" and a.dtype.kind == "f":
            def key(x):
                x = x.astype(np.float32) if x.dtype != np.float64 else x
                w = 32 if x.dtype == np.float32 else 64
                i = x.view(np.int32 if w == 32 else np.int64)
                mask = np.iinfo(i.dtype).max
                return np.where(i < 0, i ^ mask, i)
            a, b = key(a), key(b)
        with np.errstate(all="ignore"):
            return {"EQ": np.equal, "NE": np.not_equal, "LT": np.less, "LE": np.less_equal,
                    "GT": np.greater, "GE": np.greater_equal}[d](a, b)

    def op_convert(self, op, ins, env):
        """Value conversion; float->int truncates toward zero and saturates, NaN->0 (XLA rule)."""
        x = ins[0]
        dt = op.out_types[0].dtype
        want = np.dtype(_NP[dt])
        if want == np.bool_:
            return x != 0
        if x.dtype.kind == "f" and want.kind in "iu":
            info = np.iinfo(want)
            with np.errstate(all="ignore"):
                t = np.trunc(x.astype(np.float64))
                t = np.where(np.isnan(t), 0, t)
                t = np.clip(t, float(info.min), float(info.max))
                out = np.empty(x.shape, dtype=want)
                hi = t >= float(info.max)
                lo = t <= float(info.min)
                mid = ~(hi | lo)
                out[hi] = info.max
                out[lo] = info.min
                out[mid] = t[mid].astype(want)
                return out
        with np.errstate(all="ignore"):
            return x.astype(want)

    def op_bitcast_convert(self, op, ins, env):
        x = ins[0]
        it, ot = op.in_types[0].dtype, op.out_types[0].dtype
        if it == "bf16":
            x = f32_to_bf16_bits(x)
        x = np.ascontiguousarray(x)
        if ot == "bf16":
            return bf16_bits_to_f32(x.view(np.uint16).reshape(op.out_types[0].shape))
        return x.view(_NP[ot]).reshape(op.out_types[0].shape)

    def op_reduce_precision(self, op, ins, env):
        x = ins[0].astype(np.float32)
        eb, mb = int(op.attrs["exponent_bits"]), int(op.attrs["mantissa_bits"])
        u = x.view(np.uint32).copy()
        if mb < 23:
            sh = 23 - mb
            lsb = (u >> np.uint32(sh)) & np.uint32(1)
            rnd = np.uint32((1 << (sh - 1)) - 1) + lsb
            nan = np.isnan(x)
            u2 = (u + rnd) & np.uint32(~((1 << sh) - 1) & 0xFFFFFFFF)
            u = np.where(nan, u, u2)
        y = u.view(np.float32)
        if eb < 8:
            maxexp = (1 << (eb - 1)) - 1
            minexp = 1 - maxexp
            e = ((u >> np.uint32(23)) & np.uint32(0xFF)).astype(np.int32) - 127
            sign = np.signbit(y)
            big = (e > maxexp) & np.isfinite(x)
            small = (e < minexp)
            y = np.where(big, np.where(sign, -np.inf, np.inf), y)
            y = np.where(small & ~np.isnan(x), np.where(sign, -0.0, 0.0), y)
        return y.astype(np.float32)

    # ------------------------------------------------------------------
    # shape / data movement (reference: ops/shape.cc:260-270, ops/slice.cc:280-285)
    # ------------------------------------------------------------------
    def op_constant(self, op, ins, env): return op.attrs["value"]

    def op_iota(self, op, ins, env):
        t = op.out_types[0]
        d = op.attrs["iota_dimension"]
        shp = [1] * len(t.shape)
        shp[d] = t.shape[d]
        return np.broadcast_to(np.arange(t.shape[d]).reshape(shp), t.shape).astype(_NP[t.dtype])

    def op_reshape(self, op, ins, env): return ins[0].reshape(op.out_types[0].shape)

    def op_broadcast_in_dim(self, op, ins, env):
        x = ins[0]
        dims = op.attrs.get("dims", op.attrs.get("broadcast_dimensions"))
        shape = op.out_types[0].shape
        shp = [1] * len(shape)
        for k, d in enumerate(dims):
            shp[d] = x.shape[k]
        return np.broadcast_to(x.reshape(shp), shape).copy()

    def op_transpose(self, op, ins, env):
        return np.ascontiguousarray(np.transpose(ins[0], op.attrs.get("dims", op.attrs.get("permutation"))))

    def op_reverse(self, op, ins, env):
        return np.flip(ins[0], axis=tuple(op.attrs.get("dims", op.attrs.get("dimensions")))).copy()

    def op_concatenate(self, op, ins, env):
        return np.concatenate(ins, axis=op.attrs.get("dim", op.attrs.get("dimension")))

    def op_slice(self, op, ins, env):
        sl = tuple(slice(s, l, st) for s, l, st in zip(op.attrs["start_indices"], op.attrs["limit_indices"], op.attrs["strides"]))
        return ins[0][sl].copy()

    @staticmethod
    def _clamped_starts(starts, opshape, sizes):
        """start = max(0, min(start, dim - size)) (slice.cc:90-107)."""
        out = []
        for s, d, z in zip(starts, opshape, sizes):
            out.append(int(max(0, min(int(np.asarray(s).reshape(())), d - z))))
        return out

    def op_dynamic_slice(self, op, ins, env):
        x = ins[0]
        sizes = op.attrs.get("sizes", op.attrs.get("slice_sizes"))
        st = self._clamped_starts(ins[1:], x.shape, sizes)
        return x[tuple(slice(s, s + z) for s, z in zip(st, sizes))].copy()

    def op_dynamic_update_slice(self, op, ins, env):
        x, u = ins[0], ins[1]
        st = self._clamped_starts(ins[2:], x.shape, u.shape)
        out = x.copy()
        out[tuple(slice(s, s + z) for s, z in zip(st, u.shape))] = u
        return out

    def op_pad(self, op, ins, env):
        """Interior dilation first, then edge padding; negative edge padding crops (slice.cc:202-276)."""
        x, pv = ins
        lo, hi, it = op.attrs["low"], op.attrs["high"], op.attrs["interior"]
        shp = [d + max(d - 1, 0) * i for d, i in zip(x.shape, it)]
        y = np.full(shp, pv, dtype=x.dtype)
        y[tuple(slice(0, None, i + 1) for i in it)] = x
        out_shape = op.out_types[0].shape
        out = np.full(out_shape, pv, dtype=x.dtype)
        src, dst = [], []
        for d in range(x.ndim):
            s0 = max(0, -lo[d])
            s1 = shp[d] - max(0, -hi[d])
            d0 = max(0, lo[d])
            src.append(slice(s0, max(s0, s1)))
            dst.append(slice(d0, d0 + max(0, s1 - s0)))
        out[tuple(dst)] = y[tuple(src)]
        return out

    # ------------------------------------------------------------------
    # window reductions (reference: ops/reduction.cc:165-626)
    # ------------------------------------------------------------------
    @staticmethod
    def _window_attrs(op, rank):
        def ints(name, dflt):
            v = op.attrs.get(name)
            if v is None:
                return [dflt] * rank
            v = np.asarray(v).reshape(-1)
            return [int(x) for x in (v if v.size == rank else np.full(rank, v[0] if v.size else dflt))]
        pad = op.attrs.get("padding")
        if isinstance(pad, tuple):      # dense literal: (values, type)
            pad = pad[0]
        if pad is None:
            pad = np.zeros((rank, 2), np.int64)
        pad = np.asarray(pad)
        pad = np.broadcast_to(pad.reshape(-1, 2) if pad.size == 2 * rank else np.full((rank, 2), int(pad.reshape(-1)[0]) if pad.size else 0), (rank, 2))
        return ints("window_dimensions", 1), ints("window_strides", 1), ints("base_dilations", 1), ints("window_dilations", 1), pad.astype(np.int64)

    def op_reduce_window(self, op, ins, env):
        """Every output element is the reducer folded, in row-major window order and starting from the
        init value, over its window of the operand padded (and base-dilated) with the init value.
        Evaluated one output element at a time with the reducer region itself."""
        x, init = ins
        rank = x.ndim
        wd, ws, bd, wdil, pad = self._window_attrs(op, rank)
        body = op.regions[0]
        dil = [d + max(d - 1, 0) * (b - 1) for d, b in zip(x.shape, bd)]
        P = np.full([dil[d] + int(pad[d, 0]) + int(pad[d, 1]) for d in range(rank)], init, dtype=x.dtype)
        valid = np.zeros(P.shape, dtype=bool)
        P[tuple(slice(int(pad[d, 0]), int(pad[d, 0]) + dil[d], bd[d]) for d in range(rank))] = x
        out_shape = op.out_types[0].shape
        out = np.empty(out_shape, dtype=x.dtype)
        import itertools
        for o in itertools.product(*[range(n) for n in out_shape]):
            acc = np.asarray(init)
            for t in itertools.product(*[range(k) for k in wd]):
                pos = tuple(o[d] * ws[d] + t[d] * wdil[d] for d in range(rank))
                acc = np.asarray(self._run_region(body, [acc, np.asarray(P[pos])], env)[0])
            out[o] = acc
        return out

    def op_select_and_scatter(self, op, ins, env):
        """For every window of the operand (row-major), the select region picks one element by a running
        comparison over the in-bounds window elements; the scatter region adds the window's source value
        to that element of the result, which starts as the init value."""
        x, src, init = ins
        rank = x.ndim
        wd, ws, _, _, pad = self._window_attrs(op, rank)
        select, scatter = op.regions
        out = np.full(x.shape, init, dtype=x.dtype)
        import itertools
        for w in itertools.product(*[range(n) for n in src.shape]):
            best = None
            for t in itertools.product(*[range(k) for k in wd]):
                pos = tuple(w[d] * ws[d] - int(pad[d, 0]) + t[d] for d in range(rank))
                if any(p < 0 or p >= x.shape[d] for d, p in enumerate(pos)):
                    continue
                if best is None or not bool(np.asarray(self._run_region(select, [np.asarray(x[best]), np.asarray(x[pos])], env)[0])):
                    best = pos
            if best is not None:
                out[best] = np.asarray(self._run_region(scatter, [np.asarray(out[best]), np.asarray(src[w])], env)[0])
        return out

    # ------------------------------------------------------------------
    # reductions (reference: ops/reduction.cc:83-162)
    # ------------------------------------------------------------------
    def op_reduce(self, op, ins, env):
        k = len(ins) // 2
        xs, inits = ins[:k], ins[k:]
        dims = tuple(op.attrs["dimensions"])
        body = op.regions[0]
        if k == 1 and len(body.ops) == 2 and body.ops[0].name.startswith("stablehlo.") \
                and set(body.ops[0].operands) == set(body.args) and len(dims) > 0:
            kind = body.ops[0].name[10:]
            x, init = xs[0], inits[0]
            dt = op.out_types[0].dtype
            red = None
            with np.errstate(all="ignore"):
                if kind == "add":
                    if dt in FLOATS:
                        red = np.sum(x.astype(self.accum), axis=dims) + init.astype(self.accum)
                    elif dt == "i1":
                        red = np.any(x, axis=dims) | init
                    else:
                        red = np.add.reduce(x, axis=dims, dtype=x.dtype) + init
                elif kind == "multiply":
                    red = (np.prod(x.astype(self.accum), axis=dims) * init) if dt in FLOATS else np.multiply.reduce(x, axis=dims, dtype=x.dtype) * init
                elif kind == "maximum":
                    red = np.maximum(np.max(x, axis=dims, initial=None) if x.size else np.full(op.out_types[0].shape, init), init)
                elif kind == "minimum":
                    red = np.minimum(np.min(x, axis=dims, initial=None) if x.size else np.full(op.out_types[0].shape, init), init)
                elif kind == "and":
                    red = np.bitwise_and.reduce(x, axis=dims) & init if x.size else np.full(op.out_types[0].shape, init)
                elif kind == "or":
                    red = np.bitwise_or.reduce(x, axis=dims) | init if x.size else np.full(op.out_types[0].shape, init)
            if red is not None:
                return [red]
        # generic fold in row-major order of the reduced dims
        keep = [d for d in range(xs[0].ndim) if d not in dims]
        perm = list(dims) + keep
        xt = [np.transpose(x, perm).reshape((-1,) + tuple(x.shape[d] for d in keep)) for x in xs]
        acc = [np.broadcast_to(i, xt[0].shape[1:]).astype(i.dtype).copy() for i in inits]
        for r in range(xt[0].shape[0]):
            acc = self._run_region(body, acc + [x[r] for x in xt], env, vectorized=True)
        return acc

    # ------------------------------------------------------------------
    # contractions (reference: ops/linalg.cc:89-250, 253-550)
    # ------------------------------------------------------------------
    def op_dot_general(self, op, ins, env):
        a, b = ins
        if "dot_dimension_numbers" in op.attrs:
            d = op.attrs["dot_dimension_numbers"][1]
            ba, bb = d.get("lhs_batching_dimensions", []), d.get("rhs_batching_dimensions", [])
            ca, cb = d.get("lhs_contracting_dimensions", []), d.get("rhs_contracting_dimensions", [])
        else:
            ba, bb = op.attrs.get("batching_dims", ([], []))
            ca, cb = op.attrs.get("contracting_dims", ([], []))
        fa = [i for i in range(a.ndim) if i not in ca and i not in ba]
        fb = [i for i in range(b.ndim) if i not in cb and i not in bb]
        isf = a.dtype.kind == "f"
        acc = self.accum if isf else (np.int64 if a.dtype.kind in "iub" else a.dtype)
        at = np.transpose(a, list(ba) + fa + list(ca)).astype(acc)
        bt = np.transpose(b, list(bb) + list(cb) + fb).astype(acc)
        B = int(np.prod([a.shape[i] for i in ba])) if ba else 1
        M = int(np.prod([a.shape[i] for i in fa])) if fa else 1
        K = int(np.prod([a.shape[i] for i in ca])) if ca else 1
        N = int(np.prod([b.shape[i] for i in fb])) if fb else 1
        r = np.matmul(at.reshape(B, M, K), bt.reshape(B, K, N))
        if op.out_types[0].dtype == "i1":
            r = r != 0
        return r.reshape(op.out_types[0].shape)

    def op_convolution(self, op, ins, env):
        """StableHLO order of operations: dilate lhs, pad (may be negative), dilate rhs, slide."""
        lhs, rhs = ins
        if "dim_numbers" in op.attrs:
            ls, rs, os_ = op.attrs["dim_numbers"]
            win = op.attrs.get("window", {})
            nsp = len(ls) - 2
            strides = win.get("stride", [1] * nsp)
            pad = win.get("pad", [[0, 0]] * nsp)
            ldil = win.get("lhs_dilate", [1] * nsp)
            rdil = win.get("rhs_dilate", [1] * nsp)
            wrev = win.get("reverse", [False] * nsp)
        else:
            raise NotImplementedError("generic-form convolution attributes")
        fg = int(op.attrs.get("feature_group_count", 1))
        bg = int(op.attrs.get("batch_group_count", 1))
        sp = [str(k) for k in range(nsp)]
        l_perm = [ls.index("b")] + [ls.index(s) for s in sp] + [ls.index("f")]
        r_perm = [rs.index(s) for s in sp] + [rs.index("i"), rs.index("o")]
        x = np.transpose(lhs, l_perm).astype(self.accum)
        w = np.transpose(rhs, r_perm).astype(self.accum)
        for d in range(nsp):
            if wrev[d] in (True, "true"):
                w = np.flip(w, axis=d)
        # lhs dilation
        shp = list(x.shape)
        for d in range(nsp):
            shp[1 + d] = (x.shape[1 + d] - 1) * ldil[d] + 1 if x.shape[1 + d] > 0 else 0
        xd = np.zeros(shp, dtype=x.dtype)
        xd[(slice(None),) + tuple(slice(0, None, ldil[d]) for d in range(nsp)) + (slice(None),)] = x
        # padding (negative crops)
        shp2 = list(xd.shape)
        src, dst = [slice(None)], [slice(None)]
        for d in range(nsp):
            lo, hi = pad[d]
            shp2[1 + d] = max(0, xd.shape[1 + d] + lo + hi)
            s0, s1 = max(0, -lo), xd.shape[1 + d] - max(0, -hi)
            d0 = max(0, lo)
            src.append(slice(s0, max(s0, s1)))
            dst.append(slice(d0, d0 + max(0, s1 - s0)))
        src.append(slice(None)); dst.append(slice(None))
        xp = np.zeros(shp2, dtype=x.dtype)
        xp[tuple(dst)] = xd[tuple(src)]
        # rhs dilation
        wshp = list(w.shape)
        for d in range(nsp):
            wshp[d] = (w.shape[d] - 1) * rdil[d] + 1 if w.shape[d] > 0 else 0
        wd = np.zeros(wshp, dtype=w.dtype)
        wd[tuple(slice(0, None, rdil[d]) for d in range(nsp)) + (slice(None), slice(None))] = w
        out_shape = op.out_types[0].shape
        osp = [out_shape[os_.index(s)] for s in sp]
        N = x.shape[0]
        Cin = x.shape[-1]
        O = w.shape[-1]
        G = fg * bg
        res = np.zeros([N // bg] + osp + [O], dtype=self.accum)
        # windows as strided view: [N, out..., k..., C]
        for g in range(G):
            if fg > 1:
                cs = Cin // fg
                xg = xp[..., g * cs:(g + 1) * cs]
                wg = wd[..., g * (O // fg):(g + 1) * (O // fg)]
                osl = slice(g * (O // fg), (g + 1) * (O // fg))
            elif bg > 1:
                nb = N // bg
                xg = xp[g * nb:(g + 1) * nb]
                wg = wd[..., g * (O // bg):(g + 1) * (O // bg)]
                osl = slice(g * (O // bg), (g + 1) * (O // bg))
            else:
                xg, wg, osl = xp, wd, slice(None)
            acc = np.zeros([xg.shape[0]] + osp + [wg.shape[-1]], dtype=self.accum)
            # accumulate one kernel tap at a time: a GEMM per tap, no im2col blow-up
            for tap in np.ndindex(*wd.shape[:nsp]):
                wt = wg[tap]
                if not np.any(wt):
                    continue
                sl = [slice(None)]
                for d in range(nsp):
                    sl.append(slice(tap[d], tap[d] + (osp[d] - 1) * strides[d] + 1, strides[d]))
                sl.append(slice(None))
                patch = xg[tuple(sl)]
                acc += np.matmul(patch.reshape(-1, patch.shape[-1]), wt).reshape(acc.shape)
            res[..., osl] = acc
        # to output layout
        cur = ["b"] + sp + ["f"]
        return np.transpose(res, [cur.index(c) for c in os_])

    # ------------------------------------------------------------------
    # gather / scatter (reference: ops/gather_scatter.cc:200-294, 296-699)
    # ------------------------------------------------------------------
    @staticmethod
    def _dn(op, key):
        v = op.attrs[key]
        return v[1] if isinstance(v, tuple) else v

    def op_gather(self, op, ins, env):
        operand, idx = ins
        dn = self._dn(op, "dimension_numbers")
        offset_dims = dn.get("offset_dims", [])
        collapsed = dn.get("collapsed_slice_dims", [])
        obatch = dn.get("operand_batching_dims", [])
        ibatch = dn.get("start_indices_batching_dims", [])
        sim = dn.get("start_index_map", [])
        ivd = dn.get("index_vector_dim", idx.ndim)
        sizes = op.attrs["slice_sizes"]
        out_shape = op.out_types[0].shape
        if ivd == idx.ndim:
            idx = idx[..., None]
        idxm = np.moveaxis(idx, ivd, -1).astype(np.int64)       # [batch..., K]
        batch_dims_out = [d for d in range(len(out_shape)) if d not in offset_dims]
        grids = np.indices(out_shape, sparse=True)
        bidx = tuple(grids[d] for d in batch_dims_out)
        # operand dims that carry an offset
        off_operand_dims = [d for d in range(operand.ndim) if d not in collapsed and d not in obatch]
        index = [0] * operand.ndim
        for d in range(operand.ndim):
            index[d] = np.zeros((), dtype=np.int64)
        for k, d in enumerate(sim):
            start = idxm[bidx + (k,)] if bidx else idxm[..., k].reshape(())
            start = np.clip(start, 0, operand.shape[d] - sizes[d])   # clamp rule gather_scatter.cc:233-239
            index[d] = index[d] + start
        # batching dims: position in the batch index space (index_vector_dim removed)
        idx_batch_axes = [a for a in range(idx.ndim) if a != ivd]
        for od, ib in zip(obatch, ibatch):
            pos = idx_batch_axes.index(ib)
            index[od] = index[od] + grids[batch_dims_out[pos]]
        for k, d in enumerate(off_operand_dims):
            index[d] = index[d] + grids[offset_dims[k]]
        index = np.broadcast_arrays(*index) if operand.ndim else []
        return operand[tuple(index)].reshape(out_shape)

    def op_scatter(self, op, ins, env):
        """Updates are applied in row-major order of the update tensor, one after
        the other (the order XLA's CPU backend uses), so duplicate indices
        accumulate deterministically.  A window that does not fit entirely inside
        the operand is dropped."""
        k = len(ins) // 2 if len(ins) > 3 else 1
        operand, idx, upd = ins[0], ins[-2] if len(ins) == 3 else ins[k], ins[-1]
        assert len(ins) == 3, "variadic scatter not needed on this path"
        dn = self._dn(op, "scatter_dimension_numbers")
        uwd = dn.get("update_window_dims", [])
        iwd = dn.get("inserted_window_dims", [])
        ibd = dn.get("input_batching_dims", [])
        sibd = dn.get("scatter_indices_batching_dims", [])
        sdo = dn.get("scatter_dims_to_operand_dims", [])
        ivd = dn.get("index_vector_dim", idx.ndim)
        if ivd == idx.ndim:
            idx = idx[..., None]
        idxm = np.moveaxis(idx, ivd, -1).astype(np.int64)
        scatter_dims_upd = [d for d in range(upd.ndim) if d not in uwd]
        grids = np.indices(upd.shape, sparse=True)
        bidx = tuple(grids[d] for d in scatter_dims_upd)
        win_operand_dims = [d for d in range(operand.ndim) if d not in iwd and d not in ibd]
        win_sizes = {d: upd.shape[uwd[k_]] for k_, d in enumerate(win_operand_dims)}
        index = [np.zeros((), dtype=np.int64) for _ in range(operand.ndim)]
        inb = np.ones((), dtype=bool)
        for k_, d in enumerate(sdo):
            start = idxm[bidx + (k_,)] if bidx else idxm[..., k_].reshape(())
            ws = win_sizes.get(d, 1)
            inb = inb & (start >= 0) & (start <= operand.shape[d] - ws)
            index[d] = index[d] + start
        idx_batch_axes = [a for a in range(idx.ndim) if a != ivd]
        for od, ib in zip(ibd, sibd):
            pos = idx_batch_axes.index(ib)
            index[od] = index[od] + grids[scatter_dims_upd[pos]]
        for k_, d in enumerate(win_operand_dims):
            index[d] = index[d] + grids[uwd[k_]]
        bc = np.broadcast_arrays(*(index + [inb, np.zeros(upd.shape, dtype=bool)]))
        index, inb = bc[:-2], bc[-2]
        flat = np.ravel_multi_index([i.reshape(-1) for i in index], operand.shape, mode="clip") if operand.ndim else np.zeros(upd.size, np.int64)
        inb = inb.reshape(-1)
        flat = flat[inb]
        u = upd.reshape(-1)[inb]
        out = operand.copy().reshape(-1)
        body = op.regions[0]
        kind = None
        if len(body.ops) == 1 and body.ops[0].name == "return" and body.ops[0].operands == [body.args[1]]:
            kind = "set"
        elif len(body.ops) == 2 and set(body.ops[0].operands) == set(body.args):
            kind = body.ops[0].name.replace("stablehlo.", "")
            if kind == "subtract" and body.ops[0].operands != body.args:
                kind = None
        stepwise = {"add": np.add, "subtract": np.subtract, "multiply": np.multiply}
        with np.errstate(all="ignore"):
            if op.out_types[0].dtype == "bf16" and kind in stepwise and self.round_intermediates:
                # The body works on bf16 scalars: every application rounds.  Updates are applied in order; round r
                # applies the r-th update of every element at once (an element occurs at most once per round).
                order = np.argsort(flat, kind="stable")
                sf = flat[order]
                first = np.r_[True, sf[1:] != sf[:-1]] if sf.size else np.zeros(0, bool)
                start = np.maximum.accumulate(np.where(first, np.arange(sf.size), 0)) if sf.size else sf
                occurrence = np.empty(sf.size, np.int64)
                occurrence[order] = np.arange(sf.size) - start
                for r in range(int(occurrence.max()) + 1 if sf.size else 0):
                    sel = occurrence == r
                    out[flat[sel]] = round_bf16(stepwise[kind](out[flat[sel]], u[sel]).astype(np.float32))
            elif kind == "set":
                out[flat] = u
            elif kind == "add":
                if out.dtype == np.bool_:
                    np.logical_or.at(out, flat, u)
                else:
                    np.add.at(out, flat, u)
            elif kind == "subtract":
                np.subtract.at(out, flat, u)
            elif kind == "multiply":
                np.multiply.at(out, flat, u)
            elif kind == "minimum":
                np.minimum.at(out, flat, u)
            elif kind == "maximum":
                np.maximum.at(out, flat, u)
            else:
                t = op.out_types[0]
                st = TType((), t.dtype)
                for j in range(flat.size):
                    r = self._run_region(body, [np.asarray(out[flat[j]]), np.asarray(u[j])], env)[0]
                    out[flat[j]] = _cast_result(r, st)
        return out.reshape(operand.shape)

    # ------------------------------------------------------------------
    # control flow (reference: ops/control_flow.cc:702-989, 992-1277)
    # ------------------------------------------------------------------
    def op_while(self, op, ins, env):
        cond, body = op.regions
        state = list(ins)
        while bool(np.asarray(self._run_region(cond, state, env)[0]).reshape(())):
            state = [_cast_result(v, t) for v, t in zip(self._run_region(body, state, env), op.out_types)]
        return state

    def op_case(self, op, ins, env):
        """Out-of-range index selects the last branch (control_flow.cc:672-675)."""
        i = int(np.asarray(ins[0]).reshape(()))
        nb = len(op.regions)
        if i < 0 or i >= nb:
            i = nb - 1
        return self._run_region(op.regions[i], [], env)

    def op_call(self, op, ins, env):
        f = self.funcs[op.attrs["callee"]]
        return self._run_region(f.body, ins, {})

    def op_composite(self, op, ins, env):
        """stablehlo.composite runs its decomposition function (reference: ops/control_flow.cc:2242-2262)."""
        f = self.funcs[str(op.attrs["decomposition"]).lstrip("@")]
        return self._run_region(f.body, ins, {})

    def op_optimization_barrier(self, op, ins, env): return list(ins)

    # -- one device only: collectives pass through, ids are zero, tokens are scalar placeholders
    def _module_count(self, key):
        v = self.module_attributes.get(key, 1)
        if isinstance(v, tuple):
            v = v[0]
        return int(np.asarray(v).reshape(-1)[0])

    def op_all_reduce(self, op, ins, env):
        """stablehlo.all_reduce over one device forwards its operands; a replica group with more than one member
        is an error (reference: src/pjrt_plugin/ops/collectives.cc:20-48: the last dimension of a rank-2
        `replica_groups`, else its element count, decides)."""
        groups = op.attrs.get("replica_groups")
        if groups is not None:
            g = np.asarray(groups[0] if isinstance(groups, tuple) else groups)
            if g.size and (g.shape[-1] if g.ndim >= 2 else g.size) > 1:
                raise ValueError("stablehlo.all_reduce: multi-device all_reduce is not supported")
        if len(ins) != len(op.results):
            raise ValueError("stablehlo.all_reduce: operand/result count mismatch")
        return list(ins)

    def op_partition_id(self, op, ins, env):
        """Zero, of the result's integer type, when the module declares one partition (reference:
        src/pjrt_plugin/ops/collectives.cc:56-79)."""
        if self._module_count("mhlo.num_partitions") != 1:
            raise ValueError("stablehlo.partition_id: multi-partition execution is not supported")
        t = op.out_types[0]
        if t.shape != ():
            raise ValueError("stablehlo.partition_id: result must be a scalar tensor")
        return np.zeros((), dtype=_NP[t.dtype])

    def op_replica_id(self, op, ins, env):
        """The replica counterpart of partition_id (the reference registers no handler for it)."""
        if self._module_count("mhlo.num_replicas") != 1:
            raise ValueError("stablehlo.replica_id: multi-replica execution is not supported")
        t = op.out_types[0]
        if t.shape != ():
            raise ValueError("stablehlo.replica_id: result must be a scalar tensor")
        return np.zeros((), dtype=_NP[t.dtype])

    def op_create_token(self, op, ins, env):
        """A token carries no data; it is the f32 scalar 0 wherever a value must stand for it, also as an argument
        or result of main (reference: src/pjrt_plugin/ops/control_flow.cc:2266-2288)."""
        return np.float32(0.0).reshape(())

    def op_after_all(self, op, ins, env):
        """A fresh placeholder; the operand tokens are ignored (reference: ops/control_flow.cc:2283-2288)."""
        return np.float32(0.0).reshape(())

    def op_sort(self, op, ins, env):
        """stablehlo.sort: the comparator region decides, ties keep their order (the reference sorts by the first
        operand with a direction read off the comparator, src/pjrt_plugin/ops/sort_fft_complex.cc:145-216; for the
        comparators JAX emits both agree).  Evaluated without a sorting routine: the comparator is run on all pairs
        of a slice at once, and element i lands at (number of j before i) where j is before i if cmp(j, i), or
        neither cmp(j, i) nor cmp(i, j) and j < i."""
        dim = int(op.attrs["dimension"])
        xs = [np.asarray(x) for x in ins]
        if xs[0].ndim == 0:
            return [x.copy() for x in xs]
        if dim < 0:
            dim += xs[0].ndim
        moved = [np.moveaxis(x, dim, -1) for x in xs]
        L = moved[0].shape[-1]
        lead = moved[0].shape[:-1]
        flat = [m.reshape(-1, L) for m in moved]
        outs = [np.empty_like(f) for f in flat]
        body = op.regions[0]
        idx = np.arange(L)
        step = max(1, min(L, (1 << 23) // max(L, 1)))      # rows of the all-pairs table evaluated at once
        for r in range(flat[0].shape[0]):
            pos = np.empty(L, dtype=np.int64)
            for i0 in range(0, L, step):
                i1 = min(L, i0 + step)
                fwd, rev = [], []
                for f in flat:
                    xi = np.broadcast_to(f[r][i0:i1, None], (i1 - i0, L))
                    xj = np.broadcast_to(f[r][None, :], (i1 - i0, L))
                    fwd += [xi, xj]
                    rev += [xj, xi]
                lt_ij = np.asarray(self._run_region(body, fwd, env, vectorized=True)[0]).astype(bool)   # cmp(x_i, x_j)
                lt_ji = np.asarray(self._run_region(body, rev, env, vectorized=True)[0]).astype(bool)   # cmp(x_j, x_i)
                before = lt_ji | (~lt_ij & ~lt_ji & (idx[None, :] < idx[i0:i1, None]))                   # j sorts before i
                pos[i0:i1] = before.sum(axis=1)
            perm = np.empty(L, dtype=np.int64)
            perm[pos] = idx
            for f, o in zip(flat, outs):
                o[r] = f[r][perm]
        return [np.moveaxis(o.reshape(lead + (L,)), -1, dim) for o in outs]

    def op_chlo_top_k(self, op, ins, env):
        """Largest k along the last dim, equal values in ascending position (reference: TopKImplFn,
        src/pjrt_plugin/ops/sort_fft_complex.cc:40-82); floats in total order (NaN above +inf, -0.0 below +0.0).
        Selection by counting: element i has rank #{j: x_j > x_i} + #{j < i: x_j == x_i}."""
        x = np.asarray(ins[0])
        k = int(op.attrs["k"])
        key = _total_order_key(x) if x.dtype.kind == "f" else x
        a, b = key[..., :, None], key[..., None, :]
        L = x.shape[-1]
        idx = np.arange(L)
        rank = (b > a).sum(-1) + ((b == a) & (idx[None, :] < idx[:, None])).sum(-1)
        order = np.empty(x.shape, dtype=np.int64)
        np.put_along_axis(order, rank, np.broadcast_to(idx, x.shape), axis=-1)
        order = order[..., :k]
        return [np.take_along_axis(x, order, -1), order.astype(_NP[op.out_types[1].dtype])]

    def op_rng_bit_generator(self, op, ins, env):
        """State rule of the reference (src/pjrt_plugin/ops/control_flow.cc:2301-2360): state = [key, counter, ...] as
        ui64, the counter grows by ceil(output bytes / 16).  The bits themselves are implementation-defined (the
        reference takes MLX's); this build defines element i as threefry2x32(key halves; (i, low half of the counter)),
        word 0 for types up to 32 bits (truncated), both words for 64-bit types.  PARITY UNPINNED for the bit values."""
        state = np.asarray(ins[0], dtype=np.uint64)
        t = op.out_types[1]
        n = int(np.prod(t.shape, dtype=np.int64))
        dt = _NP[t.dtype]
        esz = np.dtype(dt).itemsize
        new_state = state.copy()
        new_state[1] = np.uint64((int(state[1]) + (n * esz + 15) // 16) & ((1 << 64) - 1))
        k0 = np.uint32(int(state[0]) & 0xFFFFFFFF)
        k1 = np.uint32(int(state[0]) >> 32)
        c0 = np.arange(n, dtype=np.uint32)
        c1 = np.full(n, int(state[1]) & 0xFFFFFFFF, dtype=np.uint32)
        x0, x1 = threefry2x32(k0, k1, c0, c1)
        if esz == 8:
            bits = (x0.astype(np.uint64) | (x1.astype(np.uint64) << np.uint64(32))).view(dt)
        elif esz == 4:
            bits = x0.view(dt)
        else:
            bits = x0.astype(np.dtype("u%d" % esz)).view(dt)
        return [new_state, bits.reshape(t.shape)]

    def op_custom_call(self, op, ins, env):
        tgt = op.attrs.get("call_target_name")
        if tgt in ("Sharding", "SPMDFullToShardShape", "SPMDShardToFullShape"):
            return ins[0]
        if tgt == "mhlo.topk":      # the older spelling of chlo.top_k (reference: ops/control_flow.cc:1461-1477)
            op.attrs["k"] = op.out_types[0].shape[-1]
            return self.op_chlo_top_k(op, ins, env)
        if isinstance(tgt, str) and tgt.startswith("mhlo.") and hasattr(self, "op_chlo_" + tgt[5:]) and len(ins) == 1:
            return getattr(self, "op_chlo_" + tgt[5:])(op, ins, env)
        if isinstance(tgt, str) and tgt.split(".", 1)[0] in ("mps", "mi355x"):
            fn = getattr(self, "fused_" + tgt.split(".", 1)[1], None)
            if fn is not None:
                import json
                cfg = op.attrs.get("backend_config") or ""
                cfg = json.loads(cfg) if isinstance(cfg, str) and cfg.strip() else {}
                outs = fn([np.asarray(a) for a in ins], cfg)
                return [np.asarray(o, dtype=np.float64) for o in outs]      # rounded once to the declared type by the caller
        raise NotImplementedError(f"oracle: custom_call {tgt}")

    # ------------------------------------------------------------------
    # fused-op custom calls of the reference's Python layer (src/jax_plugins/mps/ops.py:52-596; executor side
    # src/pjrt_plugin/ops/control_flow.cc:1484-2020), evaluated in float64 from the operands as given
    # ------------------------------------------------------------------
    @staticmethod
    def _sdpa_probabilities(q, k, v, mask, causal, scale):
        """softmax(scale q k^T [masked]) with key / value heads repeated to the query heads (ops.py:63-76, 99-107)."""
        q, k, v = (a.astype(np.float64) for a in (q, k, v))
        groups = q.shape[1] // k.shape[1]
        k, v = np.repeat(k, groups, axis=1), np.repeat(v, groups, axis=1)
        s = np.einsum("bnth,bnsh->bnts", q, k) * scale
        lowest = float(np.finfo(np.float32).min)
        if causal:
            T, S = q.shape[2], k.shape[2]
            visible = np.arange(S)[None, :] <= np.arange(T)[:, None] + (S - T)
            s = np.where(visible[None, None], s, lowest)
        elif mask is not None:
            if mask.dtype == np.bool_:
                s = np.where(np.broadcast_to(mask, s.shape), s, lowest)
            else:
                s = s + mask.astype(np.float64)
        e = np.exp(s - s.max(-1, keepdims=True))
        return q, k, v, e / e.sum(-1, keepdims=True), groups

    def fused_sdpa(self, ins, cfg, causal=False):
        q, k, v = ins[:3]
        _, _, v64, p, _ = self._sdpa_probabilities(q, k, v, None if causal else ins[3], causal, float(cfg.get("scale", 1.0)))
        return [np.einsum("bnts,bnsh->bnth", p, v64)]

    def fused_sdpa_causal(self, ins, cfg):
        return self.fused_sdpa(ins, cfg, causal=True)

    def fused_sdpa_bwd(self, ins, cfg, causal=False):
        q, k, v = ins[:3]
        g = ins[-1].astype(np.float64)
        scale = float(cfg.get("scale", 1.0))
        q64, k64, v64, p, groups = self._sdpa_probabilities(q, k, v, None if causal else ins[3], causal, scale)
        dv = np.einsum("bnts,bnth->bnsh", p, g)
        dp = np.einsum("bnth,bnsh->bnts", g, v64)
        ds = p * (dp - (dp * p).sum(-1, keepdims=True)) * scale
        dq = np.einsum("bnts,bnsh->bnth", ds, k64)
        dk = np.einsum("bnts,bnth->bnsh", ds, q64)
        if groups > 1:
            B, N, S, H = dk.shape
            dk = dk.reshape(B, N // groups, groups, S, H).sum(2)
            dv = dv.reshape(B, N // groups, groups, S, H).sum(2)
        return [dq, dk, dv]

    def fused_sdpa_causal_bwd(self, ins, cfg):
        return self.fused_sdpa_bwd(ins, cfg, causal=True)

    def fused_rms_norm(self, ins, cfg):
        x, w = (a.astype(np.float64) for a in ins)
        return [x / np.sqrt((x * x).mean(-1, keepdims=True) + float(cfg.get("eps", 1e-6))) * w]

    def fused_rms_norm_bwd(self, ins, cfg):
        x, w, g = (a.astype(np.float64) for a in ins)
        r = 1.0 / np.sqrt((x * x).mean(-1, keepdims=True) + float(cfg.get("eps", 1e-6)))
        xn, gw = x * r, g * w
        dx = r * (gw - xn * (gw * xn).mean(-1, keepdims=True))
        return [dx, (g * xn).reshape(-1, x.shape[-1]).sum(0)]

    def fused_layer_norm(self, ins, cfg):
        x, w, b = (a.astype(np.float64) for a in ins)
        d = x - x.mean(-1, keepdims=True)
        return [d / np.sqrt((d * d).mean(-1, keepdims=True) + float(cfg.get("eps", 1e-5))) * w + b]

    def fused_layer_norm_bwd(self, ins, cfg):
        x, w, b, g = (a.astype(np.float64) for a in ins)
        d = x - x.mean(-1, keepdims=True)
        r = 1.0 / np.sqrt((d * d).mean(-1, keepdims=True) + float(cfg.get("eps", 1e-5)))
        xn, gw = d * r, g * w
        dx = r * (gw - gw.mean(-1, keepdims=True) - xn * (gw * xn).mean(-1, keepdims=True))
        return [dx, (g * xn).reshape(-1, x.shape[-1]).sum(0), g.reshape(-1, x.shape[-1]).sum(0)]

    @staticmethod
    def _rope(x, offset, cfg, inverse):
        """Rotation of the first `dims` features of (..., T, D) by (position + offset) * rope_scale * base^(-2i/dims):
        halves (x[i], x[i + dims/2]) as in ops.py:418-438, or neighbouring pairs when "traditional"."""
        x = x.astype(np.float64)
        D, T = x.shape[-1], x.shape[-2]
        dims = int(cfg.get("dims", D))
        half = dims // 2
        pos = (np.arange(T, dtype=np.float64) + float(np.asarray(offset).reshape(()))) * float(cfg.get("rope_scale", 1.0))
        ang = pos[:, None] * float(cfg.get("base", 10000.0)) ** (-2.0 * np.arange(half) / dims)[None, :]
        c, s = np.cos(ang), np.sin(ang) * (-1.0 if inverse else 1.0)
        out = x.copy()
        if cfg.get("traditional", False):
            a, b = x[..., 0:dims:2], x[..., 1:dims:2]
            out[..., 0:dims:2], out[..., 1:dims:2] = a * c - b * s, b * c + a * s
        else:
            a, b = x[..., :half], x[..., half:dims]
            out[..., :half], out[..., half:dims] = a * c - b * s, b * c + a * s
        return out

    def fused_rope(self, ins, cfg):
        return [self._rope(ins[0], ins[1], cfg, False)]

    def fused_rope_bwd(self, ins, cfg):
        return [self._rope(ins[2], ins[1], cfg, True)]

    def fused_gelu(self, ins, cfg):
        x = ins[0].astype(np.float64)
        return [0.5 * x * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))]

    def fused_gelu_bwd(self, ins, cfg):
        x, g = (a.astype(np.float64) for a in ins)
        c0, c1 = math.sqrt(2.0 / math.pi), 0.044715
        th = np.tanh(c0 * (x + c1 * x ** 3))
        return [g * (0.5 * (1.0 + th) + 0.5 * x * (1.0 - th * th) * c0 * (1.0 + 3.0 * c1 * x * x))]


def _total_order_key(x):
    """Signed integer key whose order is the IEEE total order of the floats (sign-magnitude bits made monotonic)."""
    x = np.asarray(x)
    bits = {2: np.int16, 4: np.int32, 8: np.int64}[x.dtype.itemsize]
    i = x.view(bits).astype(np.int64)
    top = np.int64(1) << (8 * x.dtype.itemsize - 1)
    return np.where(i < 0, -(i + top) - 1, i)


def threefry2x32(k0, k1, c0, c1):
    """Threefry-2x32 with 20 rounds (Salmon et al., Random123), on uint32 arrays; checked against the published
    known-answer vectors in tests/test_oracle_pins.py."""
    with np.errstate(over="ignore"):
        k0 = np.asarray(k0, np.uint32); k1 = np.asarray(k1, np.uint32)
        x0 = np.asarray(c0, np.uint32).copy(); x1 = np.asarray(c1, np.uint32).copy()
        ks = [k0, k1, k0 ^ k1 ^ np.uint32(0x1BD11BDA)]
        rotl = lambda x, r: (x << np.uint32(r)) | (x >> np.uint32(32 - r))
        x0 = x0 + ks[0]
        x1 = x1 + ks[1]
        rots = [(13, 15, 26, 6), (17, 29, 16, 24)]
        for blk in range(5):
            for r in rots[blk % 2]:
                x0 = x0 + x1
                x1 = rotl(x1, r) ^ x0
            x0 = x0 + ks[(blk + 1) % 3]
            x1 = x1 + ks[(blk + 2) % 3] + np.uint32(blk + 1)
        return x0, x1


def run_text(text: str, *args, accum="f64"):
    return Oracle(text, accum=accum).run(*args)
