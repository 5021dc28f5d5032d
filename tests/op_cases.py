"""Per-op parity cases: small StableHLO modules with seeded inputs.

The shapes and edge cases restate the reference's own per-op configs
(tests/configs/{unary,binary,conversion,shape,slice,matmul,conv,reduction,control_flow}.py):
each case is one module that goes through PJRT_Client_Compile / Execute and is
compared with the CPU oracle on the same inputs (bit-exact for integer, boolean
and data-movement results; 1e-5 relative for f32; 2e-2 for bf16).
"""
from __future__ import annotations

import sys
from dataclasses import dataclass
from pathlib import Path
from typing import Callable, List

import numpy as np

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

from jax_mps_amd.shlo.builder import Builder, Val, _NP  # noqa: E402

_MLIR = {np.dtype(v): k for k, v in _NP.items()}


@dataclass
class Case:
    name: str
    text: str
    inputs: List[np.ndarray]
    dtypes: List[str]
    exact: bool = False


_cases: List[Callable[[], Case]] = []


def case(name, fn, *inputs, dtypes=None, exact=False):
    def make():
        b = Builder("jit_" + name.replace("-", "_").replace(".", "_"))
        dts = list(dtypes) if dtypes else [_MLIR[np.asarray(a).dtype] for a in inputs]
        args = [b.arg(np.asarray(a).shape, d) for a, d in zip(inputs, dts)]
        out = fn(b, *args)
        if isinstance(out, Val):
            out = [out]
        b.ret(*out)
        return Case(name, b.text(), [np.asarray(a) for a in inputs], dts, exact)
    make.case_name = name
    _cases.append(make)

def text_case(name, text, *inputs, dtypes=None, exact=False):
    """A program given as StableHLO text (for forms the builder does not write)."""
    def make():
        dts = list(dtypes) if dtypes else [_MLIR[np.asarray(a).dtype] for a in inputs]
        return Case(name, text, [np.asarray(a) for a in inputs], dts, exact)
    make.case_name = name
    _cases.append(make)


def rng(seed):
    return np.random.default_rng(seed)


def f32(seed, *shape, lo=-2.0, hi=2.0):
    return rng(seed).uniform(lo, hi, size=shape).astype(np.float32)


def i32(seed, *shape, lo=-50, hi=50):
    return rng(seed).integers(lo, hi, size=shape).astype(np.int32)


# ------------------------------------------------------------------ unary (tests/configs/unary.py)
for k, (op, lo, hi) in enumerate([
        ("exp", -4, 4), ("log", 0.1, 9), ("sqrt", 0, 9), ("rsqrt", 0.1, 9), ("tanh", -4, 4), ("logistic", -6, 6),
        ("abs", -3, 3), ("neg", -3, 3), ("sign", -3, 3), ("floor", -3, 3)]):
    case("unary-" + op, (lambda o: lambda b, x: getattr(b, o)(x))(op), f32(k, 7, 33, lo=lo, hi=hi))
for k, op in enumerate(["sine", "cosine", "ceil", "log_plus_one", "exponential_minus_one", "round_nearest_even",
                        "round_nearest_afz", "cbrt", "tan"]):
    case("unary-" + op, (lambda o: lambda b, x: b._unary(o, x))(op), f32(20 + k, 5, 17, lo=-1.2 if op != "log_plus_one" else -0.5, hi=1.2))
case("unary-specials", lambda b, x: [b.exp(x), b.sign(x), b.abs(x), b._unary("is_finite", x), b.neg(x)],
     np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-40, -3.5, 88.0], np.float32))
case("round-half", lambda b, x: [b._unary("round_nearest_even", x), b._unary("round_nearest_afz", x)],
     np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.49, -3.51], np.float32), exact=True)
# where |x| + 0.5 is not a number of the type the reference's formula rounds the sum first (ops/arithmetic.cc:316-327)
_AFZ = [0.49999997, -0.49999997, 0.5, 8388609.0, -8404769.0, 12606725.0, 16777215.0, 8388608.0, 4194303.5, -4194304.5, 1e-45, np.inf, -np.inf, np.nan, -0.0, 3e38]
case("round-half-away-where-the-sum-rounds", lambda b, x: b._unary("round_nearest_afz", x), np.array(_AFZ, np.float32), exact=True)
case("round-half-away-where-the-sum-rounds-bf16", lambda b, x: b._unary("round_nearest_afz", x),
     np.array([0.498046875, -0.498046875, 0.5, 129.0, -131.0, 255.0, 127.5, 64.5, -2.5, 1.0, 256.0, 3e38], np.float32), dtypes=["bf16"], exact=True)
case("round-half-away-where-the-sum-rounds-f16", lambda b, x: b._unary("round_nearest_afz", x),
     np.array([0.49975586, -0.49975586, 0.5, 1025.0, -1027.0, 2047.0, 1023.5, 512.5, -2.5, 65504.0], np.float16), exact=True)
# a product narrowed to f16 is rounded to f32 first and keeps the sign of a zero
case("convert-f16-of-a-product", lambda b, x, y: [b.convert(b.convert(b.mul(x, y), "f16"), "f32"), b.div(1.0, b.convert(b.convert(b.mul(b.abs(x), x), "f16"), "f32"))],
     np.array([-0.0, 0.0, 1.0009766, 3.0, -1e-5, 1e-30, 255.9, -0.0], np.float32), np.array([0.0, -0.0, 1.0009766, 0.33333334, 1e-4, -1e-30, 255.9, -5.0], np.float32), exact=True)
# tanh of a 16-bit float near zero is the argument itself, not the cancelled difference of two exponentials
case("tanh-bf16-near-zero", lambda b, x: b.tanh(x), np.array([1e-8, -1e-8, 3e-5, -2e-4, 1e-3, 0.05, 0.0996, 0.1004, -0.3, 1e-19, 0.0, 2.5], np.float32), dtypes=["bf16"])
case("tanh-f16-near-zero", lambda b, x: b.tanh(x), np.array([6e-8, -6e-8, 3e-5, -2e-4, 1e-3, 0.05, 0.0996, 0.1004, -0.3, 0.0, 2.5], np.float16))
# of two zeros of different sign maximum and minimum return the second operand (x > y ? x : y after the NaN test)
case("maximum-minimum-of-signed-zeros", lambda b, x, y: [b.div(1.0, b.maximum(x, y)), b.div(1.0, b.minimum(x, y))],
     np.array([0.0, -0.0, 0.0, -0.0, np.nan, 1.0, -0.0], np.float32), np.array([-0.0, 0.0, 0.0, -0.0, -0.0, np.nan, 1e-45], np.float32), exact=True)

# ------------------------------------------------------------------ binary (tests/configs/binary.py)
for k, op in enumerate(["add", "sub", "mul", "div", "maximum", "minimum"]):
    case("binary-" + op, (lambda o: lambda b, x, y: getattr(b, o)(x, y))(op), f32(40 + k, 9, 20), f32(60 + k, 9, 20, lo=0.5, hi=3))
case("binary-power", lambda b, x, y: b.power(x, y), f32(70, 6, 11, lo=0.2, hi=3), f32(71, 6, 11))
case("binary-remainder-float", lambda b, x, y: b.remainder(x, y), f32(72, 6, 11, lo=-9, hi=9), f32(73, 6, 11, lo=0.5, hi=3))
case("binary-atan2", lambda b, x, y: b._binary("atan2", x, y), f32(74, 6, 11), f32(75, 6, 11))
case("binary-broadcast-scalar", lambda b, x, y: b.add(b.mul(x, 2.5), b.broadcast_in_dim(y, x.shape, [])), f32(76, 3, 5, 8), f32(77))
case("binary-nan-propagation", lambda b, x, y: [b.maximum(x, y), b.minimum(x, y)],
     np.array([1.0, np.nan, 3.0, np.nan, -0.0, 0.0], np.float32), np.array([np.nan, 2.0, -np.inf, np.nan, 0.0, -0.0], np.float32))
# integer semantics (arithmetic.cc:46-83, 496-513; mlx_executable.cc:293-301)
case("int-arith", lambda b, x, y: [b.add(x, y), b.sub(x, y), b.mul(x, y), b.maximum(x, y), b.minimum(x, y)], i32(80, 6, 9), i32(81, 6, 9), exact=True)
case("int-div-rem", lambda b, x, y: [b.div(x, y), b.remainder(x, y)],
     np.array([7, -7, 7, -7, 0, 5, -5, 2147483647, -2147483648], np.int32), np.array([2, 2, -2, -2, 3, 0, 0, -1, 1], np.int32), exact=True)
case("int-bitwise", lambda b, x, y: [b.and_(x, y), b.or_(x, y), b.xor(x, y), b.not_(x)], i32(82, 33, lo=-2**31, hi=2**31 - 1), i32(83, 33, lo=-2**31, hi=2**31 - 1), exact=True)
case("int-shifts", lambda b, x, s: [b.shift_left(x, s), b.shift_right_logical(x, s), b._binary("shift_right_arithmetic", x, s)],
     np.array([1, -1, 12345, -12345, 2**30, -2**31, 7, 7], np.int32), np.array([0, 1, 31, 4, 32, 33, -1, 100], np.int32), exact=True)
case("uint-shifts", lambda b, x, s: [b.shift_left(x, s), b.shift_right_logical(x, s)],
     np.array([1, 0xFFFFFFFF, 12345, 2**31], np.uint32), np.array([31, 32, 4, 40], np.uint32), exact=True)
case("int-popcnt-clz", lambda b, x: [b._unary("popcnt", x), b._unary("count_leading_zeros", x)],
     np.array([0, 1, -1, 255, 2**30, -2**31, 16777217], np.int32), exact=True)
case("int-power", lambda b, x, y: b.power(x, y), np.array([2, 3, -2, 1, -1, 5, 0], np.int32), np.array([10, 4, 3, -5, -3, -1, 0], np.int32), exact=True)
case("bool-logic", lambda b, x, y: [b.and_(x, y), b.or_(x, y), b.xor(x, y), b.not_(x)],
     np.array([True, True, False, False]), np.array([True, False, True, False]), exact=True)

# ------------------------------------------------------------------ compare / select / clamp
for d in ["EQ", "NE", "LT", "LE", "GT", "GE"]:
    case("compare-f32-" + d, (lambda dd: lambda b, x, y: b.compare(x, y, dd))(d),
         np.array([1.0, 2.0, 2.0, np.nan, -0.0, np.inf], np.float32), np.array([2.0, 2.0, 1.0, 1.0, 0.0, np.inf], np.float32), exact=True)
case("compare-i32", lambda b, x, y: [b.compare(x, y, "LT"), b.compare(x, y, "GE")], i32(90, 40, lo=-3, hi=3), i32(91, 40, lo=-3, hi=3), exact=True)
# integer arithmetic wraps, for signed types too, and nothing downstream may be simplified as if it could not: the square of
# a 32-bit number can be negative, x - y can exceed x, x + 1 can be below x
_I32_WIDE = np.array([1790545064, -1206374848, 46341, -46341, 2**31 - 1, -2**31, 65536, 3, 0, -1], np.int32)
_I64_WIDE = np.array([-6927189342267442211, 2**63 - 1, -2**63, 5, -5, 2**62, -2**62 - 1, 0], np.int64)
case("signed-overflow-square-then-remainder", lambda b, x: b.remainder(b.mul(x, x), b.or_(x, 1)), _I32_WIDE, exact=True)
case("signed-overflow-difference-then-compare", lambda b, x, y: b.compare(x, b.sub(x, y), "GE"), _I64_WIDE, _I64_WIDE[::-1].copy(), exact=True)
case("signed-overflow-increment-then-compare", lambda b, x: [b.compare(b.add(x, 1), x, "GT"), b.compare(b.sub(x, 1), x, "LT")], _I32_WIDE, exact=True)
case("signed-overflow-negate-abs-most-negative", lambda b, x: [b.neg(x), b.abs(x), b.div(b.abs(x), 3)], _I32_WIDE, exact=True)
case("signed-overflow-sum-reduction", lambda b, x: [b.compare(b.reduce_sum(x, [0]), 0, "LT"), b.reduce_sum(x, [0])],
     np.array([[2**31 - 1, 2**30, 5], [1, 2**30, -5], [0, 1, 0]], np.int32), exact=True)
case("divide-i64-most-negative", lambda b, x, y: [b.div(x, y), b.remainder(x, y)], np.array([-2**63, -2**63, -2**63, -2**63 + 1, 2**63 - 1, -2**63], np.int64),
     np.array([-2**63 + 1, -1, 2**62 - 1, -1, -2**63, 0], np.int64), exact=True)
# an unsigned divisor of all ones is an ordinary number (the same bits mean -1 for a signed type, the one divisor that overflows)
case("divide-unsigned-by-all-ones-u8", lambda b, x, y: [b.div(x, y), b.remainder(x, y)], np.array([251, 1, 255, 0, 254, 7], np.uint8), np.array([255, 255, 255, 255, 255, 0], np.uint8), exact=True)
case("divide-unsigned-by-all-ones-u32", lambda b, x, y: [b.div(x, y), b.remainder(x, y)], np.array([4197786975, 2**32 - 1, 0, 2**32 - 2], np.uint32), np.array([2**32 - 1] * 4, np.uint32), exact=True)
case("divide-unsigned-by-all-ones-u64", lambda b, x, y: [b.div(x, y), b.remainder(x, y)], np.array([2**64 - 1, 2**64 - 5, 12, 2**63], np.uint64), np.array([2**64 - 1, 2**64 - 1, 2**64 - 1, 3], np.uint64), exact=True)
case("compare-u32", lambda b, x, y: b.compare(x, y, "LT"), np.array([1, 0xFFFFFFFF, 5], np.uint32), np.array([0xFFFFFFFF, 1, 5], np.uint32), exact=True)
case("compare-totalorder", lambda b, x, y: b.compare(x, y, "LT", "TOTALORDER"),
     np.array([-0.0, 0.0, 1.0, -np.inf, -1.0], np.float32), np.array([0.0, -0.0, 2.0, np.inf, -2.0], np.float32), exact=True)
case("select", lambda b, p, x, y: b.select(p, x, y), rng(92).integers(0, 2, size=(5, 12)).astype(bool), f32(93, 5, 12), f32(94, 5, 12), exact=True)
case("select-scalar-pred", lambda b, p, x, y: b.select(b.broadcast_in_dim(p, x.shape, []), x, y), np.array(True), f32(95, 4, 4), f32(96, 4, 4), exact=True)
case("clamp", lambda b, x: b.clamp(-0.5, x, 0.75), f32(97, 6, 10), exact=True)
case("clamp-int", lambda b, x: b.clamp(-3, x, 4), i32(98, 30), exact=True)

# ------------------------------------------------------------------ conversions (tests/configs/conversion.py)
case("convert-f32-i32", lambda b, x: b.convert(x, "i32"),
     np.array([0.9, -0.9, 1.5, -1.5, 3e9, -3e9, np.nan, np.inf, -np.inf, 2147483520.0], np.float32), exact=True)
case("convert-f32-u8", lambda b, x: b.convert(x, "ui8"), np.array([0.9, -5.0, 255.9, 300.0, np.nan], np.float32), exact=True)
case("convert-i32-f32", lambda b, x: b.convert(x, "f32"), np.array([0, 1, -1, 16777217, 2**31 - 1, -2**31], np.int32), exact=True)
case("convert-f32-bf16-f32", lambda b, x: b.convert(b.convert(x, "bf16"), "f32"), f32(100, 9, 16, lo=-100, hi=100), exact=True)
case("convert-f32-f16", lambda b, x: b.convert(b.convert(x, "f16"), "f32"), f32(101, 33, lo=-100, hi=100), exact=True)
case("convert-bool", lambda b, x: [b.convert(x, "i1"), b.convert(b.convert(x, "i1"), "f32")], np.array([0.0, 1.0, -2.0, np.nan, 0.5], np.float32), exact=True)
case("convert-i64-i32", lambda b, x: b.convert(x, "i32"), np.array([2**40 + 5, -1, 2**31], np.int64), exact=True)
case("bitcast-f32-i32", lambda b, x: b.bitcast_convert(x, "i32"), np.array([1.0, -0.0, np.inf, 1e-40], np.float32), exact=True)
case("bitcast-i32-f32", lambda b, x: b.bitcast_convert(x, "f32"), np.array([0x3F800000, 0x7F800000, 1], np.int32), exact=True)

# ------------------------------------------------------------------ shape ops (tests/configs/shape.py)
case("broadcast_in_dim", lambda b, x: b.broadcast_in_dim(x, (4, 3, 5), [1]), f32(110, 3), exact=True)
case("broadcast-expand-unit", lambda b, x: b.broadcast_in_dim(x, (4, 3, 5), [0, 1, 2]), f32(111, 4, 1, 5), exact=True)
case("reshape", lambda b, x: b.reshape(x, (6, 20)), f32(112, 3, 8, 5), exact=True)
case("reshape-after-transpose", lambda b, x: b.reshape(b.transpose(x, [1, 0, 2]), (8, 15)), f32(113, 3, 8, 5), exact=True)
case("transpose-2d", lambda b, x: b.transpose(x, [1, 0]), f32(114, 37, 65), exact=True)
case("transpose-4d", lambda b, x: b.transpose(x, [0, 2, 1, 3]), f32(115, 2, 5, 3, 8), exact=True)
case("reverse", lambda b, x: b.reverse(x, [0, 2]), f32(116, 3, 4, 5), exact=True)
case("concatenate", lambda b, x, y, z: b.concatenate([x, y, z], 1), f32(117, 3, 2), f32(118, 3, 5), f32(119, 3, 1), exact=True)
case("concatenate-dim0", lambda b, x, y: b.concatenate([x, y], 0), f32(120, 3, 8), f32(121, 5, 8), exact=True)
case("iota", lambda b, x: b.add(x, b.convert(b.iota((4, 6), 1), "f32")), f32(122, 4, 6), exact=True)
case("slice", lambda b, x: b.slice(x, [1, 0, 2], [3, 4, 8], [1, 2, 3]), f32(123, 4, 4, 9), exact=True)
case("pad", lambda b, x: b.pad(x, -1.0, [1, 0], [2, 3], [0, 1]), f32(124, 3, 4), exact=True)
case("pad-negative", lambda b, x: b.pad(x, 0.5, [-1, 2], [1, -2], [0, 0]), f32(125, 4, 6), exact=True)
case("pad-interior-negative", lambda b, x: b.pad(x, 9.0, [-1, 0], [-1, 1], [2, 0]), f32(126, 4, 3), exact=True)
case("dynamic_slice", lambda b, x, i, j: b.dynamic_slice(x, [i, j], [2, 3]), f32(127, 5, 7), np.int32(2), np.int32(3), exact=True)
case("dynamic_slice-clamped", lambda b, x, i, j: b.dynamic_slice(x, [i, j], [2, 3]), f32(128, 5, 7), np.int32(9), np.int32(-4), exact=True)
case("dynamic_update_slice", lambda b, x, u, i, j: b.dynamic_update_slice(x, u, [i, j]), f32(129, 5, 7), f32(130, 2, 3), np.int32(1), np.int32(2), exact=True)
case("dynamic_update_slice-clamped", lambda b, x, u, i, j: b.dynamic_update_slice(x, u, [i, j]), f32(131, 5, 7), f32(132, 2, 3), np.int32(7), np.int32(-2), exact=True)
case("dynamic_update_slice-scalar", lambda b, x, u: b.dynamic_update_slice(x, u, []), f32(133), f32(134), exact=True)
case("bf16-elementwise", lambda b, x, y: b.add(b.mul(x, y), b.tanh(x)), f32(135, 16, 24), f32(136, 16, 24), dtypes=["bf16", "bf16"])

# ------------------------------------------------------------------ gather (tests/configs/slice.py:33-43,217-240,391-456)
case("gather-take-rows", lambda b, x, i: b.take_rows(x, i), f32(140, 5, 3), np.array([0, 2, 4], np.int32), exact=True)
case("gather-take-negative-and-oob", lambda b, x, i: b.take_rows(x, i), f32(141, 5, 3), np.array([-1, 4, 5, -6, 0], np.int32))
case("gather-multi-index-point", lambda b, x, i: b.gather(x, i, offset_dims=[], collapsed_slice_dims=[0, 1], start_index_map=[0, 1],
                                                          index_vector_dim=1, slice_sizes=[1, 1]),
     f32(142, 4, 4), np.stack([np.arange(4), np.arange(4)], 1).astype(np.int32), exact=True)
case("gather-batched-single-axis", lambda b, x, i: b.gather(x, b.reshape(i, (3, 1)), offset_dims=[], collapsed_slice_dims=[1],
                                                            operand_batching_dims=[0], start_indices_batching_dims=[0],
                                                            start_index_map=[1], index_vector_dim=1, slice_sizes=[1, 1]),
     f32(143, 3, 10), np.array([7, 0, 9], np.int32), exact=True)
case("gather-partial-reversed-index-map", lambda b, x, i: b.gather(x, i, offset_dims=[1], collapsed_slice_dims=[0, 2], start_index_map=[2, 0],
                                                                   index_vector_dim=1, slice_sizes=[1, 4, 1]),
     f32(144, 3, 4, 5), np.array([[3, 2]], np.int32), exact=True)
case("gather-partial-scalar-indices", lambda b, x, i: b.gather(x, i, offset_dims=[0], collapsed_slice_dims=[0, 2], start_index_map=[0, 2],
                                                               index_vector_dim=0, slice_sizes=[1, 4, 1]),
     f32(145, 3, 4, 5), np.array([1, 0], np.int32), exact=True)
case("gather-multi-dim-no-collapse", lambda b, x, i: b.gather(x, i, offset_dims=[0, 1, 2], collapsed_slice_dims=[], start_index_map=[1, 2],
                                                              index_vector_dim=1, slice_sizes=[2, 1, 1]) if False else
     b.gather(x, i, offset_dims=[1, 2, 3], collapsed_slice_dims=[], start_index_map=[1, 2], index_vector_dim=1, slice_sizes=[2, 1, 1]),
     f32(146, 2, 3, 3), np.array([[0, 1], [1, 2], [0, 0]], np.int32), exact=True)
case("gather-clamped-window", lambda b, x, i: b.gather(x, i, offset_dims=[1], collapsed_slice_dims=[], start_index_map=[0],
                                                       index_vector_dim=1, slice_sizes=[3]),
     f32(147, 8), np.array([[0], [6], [7], [-2]], np.int32), exact=True)
case("gather-large-int32", lambda b, x, i: b.take_rows(x, i), np.array([[16777217], [2**30], [2**31 - 1]], np.int32), np.array([1, 0, 2], np.int32), exact=True)
case("gather-large-uint32", lambda b, x, i: b.take_rows(x, i), np.array([[16777217], [2**30], [2**31 - 1]], np.uint32), np.array([1], np.int32), exact=True)
case("gather-large-int64", lambda b, x, i: b.take_rows(x, i), np.array([[2**40], [2**50], [2**62]], np.int64), np.array([2, 0], np.int32), exact=True)


def _row_scatter(body, **kw):
    def f(b, x, i, u):
        return b.scatter(x, b.reshape(i, (i.shape[0], 1)), u, update_window_dims=list(range(1, u.ndim)), inserted_window_dims=[0],
                         scatter_dims_to_operand_dims=[0], index_vector_dim=1, body=body, **kw)
    return f


# ------------------------------------------------------------------ scatter (tests/configs/slice.py:175-216,241-295)
case("scatter-add", _row_scatter("add"), np.zeros((10, 4), np.float32), np.array([0, 2, 5], np.int32), np.ones((3, 4), np.float32), exact=True)
case("scatter-add-duplicates", _row_scatter("add"), f32(150, 10, 4), np.array([3, 3, 0, 3, 9, 0, 3], np.int32), f32(151, 7, 4), exact=True)
case("scatter-add-oob-dropped", _row_scatter("add"), f32(152, 6, 5), np.array([0, 6, -1, 5, 100], np.int32), f32(153, 5, 5), exact=True)
case("scatter-set", _row_scatter("set"), f32(154, 5, 3), np.array([0, 2], np.int32), f32(155, 2, 3), exact=True)
# element types the scatter kernels do not take run on the 32-bit type that holds them (and narrow index types on int32)
case("scatter-set-bool-mask", _row_scatter("set"), np.zeros((10, 4), np.bool_), np.array([3, 7, 3, 12, -1], np.int32), rng(160).random((5, 4)) > 0.4, dtypes=["i1", "i32", "i1"], exact=True)
case("scatter-add-bool-is-or", _row_scatter("add"), rng(161).random((6, 3)) > 0.7, np.array([0, 0, 5, 2], np.int64), rng(162).random((4, 3)) > 0.5, dtypes=["i1", "i64", "i1"], exact=True)
case("scatter-add-u8-wraps", _row_scatter("add"), rng(163).integers(0, 256, size=(5, 6)).astype(np.uint8), np.array([1, 1, 1, 4, 0, 1], np.int32),
     rng(164).integers(100, 256, size=(6, 6)).astype(np.uint8), exact=True)
case("scatter-min-i8-u8-indices", _row_scatter("min"), rng(165).integers(-128, 128, size=(7, 5)).astype(np.int8), np.array([6, 0, 6, 3, 200], np.uint8),
     rng(166).integers(-128, 128, size=(5, 5)).astype(np.int8), exact=True)
case("scatter-mul-i16-wraps-i16-indices", _row_scatter("mul"), rng(167).integers(-300, 300, size=(4, 3)).astype(np.int16), np.array([2, 2, 2, 0, -1], np.int16),
     rng(168).integers(-300, 300, size=(5, 3)).astype(np.int16), exact=True)
case("scatter-set-i64-as-two-halves", _row_scatter("set"), np.array([[2**40 + 5, -1], [7, -2**63], [2**63 - 1, 0], [3, 4]], np.int64), np.array([2, 0, 2, 9], np.int32),
     np.array([[-2**50, 11], [2**33, -2**33], [12345678901234, -98765432109876], [1, 1]], np.int64), exact=True)
case("scatter-set-u64-rank-3-i64-indices", _row_scatter("set"), rng(171).integers(0, 2**63, size=(5, 2, 3)).astype(np.uint64) * np.uint64(2), np.array([4, 1, 4], np.int64),
     rng(172).integers(0, 2**63, size=(3, 2, 3)).astype(np.uint64) * np.uint64(2) + np.uint64(1), exact=True)
case("scatter-add-f16", _row_scatter("add"), f32(169, 9, 8, lo=-1, hi=1).astype(np.float16), np.array([4, 4, 0, 8, 4], np.int32), f32(170, 5, 8, lo=-1, hi=1).astype(np.float16))
case("scatter-mul", _row_scatter("mul", unique_indices=True), np.ones((10, 4), np.float32), np.array([0, 2, 5], np.int32), np.full((3, 4), 2.0, np.float32), exact=True)
case("scatter-min", _row_scatter("min"), f32(156, 10, 4), np.array([0, 2, 5], np.int32), f32(157, 3, 4), exact=True)
case("scatter-max", _row_scatter("max"), f32(158, 10, 4), np.array([0, 2, 2], np.int32), f32(159, 3, 4), exact=True)
case("scatter-large-int32", _row_scatter("set"), np.zeros((5, 1), np.int32), np.array([1], np.int32), np.array([[2**30]], np.int32), exact=True)
case("scatter-large-uint32", _row_scatter("set"), np.zeros((5, 1), np.uint32), np.array([2], np.int32), np.array([[16777217]], np.uint32), exact=True)
case("scatter-add-many", _row_scatter("add"), f32(160, 300, 70), rng(161).integers(0, 300, size=1000).astype(np.int32), f32(162, 1000, 70), exact=True)

# scatter forms other than whole rows along dim 0 (lowered to an element scatter with computed keys)
case("scatter-point-2d-add", lambda b, x, i, u: b.scatter(x, i, u, update_window_dims=[], inserted_window_dims=[0, 1], scatter_dims_to_operand_dims=[0, 1], index_vector_dim=1),
     f32(1940, 6, 7), np.array([[0, 0], [5, 6], [2, 3], [2, 3], [6, 0], [-1, 2], [2, 3]], np.int32), f32(1941, 7), exact=True)
case("scatter-along-dim1-set", lambda b, x, i, u: b.scatter(x, i, u, update_window_dims=[0], inserted_window_dims=[1], scatter_dims_to_operand_dims=[1], index_vector_dim=1, body="set"),
     f32(1942, 5, 8), np.array([[7], [0], [3]], np.int32), f32(1943, 5, 3), exact=True)
case("scatter-window-2x3-add", lambda b, x, i, u: b.scatter(x, i, u, update_window_dims=[1, 2], inserted_window_dims=[], scatter_dims_to_operand_dims=[0, 1], index_vector_dim=1),
     f32(1944, 10, 12), np.array([[0, 0], [8, 9], [3, 4], [4, 5], [9, 9], [8, 10]], np.int32), f32(1945, 6, 2, 3), exact=True)
case("scatter-index-vector-dim0-max", lambda b, x, i, u: b.scatter(x, i, u, update_window_dims=[], inserted_window_dims=[0, 1], scatter_dims_to_operand_dims=[1, 0], index_vector_dim=0, body="max"),
     f32(1946, 4, 9), np.array([[8, 0, 3, 3, 8], [3, 0, 1, 1, 3]], np.int32), f32(1947, 5), exact=True)
case("scatter-batched-dims-add", lambda b, x, i, u: b.scatter(x, i, u, update_window_dims=[], inserted_window_dims=[1], scatter_dims_to_operand_dims=[1], index_vector_dim=2,
                                                              input_batching_dims=[0], scatter_indices_batching_dims=[0]),
     f32(1948, 3, 10), rng(1949).integers(0, 10, size=(3, 6, 1)).astype(np.int32), f32(1950, 3, 6), exact=True)
case("scatter-point-int32-many", lambda b, x, i, u: b.scatter(x, i, u, update_window_dims=[], inserted_window_dims=[0, 1], scatter_dims_to_operand_dims=[0, 1], index_vector_dim=1),
     rng(1951).integers(-9, 9, size=(20, 30)).astype(np.int32), rng(1952).integers(0, 20, size=(2000, 2)).astype(np.int32), rng(1953).integers(-100, 100, size=(2000,)).astype(np.int32), exact=True)

# hot rows: runs of equal indices longer than the LDS index tile (256) and the staging round (128), next to short runs
def _hot(seed, n, rows):
    r = rng(seed)
    idx = np.where(r.random(n) < 0.7, r.integers(0, 3, size=n) * 7, r.integers(0, rows, size=n))
    return idx.astype(np.int32)
case("scatter-add-hot-rows", _row_scatter("add"), f32(163, 40, 100), _hot(164, 1500, 40), f32(165, 1500, 100), exact=True)
case("scatter-add-hot-rows-int", _row_scatter("add"), rng(166).integers(-5, 5, size=(30, 70)).astype(np.int32), _hot(167, 900, 30),
     rng(168).integers(-1000, 1000, size=(900, 70)).astype(np.int32), exact=True)
case("scatter-max-hot-rows", _row_scatter("max"), f32(169, 25, 64), _hot(1690, 600, 25), f32(1691, 600, 64), exact=True)
case("scatter-add-hot-rows-exactly-16", _row_scatter("add"), f32(1692, 8, 33), np.array([5] * 16 + [2] * 15 + [7] * 17, np.int32), f32(1693, 48, 33), exact=True)

# very long runs (at least 256 updates of one row: narrow column chunks, 1024 updates staged per round), run lengths at the
# tier boundaries, the single-workgroup sort (at most 8192 updates) with one to three digit passes, and the general sort
def _runs(seed, *lengths_by_row):
    idx = np.concatenate([np.full(n, row, np.int32) for row, n in lengths_by_row])
    return rng(seed).permutation(idx).astype(np.int32)
case("scatter-add-very-long-run-three-rounds", _row_scatter("add"), f32(2600, 20, 13),
     np.where(rng(2601).random(3000) < 0.8, 3, rng(2602).integers(0, 20, size=3000)).astype(np.int32), f32(2603, 3000, 13), exact=True)
case("scatter-add-run-lengths-at-the-tier-boundaries", _row_scatter("add"), f32(2604, 12, 20),
     _runs(2605, (1, 255), (2, 256), (3, 257), (4, 1024), (5, 1025), (6, 15), (7, 16), (8, 17), (9, 1)), f32(2606, 2866, 20), exact=True)
case("scatter-max-very-long-run", _row_scatter("max"), f32(2607, 6, 9), _runs(2608, (0, 700), (5, 300), (2, 40)), f32(2609, 1040, 9), exact=True)
case("scatter-add-very-long-run-bf16", _row_scatter("add"), f32(2610, 6, 24, lo=-1, hi=1), _runs(2611, (4, 600), (1, 90), (0, 3)), f32(2612, 693, 24, lo=-1, hi=1),
     dtypes=["bf16", "i32", "bf16"], exact=True)
case("scatter-add-row-numbers-of-17-bits", _row_scatter("add"), f32(2613, 70000, 4),
     np.concatenate([rng(2614).integers(-5, 70010, size=4000), np.full(300, 69999), np.full(20, 65536)]).astype(np.int32)[rng(2615).permutation(4320)],
     f32(2616, 4320, 4), exact=True)
case("scatter-add-row-numbers-of-8-bits-int64-indices", _row_scatter("add"), f32(2617, 200, 6), rng(2618).integers(0, 200, size=8192).astype(np.int64),
     f32(2619, 8192, 6), exact=True)
case("scatter-add-more-updates-than-one-workgroup-sorts", _row_scatter("add"), f32(2620, 50, 10),
     np.where(rng(2621).random(9000) < 0.3, 7, rng(2622).integers(0, 50, size=9000)).astype(np.int32), f32(2623, 9000, 10), exact=True)

# a chain whose every link reads its input at two positions (v + reverse(v)): fused naively, link n evaluates the first value at 2^n
# positions; values evaluated at more than a few dozen positions are stored instead
def _mirrored_chain(links):
    def f(b, x):
        v = x
        for _ in range(links):
            t = b.tanh(v)
            v = b.mul(b.add(t, b.reverse(t, [0])), 0.5)
        return v
    return f


case("elementwise-chain-read-at-mirrored-positions-12-links", _mirrored_chain(12), f32(2800, 6, 40, lo=-1, hi=1))
case("elementwise-chain-read-at-mirrored-positions-40-links", _mirrored_chain(40), f32(2801, 6, 40, lo=-1, hi=1))


# x.at[i].add(u) as JAX lowers it: negative indices wrapped, updates of out-of-range rows selected to zero, then a scatter that drops those
# rows anyway.  The select is not computed (the scatter reads u); a mask that is not the scatter's own range check stays.
def _masked_scatter(lo_bound=0, hi_slack=0, other_index=False, body="add"):
    def f(b, x, i, u, *more):
        rows = x.shape[0]
        wrapped = b.select(b.compare(i, 0, "LT"), b.add(i, rows), i)
        checked = more[0] if other_index else wrapped
        ok = b.and_(b.compare(checked, lo_bound, "GE"), b.compare(checked, rows - 1 + hi_slack, "LE"))
        mask = b.broadcast_in_dim(ok, u.shape, [0])
        masked = b.select(mask, u, b.zeros(u.shape))
        return b.scatter(x, b.reshape(wrapped, (i.shape[0], 1)), masked, update_window_dims=[1], inserted_window_dims=[0],
                         scatter_dims_to_operand_dims=[0], index_vector_dim=1, body=body)
    return f


_MASKED = (f32(2650, 12, 6), np.array([0, 11, -1, 12, 40, -12, -13, 5, 5, -30, 3], np.int32), f32(2651, 11, 6))
case("scatter-add-updates-masked-by-the-range-check", _masked_scatter(), *_MASKED, exact=True)
case("scatter-add-updates-masked-by-a-narrower-check", _masked_scatter(lo_bound=2), *_MASKED, exact=True)
case("scatter-add-updates-masked-by-another-index", _masked_scatter(other_index=True), *_MASKED, np.array([0, 1, 2, 3, 4, 5, 60, 7, -8, 9, 10], np.int32), exact=True)
case("scatter-max-updates-masked-by-the-range-check", _masked_scatter(body="max"), *_MASKED, exact=True)
case("scatter-add-updates-masked-int64-indices", _masked_scatter(), _MASKED[0], _MASKED[1].astype(np.int64), _MASKED[2], exact=True)


# the operand is a splat constant (zeros a gradient is scattered into): the scatter writes it itself, in the launch that sorts
def _scatter_into(value, rows, cols, dtype="f32", body="add"):
    def f(b, i, u):
        x = b.constant(value, dtype, (rows, cols))
        return b.scatter(x, b.reshape(i, (i.shape[0], 1)), u, update_window_dims=[1], inserted_window_dims=[0], scatter_dims_to_operand_dims=[0],
                         index_vector_dim=1, body=body)
    return f
case("scatter-add-into-zeros", _scatter_into(0.0, 300, 70), rng(2630).integers(0, 300, size=1000).astype(np.int32), f32(2631, 1000, 70), exact=True)
case("scatter-add-into-zeros-odd-size", _scatter_into(0.0, 31, 3), rng(2632).integers(-2, 33, size=200).astype(np.int32), f32(2633, 200, 3), exact=True)
case("scatter-max-into-splat", _scatter_into(-0.25, 40, 9, body="max"), _hot(2634, 700, 40), f32(2635, 700, 9), exact=True)
case("scatter-add-into-ones-bf16", _scatter_into(1.0, 17, 5, dtype="bf16"), rng(2636).integers(0, 17, size=64).astype(np.int32), f32(2637, 64, 5, lo=-1, hi=1),
     dtypes=["i32", "bf16"], exact=True)
case("scatter-add-into-int-splat", _scatter_into(7, 20, 6, dtype="i32"), rng(2638).integers(0, 20, size=90).astype(np.int32),
     rng(2639).integers(-100, 100, size=(90, 6)).astype(np.int32), exact=True)
case("scatter-add-into-zeros-more-updates-than-one-workgroup-sorts", _scatter_into(0.0, 64, 12), rng(2640).integers(0, 64, size=8200).astype(np.int32),
     f32(2641, 8200, 12), exact=True)
def _scatter_splat_read_twice(b, i, u):
    x = b.constant(0.0, "f32", (50, 8))
    y = b.scatter(x, b.reshape(i, (i.shape[0], 1)), u, update_window_dims=[1], inserted_window_dims=[0], scatter_dims_to_operand_dims=[0], index_vector_dim=1)
    return [y, b.add(x, 1.0)]
case("scatter-add-into-zeros-that-something-else-reads", _scatter_splat_read_twice, rng(2642).integers(0, 50, size=120).astype(np.int32), f32(2643, 120, 8), exact=True)

# ------------------------------------------------------------------ dot_general (tests/configs/matmul.py:19-249)
case("dot-matmul", lambda b, x, y: b.matmul(x, y), f32(170, 33, 70), f32(171, 70, 45))
case("dot-vector-matrix", lambda b, x, y: b.dot_general(x, y, ([0], [0])), f32(172, 70), f32(173, 70, 45))
case("dot-matrix-vector", lambda b, x, y: b.dot_general(x, y, ([1], [0])), f32(174, 33, 70), f32(175, 70))
case("dot-inner", lambda b, x, y: b.dot_general(x, y, ([0], [0])), f32(176, 129), f32(177, 129))
case("dot-transposed-lhs", lambda b, x, y: b.dot_general(x, y, ([0], [0])), f32(178, 70, 33), f32(179, 70, 45))
case("dot-transposed-rhs", lambda b, x, y: b.dot_general(x, y, ([1], [1])), f32(180, 33, 70), f32(181, 45, 70))
case("dot-batched", lambda b, x, y: b.dot_general(x, y, ([2], [1]), ([0], [0])), f32(182, 5, 17, 40), f32(183, 5, 40, 23))
case("dot-batched-attention-layout", lambda b, q, k: b.dot_general(q, k, ([3], [3]), ([0, 2], [0, 2])), f32(184, 2, 9, 3, 16), f32(185, 2, 11, 3, 16))
case("dot-two-contracting", lambda b, x, y: b.dot_general(x, y, ([1, 2], [0, 1])), f32(186, 6, 4, 5), f32(187, 4, 5, 7))
case("dot-bf16", lambda b, x, y: b.matmul(x, y), f32(188, 40, 96), f32(189, 96, 72), dtypes=["bf16", "bf16"])
case("dot-bf16-f32-out", lambda b, x, y: b.dot_general(x, y, ([1], [0]), out_dtype="f32"), f32(190, 40, 96), f32(191, 96, 72), dtypes=["bf16", "bf16"])
# bf16 layouts of the tiled MFMA kernel: k-contiguous and m/n-contiguous operands, ragged tiles, batches
case("dot-bf16-tiled-kn", lambda b, x, y: b.matmul(x, y), f32(1900, 200, 136), f32(1901, 136, 328), dtypes=["bf16", "bf16"])
case("dot-bf16-tiled-rhs-kmajor", lambda b, x, y: b.dot_general(x, y, ([1], [1])), f32(1902, 150, 72), f32(1903, 90, 72), dtypes=["bf16", "bf16"])
case("dot-bf16-tiled-lhs-mmajor", lambda b, x, y: b.dot_general(x, y, ([0], [0])), f32(1904, 100, 136), f32(1905, 100, 72), dtypes=["bf16", "bf16"])
case("dot-bf16-tiled-lhs-mmajor-rhs-kmajor", lambda b, x, y: b.dot_general(x, y, ([0], [1])), f32(1906, 68, 264), f32(1907, 130, 68), dtypes=["bf16", "bf16"])
case("dot-bf16-tiled-attention-qk", lambda b, q, k: b.dot_general(q, k, ([3], [3]), ([0, 2], [0, 2])), f32(1908, 2, 128, 3, 64), f32(1909, 2, 128, 3, 64), dtypes=["bf16", "bf16"])
case("dot-bf16-tiled-attention-pv", lambda b, p, v: b.dot_general(p, v, ([3], [1]), ([0, 1], [0, 2])), f32(1910, 2, 3, 128, 128), f32(1911, 2, 128, 3, 64), dtypes=["bf16", "bf16"])
case("dot-bf16-tiled-big", lambda b, x, y: b.matmul(x, y), f32(1912, 1024, 192, lo=-1, hi=1), f32(1913, 192, 1024, lo=-1, hi=1), dtypes=["bf16", "bf16"])
case("dot-bf16-tiled-f32-out", lambda b, x, y: b.dot_general(x, y, ([1], [0]), out_dtype="f32"), f32(1914, 130, 200), f32(1915, 200, 136), dtypes=["bf16", "bf16"])
case("dot-bf16-async-nt", lambda b, x, y: b.dot_general(x, y, ([1], [1])), f32(1916, 200, 192, lo=-1, hi=1), f32(1917, 328, 192, lo=-1, hi=1), dtypes=["bf16", "bf16"])
case("dot-bf16-async-nt-long-k", lambda b, x, y: b.dot_general(x, y, ([1], [1]), out_dtype="f32"), f32(1918, 300, 1024, lo=-1, hi=1), f32(1919, 130, 1024, lo=-1, hi=1), dtypes=["bf16", "bf16"])
case("dot-bf16-async-nt-one-slab", lambda b, x, y: b.dot_general(x, y, ([1], [1])), f32(1920, 70, 64), f32(1921, 50, 64), dtypes=["bf16", "bf16"])
case("dot-bf16-async-nt-big", lambda b, x, y: b.dot_general(x, y, ([1], [1])), f32(1922, 1024, 512, lo=-1, hi=1), f32(1923, 768, 512, lo=-1, hi=1), dtypes=["bf16", "bf16"])
# integer contractions are lowered to broadcast-multiply-reduce (exact, wrap-around)
def i32(seed, *shape, lo=-1000, hi=1000):
    return rng(seed).integers(lo, hi, size=shape).astype(np.int32)
# n-contiguous rhs (a dense layer's [in, out] weights) read in place by the LDS-ring kernel, one case per tile shape
case("dot-bf16-async-nn-edges", lambda b, x, y: b.matmul(x, y), f32(1950, 200, 128, lo=-1, hi=1), f32(1951, 128, 328, lo=-1, hi=1), dtypes=["bf16", "bf16"])
case("dot-bf16-async-nn-narrow", lambda b, x, y: b.matmul(x, y), f32(1952, 300, 64, lo=-1, hi=1), f32(1953, 64, 72, lo=-1, hi=1), dtypes=["bf16", "bf16"])
case("dot-bf16-async-nn-batched", lambda b, x, y: b.dot_general(x, y, ([2], [1]), ([0], [0])), f32(1954, 3, 130, 64, lo=-1, hi=1), f32(1955, 3, 64, 136, lo=-1, hi=1), dtypes=["bf16", "bf16"])
case("dot-bf16-async-nn-128x64", lambda b, x, y: b.matmul(x, y), f32(1956, 2048, 128, lo=-1, hi=1), f32(1957, 128, 3072, lo=-1, hi=1), dtypes=["bf16", "bf16"])
case("dot-bf16-async-nn-128x128", lambda b, x, y: b.dot_general(x, y, ([1], [0]), out_dtype="f32"), f32(1958, 4096, 128, lo=-1, hi=1), f32(1959, 128, 6144, lo=-1, hi=1), dtypes=["bf16", "bf16"])
case("dot-bf16-async-nn-256x128", lambda b, x, y: b.matmul(x, y), f32(1960, 4096, 192, lo=-1, hi=1), f32(1961, 192, 8200, lo=-1, hi=1), dtypes=["bf16", "bf16"])
# bias added by the GEMM kernels' own epilogue (dot_general -> add(broadcast(bias)) with no other reader of the product)
def _linear(b, x, w, bias):
    y = b.dot_general(x, w, ([x.ndim - 1], [0]))
    return b.add(y, b.broadcast_in_dim(bias, y.shape, [y.ndim - 1]))


case("dot-bias-f32-small", _linear, f32(1970, 33, 70), f32(1971, 70, 45), f32(1972, 45))
case("dot-bias-f32-igemm", _linear, f32(1973, 520, 384, lo=-1, hi=1), f32(1974, 384, 1030, lo=-1, hi=1), f32(1975, 1030))
case("dot-bias-f32-3d", _linear, f32(1976, 4, 9, 70), f32(1977, 70, 24), f32(1978, 24))
case("dot-bias-bf16-async", _linear, f32(1979, 200, 128, lo=-1, hi=1), f32(1980, 128, 328, lo=-1, hi=1), f32(1981, 328), dtypes=["bf16", "bf16", "bf16"])
case("dot-bias-bf16-tiled", _linear, f32(1982, 200, 136, lo=-1, hi=1), f32(1983, 136, 328, lo=-1, hi=1), f32(1984, 328), dtypes=["bf16", "bf16", "bf16"])
case("dot-bias-bf16-odd", _linear, f32(1985, 37, 50, lo=-1, hi=1), f32(1986, 50, 29, lo=-1, hi=1), f32(1987, 29), dtypes=["bf16", "bf16", "bf16"])
# maximum(x, 0) on a small fp32 product is applied while the product is stored; a mask compare(x, 0, GT) next to it reads the
# activation instead (same truth value), so the value before the activation needs no memory
def _nan_row(seed, *shape):
    a = f32(seed, *shape)
    a[1, 3] = np.nan
    return a
case("dot-bias-relu-f32-small", lambda b, x, w, c: b.maximum(_linear(b, x, w, c), 0.0), f32(2660, 33, 70), f32(2661, 70, 45), f32(2662, 45))
case("dot-relu-f32-small-no-bias-zero-first", lambda b, x, w: b.maximum(b.constant(0.0, "f32", (33, 45)), b.matmul(x, w)), f32(2663, 33, 70), f32(2664, 70, 45))
case("dot-bias-relu-f32-small-nan-stays", lambda b, x, w, c: b.maximum(_linear(b, x, w, c), 0.0), _nan_row(2665, 33, 70), f32(2666, 70, 45), f32(2667, 45))
def _relu_and_mask(b, x, w, c, g):
    z = _linear(b, x, w, c)
    return [b.maximum(z, 0.0), b.select(b.compare(z, b.constant(0.0, "f32", z.shape), "GT"), g, b.constant(0.0, "f32", z.shape))]
case("dot-bias-relu-f32-small-mask-from-activation", _relu_and_mask, f32(2668, 33, 70), f32(2669, 70, 45), f32(2670, 45), f32(2671, 33, 45))
case("dot-bias-relu-f32-small-value-before-also-read", lambda b, x, w, c: (lambda z: [b.maximum(z, 0.0), b.mul(z, 2.0)])(_linear(b, x, w, c)),
     f32(2672, 33, 70), f32(2673, 70, 45), f32(2674, 45))
case("dot-relu-f32-igemm-not-small", lambda b, x, w: b.maximum(b.matmul(x, w), 0.0), f32(2675, 520, 384, lo=-1, hi=1), f32(2676, 384, 1030, lo=-1, hi=1))
def _two_products_relu(b, x, w, h, u, c):
    y = b.add(b.matmul(x, w), b.matmul(h, u))
    return b.maximum(b.add(y, b.broadcast_in_dim(c, y.shape, [1])), 0.0)
case("dot-sum-two-products-bias-relu", _two_products_relu, f32(2677, 20, 30), f32(2678, 30, 40), f32(2679, 20, 50), f32(2680, 50, 40), f32(2681, 40))
case("dot-bias-computed", lambda b, x, w, c: _linear(b, x, w, b.mul(c, c)), f32(1988, 33, 70), f32(1989, 70, 45), f32(1990, 45))
case("dot-bias-depends-on-a-later-product", lambda b, x, w, v: (lambda y, z: b.add(y, b.broadcast_in_dim(b.neg(b.reshape(z, (45,))), y.shape, [1])))(b.matmul(x, w), b.matmul(v, w)),
     f32(1994, 33, 70), f32(1995, 70, 45), f32(1996, 1, 70))
case("dot-bias-product-read-twice", lambda b, x, w, c: (lambda y: b.mul(b.add(y, b.broadcast_in_dim(c, y.shape, [1])), y))(b.matmul(x, w)),
     f32(1991, 33, 70), f32(1992, 70, 45), f32(1993, 45))

# tanh-form GELU after a bf16 product: applied by the GEMM kernels while they store (recognised by what the chain computes)
def _gelu_builder(b, y):
    from jax_mps_amd.shlo.builder import gelu_tanh
    return gelu_tanh(b, y)


def _gelu_jax_order(b, y):   # jax.nn.gelu(approximate=True): x * (0.5 * (1 + tanh(c * (x + 0.044715 * x^3))))
    inner = b.mul(b.add(y, b.mul(b.mul(b.mul(y, y), y), 0.044715)), 0.7978845608028654)
    return b.mul(y, b.mul(b.add(b.tanh(inner), 1.0), 0.5))


case("dot-gelu-bf16-async", lambda b, x, w, c: _gelu_builder(b, _linear(b, x, w, c)), f32(2101, 256, 128, lo=-1, hi=1), f32(2102, 128, 320, lo=-1, hi=1), f32(2103, 320),
     dtypes=["bf16", "bf16", "bf16"])
case("dot-gelu-bf16-jax-order-no-bias", lambda b, x, w: _gelu_jax_order(b, b.matmul(x, w)), f32(2104, 200, 128, lo=-1, hi=1), f32(2105, 128, 328, lo=-1, hi=1), dtypes=["bf16", "bf16"])
case("dot-gelu-bf16-tiled", lambda b, x, w, c: _gelu_builder(b, _linear(b, x, w, c)), f32(2106, 200, 136, lo=-1, hi=1), f32(2107, 136, 328, lo=-1, hi=1), f32(2108, 328),
     dtypes=["bf16", "bf16", "bf16"])
case("dot-gelu-bf16-odd", lambda b, x, w, c: _gelu_jax_order(b, _linear(b, x, w, c)), f32(2109, 37, 50, lo=-2, hi=2), f32(2110, 50, 29, lo=-2, hi=2), f32(2111, 29), dtypes=["bf16", "bf16", "bf16"])
case("dot-gelu-bf16-3d-wide-range", lambda b, x, w, c: _gelu_builder(b, _linear(b, x, w, c)), f32(2112, 4, 64, 64, lo=-3, hi=3), f32(2113, 64, 128, lo=-3, hi=3), f32(2114, 128, lo=-8, hi=8),
     dtypes=["bf16", "bf16", "bf16"])
case("dot-gelu-bf16-zero-cubic-term", lambda b, x, w, c: (lambda y: b.mul(b.mul(y, 0.5), b.add(b.tanh(b.mul(y, 0.8)), 1.0)))(_linear(b, x, w, c)), f32(2124, 128, 128, lo=-1, hi=1),
     f32(2125, 128, 128, lo=-1, hi=1), f32(2126, 128), dtypes=["bf16", "bf16", "bf16"])
# chains that must stay kernels of their own: the sum is read twice; the function is not a GELU; the result is f32
case("dot-gelu-bf16-sum-read-twice", lambda b, x, w, c: (lambda y: b.add(_gelu_builder(b, y), y))(_linear(b, x, w, c)), f32(2115, 128, 128, lo=-1, hi=1), f32(2116, 128, 128, lo=-1, hi=1),
     f32(2117, 128), dtypes=["bf16", "bf16", "bf16"])
case("dot-not-gelu-bf16", lambda b, x, w, c: (lambda y: b.mul(y, b.tanh(y)))(_linear(b, x, w, c)), f32(2118, 128, 128, lo=-1, hi=1),
     f32(2119, 128, 128, lo=-1, hi=1), f32(2120, 128), dtypes=["bf16", "bf16", "bf16"])
case("dot-gelu-f32", lambda b, x, w, c: _gelu_builder(b, _linear(b, x, w, c)), f32(2121, 33, 70), f32(2122, 70, 45), f32(2123, 45))


# add(dot, dot) of two small fp32 products is one launch (the recurrent cell's x*Wi + h*Wh), with the bias on top
case("dot-sum-two-products", lambda b, x, wi, h, wh: b.add(b.matmul(x, wi), b.matmul(h, wh)), f32(2020, 33, 70), f32(2021, 70, 45), f32(2022, 33, 19), f32(2023, 19, 45))
case("dot-sum-two-products-bias", lambda b, x, wi, h, wh, c: (lambda y: b.add(y, b.broadcast_in_dim(c, y.shape, [1])))(b.add(b.matmul(x, wi), b.matmul(h, wh))),
     f32(2024, 64, 128), f32(2025, 128, 200), f32(2026, 64, 256), f32(2027, 256, 200), f32(2028, 200))
case("dot-sum-two-products-work-between", lambda b, x, wi, h, wh: b.add(b.matmul(x, wi), b.matmul(b.tanh(b.add(h, h)), wh)), f32(2029, 33, 70), f32(2030, 70, 45), f32(2031, 33, 19), f32(2032, 19, 45))
case("dot-sum-two-products-transposed", lambda b, x, wi, h, wh: b.add(b.dot_general(x, wi, ([0], [1])), b.dot_general(h, wh, ([1], [1]))), f32(2033, 70, 33), f32(2034, 45, 70), f32(2035, 33, 19), f32(2036, 45, 19))
case("dot-sum-one-product-large", lambda b, x, wi, h, wh: b.add(b.matmul(x, wi), b.matmul(h, wh)), f32(2037, 520, 384, lo=-1, hi=1), f32(2038, 384, 1030, lo=-1, hi=1), f32(2039, 520, 16), f32(2040, 16, 1030))
case("dot-sum-product-read-twice", lambda b, x, wi, h, wh: (lambda p, q: b.mul(b.add(p, q), q))(b.matmul(x, wi), b.matmul(h, wh)), f32(2041, 33, 70), f32(2042, 70, 45), f32(2043, 33, 19), f32(2044, 19, 45))


# softmax(scale * q k^T [masked]) v as JAX's XLA path spells it: one fused launch when the operands are bf16 (tests/
# test_gpu_ops.py holds bf16 results to 2e-2); layouts, tails, masks and head sizes the fused kernel has to get right
def _sdpa(b, q, k, v, mask=None, scale=None, layout="BTNH", merge=True):
    import math as _m
    if layout == "BTNH":
        logits = b.dot_general(q, k, ([3], [3]), ([0, 2], [0, 2]), out_dtype="f32")          # B N T S
    else:
        logits = b.dot_general(q, k, ([3], [3]), ([0, 1], [0, 1]), out_dtype="f32")
    if scale is not None:
        logits = b.mul(logits, float(scale))
    if mask is not None:
        keep = b.compare(mask, 0, "NE")
        logits = b.select(b.broadcast_in_dim(keep, logits.shape, [0, 1, 2, 3]), logits, b.full_like(logits, float(-0.7 * np.finfo(np.float32).max)))
    from jax_mps_amd.programs.configs import softmax as _softmax
    probs = b.convert(_softmax(b, logits, -1), q.dtype)
    if layout == "BTNH":
        enc = b.dot_general(probs, v, ([3], [1]), ([0, 1], [0, 2]))                             # B N T H
    else:
        enc = b.dot_general(probs, v, ([3], [2]), ([0, 1], [0, 1]))
    if merge:
        bt, n, t, h = enc.shape
        enc = b.reshape(b.transpose(enc, [0, 2, 1, 3]), (bt, t, n * h))
    return enc


_B16 = ["bf16", "bf16", "bf16"]
case("attention-bf16-128x128-h64", lambda b, q, k, v: _sdpa(b, q, k, v, scale=0.125), f32(2200, 2, 128, 3, 64, lo=-1, hi=1), f32(2201, 2, 128, 3, 64, lo=-1, hi=1), f32(2202, 2, 128, 3, 64, lo=-1, hi=1), dtypes=_B16)
case("attention-bf16-tails", lambda b, q, k, v: _sdpa(b, q, k, v, scale=0.125), f32(2203, 2, 50, 2, 64, lo=-1, hi=1), f32(2204, 2, 70, 2, 64, lo=-1, hi=1), f32(2205, 2, 70, 2, 64, lo=-1, hi=1), dtypes=_B16)
case("attention-bf16-key-mask", lambda b, q, k, v, m: _sdpa(b, q, k, v, mask=m, scale=0.125), f32(2206, 3, 40, 2, 64, lo=-1, hi=1), f32(2207, 3, 96, 2, 64, lo=-1, hi=1),
     f32(2208, 3, 96, 2, 64, lo=-1, hi=1), (rng(2209).uniform(size=(3, 1, 1, 96)) < 0.7).astype(np.int32), dtypes=_B16 + ["i32"])
case("attention-bf16-full-mask", lambda b, q, k, v, m: _sdpa(b, q, k, v, mask=m, scale=0.2), f32(2210, 2, 64, 2, 64, lo=-1, hi=1), f32(2211, 2, 64, 2, 64, lo=-1, hi=1),
     f32(2212, 2, 64, 2, 64, lo=-1, hi=1), np.tril(np.ones((64, 64), np.int32))[None, None].repeat(2, 0), dtypes=_B16 + ["i32"])
case("attention-bf16-h128-long-keys", lambda b, q, k, v: _sdpa(b, q, k, v, scale=0.09), f32(2213, 1, 200, 2, 128, lo=-1, hi=1), f32(2214, 1, 300, 2, 128, lo=-1, hi=1), f32(2215, 1, 300, 2, 128, lo=-1, hi=1), dtypes=_B16)
case("attention-bf16-bnth-no-merge-no-scale", lambda b, q, k, v: _sdpa(b, q, k, v, layout="BNTH", merge=False), f32(2216, 2, 3, 72, 64, lo=-0.5, hi=0.5), f32(2217, 2, 3, 100, 64, lo=-0.5, hi=0.5),
     f32(2218, 2, 3, 100, 64, lo=-0.5, hi=0.5), dtypes=_B16)
case("attention-bf16-h32-not-fused", lambda b, q, k, v: _sdpa(b, q, k, v, scale=0.18), f32(2219, 2, 64, 2, 32, lo=-1, hi=1), f32(2220, 2, 64, 2, 32, lo=-1, hi=1), f32(2221, 2, 64, 2, 32, lo=-1, hi=1), dtypes=_B16)
case("attention-bf16-probabilities-read-twice", lambda b, q, k, v: (lambda lg: [b.convert(lg, "bf16"), b.dot_general(b.convert(lg, "bf16"), v, ([3], [1]), ([0, 1], [0, 2]))])(
     __import__("jax_mps_amd.programs.configs", fromlist=["softmax"]).softmax(b, b.dot_general(q, k, ([3], [3]), ([0, 2], [0, 2]), out_dtype="f32"), -1)),
     f32(2222, 2, 64, 2, 64, lo=-1, hi=1), f32(2223, 2, 64, 2, 64, lo=-1, hi=1), f32(2224, 2, 64, 2, 64, lo=-1, hi=1), dtypes=_B16)


# dimension numbers whose operand dims do not collapse to one strided matrix per batch (free dims on both sides of a contracted
# one, contracted dims in another order on the other side, batch dims apart): a transposed copy is made first
case("dot-general-vector-times-the-middle-dim", lambda b, v, t: b.dot_general(v, t, ([0], [1])), f32(2300, 5), f32(2301, 4, 5, 6))
case("dot-general-three-contracted-dims-in-another-order", lambda b, x, y: b.dot_general(x, y, ([3, 1, 2], [3, 1, 0])), f32(2302, 3, 4, 3, 2), f32(2303, 3, 4, 4, 2))
case("dot-general-batch-dim-between-contracted-dims", lambda b, x, y: b.dot_general(x, y, ([1, 2], [3, 1]), ([0], [2])), f32(2304, 3, 3, 2), f32(2305, 4, 2, 3, 3))
case("dot-general-free-dims-around-a-contracted-one-bf16", lambda b, x, y: b.dot_general(x, y, ([3], [2])), f32(2306, 4, 5, 2, 5, lo=-1, hi=1), f32(2307, 3, 2, 5, 2, lo=-1, hi=1),
     dtypes=["bf16", "bf16"])
case("dot-general-tensordot-two-axes-swapped", lambda b, x, y: b.tanh(b.dot_general(x, y, ([0, 2], [1, 0]))), f32(2308, 16, 7, 33, lo=-1, hi=1), f32(2309, 33, 16, 9, lo=-1, hi=1))

# float16 products and convolutions: widened to the float32 path, the result narrowed once
case("dot-f16-bias-tanh", lambda b, x, w, c: b.tanh(b.add(b.matmul(x, w), b.broadcast_in_dim(c, (16, 8), [1]))),
     f32(2310, 16, 32, lo=-1, hi=1).astype(np.float16), f32(2311, 32, 8, lo=-0.3, hi=0.3).astype(np.float16), f32(2312, 8).astype(np.float16))
case("dot-f16-batched-f32-result", lambda b, x, w: b.dot_general(x, w, ([2], [1]), ([0], [0]), out_dtype="f32"),
     f32(2313, 3, 20, 64, lo=-1, hi=1).astype(np.float16), f32(2314, 3, 64, 24, lo=-1, hi=1).astype(np.float16))
case("conv-f16-3x3-pad1", lambda b, x, f: b.conv(x, f, padding=((1, 1), (1, 1))), f32(2315, 2, 8, 8, 16, lo=-1, hi=1).astype(np.float16),
     f32(2316, 3, 3, 16, 8, lo=-0.2, hi=0.2).astype(np.float16))

# bitcast_convert between element types of different width (x.view(dtype)): a last dim of wide / narrow elements, least
# significant first, appears or is folded away
def _bitcast_to(b, x, dtype, shape):
    v = b._new(shape, dtype)
    b._emit(f"{v.name} = stablehlo.bitcast_convert {x.name} : ({x.type}) -> {v.type}")
    return v
case("bitcast-f32-to-four-u8", lambda b, x: _bitcast_to(b, x, "ui8", (3, 5, 4)), f32(2320, 3, 5), exact=True)
case("bitcast-i64-to-two-i32-and-back", lambda b, x: (lambda h: [h, _bitcast_to(b, h, "i64", (7,))])(_bitcast_to(b, x, "i32", (7, 2))),
     np.array([0, 1, -1, 2**40 + 5, -2**63, 2**63 - 1, 123456789012345], np.int64), exact=True)
case("bitcast-four-u8-to-f32", lambda b, x: _bitcast_to(b, x, "f32", (6,)), rng(2321).integers(0, 256, size=(6, 4)).astype(np.uint8), exact=True)
case("bitcast-two-bf16-to-u32-and-f32-to-two-f16", lambda b, x, y: [_bitcast_to(b, x, "ui32", (5,)), _bitcast_to(b, y, "f16", (5, 2))],
     f32(2322, 5, 2), f32(2323, 5), dtypes=["bf16", "f32"], exact=True)

# independent small products next to each other share one launch (the gradients of one recurrent step)
case("dot-group-three-independent", lambda b, dz, wh, h, x: [b.dot_general(dz, wh, ([1], [1])), b.dot_general(h, dz, ([0], [0])), b.dot_general(x, dz, ([0], [0]))],
     f32(2050, 20, 96), f32(2051, 40, 96), f32(2052, 20, 40), f32(2053, 20, 24))
case("dot-group-second-reads-first", lambda b, x, w1, w2: (lambda y: [y, b.matmul(y, w2)])(b.matmul(x, w1)), f32(2054, 20, 30), f32(2055, 30, 40), f32(2056, 40, 10))


# operands that are slice / reshape / transpose chains over a buffer are read through strides (no copy kernel)
def _qkv_attention_logits(b, x, w, bias, heads):
    bt, s, _ = x.shape
    hd = w.shape[1] // (3 * heads)
    qkv = b.reshape(_linear(b, x, w, bias), (bt, s, 3, heads, hd))
    q, k, v = (b.reshape(b.slice(qkv, [0, 0, i, 0, 0], [bt, s, i + 1, heads, hd]), (bt, s, heads, hd)) for i in range(3))
    logits = b.dot_general(q, k, ([3], [3]), ([0, 2], [0, 2]))      # B H T S
    return b.dot_general(logits, v, ([3], [1]), ([0, 1], [0, 2]))   # B H T D


case("dot-view-qkv-split-f32", lambda b, x, w, c: _qkv_attention_logits(b, x, w, c, 2), f32(2000, 3, 10, 24, lo=-1, hi=1), f32(2001, 24, 48, lo=-1, hi=1), f32(2002, 48))
case("dot-view-qkv-split-bf16", lambda b, x, w, c: _qkv_attention_logits(b, x, w, c, 3), f32(2003, 2, 128, 64, lo=-1, hi=1), f32(2004, 64, 576, lo=-0.3, hi=0.3), f32(2005, 576, lo=-0.3, hi=0.3),
     dtypes=["bf16", "bf16", "bf16"])
case("dot-view-strided-slice-of-argument", lambda b, x, y: b.matmul(b.slice(x, [1, 2], [33, 70], [2, 1]), b.slice(y, [0, 3], [68, 45], [1, 2])), f32(2006, 33, 70), f32(2007, 70, 45))
case("dot-view-transpose-of-argument", lambda b, x, y: b.matmul(b.transpose(x, [1, 0]), b.transpose(y, [1, 0])), f32(2008, 70, 33), f32(2009, 45, 70))
case("dot-view-reshape-merging-dims", lambda b, x, y: b.matmul(b.reshape(b.slice(x, [0, 0, 0], [4, 6, 35]), (24, 35)), y), f32(2010, 4, 6, 40), f32(2011, 35, 12))
case("dot-view-reshape-not-a-view", lambda b, x, y: b.matmul(b.reshape(b.slice(x, [0, 0, 0], [4, 5, 35]), (20, 35)), y), f32(2012, 4, 6, 35), f32(2013, 35, 12))
case("dot-view-same-buffer-twice", lambda b, x: b.dot_general(b.slice(x, [0, 0], [16, 40]), b.slice(x, [16, 0], [32, 40]), ([1], [1])), f32(2014, 32, 40))
case("dot-int32-matmul", lambda b, x, y: b.matmul(x, y), i32(1930, 33, 70), i32(1931, 70, 45), exact=True)
case("dot-int32-batched-attention-layout", lambda b, q, k: b.dot_general(q, k, ([3], [3]), ([0, 2], [0, 2])), i32(1932, 2, 9, 3, 16), i32(1933, 2, 11, 3, 16), exact=True)
case("dot-int32-wraps", lambda b, x, y: b.matmul(x, y), i32(1934, 8, 300, lo=-2**30, hi=2**30), i32(1935, 300, 8, lo=-2**30, hi=2**30), exact=True)
case("dot-uint32-above-2p24", lambda b, x, y: b.matmul(x, y), rng(1936).integers(0, 2**20, size=(5, 40)).astype(np.uint32), rng(1937).integers(0, 2**11, size=(40, 6)).astype(np.uint32), exact=True)
case("dot-large-k", lambda b, x, y: b.matmul(x, y), f32(192, 64, 3000, lo=-1, hi=1), f32(193, 3000, 64, lo=-1, hi=1))
# fp32 products by size class: small ones run on the K-split-in-workgroup kernel (16- or 32-wide tiles), larger
# unbatched ones on the implicit-GEMM kernel, larger batched ones on the strided tile kernel
case("dot-f32-small-tile32-batched", lambda b, x, y: b.dot_general(x, y, ([2], [1]), ([0], [0])), f32(1940, 6, 300, 200, lo=-1, hi=1), f32(1941, 6, 200, 300, lo=-1, hi=1))
case("dot-f32-small-tile32-transposed", lambda b, x, y: b.dot_general(x, y, ([0], [1])), f32(1942, 77, 500, lo=-1, hi=1), f32(1943, 610, 77, lo=-1, hi=1))
case("dot-f32-igemm", lambda b, x, y: b.matmul(x, y), f32(1944, 520, 384, lo=-1, hi=1), f32(1945, 384, 1030, lo=-1, hi=1))
case("dot-f32-strided-batched", lambda b, x, y: b.dot_general(x, y, ([2], [1]), ([0], [0])), f32(1946, 8, 330, 256, lo=-1, hi=1), f32(1947, 8, 256, 330, lo=-1, hi=1))


def _conv(**kw):
    return lambda b, x, w: b.conv(x, w, **kw)


def _same(n, k, s, d=1):
    out = -(-n // s)
    tot = max((out - 1) * s + (k - 1) * d + 1 - n, 0)
    return (tot // 2, tot - tot // 2)


# ------------------------------------------------------------------ convolution (tests/configs/conv.py:9-224)
u = lambda seed, *shape: f32(seed, *shape, lo=-1, hi=1)
case("conv-SAME", _conv(padding=(_same(8, 3, 1),) * 2), u(200, 2, 8, 8, 3), u(201, 3, 3, 3, 8))
case("conv-NCHW-OIHW", _conv(padding=(_same(8, 3, 1),) * 2, dn=("bf01", "oi01", "bf01")), u(202, 1, 3, 8, 8), u(203, 16, 3, 3, 3))
case("conv-1d-NWC", _conv(strides=(2,), padding=(_same(16, 3, 2),), dn=("b0f", "0io", "b0f")), u(204, 2, 16, 3), u(205, 3, 3, 4))
case("conv-stride2-SAME", _conv(strides=(2, 2), padding=(_same(8, 3, 2),) * 2), u(206, 2, 8, 8, 3), u(207, 3, 3, 3, 8))
case("conv-stride2-asymmetric", _conv(strides=(2, 2), padding=((1, 0), (1, 0))), u(208, 2, 8, 8, 3), u(209, 3, 3, 3, 8))
case("conv-5x5-stride2", _conv(strides=(2, 2), padding=(_same(16, 5, 2),) * 2), u(210, 2, 16, 16, 3), u(211, 5, 5, 3, 8))
case("conv-stride2-dilated", _conv(strides=(2, 2), padding=(_same(16, 3, 2, 2),) * 2, rhs_dilation=(2, 2)), u(212, 2, 16, 16, 3), u(213, 3, 3, 3, 8))
case("conv-stride2-VALID", _conv(strides=(2, 2)), u(214, 2, 9, 9, 3), u(215, 3, 3, 3, 8))
case("conv-1d-stride2-dilated", _conv(strides=(2,), padding=(_same(32, 3, 2, 2),), rhs_dilation=(2,), dn=("b0f", "0io", "b0f")), u(216, 2, 32, 3), u(217, 3, 3, 4))
case("conv-lhs_dilation-neg_padding", _conv(padding=((0, -1), (0, 0)), lhs_dilation=(2, 1)), u(218, 1, 6, 7, 4), u(219, 1, 2, 4, 2))
case("conv-lhs_dilation-only", _conv(lhs_dilation=(2, 1)), u(220, 1, 6, 7, 4), u(221, 1, 2, 4, 2))
case("conv-large-kernel", _conv(padding=(_same(4, 8, 1),) * 2), u(222, 1, 4, 4, 3), u(223, 8, 8, 3, 16))
case("conv-batch_group_count_2", _conv(dn=("bf01", "oi01", "bf01"), batch_group_count=2), u(224, 4, 1, 6, 7), u(225, 2, 1, 1, 2))
case("conv-batch_group_count_3-multi_filter", _conv(padding=((1, 1), (1, 1)), batch_group_count=3), u(226, 6, 5, 5, 2), u(227, 3, 3, 2, 6))
case("conv-depthwise", _conv(padding=((1, 1), (1, 1)), feature_group_count=6), u(228, 2, 7, 7, 6), u(229, 3, 3, 1, 12))
case("conv-grouped", _conv(padding=((1, 1), (1, 1)), feature_group_count=2), u(230, 2, 7, 7, 8), u(231, 3, 3, 4, 6))
case("conv-1x1", _conv(), u(232, 3, 9, 9, 20), u(233, 1, 1, 20, 24))
case("conv-resnet-block-shape", _conv(padding=((1, 1), (1, 1))), u(234, 4, 16, 16, 64), u(235, 3, 3, 64, 64))
case("conv-wgrad-form", lambda b, x, g: b.conv(x, g, strides=(1, 1), padding=((1, 1), (1, 1)), rhs_dilation=(2, 2), dn=("f01b", "i01o", "01bf")),
     u(236, 4, 16, 16, 24), u(237, 4, 8, 8, 40))
case("conv-dgrad-form", lambda b, g, w: b.conv(g, b.reverse(w, [0, 1]), strides=(1, 1), padding=((1, 2), (1, 2)), lhs_dilation=(2, 2), dn=("b01f", "01oi", "b01f")),
     u(238, 4, 8, 8, 40), u(239, 3, 3, 24, 40))
# shapes that reach the vectorised tile loaders and the split-K path of the implicit-GEMM kernel
case("conv-fwd-vector-loaders", _conv(padding=((1, 1), (1, 1))), u(242, 8, 12, 12, 32), u(243, 3, 3, 32, 64))
case("conv-fwd-stride2-vector", _conv(strides=(2, 2), padding=((0, 1), (0, 1))), u(244, 8, 12, 12, 32), u(245, 3, 3, 32, 64))
case("conv-fwd-128-tile", _conv(padding=((1, 1), (1, 1))), u(246, 16, 32, 32, 16), u(247, 3, 3, 16, 128))
case("conv-dgrad-vector", lambda b, g, w: b.conv(g, b.reverse(w, [0, 1]), strides=(1, 1), padding=((1, 2), (1, 2)), lhs_dilation=(2, 2), dn=("b01f", "01oi", "b01f")),
     u(248, 8, 6, 6, 64), u(249, 3, 3, 32, 64))
# input-dilated convolutions run one launch per residue class of the output positions
case("conv-dgrad-classes-odd", lambda b, g, w: b.conv(g, b.reverse(w, [0, 1]), strides=(1, 1), padding=((1, 1), (2, 1)), lhs_dilation=(2, 3), dn=("b01f", "01oi", "b01f")),
     u(1300, 4, 7, 5, 32), u(1301, 3, 3, 16, 32))
case("conv-dgrad-classes-repacked", lambda b, g, w: b.conv(g, b.reverse(w, [0, 1]), strides=(1, 1), padding=((1, 2), (1, 2)), lhs_dilation=(2, 2), dn=("b01f", "01oi", "b01f")),
     u(1302, 16, 8, 8, 32), u(1303, 3, 3, 16, 32))
case("conv-dilated-5x5-classes", _conv(padding=((2, 2), (0, 3)), lhs_dilation=(2, 2)), u(1304, 2, 9, 6, 16), u(1305, 5, 5, 16, 8))
case("conv-wgrad-vector", lambda b, x, g: b.conv(x, g, strides=(1, 1), padding=((0, 1), (0, 1)), rhs_dilation=(2, 2), dn=("f01b", "i01o", "01bf")),
     u(250, 16, 12, 12, 8), u(251, 16, 6, 6, 32))
case("conv-wgrad-stride1-vector", lambda b, x, g: b.conv(x, g, strides=(1, 1), padding=((1, 1), (1, 1)), dn=("f01b", "i01o", "01bf")),
     u(252, 32, 8, 8, 64), u(253, 32, 8, 8, 64))
case("conv-1x1-stride2-vector", _conv(strides=(2, 2)), u(254, 8, 8, 8, 64), u(255, 1, 1, 64, 128))
# branches of the vector-loader kernel: windows too large for the per-tap offset table (offsets recomputed per tap),
# output features that are no multiple of the tile, rows that are no multiple of the tile, residue classes of
# different sizes sharing one launch
case("conv-fwd-11x11-no-tap-table", _conv(padding=((5, 5), (5, 5))), u(1310, 2, 16, 16, 16), u(1311, 11, 11, 16, 32))
case("conv-wgrad-144-taps-no-tap-table", lambda b, x, g: b.conv(x, g, strides=(1, 1), padding=((1, 1), (1, 1)), dn=("f01b", "i01o", "01bf")),
     u(1312, 32, 12, 12, 64), u(1313, 32, 12, 12, 64))
case("conv-fwd-100-features", _conv(padding=((1, 1), (1, 1))), u(1314, 4, 10, 10, 32), u(1315, 3, 3, 32, 100))
case("conv-fwd-147-rows", _conv(padding=((1, 1), (1, 1))), u(1316, 3, 7, 7, 48), u(1317, 3, 3, 48, 64))
case("conv-dgrad-classes-share-a-launch-odd", lambda b, g, w: b.conv(g, b.reverse(w, [0, 1]), strides=(1, 1), padding=((1, 1), (1, 1)), lhs_dilation=(2, 2), dn=("b01f", "01oi", "b01f")),
     u(1318, 4, 7, 5, 32), u(1319, 3, 3, 16, 32))
# batch-norm statistics taken from the convolution's accumulators: the sum and the sum of squares over every dim but the
# features, right after the convolution (ragged rows and two feature tiles included), and the same sums when the
# convolution cannot deliver them (a split of K) or must not (another reduction kind)
def _conv_stats(padding=((1, 1), (1, 1)), kind="add"):
    def f(b, x, w):
        y = b.conv(x, w, padding=padding)
        axes = list(range(y.ndim - 1))
        if kind == "add":
            return [y, b.reduce_sum(y, axes), b.reduce_sum(b.mul(y, y), axes)]
        return [y, b.reduce_max(y, axes), b.reduce_sum(b.mul(y, y), axes)]
    return f


# (the kernel delivers them only when it runs unsplit, i.e. with a few hundred output tiles; positive inputs, so that the
# sums do not cancel and the elementwise bound is a relative one)
case("conv-statistics-from-accumulators", _conv_stats(), f32(1320, 24, 32, 32, 16, lo=0.05, hi=1.0), f32(1321, 3, 3, 16, 64, lo=0.05, hi=1.0))
case("conv-statistics-ragged-rows-two-feature-tiles", _conv_stats(), f32(1322, 12, 31, 31, 16, lo=0.05, hi=1.0), f32(1323, 3, 3, 16, 128, lo=0.05, hi=1.0))
case("conv-statistics-100-features", _conv_stats(), f32(1324, 12, 31, 31, 16, lo=0.05, hi=1.0), f32(1325, 3, 3, 16, 100, lo=0.05, hi=1.0))
case("conv-statistics-split-k-stays-unfused", _conv_stats(), f32(1326, 2, 4, 4, 256, lo=0.05, hi=1.0), f32(1327, 3, 3, 256, 64, lo=0.05, hi=1.0))
case("conv-statistics-max-stays-unfused", _conv_stats(kind="max"), f32(1328, 24, 32, 32, 16, lo=0.05, hi=1.0), f32(1329, 3, 3, 16, 64, lo=0.05, hi=1.0))
case("conv-bf16", _conv(padding=((1, 1), (1, 1))), u(240, 2, 8, 8, 16), u(241, 3, 3, 16, 8), dtypes=["bf16", "bf16"])

# ------------------------------------------------------------------ reduce (tests/configs/reduction.py:8-39)
case("reduce-sum-all", lambda b, x: b.reduce_sum(x, [0, 1]), f32(250, 37, 53))
case("reduce-sum-rows", lambda b, x: b.reduce_sum(x, [1]), f32(251, 37, 53))
case("reduce-sum-cols", lambda b, x: b.reduce_sum(x, [0]), f32(252, 37, 53))
case("reduce-sum-middle", lambda b, x: b.reduce_sum(x, [1]), f32(253, 5, 19, 12))
case("reduce-sum-outer-two", lambda b, x: b.reduce_sum(x, [0, 1, 2]), f32(254, 4, 9, 9, 16))
case("reduce-sum-nonadjacent", lambda b, x: b.reduce_sum(x, [0, 2]), f32(255, 6, 7, 8))
case("reduce-max", lambda b, x: b.reduce_max(x, [1]), f32(256, 21, 130), exact=True)
case("reduce-min", lambda b, x: b.reduce_min(x, [0]), f32(257, 21, 130), exact=True)
case("reduce-prod", lambda b, x: b._reduce(x, [1], "multiply", 1.0), f32(258, 9, 12, lo=0.5, hi=1.5))
case("reduce-sum-int", lambda b, x: b.reduce_sum(x, [0]), i32(259, 100, 7), exact=True)
case("reduce-and-or", lambda b, x: [b._reduce(x, [1], "and", True), b._reduce(x, [1], "or", False)], rng(260).integers(0, 2, size=(6, 9)).astype(bool), exact=True)
case("reduce-long-row", lambda b, x: b.reduce_sum(x, [1]), f32(261, 3, 70000, lo=-1, hi=1))
case("reduce-tall-column", lambda b, x: b.reduce_sum(x, [0]), f32(262, 50000, 24, lo=-1, hi=1))
case("reduce-full-large", lambda b, x: b.reduce_sum(x, [0]), f32(263, 1 << 20, lo=-1, hi=1))
case("reduce-siblings", lambda b, x: [b.reduce_sum(x, [0, 1, 2]), b.reduce_sum(b.mul(x, x), [0, 1, 2])], f32(264, 8, 12, 12, 32))
case("reduce-fused-input", lambda b, x, m: b.reduce_sum(b.mul(b.sub(x, b.broadcast_in_dim(m, x.shape, [1])), 2.0), [0]), f32(265, 300, 40), f32(266, 40))
case("reduce-bf16", lambda b, x: b.reduce_sum(x, [1]), f32(267, 12, 256), dtypes=["bf16"])
case("softmax-rows", lambda b, x: __import__("jax_mps_amd.shlo.builder", fromlist=["softmax"]).softmax(b, x, -1), f32(268, 33, 100))
case("layer-norm", lambda b, x, s, t: __import__("jax_mps_amd.shlo.builder", fromlist=["layer_norm"]).layer_norm(b, x, s, t, 1e-5), f32(269, 20, 96), f32(270, 96), f32(271, 96))
# row programs at row lengths that take the different walk forms: several unrolled walks with values kept in registers
# between them (the last one ragged), one element per lane, long rows walked by loops, 16-bit rows
def _softmax_of(b, x):
    from jax_mps_amd.shlo.builder import softmax
    return softmax(b, x, -1)


def _layer_norm_of(b, x, s, t):
    from jax_mps_amd.shlo.builder import layer_norm
    return layer_norm(b, x, s, t, 1e-5)


case("softmax-rows-1000", _softmax_of, f32(2730, 37, 1000, lo=-6, hi=6))
case("softmax-rows-777", _softmax_of, f32(2731, 19, 777, lo=-6, hi=6))
case("softmax-rows-5000", _softmax_of, f32(2732, 7, 5000, lo=-6, hi=6))
case("softmax-rows-bf16-768", _softmax_of, f32(2733, 24, 768, lo=-4, hi=4), dtypes=["bf16"])
case("layer-norm-768-bf16", _layer_norm_of, f32(2734, 40, 768), f32(2735, 768), f32(2736, 768), dtypes=["bf16", "bf16", "bf16"])
case("layer-norm-1536", _layer_norm_of, f32(2737, 12, 1536), f32(2738, 1536), f32(2739, 1536))
# per-channel chains with a division and a square root that a large kernel reads through a broadcast: stored by the pass
# that folds the sums they depend on, or by a kernel of their own when they depend on no reduction
def _bn_like(b, x, g):
    n = float(x.shape[0] * x.shape[1])
    mean = b.div(b.reduce_sum(x, [0, 1]), n)
    var = b.sub(b.div(b.reduce_sum(b.mul(x, x), [0, 1]), n), b.mul(mean, mean))
    scale = b.div(g, b.sqrt(b.add(b.maximum(var, 0.0), 1e-5)))
    return b.mul(b.sub(x, b.broadcast_in_dim(mean, x.shape, [2])), b.broadcast_in_dim(scale, x.shape, [2]))


case("per-channel-chain-after-reduce", _bn_like, f32(2740, 96, 50, 64), f32(2741, 64, lo=0.5, hi=1.5))
case("per-channel-chain-no-reduce", lambda b, x, g, v: b.mul(x, b.broadcast_in_dim(b.div(g, b.sqrt(b.add(v, 1e-3))), x.shape, [2])),
     f32(2742, 96, 50, 64), f32(2743, 64, lo=0.5, hi=1.5), f32(2744, 64, lo=0.1, hi=2.0))
# a large elementwise value (batch norm's masked gradient) that a column reduction reads first and elementwise ops read later: the
# reduction's pass stores it on the way (unless the input is small enough for a one-launch reduction of a few workgroups), next to
# sibling reductions, in bf16, and when it is also a result
def _masked_grad_sums(b, x, dy, kept=(3,), also_return=False):
    red = [d for d in range(x.ndim) if d not in kept]
    g = b.select(b.compare(x, b.constant(0.0, x.dtype, x.shape), "GT"), dy, b.constant(0.0, x.dtype, x.shape))
    s1 = b.reduce_sum(g, red)
    s2 = b.reduce_sum(b.mul(g, x), red)
    n = float(np.prod([x.shape[d] for d in red]))
    dx = b.sub(b.sub(g, b.broadcast_in_dim(b.div(s1, n), x.shape, list(kept))), b.mul(x, b.broadcast_in_dim(b.div(s2, n), x.shape, list(kept))))
    return [dx, g] if also_return else dx
case("reduce-column-stores-its-input-two-passes", _masked_grad_sums, f32(2750, 32, 16, 32, 32, lo=-1, hi=1), f32(2751, 32, 16, 32, 32, lo=-1, hi=1))
case("reduce-column-small-input-stored-by-one-pass", lambda b, x, dy: _masked_grad_sums(b, x, dy, kept=(1,)), f32(2752, 128, 512, lo=-1, hi=1), f32(2753, 128, 512, lo=-1, hi=1))
case("reduce-column-tiny-input-keeps-its-own-kernel", lambda b, x, dy: _masked_grad_sums(b, x, dy, kept=(1,)), f32(2761, 24, 96, lo=-1, hi=1), f32(2762, 24, 96, lo=-1, hi=1))
case("reduce-column-stores-its-input-bf16", _masked_grad_sums, f32(2754, 16, 16, 32, 64, lo=-1, hi=1), f32(2755, 16, 16, 32, 64, lo=-1, hi=1), dtypes=["bf16", "bf16"])
case("reduce-column-stores-its-input-also-a-result", lambda b, x, dy: _masked_grad_sums(b, x, dy, also_return=True),
     f32(2756, 32, 16, 16, 64, lo=-1, hi=1), f32(2757, 32, 16, 16, 64, lo=-1, hi=1))
case("reduce-column-input-read-by-a-product-first", lambda b, x, dy, w: (lambda g: [b.matmul(b.reshape(g, (4096, 32)), w), b.reduce_sum(g, [0, 1, 2])])(
     b.select(b.compare(x, b.constant(0.0, "f32", x.shape), "GT"), dy, b.constant(0.0, "f32", x.shape))),
     f32(2758, 16, 16, 16, 32, lo=-1, hi=1), f32(2759, 16, 16, 16, 32, lo=-1, hi=1), f32(2760, 32, 8))
# a reduction finished in one launch whose per-output values ride in the same launch
case("reduce-then-scale-one-pass", lambda b, x: b.div(b.reduce_sum(x, [0]), 300.0), f32(2745, 300, lo=-1, hi=1))
case("reduce-rows-then-scale-one-pass", lambda b, x, w: b.mul(b.reduce_sum(x, [1]), w), f32(2746, 70, 90, lo=-1, hi=1), f32(2747, 70))
# readers of a finished reduction that take it from another position get no place in the pass that finishes it
case("reduce-result-read-transposed", lambda b, x: b.transpose(b.reduce_sum(x, [1]), [1, 0]), f32(2763, 16, 2, 16, lo=-1, hi=1))
case("reduce-result-read-through-slices-and-a-concatenation",
     lambda b, x: (lambda s: b.concatenate([b.slice(s, [0, 0], [8, 8]), b.slice(b.exp(s), [0, 8], [8, 16])], 1))(b.reduce_sum(x, [1])),
     f32(2764, 8, 2, 16, lo=-1, hi=1))
case("reduce-result-read-reversed-and-in-place", lambda b, x: (lambda s: b.add(b.mul(s, 0.5), b.reverse(s, [0])))(b.reduce_max(x, [0])),
     f32(2765, 40, 24, lo=-1, hi=1))
# per-output values that read a padded or concatenated operand (a guarded read) next to the finished result
case("reduce-column-one-pass-scaled-by-a-padded-vector", lambda b, x, w: b.mul(b.reduce_sum(x, [0]), b.pad(w, 1.5, [2], [2])),
     f32(2766, 40, 24, lo=-1, hi=1), f32(2767, 20))
case("reduce-rows-one-pass-scaled-by-a-concatenation", lambda b, x, u, w: b.mul(b.reduce_sum(x, [1]), b.concatenate([u, b.exp(w)], 0)),
     f32(2768, 70, 90, lo=-1, hi=1), f32(2769, 30), f32(2770, 40))
case("reduce-column-two-passes-scaled-by-a-padded-vector", lambda b, x, w: b.mul(b.reduce_sum(x, [0]), b.pad(w, -2.0, [4], [0])),
     f32(2771, 16384, 64, lo=-1, hi=1), f32(2772, 60))
# a reduction over no elements returns its init value
case("reduce-over-an-empty-tensor", lambda b, x, y: [b.reduce_sum(x, [0]), b.reduce_max(x, [0]), b.add(b.reduce_sum(x, [0]), y)],
     np.zeros((0, 4), np.float32), f32(2773, 4), exact=True)
case("argmax-over-an-empty-dim", lambda b, x: b.argmax(x, 1), np.zeros((3, 0), np.float32), exact=True)
# a small sum that a product step writes itself (bias, addend, second product) and that two readers share, one of them a
# product: the readers load the sum, the bare product is not in memory to recompute it from
case("dot-bias-sum-read-by-a-product-and-a-kernel", lambda b, x, w, c, u: (lambda y: b.mul(y, b.logistic(b.matmul(y, u))))(b.add(b.matmul(x, w), b.broadcast_in_dim(c, (4, 8), [1]))),
     f32(2780, 4, 64, lo=-1, hi=1), f32(2781, 64, 8, lo=-0.3, hi=0.3), f32(2782, 8), f32(2783, 8, 8, lo=-0.5, hi=0.5))
case("dot-addend-sum-read-by-a-product-and-a-kernel", lambda b, x, w, y0, u: (lambda y: b.mul(y, b.tanh(b.matmul(y, u))))(b.add(b.tanh(y0), b.matmul(x, w))),
     f32(2784, 16, 24, lo=-1, hi=1), f32(2785, 24, 8, lo=-0.3, hi=0.3), f32(2786, 16, 8), f32(2787, 8, 8, lo=-0.5, hi=0.5))
case("dot-two-products-sum-read-by-a-product-and-a-kernel", lambda b, x, w, h, v, u: (lambda y: b.add(y, b.matmul(y, u)))(b.add(b.matmul(x, w), b.matmul(h, v))),
     f32(2788, 16, 24, lo=-1, hi=1), f32(2789, 24, 8, lo=-0.3, hi=0.3), f32(2790, 16, 12, lo=-1, hi=1), f32(2791, 12, 8, lo=-0.3, hi=0.3), f32(2792, 8, 8, lo=-0.5, hi=0.5))
def _gated_loop(b, x, w, c, u):
    zero = b.constant(0, "i32")
    def body(i, h):
        y = b.add(b.matmul(h, w), b.broadcast_in_dim(c, (4, 8), [1]))
        return [b.add(i, 1), b.mul(y, b.logistic(b.matmul(y, u)))]
    return b.while_loop([zero, x], lambda i, h: b.compare(i, 3, "LT"), body)[1]
case("while-dot-bias-sum-read-by-a-product-and-a-kernel", _gated_loop, f32(2793, 4, 8, lo=-1, hi=1), f32(2794, 8, 8, lo=-0.6, hi=0.6), f32(2795, 8), f32(2796, 8, 8, lo=-0.5, hi=0.5))
# a row program whose per-row result is an output of its own and is also read back, broadcast, by the full-shape result
case("row-program-per-row-result-returned-and-read-back", lambda b, x, y: (lambda v: (lambda r: [r, b.sub(v, b.broadcast_in_dim(r, (378, 2), [0]))])(
     b.rsqrt(b.add(b.abs(b.mul(b.reduce_sum(v, [1]), 0.5)), 1e-3))))(b.mul(x, y)), f32(2797, 378, 2, lo=-1, hi=1), f32(2798, 378, 2, lo=-1, hi=1))
case("row-program-per-row-result-returned-and-read-back-wide", lambda b, x: (lambda m: [m, b.exp(b.sub(x, b.broadcast_in_dim(m, (50, 700), [0])))])(b.reduce_max(x, [1])),
     f32(2799, 50, 700, lo=-2, hi=2))
case("argmax", lambda b, x: b.argmax(x, 1), f32(272, 9, 31), exact=True)
case("argmax-leading-dim", lambda b, x: b.argmax(x, 0), f32(2720, 150, 7), exact=True)
case("argmax-middle-dim-long", lambda b, x: b.argmax(x, 1), f32(2721, 3, 1000, 5), exact=True)
case("argmax-ties-first-occurrence", lambda b, x: b.argmax(x, 1),
     np.array([[1, 3, 3, 2], [5, 5, 5, 5], [-1, -2, -1, -3], [0, -0.0, 0, 0]], np.float32), exact=True)
case("argmax-nan-wins", lambda b, x: b.argmax(x, 1), np.array([[1, np.nan, 3, np.nan], [np.inf, 2, np.inf, 1], [-np.inf, -np.inf, -np.inf, -np.inf]], np.float32), exact=True)
case("argmax-of-fused-input", lambda b, x, y: b.argmax(b.add(b.mul(x, y), 1.0), 1), f32(2722, 64, 10), f32(2723, 64, 10), exact=True)

# ------------------------------------------------------------------ control flow (tests/configs/control_flow.py:66-80,232-263,389-458)
def _sum_to_n(b, n, x):
    # fori-style loop: i from 0 while i < n; acc += x * i
    zero = b.constant(0, "i32")
    out = b.while_loop([zero, b.zeros(x.shape)], lambda i, acc: b.compare(i, n, "LT"),
                       lambda i, acc: [b.add(i, 1), b.add(acc, b.mul(x, b._bcast_np(b.convert(i, "f32"), x.shape)))])
    return out[1]


case("while-sum-0-4", lambda b, x: _sum_to_n(b, 5, x), np.ones((3,), np.float32), exact=True)
case("while-130-iterations", lambda b, x: _sum_to_n(b, 130, x), f32(280, 8), )
case("while-zero-trip", lambda b, x: _sum_to_n(b, 0, x), f32(281, 4), exact=True)


def _dynamic_while(b, x, limit):
    # value-dependent condition: double until the sum exceeds the limit
    out = b.while_loop([x], lambda v: b.compare(b.reduce_sum(v, [0]), limit, "LT"), lambda v: [b.mul(v, 2.0)])
    return out[0]


case("while-value-dependent", _dynamic_while, np.array([1.0, 2.0, 3.0], np.float32), np.float32(100.0), exact=True)


def _traced_bound(b, x, n):
    zero = b.constant(0, "i32")
    out = b.while_loop([zero, x], lambda i, v: b.compare(i, n, "LT"), lambda i, v: [b.add(i, 1), b.add(v, 1.5)])
    return out[1]


case("while-traced-bound", _traced_bound, f32(282, 5), np.int32(7), exact=True)


def _nested(b, x):
    zero = b.constant(0, "i32")

    def outer_body(i, acc):
        inner = b.while_loop([b.constant(0, "i32"), acc], lambda j, a: b.compare(j, 3, "LT"), lambda j, a: [b.add(j, 1), b.add(a, x)])
        return [b.add(i, 1), b.mul(inner[1], 0.5)]
    return b.while_loop([zero, b.zeros(x.shape)], lambda i, acc: b.compare(i, 4, "LT"), outer_body)[1]


case("while-nested", _nested, f32(283, 6))


def _scan_dus(b, xs):
    # scan that stacks running sums: carries (i, acc, out[T, n])
    T, n = xs.shape
    z = b.constant(0, "i32")

    def body(i, acc, out):
        x_t = b.reshape(b.dynamic_slice(xs, [i, b.constant(0, "i32")], [1, n]), (n,))
        acc2 = b.add(acc, x_t)
        return [b.add(i, 1), acc2, b.dynamic_update_slice(out, b.reshape(acc2, (1, n)), [i, b.constant(0, "i32")])]
    return b.while_loop([z, b.zeros((n,)), b.zeros((T, n))], lambda i, a, o: b.compare(i, T, "LT"), body)[2]


case("while-scan-cumsum", _scan_dus, f32(284, 9, 5))


def _swap(b, x, y):
    z = b.constant(0, "i32")
    r = b.while_loop([z, x, y], lambda i, p, q: b.compare(i, 3, "LT"), lambda i, p, q: [b.add(i, 1), q, b.add(p, 1.0)])
    return [r[1], r[2]]


case("while-swapped-carries", _swap, f32(285, 4), f32(286, 4), exact=True)


# loop carries written in place by their producer: the cases where that is and is not allowed
def _loop(b, init, body, trips=5):
    z = b.constant(0, "i32")
    r = b.while_loop([z] + list(init), lambda i, *c: b.compare(i, trips, "LT"), lambda i, *c: [b.add(i, 1)] + list(body(i, *c)))
    return r[1:]


case("while-carry-in-place-elementwise", lambda b, c, f: _loop(b, [c], lambda i, cc: [b.add(b.mul(cc, f), 1.0)]), f32(2300, 6, 40), f32(2301, 6, 40, lo=0.5, hi=1.0), exact=True)
case("while-carry-two-updated-together", lambda b, x, y: _loop(b, [x, y], lambda i, p, q: [b.add(p, q), b.sub(p, q)]), f32(2302, 33), f32(2303, 33, lo=-0.1, hi=0.1))
case("while-carry-read-shifted-by-producer", lambda b, x: _loop(b, [x], lambda i, p: [b.add(p, b.reverse(p, [0]))]), f32(2304, 64, lo=-0.1, hi=0.1))
case("while-carry-rolled", lambda b, x: _loop(b, [x], lambda i, p: [b.concatenate([b.slice(p, [1], [50]), b.slice(p, [0], [1])], 0)]), f32(2305, 50), exact=True)
case("while-carry-old-value-read-after-producer", lambda b, x, w: _loop(b, [x, b.zeros((8, 8))], lambda i, p, acc: (lambda pn: [pn, b.add(acc, b.matmul(p, w))])(b.add(p, 1.0))),
     f32(2306, 8, 8, lo=-0.5, hi=0.5), f32(2307, 8, 8, lo=-0.5, hi=0.5))
case("while-carry-new-value-read-after-producer", lambda b, x, w: _loop(b, [x, b.zeros((8, 8))], lambda i, p, acc: (lambda pn: [pn, b.add(acc, b.matmul(pn, w))])(b.mul(p, 0.9))),
     f32(2308, 8, 8, lo=-0.5, hi=0.5), f32(2309, 8, 8, lo=-0.5, hi=0.5))
case("while-carry-broadcast-row-of-itself", lambda b, x: _loop(b, [x], lambda i, p: [b.add(p, b.broadcast_in_dim(b.reshape(b.slice(p, [0, 0], [1, 16]), (16,)), (4, 16), [1]))]), f32(2310, 4, 16, lo=-0.1, hi=0.1))


# products of a loop-invariant operand with the counter-selected slice of a loop-invariant tensor are taken over the whole tensor
# ahead of the loop (one large product instead of one small one per iteration); the body reads slice i of the result, and slices of
# tensors the loop never writes are addressed by the host.  Reference: the scan path of ops/control_flow.cc:702-989.
def _rnn(b, xs, w, u, index=lambda b, i, T: i, trips=None, carry_xs=False, axis=0):
    T = xs.shape[axis]
    rest = [d for k, d in enumerate(xs.shape) if k != axis]
    h0 = b.constant(0.0, xs.dtype, (rest[0], u.shape[0]))
    zero = b.constant(0, "i32")

    def step(i, h, seq):
        starts = [zero] * xs.ndim
        starts[axis] = index(b, i, T)
        sizes = list(xs.shape)
        sizes[axis] = 1
        x_t = b.reshape(b.dynamic_slice(seq, starts, sizes), rest)
        return b.tanh(b.add(b.matmul(x_t, w), b.matmul(h, u)))
    n = trips if trips is not None else T
    if carry_xs:   # the sequence travels as a carry that the body hands on unchanged, as jax.lax.scan passes its constants
        r = b.while_loop([zero, h0, xs], lambda i, h, q: b.compare(i, n, "LT"), lambda i, h, q: [b.add(i, 1), step(i, h, q), q])
    else:
        r = b.while_loop([zero, h0], lambda i, h: b.compare(i, n, "LT"), lambda i, h: [b.add(i, 1), step(i, h, xs)])
    return r[1]


_RNN = (f32(2500, 12, 6, 20, lo=-1, hi=1), f32(2501, 20, 16, lo=-0.4, hi=0.4), f32(2502, 16, 16, lo=-0.4, hi=0.4))
case("while-hoist-product-of-sequence-slice", lambda b, xs, w, u: _rnn(b, xs, w, u), *_RNN)
case("while-hoist-reversed-index", lambda b, xs, w, u: _rnn(b, xs, w, u, index=lambda b, i, T: b.sub(b.constant(T - 1, "i32"), i)), *_RNN)
case("while-hoist-index-clamped-at-the-end", lambda b, xs, w, u: _rnn(b, xs, w, u, index=lambda b, i, T: b.add(i, 3)), *_RNN)
case("while-hoist-sequence-carried-unchanged", lambda b, xs, w, u: _rnn(b, xs, w, u, carry_xs=True), *_RNN)
case("while-hoist-slice-of-a-middle-dim", lambda b, xs, w, u: _rnn(b, xs, w, u, axis=1), f32(2503, 6, 12, 20, lo=-1, hi=1), _RNN[1], _RNN[2])
case("while-short-loop-over-long-sequence-keeps-its-products", lambda b, xs, w, u: _rnn(b, xs, w, u, trips=3), *_RNN)
case("while-hoist-bf16", lambda b, xs, w, u: _rnn(b, xs, w, u), *_RNN, dtypes=["bf16", "bf16", "bf16"])


def _rnn_rhs_slice(b, xs, w, u):
    # the sliced operand on the right: h' = tanh(W . x_t + U . h) with column-major states
    T, n_in, batch = xs.shape
    zero = b.constant(0, "i32")

    def body(i, h):
        x_t = b.reshape(b.dynamic_slice(xs, [i, zero, zero], [1, n_in, batch]), (n_in, batch))
        return [b.add(i, 1), b.tanh(b.add(b.matmul(w, x_t), b.matmul(u, h)))]
    return b.while_loop([zero, b.zeros((u.shape[0], batch))], lambda i, h: b.compare(i, T, "LT"), body)[1]


# (here the selected dim and the batch dim are apart in memory, so the products stay in the loop)
case("while-slice-is-the-right-operand-free-dims-apart", _rnn_rhs_slice, f32(2504, 9, 20, 6, lo=-1, hi=1), f32(2505, 16, 20, lo=-0.4, hi=0.4), f32(2506, 16, 16, lo=-0.4, hi=0.4))


def _rnn_rhs_rows(b, xs, w, u):
    # the sliced operand on the right with its free dims side by side: h' = tanh(W . x_t^T + U . h), x_t one [batch, n_in] block
    T, batch, n_in = xs.shape
    zero = b.constant(0, "i32")

    def body(i, h):
        x_t = b.reshape(b.dynamic_slice(xs, [i, zero, zero], [1, batch, n_in]), (batch, n_in))
        return [b.add(i, 1), b.tanh(b.add(b.dot_general(w, x_t, ([1], [1])), b.matmul(u, h)))]
    return b.while_loop([zero, b.zeros((u.shape[0], batch))], lambda i, h: b.compare(i, T, "LT"), body)[1]


case("while-hoist-slice-is-the-right-operand", _rnn_rhs_rows, f32(2508, 9, 6, 20, lo=-1, hi=1), f32(2505, 16, 20, lo=-0.4, hi=0.4), f32(2506, 16, 16, lo=-0.4, hi=0.4))


def _two_loops_one_product(b, xs, w, u):
    # a forward loop that stacks its states and a backward loop that recomputes x_t . W: both read one whole product
    T, batch, n_in = xs.shape
    n = u.shape[0]
    zero = b.constant(0, "i32")

    def fwd(i, h, hs):
        x_t = b.reshape(b.dynamic_slice(xs, [i, zero, zero], [1, batch, n_in]), (batch, n_in))
        h2 = b.tanh(b.add(b.matmul(x_t, w), b.matmul(h, u)))
        return [b.add(i, 1), h2, b.dynamic_update_slice(hs, b.reshape(h, (1, batch, n)), [i, zero, zero])]
    f = b.while_loop([zero, b.zeros((batch, n)), b.zeros((T, batch, n))], lambda i, h, hs: b.compare(i, T, "LT"), fwd)
    hs = f[2]

    def bwd(i, g, gw, gu):
        t = b.sub(b.constant(T - 1, "i32"), i)
        x_t = b.reshape(b.dynamic_slice(xs, [t, zero, zero], [1, batch, n_in]), (batch, n_in))
        h_t = b.reshape(b.dynamic_slice(hs, [t, zero, zero], [1, batch, n]), (batch, n))
        y = b.tanh(b.add(b.matmul(x_t, w), b.matmul(h_t, u)))
        gz = b.mul(g, b.sub(1.0, b.mul(y, y)))
        return [b.add(i, 1), b.dot_general(gz, u, ([1], [1])), b.add(gw, b.dot_general(x_t, gz, ([0], [0]))), b.add(gu, b.dot_general(h_t, gz, ([0], [0])))]
    r = b.while_loop([zero, f[1], b.zeros(w.shape), b.zeros(u.shape)], lambda i, g, gw, gu: b.compare(i, T, "LT"), bwd)
    return [f[1], r[1], r[2], r[3]]


case("while-hoist-two-loops-share-the-whole-product", _two_loops_one_product, *_RNN)


def _slice_of_a_changing_carry(b, buf, w):
    # the sliced tensor is a carry that the body rewrites (row i + 1 from row i): neither the product nor the slice may leave the loop
    T, n = buf.shape
    zero = b.constant(0, "i32")

    def body(i, cur, acc):
        row = b.reshape(b.dynamic_slice(cur, [i, zero], [1, n]), (1, n))
        y = b.tanh(b.matmul(row, w))
        nxt = b.dynamic_update_slice(cur, b.add(y, b.reshape(b.dynamic_slice(cur, [b.add(i, 1), zero], [1, n]), (1, n))), [b.add(i, 1), zero])
        return [b.add(i, 1), nxt, b.add(acc, y)]
    r = b.while_loop([zero, buf, b.zeros((1, n))], lambda i, c, a: b.compare(i, T - 1, "LT"), body)
    return [r[1], r[2]]


case("while-slice-of-a-carry-the-body-rewrites", _slice_of_a_changing_carry, f32(2509, 9, 24, lo=-1, hi=1), f32(2510, 24, 24, lo=-0.3, hi=0.3))


def _slices_named_by_the_host(b, xs):
    # xs[i] read elementwise, and a two-row block at 2 * i: contiguous blocks of a tensor the loop never writes
    T, n = xs.shape
    zero = b.constant(0, "i32")

    def body(i, acc):
        row = b.reshape(b.dynamic_slice(xs, [i, zero], [1, n]), (n,))
        pair = b.dynamic_slice(xs, [b.mul(i, 2), zero], [2, n])
        return [b.add(i, 1), b.add(b.mul(acc, 0.5), b.add(b.exp(row), b.reduce_sum(pair, [0])))]
    return b.while_loop([zero, b.zeros((n,))], lambda i, acc: b.compare(i, T // 2, "LT"), body)[1]


case("while-slices-of-an-invariant-tensor", _slices_named_by_the_host, f32(2507, 10, 48, lo=-1, hi=1))


# a scatter inside a counted loop (its launches are replayed from a captured graph): splat operand written by the scatter, a very
# long run, and the result accumulated into a carry
def _scatter_in_loop(b, i, u):
    def body(t, acc):
        x = b.constant(0.0, "f32", (24, 10))
        scale = b.broadcast_in_dim(b.reshape(b.convert(b.add(t, 1), "f32"), (1, 1)), u.shape, (0, 1))
        y = b.scatter(x, b.reshape(i, (i.shape[0], 1)), b.mul(u, scale), update_window_dims=[1], inserted_window_dims=[0],
                      scatter_dims_to_operand_dims=[0], index_vector_dim=1)
        return [b.add(acc, y)]
    return _loop(b, [b.constant(0.0, "f32", (24, 10))], body, trips=4)[0]
case("scatter-add-into-zeros-inside-a-loop", _scatter_in_loop, _runs(2650, (3, 300), (20, 40), (7, 5), (0, 1)), f32(2651, 346, 10), exact=True)

def _case3(b, idx, x):
    return b.case(idx, [lambda: b.mul(x, 2.0), lambda: b.add(x, 10.0), lambda: b.neg(x)], [(x.shape, "f32")])[0]


for k, v in enumerate([0, 1, 2, 5, -1]):
    case(f"case-index-{v}", _case3, np.int32(v), f32(290 + k, 4), exact=True)


# ---- loops whose trip count depends on data (they run in chunks on the device, the host reads one flag per chunk) and
# cases inside loops (all branches run, the selected result is kept)
def _collatz(b, n):
    # steps until n reaches 1 (27 takes 111 steps: several chunks, then iterations past the end that must change nothing)
    one, two, three = b.constant(1, "i32"), b.constant(2, "i32"), b.constant(3, "i32")

    def body(v, steps):
        even = b.compare(b.remainder(v, two), b.constant(0, "i32"), "EQ")
        return [b.select(even, b.div(v, two), b.add(b.mul(v, three), one)), b.add(steps, 1)]
    r = b.while_loop([n, b.constant(0, "i32")], lambda v, steps: b.compare(v, one, "GT"), body)
    return [r[0], r[1]]


for start in (27, 1, 6, 97, 871):
    case(f"while-dynamic-collatz-{start}", _collatz, np.int32(start), exact=True)


def _dynamic_scan(b, xs, limit):
    # carries updated by dynamic_update_slice and a running sum; stops when the sum passes a limit given at run time
    T, n = xs.shape
    z = b.constant(0, "i32")

    def body(i, acc, out):
        x_t = b.reshape(b.dynamic_slice(xs, [i, z], [1, n]), (n,))
        acc2 = b.add(acc, x_t)
        return [b.add(i, 1), acc2, b.dynamic_update_slice(out, b.reshape(acc2, (1, n)), [i, z])]

    def cond(i, acc, out):
        return b.and_(b.compare(i, T, "LT"), b.compare(b.reduce_sum(acc, [0]), limit, "LT"))
    r = b.while_loop([z, b.zeros((n,)), b.zeros((T, n))], cond, body)
    return [r[0], r[1], r[2]]


case("while-dynamic-scan-stops-early", _dynamic_scan, f32(2400, 40, 6, lo=0.0, hi=1.0), np.float32(30.0))
case("while-dynamic-scan-runs-out", _dynamic_scan, f32(2401, 40, 6, lo=0.0, hi=1.0), np.float32(1e9))
case("while-dynamic-zero-trip", _dynamic_scan, f32(2402, 40, 6, lo=0.0, hi=1.0), np.float32(-1.0), exact=True)


def _dynamic_nested(b, n, x):
    # outer loop bounded by an argument; inner loop halves a value until it is small (also data dependent); on the
    # iterations queued past the end of the outer loop the inner one must not run at all
    z = b.constant(0, "i32")

    def outer(i, acc):
        start = b.add(b._bcast_np(b.convert(i, "f32"), x.shape), x)
        inner = b.while_loop([start, b.constant(0, "i32")], lambda v, k: b.compare(b.reduce_max(b.abs(v), [0]), 0.25, "GT"),
                             lambda v, k: [b.mul(v, 0.5), b.add(k, 1)])
        return [b.add(i, 1), b.add(acc, b.convert(inner[1], "f32"))]
    r = b.while_loop([z, b.constant(0.0, "f32")], lambda i, acc: b.compare(i, n, "LT"), outer)
    return [r[0], r[1]]


case("while-dynamic-nested", _dynamic_nested, np.int32(6), f32(2403, 5, lo=0.5, hi=1.0), exact=True)


def _case_in_loop(b, sel, x):
    # a three-way switch on a value read from an argument vector inside a counted loop
    z = b.constant(0, "i32")

    def body(i, acc):
        idx = b.reshape(b.dynamic_slice(sel, [i], [1]), ())
        y = b.case(idx, [lambda: b.mul(acc, 2.0), lambda: b.add(acc, x), lambda: b.neg(acc)], [(x.shape, "f32")])[0]
        return [b.add(i, 1), y]
    return b.while_loop([z, x], lambda i, acc: b.compare(i, 8, "LT"), body)[1]


case("case-inside-counted-loop", _case_in_loop, np.array([0, 1, 2, 1, 7, -3, 0, 1], np.int32), f32(2404, 6), exact=True)


def _case_in_dynamic_loop(b, sel, x, n):
    z = b.constant(0, "i32")

    def body(i, acc):
        idx = b.reshape(b.dynamic_slice(sel, [i], [1]), ())
        y = b.case(idx, [lambda: b.mul(acc, 0.5), lambda: b.add(acc, x)], [(x.shape, "f32")])[0]
        return [b.add(i, 1), y]
    return b.while_loop([z, x], lambda i, acc: b.compare(i, n, "LT"), body)[1]


case("case-inside-dynamic-loop", _case_in_dynamic_loop, np.array([0, 1, 1, 0, 1, 1, 1, 0, 0, 1], np.int32), f32(2405, 6), np.int32(7), exact=True)

# ------------------------------------------------------------------ one device: collectives, ids, tokens
# (reference tests: tests/configs/collectives.py:35-56 run pmap(pmean) and pmap(axis_index) over one device;
# tests/test_control_flow_compile.py:95-133 pass tokens into, through and out of jitted functions.  The programs
# below are the text such functions lower to, written by hand.)
text_case("all-reduce-one-device-pmean", """module @pmap_f attributes {mhlo.num_partitions = 1 : i32, mhlo.num_replicas = 1 : i32} {
  func.func public @main(%arg0: tensor<1x4xf32>) -> tensor<1x4xf32> {
    %0 = stablehlo.reshape %arg0 : (tensor<1x4xf32>) -> tensor<4xf32>
    %1 = "stablehlo.all_reduce"(%0) <{replica_groups = dense<0> : tensor<1x1xi64>}> ({
    ^bb0(%arg1: tensor<f32>, %arg2: tensor<f32>):
      %5 = stablehlo.add %arg1, %arg2 : tensor<f32>
      stablehlo.return %5 : tensor<f32>
    }) : (tensor<4xf32>) -> tensor<4xf32>
    %cst = stablehlo.constant dense<1.000000e+00> : tensor<f32>
    %2 = stablehlo.broadcast_in_dim %cst, dims = [] : (tensor<f32>) -> tensor<4xf32>
    %3 = stablehlo.divide %1, %2 : tensor<4xf32>
    %4 = stablehlo.reshape %3 : (tensor<4xf32>) -> tensor<1x4xf32>
    return %4 : tensor<1x4xf32>
  }
}
""", f32(2501, 1, 4), exact=True)

text_case("all-reduce-one-device-two-operands", """module @jit_f attributes {mhlo.num_partitions = 1 : i32, mhlo.num_replicas = 1 : i32} {
  func.func public @main(%arg0: tensor<3x5xf32>, %arg1: tensor<7xi32>) -> (tensor<3x5xf32>, tensor<7xi32>) {
    %0 = stablehlo.multiply %arg0, %arg0 : tensor<3x5xf32>
    %1:2 = "stablehlo.all_reduce"(%0, %arg1) <{channel_handle = #stablehlo.channel_handle<handle = 1, type = 1>, replica_groups = dense<0> : tensor<1x1xi64>, use_global_device_ids}> ({
    ^bb0(%arg2: tensor<f32>, %arg3: tensor<f32>):
      %3 = stablehlo.maximum %arg2, %arg3 : tensor<f32>
      stablehlo.return %3 : tensor<f32>
    }) : (tensor<3x5xf32>, tensor<7xi32>) -> (tensor<3x5xf32>, tensor<7xi32>)
    %2 = stablehlo.add %1#1, %1#1 : tensor<7xi32>
    return %1#0, %2 : tensor<3x5xf32>, tensor<7xi32>
  }
}
""", f32(2502, 3, 5), i32(2503, 7), exact=True)

text_case("partition-id-axis-index-zero", """module @pmap_f attributes {mhlo.num_partitions = 1 : i32, mhlo.num_replicas = 1 : i32} {
  func.func public @main(%arg0: tensor<1x4xi32>) -> (tensor<1x4xi32>, tensor<ui32>) {
    %0 = stablehlo.reshape %arg0 : (tensor<1x4xi32>) -> tensor<4xi32>
    %1 = stablehlo.partition_id : tensor<ui32>
    %2 = stablehlo.convert %1 : (tensor<ui32>) -> tensor<i32>
    %3 = stablehlo.broadcast_in_dim %2, dims = [] : (tensor<i32>) -> tensor<4xi32>
    %4 = stablehlo.add %0, %3 : tensor<4xi32>
    %5 = stablehlo.reshape %4 : (tensor<4xi32>) -> tensor<1x4xi32>
    %6 = stablehlo.replica_id : tensor<ui32>
    return %5, %6 : tensor<1x4xi32>, tensor<ui32>
  }
}
""", np.arange(4, dtype=np.int32).reshape(1, 4), exact=True)

text_case("token-created-merged-and-returned", """module @jit_f {
  func.func public @main(%arg0: tensor<f32>, %arg1: !stablehlo.token) -> (tensor<f32>, !stablehlo.token) {
    %0 = stablehlo.create_token : !stablehlo.token
    %1 = stablehlo.after_all %0, %arg1 : !stablehlo.token
    %cst = stablehlo.constant dense<1.000000e+00> : tensor<f32>
    %2 = stablehlo.add %arg0, %cst : tensor<f32>
    return %2, %1 : tensor<f32>, !stablehlo.token
  }
}
""", np.float32(3.0), np.float32(7.0), exact=True)

text_case("token-argument-returned-as-is", """module @jit_f {
  func.func public @main(%arg0: !stablehlo.token, %arg1: tensor<6xf32>) -> (!stablehlo.token, tensor<6xf32>) {
    %0 = stablehlo.multiply %arg1, %arg1 : tensor<6xf32>
    return %arg0, %0 : !stablehlo.token, tensor<6xf32>
  }
}
""", np.float32(5.0), f32(2504, 6), exact=True)

text_case("token-carried-by-a-loop", """module @jit_f {
  func.func public @main(%arg0: tensor<4xf32>) -> (tensor<4xf32>, !stablehlo.token) {
    %tok = stablehlo.create_token : !stablehlo.token
    %c0 = stablehlo.constant dense<0> : tensor<i32>
    %0:3 = stablehlo.while(%iterArg = %c0, %iterArg_0 = %arg0, %iterArg_1 = %tok) : tensor<i32>, tensor<4xf32>, !stablehlo.token
     cond {
      %c3 = stablehlo.constant dense<3> : tensor<i32>
      %1 = stablehlo.compare  LT, %iterArg, %c3,  SIGNED : (tensor<i32>, tensor<i32>) -> tensor<i1>
      stablehlo.return %1 : tensor<i1>
    } do {
      %c1 = stablehlo.constant dense<1> : tensor<i32>
      %1 = stablehlo.add %iterArg, %c1 : tensor<i32>
      %2 = stablehlo.add %iterArg_0, %iterArg_0 : tensor<4xf32>
      %3 = stablehlo.after_all %iterArg_1 : !stablehlo.token
      stablehlo.return %1, %2, %3 : tensor<i32>, tensor<4xf32>, !stablehlo.token
    }
    return %0#1, %0#2 : tensor<4xf32>, !stablehlo.token
  }
}
""", f32(2505, 4), exact=True)


def all_cases() -> List[Case]:
    return [mk() for mk in _cases]


def raw_case(name, text, *inputs, dtypes, exact=False):
    """A case given as module text (forms the builder does not print)."""
    def make():
        return Case(name, text, [np.asarray(a) for a in inputs], list(dtypes), exact)
    make.case_name = name
    _cases.append(make)


raw_case("text-hex-constant-bool-list-barrier-sharding-call", """module @jit_f attributes {mhlo.num_partitions = 1 : i32, mhlo.num_replicas = 1 : i32} {
  func.func public @main(%arg0: tensor<3xf32> {mhlo.layout_mode = "default"}, %arg1: tensor<2x4xf32> {jax.buffer_donor = true}) -> (tensor<3xf32> {jax.result_info = "[0]"}, tensor<2xi1>, tensor<1x2xf32>) {
    %cst = stablehlo.constant dense<"0x0000803F0000004000004040"> : tensor<3xf32>
    %c = stablehlo.constant dense<[true, false]> : tensor<2xi1>
    %c_0 = stablehlo.constant dense<true> : tensor<i1>
    %cst_2 = stablehlo.constant dense<1.500000e+00> : tensor<3xf32>
    %0 = stablehlo.add %arg0, %cst : tensor<3xf32>
    %1 = stablehlo.multiply %0, %cst_2 : tensor<3xf32>
    %2 = stablehlo.broadcast_in_dim %c_0, dims = [] : (tensor<i1>) -> tensor<2xi1>
    %3 = stablehlo.and %c, %2 : tensor<2xi1>
    %c_3 = stablehlo.constant dense<1> : tensor<i32>
    %c_4 = stablehlo.constant dense<0> : tensor<i32>
    %4 = stablehlo.dynamic_slice %arg1, %c_4, %c_3, sizes = [1, 2] : (tensor<2x4xf32>, tensor<i32>, tensor<i32>) -> tensor<1x2xf32>
    %5 = stablehlo.custom_call @Sharding(%4) {backend_config = "", mhlo.sharding = "{replicated}"} : (tensor<1x2xf32>) -> tensor<1x2xf32>
    %6 = stablehlo.optimization_barrier %5 : tensor<1x2xf32>
    return %1, %3, %6 : tensor<3xf32>, tensor<2xi1>, tensor<1x2xf32>
  }
}
""", np.array([10, 20, 30], np.float32), np.arange(8, dtype=np.float32).reshape(2, 4), dtypes=["f32", "f32"], exact=True)


def case_names() -> List[str]:
    return [mk.case_name for mk in _cases]


def get_case(name: str) -> Case:
    for mk in _cases:
        if mk.case_name == name:
            return mk()
    raise KeyError(name)


# ------------------------------------------------------------------ sort (reference tests: tests/configs/sort.py:13-135 use
# random inputs against JAX-CPU; here the same forms, checked bit-for-bit against the oracle, which tests/test_oracle_pins.py
# pins to numpy's stable sorts)
def _with_ties(seed, *shape):
    return (np.round(f32(seed, *shape, lo=-3, hi=3) * 2) / 2 + np.float32(0.0)).astype(np.float32)   # + 0.0: no negative zeros (total order tells them apart)


_SORT_NAN = np.array([[3.0, np.nan, -1.0, 2.0, -np.inf, np.inf, -0.0, 0.0, np.nan, 2.0]], np.float32)
case("sort-1d", lambda b, x: b.sort([x]), f32(2100, 1000), exact=True)
case("sort-1d-odd-length", lambda b, x: b.sort([x]), f32(2101, 777), exact=True)
case("sort-2d-axis0", lambda b, x: b.sort([x], dimension=0), f32(2102, 37, 20), exact=True)
case("sort-3d-axis1", lambda b, x: b.sort([x], dimension=1), f32(2103, 3, 50, 7), exact=True)
case("sort-descending", lambda b, x: b.sort([x], descending=True), _with_ties(2104, 4, 64), exact=True)
case("sort-nan-and-signed-zero-total-order", lambda b, x: b.sort([x]), _SORT_NAN, exact=True)
case("sort-int32", lambda b, x: b.sort([x]), i32(2105, 5, 300, lo=-1000, hi=1000), exact=True)
case("sort-uint8", lambda b, x: b.sort([x], descending=True), rng(2106).integers(0, 256, size=(3, 100)).astype(np.uint8), exact=True)
case("sort-bool", lambda b, x: b.sort([x]), rng(2107).integers(0, 2, size=(2, 33)).astype(np.bool_), exact=True)
case("sort-key-val-stable-ties", lambda b, k, v: b.sort([k, v], dimension=1), _with_ties(2108, 4, 200), f32(2109, 4, 200), exact=True)
case("sort-argsort-descending-ties", lambda b, k: b.sort([k, b.iota(k.shape, 1, "i32")], dimension=1, descending=True), _with_ties(2110, 6, 129), exact=True)
case("sort-two-keys-lexicographic", lambda b, k0, k1, v: b.sort([k0, k1, v], dimension=0, num_keys=2),
     rng(2111).integers(0, 4, size=(500,)).astype(np.int32), _with_ties(2112, 500), f32(2113, 500), exact=True)
case("sort-custom-comparator-abs", lambda b, x: b.sort([x], comparator=lambda bb, l, r: bb.compare(bb.abs(l[0]), bb.abs(r[0]), "LT")), _with_ties(2114, 3, 100), exact=True)
case("sort-bf16-keys", lambda b, k, v: b.sort([k, v]), f32(2115, 2, 256), i32(2116, 2, 256), dtypes=["bf16", "i32"], exact=True)
case("sort-4096", lambda b, x: b.sort([x]), f32(2117, 2, 4096), exact=True)
case("sort-long-slice-in-memory", lambda b, x: b.sort([x]), f32(2119, 20000), exact=True)
case("sort-long-key-val-in-memory", lambda b, k, v: b.sort([k, v], dimension=0, descending=True), _with_ties(2120, 9000, 2), i32(2121, 9000, 2), exact=True)
case("sort-fused-producer-and-consumer", lambda b, x: b.mul(b.sort([b.neg(x)])[0], 2.0), f32(2118, 8, 100), exact=True)


# top_k (reference tests: tests/configs/sort.py:140-210): shapes of the reference's cases plus ties, NaN and a vocabulary-sized row
case("top-k-1d", lambda b, x: list(b.top_k(x, 3)), f32(2130, 16), exact=True)
case("top-k-2d-k1", lambda b, x: list(b.top_k(x, 1)), f32(2131, 4, 8), exact=True)
case("top-k-2d-k5", lambda b, x: list(b.top_k(x, 5)), f32(2132, 4, 8), exact=True)
case("top-k-4d", lambda b, x: list(b.top_k(x, 3)), f32(2133, 2, 2, 4, 8), exact=True)
case("top-k-transposed-input", lambda b, x: list(b.top_k(b.transpose(x, [2, 1, 0]), 2)), f32(2134, 2, 4, 8), exact=True)
case("top-k-equals-size", lambda b, x: list(b.top_k(x, 8)), f32(2135, 4, 8), exact=True)
case("top-k-ties-lowest-index-first", lambda b, x: list(b.top_k(x, 6)), _with_ties(2136, 5, 40), exact=True)
case("top-k-nan-first", lambda b, x: list(b.top_k(x, 4)), _SORT_NAN, exact=True)
text_case("top-k-custom-call-spelling", """module @jit_f {
  func.func public @main(%arg0: tensor<3x12xf32>) -> (tensor<3x4xf32>, tensor<3x4xi32>) {
    %0:2 = stablehlo.custom_call @mhlo.topk(%arg0) {mhlo.attributes = {k = 4 : i64, largest = true}, mhlo.version = 1 : i64} : (tensor<3x12xf32>) -> (tensor<3x4xf32>, tensor<3x4xi32>)
    return %0#0, %0#1 : tensor<3x4xf32>, tensor<3x4xi32>
  }
}
""", f32(2138, 3, 12), exact=True)
case("top-k-int32", lambda b, x: list(b.top_k(x, 7)), i32(2137, 3, 100), exact=True)
case("top-k-vocabulary-row", lambda b, x: list(b.top_k(x, 50)), f32(2138, 2, 8000), exact=True)


# ------------------------------------------------------------------ rng_bit_generator: counter update as the reference
# keeps it (src/pjrt_plugin/ops/control_flow.cc:2343-2355); bits = threefry2x32 of (key halves; element index, counter)
_RNG_STATE = np.array([0x0123456789ABCDEF, 41], dtype=np.uint64)
case("rng-bits-u32", lambda b, st: list(b.rng_bit_generator(st, (1000,), "ui32", "THREE_FRY")), _RNG_STATE, exact=True)
case("rng-bits-u32-2d-default", lambda b, st: list(b.rng_bit_generator(st, (7, 33), "ui32")), _RNG_STATE, exact=True)
case("rng-bits-u64", lambda b, st: list(b.rng_bit_generator(st, (129,), "ui64", "PHILOX")), _RNG_STATE, exact=True)
case("rng-bits-u8", lambda b, st: list(b.rng_bit_generator(st, (50,), "ui8")), _RNG_STATE, exact=True)
case("rng-bits-i32", lambda b, st: list(b.rng_bit_generator(st, (64,), "i32")), _RNG_STATE, exact=True)
case("rng-bits-chained", lambda b, st: (lambda s1, b1: (lambda s2, b2: [s2, b1, b2])(*b.rng_bit_generator(s1, (16,), "ui32")))(*b.rng_bit_generator(st, (16,), "ui32")),
     np.array([7, 0xFFFFFFFFFFFFFFFF], dtype=np.uint64), exact=True)
case("rng-uniform-floats", lambda b, st: (lambda s1, bits: b.sub(b.bitcast_convert(b.or_(b.shift_right_logical(bits, b.constant(np.uint32(9), "ui32", bits.shape)),
                                                                                        b.constant(np.uint32(0x3F800000), "ui32", bits.shape)), "f32"),
                                                               b.constant(np.float32(1), "f32", bits.shape)))(*b.rng_bit_generator(st, (4096,), "ui32")), _RNG_STATE, exact=True)


# ------------------------------------------------------------------ threefry2x32 as JAX lowers it without a custom call:
# plain ui32 adds, xors and rotations (reference kernel text: src/pjrt_plugin/ops/control_flow.cc:1351-1390); the whole
# block cipher fuses into one generated kernel.  Inputs are the Random123 known-answer vectors.
def threefry2x32(b, k0, k1, c0, c1):
    u = lambda x: b.constant(np.uint32(x), "ui32", k0.shape)
    rotl = lambda x, r: b.or_(b.shift_left(x, u(r)), b.shift_right_logical(x, u(32 - r)))
    ks = [k0, k1, b.xor(b.xor(k0, k1), u(0x1BD11BDA))]
    x0, x1 = b.add(c0, ks[0]), b.add(c1, ks[1])
    rots = [(13, 15, 26, 6), (17, 29, 16, 24)]
    for blk in range(5):
        for r in rots[blk % 2]:
            x0 = b.add(x0, x1)
            x1 = b.xor(x0, rotl(x1, r))
        x0 = b.add(x0, ks[(blk + 1) % 3])
        x1 = b.add(x1, b.add(ks[(blk + 2) % 3], u(blk + 1)))
    return x0, x1


THREEFRY_KAT = dict(
    key0=np.array([0x00000000, 0xFFFFFFFF, 0x13198A2E], np.uint32), key1=np.array([0x00000000, 0xFFFFFFFF, 0x03707344], np.uint32),
    ctr0=np.array([0x00000000, 0xFFFFFFFF, 0x243F6A88], np.uint32), ctr1=np.array([0x00000000, 0xFFFFFFFF, 0x85A308D3], np.uint32),
    out0=np.array([0x6B200159, 0x1CB996FC, 0xC4923A9C], np.uint32), out1=np.array([0x99BA4EFE, 0xBB002BE7, 0x483DF7A0], np.uint32))
case("threefry2x32-known-answers", threefry2x32, THREEFRY_KAT["key0"], THREEFRY_KAT["key1"], THREEFRY_KAT["ctr0"], THREEFRY_KAT["ctr1"], exact=True)
case("threefry2x32-stream", threefry2x32, np.full(5000, 42, np.uint32), np.full(5000, 7, np.uint32), np.arange(5000, dtype=np.uint32), np.zeros(5000, np.uint32), exact=True)


# ------------------------------------------------------------------ pooling: reduce_window / select_and_scatter (tests/configs/reduction.py:87-342)
NHWC_PAD1 = [(0, 0), (1, 1), (1, 1), (0, 0)]
case("maxpool-3x3-s2-pad1", lambda b, x: b.reduce_window(x, float("-inf"), "max", (1, 3, 3, 1), (1, 2, 2, 1), NHWC_PAD1), f32(3000, 4, 17, 15, 24), exact=True)
case("sumpool-2x2-s2", lambda b, x: b.reduce_window(x, 0.0, "add", (1, 2, 2, 1), (1, 2, 2, 1)), f32(3001, 2, 16, 16, 8))
case("minpool-dilated-window", lambda b, x: b.reduce_window(x, float("inf"), "min", (1, 2, 3, 1), (1, 1, 2, 1), [(0, 0), (1, 0), (2, 1), (0, 0)], window_dilation=(1, 2, 2, 1)), f32(3002, 2, 9, 11, 3), exact=True)
case("sumpool-base-dilation", lambda b, x: b.reduce_window(x, 0.0, "add", (2, 3), (1, 1), [(1, 1), (0, 2)], base_dilation=(2, 3)), f32(3003, 5, 6))
case("reduce_window-scalar", lambda b, x: b.reduce_window(x, 0.0, "add", (), (), []), np.float32(2.5), exact=True)
case("maxpool-bf16", lambda b, x: b.reduce_window(x, float("-inf"), "max", (1, 3, 3, 1), (1, 2, 2, 1), NHWC_PAD1), f32(3004, 2, 8, 8, 16), dtypes=["bf16"], exact=True)
case("maxpool-grad-3x3-s2-pad1", lambda b, x, g: b.select_and_scatter(x, g, 0.0, (1, 3, 3, 1), (1, 2, 2, 1), NHWC_PAD1), f32(3005, 2, 9, 8, 6), f32(3006, 2, 5, 4, 6))
case("maxpool-grad-ties", lambda b, x, g: b.select_and_scatter(x, g, 0.0, (1, 2, 2, 1), (1, 1, 1, 1)),
     np.round(f32(3007, 1, 6, 6, 2) * 2).astype(np.float32), f32(3008, 1, 5, 5, 2))
case("minpool-grad", lambda b, x, g: b.select_and_scatter(x, g, 0.0, (1, 2, 2, 1), (1, 2, 2, 1), direction="LE"), f32(3009, 2, 6, 6, 4), f32(3010, 2, 3, 3, 4))

# windows of more than 64 elements that are not cumulative sums: reduced dim after dim
case("avgpool-whole-16x16-extent", lambda b, x: b.mul(b.reduce_window(x, 0.0, "add", (1, 16, 16, 1), (1, 1, 1, 1)), 1.0 / 256), f32(3030, 2, 16, 16, 8))
case("maxpool-9x9-s2-pad4", lambda b, x: b.reduce_window(x, float("-inf"), "max", (1, 9, 9, 1), (1, 2, 2, 1), [(0, 0), (4, 4), (4, 4), (0, 0)]), f32(3031, 2, 20, 17, 4), exact=True)
case("sumpool-5x5x5-dilated-int", lambda b, x: b.reduce_window(x, 0, "add", (5, 5, 5), (2, 1, 1), [(2, 2), (0, 3), (1, 0)], (1, 2, 1), (1, 1, 2)),
     rng(3032).integers(-9, 9, size=(11, 9, 12)).astype(np.int32), exact=True)

# cumulative reductions as JAX lowers them: a reduce_window over one whole dim padded by n-1 (tests/configs/reduction.py:41-77)
case("cumsum-axis1", lambda b, x: b.reduce_window(x, 0.0, "add", (1, 300), (1, 1), [(0, 0), (299, 0)]), f32(3020, 7, 300))
case("cumsum-axis0-int", lambda b, x: b.reduce_window(x, 0, "add", (200, 1), (1, 1), [(199, 0), (0, 0)]), rng(3021).integers(-50, 50, size=(200, 9)).astype(np.int32), exact=True)
case("cummax-reverse", lambda b, x: b.reduce_window(x, float("-inf"), "max", (1, 1, 130), (1, 1, 1), [(0, 0), (0, 0), (0, 129)]), f32(3022, 3, 4, 130), exact=True)
case("cumprod-axis1", lambda b, x: b.reduce_window(x, 1.0, "mul", (1, 100), (1, 1), [(0, 0), (99, 0)]), f32(3023, 5, 100, lo=0.9, hi=1.1))


# ------------------------------------------------------------------ fused-op custom calls of the reference's Python layer
# (src/jax_plugins/mps/ops.py:52-596: the primitives lower to stablehlo.custom_call @mps.<op> with a JSON backend_config;
# executor side src/pjrt_plugin/ops/control_flow.cc:1484-2020).  Forward and backward forms, float32 and bfloat16.
def _fused(target, n_out, config=""):
    def fn(b, *args):
        shapes = {"sdpa_bwd": [0, 1, 2], "sdpa_causal_bwd": [0, 1, 2], "rms_norm_bwd": [0, 1], "layer_norm_bwd": [0, 1, 2]}.get(target, [0])
        return b.custom_call("mps." + target, list(args), [(args[k].shape, args[k].dtype) for k in shapes[:n_out]], config)
    return fn


def _sd(seed, *shape, scale=1.0):
    return (rng(seed).standard_normal(shape) * scale).astype(np.float32)


_Q, _K, _V, _G = _sd(4000, 2, 4, 24, 16), _sd(4001, 2, 4, 40, 16), _sd(4002, 2, 4, 40, 16), _sd(4003, 2, 4, 24, 16)
_KG, _VG = _sd(4004, 2, 2, 40, 16), _sd(4005, 2, 2, 40, 16)                       # two key / value heads for four query heads
_PAD_MASK = np.broadcast_to(np.arange(40)[None, None, None, :] < np.array([40, 29])[:, None, None, None], (2, 1, 1, 40)).copy()
_FULL_MASK = rng(4006).random((2, 4, 24, 40)) > 0.25
_BIAS = _sd(4007, 4, 24, 40, scale=0.5)
for dt in ("f32", "bf16"):
    d4, d5 = [dt] * 3 + ["i1"], [dt] * 3 + ["i1", dt]
    case(f"fused-sdpa-padding-mask-{dt}", _fused("sdpa", 1, '{"scale": 0.25}'), _Q, _K, _V, _PAD_MASK, dtypes=d4)
    case(f"fused-sdpa-grouped-heads-{dt}", _fused("sdpa", 1, '{"scale": 0.25}'), _Q, _KG, _VG, _PAD_MASK, dtypes=d4)
    case(f"fused-sdpa-full-mask-{dt}", _fused("sdpa", 1, '{"scale": 0.3}'), _Q, _K, _V, _FULL_MASK, dtypes=d4)
    case(f"fused-sdpa-additive-bias-{dt}", _fused("sdpa", 1, '{"scale": 0.25}'), _Q, _K, _V, _BIAS, dtypes=[dt] * 4)
    case(f"fused-sdpa-causal-{dt}", _fused("sdpa_causal", 1, '{"scale": 0.25}'), _Q, _K[:, :, :24], _V[:, :, :24], dtypes=[dt] * 3)
    case(f"fused-sdpa-causal-longer-keys-{dt}", _fused("sdpa_causal", 1, '{"scale": 0.25}'), _Q, _K, _V, dtypes=[dt] * 3)
    case(f"fused-sdpa-bwd-{dt}", _fused("sdpa_bwd", 3, '{"scale": 0.25}'), _Q, _K, _V, _PAD_MASK, _G, dtypes=d5)
    case(f"fused-sdpa-bwd-grouped-heads-{dt}", _fused("sdpa_bwd", 3, '{"scale": 0.25}'), _Q, _KG, _VG, _PAD_MASK, _G, dtypes=d5)
    case(f"fused-sdpa-causal-bwd-{dt}", _fused("sdpa_causal_bwd", 3, '{"scale": 0.25}'), _Q, _K[:, :, :24], _V[:, :, :24], _G, dtypes=[dt] * 4)
    case(f"fused-rms-norm-{dt}", _fused("rms_norm", 1, '{"eps": 1e-06}'), _sd(4010, 6, 33, 96), 1.0 + _sd(4011, 96, scale=0.1), dtypes=[dt] * 2)
    case(f"fused-rms-norm-bwd-{dt}", _fused("rms_norm_bwd", 2, '{"eps": 1e-06}'), _sd(4010, 6, 33, 96), 1.0 + _sd(4011, 96, scale=0.1), _sd(4012, 6, 33, 96),
         dtypes=[dt] * 3)
    case(f"fused-layer-norm-{dt}", _fused("layer_norm", 1, '{"eps": 1e-05}'), _sd(4013, 50, 200), 1.0 + _sd(4014, 200, scale=0.1), _sd(4015, 200, scale=0.1),
         dtypes=[dt] * 3)
    case(f"fused-layer-norm-bwd-{dt}", _fused("layer_norm_bwd", 3, '{"eps": 1e-05}'), _sd(4013, 50, 200), 1.0 + _sd(4014, 200, scale=0.1),
         _sd(4015, 200, scale=0.1), _sd(4016, 50, 200), dtypes=[dt] * 4)
    case(f"fused-rope-{dt}", _fused("rope", 1, '{"dims": 32, "traditional": false, "base": 10000.0, "rope_scale": 1.0}'), _sd(4017, 2, 3, 17, 32),
         np.int32(5), dtypes=[dt, "i32"])
    case(f"fused-rope-partial-traditional-{dt}", _fused("rope", 1, '{"dims": 16, "traditional": true, "base": 500.0, "rope_scale": 0.5}'),
         _sd(4018, 2, 3, 17, 40), np.int32(0), dtypes=[dt, "i32"])
    case(f"fused-rope-bwd-{dt}", _fused("rope_bwd", 1, '{"dims": 24, "traditional": false, "base": 10000.0, "rope_scale": 1.0}'), _sd(4019, 2, 9, 40),
         np.int32(3), _sd(4020, 2, 9, 40), dtypes=[dt, "i32", dt])
    case(f"fused-gelu-{dt}", _fused("gelu", 1), _sd(4021, 37, 130, scale=2.0), dtypes=[dt])
    case(f"fused-gelu-bwd-{dt}", _fused("gelu_bwd", 1), _sd(4021, 37, 130, scale=2.0), _sd(4022, 37, 130), dtypes=[dt] * 2)
# the attention of the DistilBERT-shaped benchmark as one custom call: 12 heads of 128 x 128 x 64, padding mask
case("fused-sdpa-encoder-heads-bf16", _fused("sdpa", 1, '{"scale": 0.125}'), _sd(4030, 2, 12, 128, 64), _sd(4031, 2, 12, 128, 64), _sd(4032, 2, 12, 128, 64),
     np.broadcast_to(np.arange(128)[None, None, None, :] < np.array([128, 77])[:, None, None, None], (2, 1, 1, 128)).copy(), dtypes=["bf16"] * 3 + ["i1"])
case("fused-sdpa-causal-encoder-heads-bf16", _fused("sdpa_causal", 1, '{"scale": 0.125}'), _sd(4030, 2, 12, 128, 64), _sd(4031, 2, 12, 128, 64),
     _sd(4032, 2, 12, 128, 64), dtypes=["bf16"] * 3)
