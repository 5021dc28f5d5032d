"""Writes tests/golden/cases.json: literal-valued cases restated from the reference's own tests
(tests/configs/slice.py:33-43,175-295,391-456; tests/configs/control_flow.py:66-80,93-206,232-263;
tests/configs/matmul.py:221-249; tests/configs/misc.py:161-167), each with the StableHLO module the
case lowers to, its inputs, and the expected outputs computed here by an independent closed form
(plain numpy indexing / arithmetic) — never by the oracle under test.

Run from the repo root:  python tests/golden/make_golden.py
"""
import json
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

from jax_mps_amd.shlo.builder import Builder, _NP  # noqa: E402

_MLIR = {np.dtype(v): k for k, v in _NP.items()}
cases = []


def add(name, fn, inputs, expected, source):
    b = Builder("golden_" + name.replace("-", "_"))
    dts = [_MLIR[np.asarray(a).dtype] for a in inputs]
    args = [b.arg(np.asarray(a).shape, d) for a, d in zip(inputs, dts)]
    out = fn(b, *args)
    out = out if isinstance(out, (list, tuple)) else [out]
    b.ret(*out)
    expected = expected if isinstance(expected, (list, tuple)) else [expected]
    cases.append(dict(
        name=name, source=source, text=b.text(),
        inputs=[dict(dtype=d, shape=list(np.asarray(a).shape), data=np.asarray(a).reshape(-1).tolist()) for a, d in zip(inputs, dts)],
        expected=[dict(dtype=str(np.asarray(e).dtype), shape=list(np.asarray(e).shape), data=np.asarray(e).reshape(-1).tolist()) for e in expected]))


def row_scatter(body, **kw):
    def f(b, x, i, u):
        return b.scatter(x, b.reshape(i, (i.shape[0], 1)), u, update_window_dims=list(range(1, u.ndim)), inserted_window_dims=[0],
                         scatter_dims_to_operand_dims=[0], index_vector_dim=1, body=body, **kw)
    return f


x53 = np.arange(15, dtype=np.float32).reshape(5, 3) * 1.5 - 4
# jnp.take(x, idx, axis=0)  (slice.py:33-37)
add("take_axis0", lambda b, x, i: b.take_rows(x, i), [x53, np.array([0, 2, 4], np.int32)], x53[[0, 2, 4]], "tests/configs/slice.py:33-37")
# x.at[idx].set(val)  (slice.py:38-43)
v23 = np.array([[9, 8, 7], [6, 5, 4]], np.float32)
e = x53.copy(); e[[0, 2]] = v23
add("at_set_rows", row_scatter("set"), [x53, np.array([0, 2], np.int32), v23], e, "tests/configs/slice.py:38-43")
# x.at[idx].add(updates) on zeros((10,4))  (slice.py:175-180)
e = np.zeros((10, 4), np.float32); e[[0, 2, 5]] += 1
add("at_add_rows", row_scatter("add"), [np.zeros((10, 4), np.float32), np.array([0, 2, 5], np.int32), np.ones((3, 4), np.float32)], e, "tests/configs/slice.py:175-180")
# x.at[idx].mul / min / max with literal operands (slice.py:187-216)
e = np.ones((10, 4), np.float32); e[[0, 2, 5]] *= 2
add("at_mul_rows", row_scatter("mul", unique_indices=True), [np.ones((10, 4), np.float32), np.array([0, 2, 5], np.int32), np.full((3, 4), 2.0, np.float32)], e, "tests/configs/slice.py:187-192")
xm = (np.arange(40, dtype=np.float32).reshape(10, 4) % 7) - 3
um = np.array([[0, 0, 0, 0], [-5, 5, -5, 5], [1, 1, 1, 1]], np.float32)
e = xm.copy(); e[[0, 2, 5]] = np.minimum(e[[0, 2, 5]], um)
add("at_min_rows", row_scatter("min"), [xm, np.array([0, 2, 5], np.int32), um], e, "tests/configs/slice.py:205-210")
e = xm.copy(); e[[0, 2, 5]] = np.maximum(e[[0, 2, 5]], um)
add("at_max_rows", row_scatter("max"), [xm, np.array([0, 2, 5], np.int32), um], e, "tests/configs/slice.py:211-216")
# duplicate indices accumulate in update order: ((0 + 1e8) + 1) - 1e8 == 0 in f32, other orders give 1
big = np.array([[1e8], [1.0], [-1e8]], np.float32)
add("at_add_order_sensitive", row_scatter("add"), [np.zeros((2, 1), np.float32), np.array([1, 1, 1], np.int32), big],
    np.array([[0.0], [np.float32(np.float32(np.float32(0 + 1e8) + 1) - 1e8)]], np.float32), "tests/configs/slice.py:175-180 (duplicate-index semantics)")
# large integers survive gather and scatter (slice.py:241-295)
for dt, vals, idx in [(np.uint32, [16777217, 2**30, 2**31 - 1], 1), (np.int32, [16777217, 2**30, 2**31 - 1], 0),
                      (np.uint64, [2**40, 2**50, 2**62], 1), (np.int64, [2**40, 2**50, 2**62], 2)]:
    a = np.array(vals, dt).reshape(3, 1)
    add(f"large_{np.dtype(dt).name}_gather", lambda b, x, i: b.take_rows(x, i), [a, np.array([idx], np.int32)], a[[idx]], "tests/configs/slice.py:241-265")
for dt, pos, val in [(np.uint32, 2, 16777217), (np.int32, 1, 2**30)]:
    z = np.zeros((5, 1), dt); e = z.copy(); e[pos] = val
    add(f"large_{np.dtype(dt).name}_scatter", row_scatter("set"), [z, np.array([pos], np.int32), np.array([[val]], dt)], e, "tests/configs/slice.py:266-281")
# x[arange(4), arange(4)]: diagonal (slice.py:217-222)
x44 = np.arange(16, dtype=np.float32).reshape(4, 4) - 3.5
add("multi_index_point_gather", lambda b, x, i: b.gather(x, i, offset_dims=[], collapsed_slice_dims=[0, 1], start_index_map=[0, 1], index_vector_dim=1, slice_sizes=[1, 1]),
    [x44, np.stack([np.arange(4), np.arange(4)], 1).astype(np.int32)], np.diag(x44).copy(), "tests/configs/slice.py:217-222")
# partial gather with reversed index map: indices [3,2] -> dim2=3, dim0=2 => x[2, :, 3] (slice.py:391-408)
x345 = np.arange(60, dtype=np.float32).reshape(3, 4, 5)
add("partial_gather_reversed_index_map", lambda b, x, i: b.gather(x, i, offset_dims=[1], collapsed_slice_dims=[0, 2], start_index_map=[2, 0], index_vector_dim=1, slice_sizes=[1, 4, 1]),
    [x345, np.array([[3, 2]], np.int32)], x345[2, :, 3][None, :].copy(), "tests/configs/slice.py:391-408")
# scalar indices, index_vector_dim=0: indices [1,0] => x[1, :, 0] (slice.py:409-425)
add("partial_gather_scalar_indices", lambda b, x, i: b.gather(x, i, offset_dims=[0], collapsed_slice_dims=[0, 2], start_index_map=[0, 2], index_vector_dim=0, slice_sizes=[1, 4, 1]),
    [x345, np.array([1, 0], np.int32)], x345[1, :, 0].copy(), "tests/configs/slice.py:409-425")
# no collapsed dims: [2,1,1] sub-tensors at (row, col) (slice.py:426-456)
x233 = np.arange(18, dtype=np.float32).reshape(2, 3, 3)
pos = np.array([[0, 1], [1, 2], [0, 0]], np.int32)
add("multi_dim_gather_no_collapse_batched", lambda b, x, i: b.gather(x, i, offset_dims=[1, 2, 3], collapsed_slice_dims=[], start_index_map=[1, 2], index_vector_dim=1, slice_sizes=[2, 1, 1]),
    [x233, pos], np.stack([x233[:, r:r + 1, c:c + 1] for r, c in pos]), "tests/configs/slice.py:426-456")
# dynamic_slice(x, (2,), (4,)) (slice.py:29-32) and the clamp rule start = max(0, min(start, dim - size))
x10 = np.arange(10, dtype=np.float32)
add("dynamic_slice_2_4", lambda b, x, i: b.dynamic_slice(x, [i], [4]), [x10, np.int32(2)], x10[2:6], "tests/configs/slice.py:29-32")
add("dynamic_slice_clamped_high", lambda b, x, i: b.dynamic_slice(x, [i], [4]), [x10, np.int32(9)], x10[6:10], "src/pjrt_plugin/ops/slice.cc:90-107")
add("dynamic_slice_clamped_low", lambda b, x, i: b.dynamic_slice(x, [i], [4]), [x10, np.int32(-3)], x10[0:4], "src/pjrt_plugin/ops/slice.cc:90-107")
e = x10.copy(); e[7:10] = [-1, -2, -3]
add("dynamic_update_slice_clamped", lambda b, x, u, i: b.dynamic_update_slice(x, u, [i]), [x10, np.array([-1, -2, -3], np.float32), np.int32(9)], e, "src/pjrt_plugin/ops/slice.cc:155-199")
# x.at[1:].set(-1.0) on zeros(2) (slice.py:346-348): window scatter written as pad-free select
# while: sum of 0..4 == 10 (control_flow.py:232-241)


def sum_loop(b, n):
    z = b.constant(0, "i32")
    r = b.while_loop([z, b.constant(0, "i32")], lambda i, s: b.compare(i, n, "LT"), lambda i, s: [b.add(i, 1), b.add(s, i)])
    return r[1]


add("while_sum_0_to_4", lambda b, n: sum_loop(b, n), [np.int32(5)], np.int32(10), "tests/configs/control_flow.py:232-241")
add("while_130_iterations", lambda b, n: sum_loop(b, n), [np.int32(130)], np.int32(130 * 129 // 2), "tests/configs/control_flow.py:389-399")
add("while_zero_trip", lambda b, n: sum_loop(b, n), [np.int32(0)], np.int32(0), "tests/configs/control_flow.py:401-410")
# switch with an out-of-range index takes the last branch (control_flow.py:140-160; ops/control_flow.cc:672-675)
for idx, want in [(0, 2.0), (1, 11.0), (2, -1.0), (7, -1.0), (-3, -1.0)]:
    add(f"switch_index_{idx}".replace("-", "minus"), lambda b, i, x: b.case(i, [lambda: b.mul(x, 2.0), lambda: b.add(x, 10.0), lambda: b.neg(x)], [((), "f32")])[0],
        [np.int32(idx), np.float32(1.0)], np.float32(want), "tests/configs/control_flow.py:140-160")
# integer semantics spelled out at the reference's call sites
add("int_divide_truncates", lambda b, x, y: b.div(x, y), [np.array([7, -7, 7, -7], np.int32), np.array([2, 2, -2, -2], np.int32)], np.array([3, -3, -3, 3], np.int32), "src/pjrt_plugin/ops/arithmetic.cc:496-513")
add("int_remainder_c_style", lambda b, x, y: b.remainder(x, y), [np.array([7, -7, 7, -7], np.int32), np.array([3, 3, -3, -3], np.int32)], np.array([1, -1, 1, -1], np.int32), "src/pjrt_plugin/ops/arithmetic.cc:46-83")
add("shift_out_of_range", lambda b, x, s: [b.shift_left(x, s), b.shift_right_logical(x, s), b._binary("shift_right_arithmetic", x, s)],
    [np.array([1, -8, -8], np.int32), np.array([32, 40, 33], np.int32)], [np.array([0, 0, 0], np.int32), np.array([0, 0, 0], np.int32), np.array([0, -1, -1], np.int32)],
    "src/pjrt_plugin/mlx_executable.cc:293-301; ops/arithmetic.cc:119-143")
add("round_half_away_from_zero", lambda b, x: b._unary("round_nearest_afz", x), [np.array([0.5, 1.5, 2.5, -0.5, -2.5], np.float32)], np.array([1, 2, 3, -1, -3], np.float32), "src/pjrt_plugin/ops/arithmetic.cc:316-327")
add("round_half_to_even", lambda b, x: b._unary("round_nearest_even", x), [np.array([0.5, 1.5, 2.5, -0.5, -2.5], np.float32)], np.array([0, 2, 2, -0.0, -2], np.float32), "src/pjrt_plugin/ops/arithmetic.cc:535-560")
add("sign_keeps_nan_and_zero", lambda b, x: b.sign(x), [np.array([-3.0, 0.0, 5.0], np.float32)], np.array([-1.0, 0.0, 1.0], np.float32), "src/pjrt_plugin/ops/arithmetic.cc:517-531")
# dot_general of small integers exact in float (matmul.py:221-249 restated in f32)
a = np.array([[1, 2, 3], [4, 5, 6]], np.float32); bb = np.array([[7, 8], [9, 10], [11, 12]], np.float32)
add("matmul_2x3_3x2", lambda b, x, y: b.matmul(x, y), [a, bb], np.array([[58, 64], [139, 154]], np.float32), "tests/configs/matmul.py:19-30")
# integer and boolean contractions with the literal operands of the reference's tests (matmul.py:221-249)
add("dot_int32", lambda b, x, y: b.dot_general(x, y, ([0], [0])), [np.array([1, 2, 3], np.int32), np.array([4, 5, 6], np.int32)], np.array(32, np.int32), "tests/configs/matmul.py:221-228")
add("matmul_int32", lambda b, x, y: b.matmul(x, y), [np.array([[1, 2], [3, 4]], np.int32), np.array([[5, 6], [7, 8]], np.int32)], np.array([[19, 22], [43, 50]], np.int32), "tests/configs/matmul.py:229-235")
add("dot_bool", lambda b, x, y: b.dot_general(x, y, ([0], [0])), [np.array([True, False, True]), np.array([True, True, False])], np.array(True), "tests/configs/matmul.py:236-242")
add("matmul_uint32", lambda b, x, y: b.matmul(x, y), [np.array([[1, 2], [3, 4]], np.uint32), np.array([[5, 6], [7, 8]], np.uint32)], np.array([[19, 22], [43, 50]], np.uint32), "tests/configs/matmul.py:243-249")
# pooling with tied values (reduction.py:296-342: "maxpool2d-tied-grad", "maxpool2d-overlapping-tied-grad", "maxpool1d-tied-grad")
tied = np.array([[[[0.0], [0.0], [1.0], [0.0]], [[0.0], [0.0], [0.0], [0.0]], [[2.0], [0.0], [0.0], [0.0]], [[0.0], [0.0], [0.0], [3.0]]]], np.float32)
add("maxpool2d_tied", lambda b, x: b.reduce_window(x, float("-inf"), "max", (1, 2, 2, 1), (1, 2, 2, 1)), [tied],
    np.array([[[[0.0], [1.0]], [[2.0], [3.0]]]], np.float32), "tests/configs/reduction.py:296-313")
# gradient of the same pooling for an all-ones cotangent: each window's first maximum receives it
tied_grad = np.zeros((1, 4, 4, 1), np.float32)
for pos in [(0, 0), (0, 2), (2, 0), (3, 3)]:
    tied_grad[0, pos[0], pos[1], 0] = 1.0
add("maxpool2d_tied_grad", lambda b, x, g: b.select_and_scatter(x, g, 0.0, (1, 2, 2, 1), (1, 2, 2, 1)), [tied, np.ones((1, 2, 2, 1), np.float32)],
    tied_grad, "tests/configs/reduction.py:296-313")
over = np.zeros((1, 5, 5, 1), np.float32)
over[0, 1, 1, 0] = over[0, 1, 2, 0] = over[0, 2, 1, 0] = 5.0
add("maxpool2d_overlapping_tied", lambda b, x: b.reduce_window(x, float("-inf"), "max", (1, 3, 3, 1), (1, 1, 1, 1)), [over],
    np.array([[5, 5, 5], [5, 5, 5], [5, 5, 0]], np.float32).reshape(1, 3, 3, 1), "tests/configs/reduction.py:315-332")
add("maxpool1d_tied", lambda b, x: b.reduce_window(x, float("-inf"), "max", (1, 2), (1, 2)), [np.array([[0, 0, 1, 1, 0, 0, 2, 0]], np.float32)],
    np.array([[0, 1, 0, 2]], np.float32), "tests/configs/reduction.py:334-342")
add("pad_edge_and_interior", lambda b, x: b.pad(x, 0.0, [1], [2], [1]), [np.array([1, 2, 3], np.float32)], np.array([0, 1, 0, 2, 0, 3, 0, 0], np.float32), "src/pjrt_plugin/ops/slice.cc:202-276")
add("pad_negative_crops", lambda b, x: b.pad(x, 9.0, [-1], [1], [0]), [np.array([1, 2, 3], np.float32)], np.array([2, 3, 9], np.float32), "src/pjrt_plugin/ops/slice.cc:202-276")



# ---------------------------------------------------------------- cases given as StableHLO text
def add_text(name, text, inputs, expected, source, tol=None):
    dts = [_MLIR[np.asarray(a).dtype] for a in inputs]
    expected = expected if isinstance(expected, (list, tuple)) else [expected]
    c = dict(
        name=name, source=source, text=text,
        inputs=[dict(dtype=d, shape=list(np.asarray(a).shape), data=np.asarray(a).reshape(-1).tolist()) for a, d in zip(inputs, dts)],
        expected=[dict(dtype=str(np.asarray(e).dtype), shape=list(np.asarray(e).shape), data=np.asarray(e).reshape(-1).tolist()) for e in expected])
    if tol:
        c["tol"] = tol
    cases.append(c)


def reduce_precision_exact(x, exponent_bits, mantissa_bits):
    """stablehlo.reduce_precision by exact rational arithmetic (no bit tricks): round the value to
    `mantissa_bits` fraction bits at its own exponent, ties to even; then an exponent above the format's
    largest becomes infinity and one below its smallest normal becomes a signed zero."""
    import math
    from fractions import Fraction
    out = np.empty(x.shape, np.float32)
    max_exp = (1 << (exponent_bits - 1)) - 1
    min_exp = 1 - max_exp
    for k, v in enumerate(x.reshape(-1).tolist()):
        if math.isnan(v) or math.isinf(v) or v == 0:
            out.reshape(-1)[k] = v
            continue
        f = Fraction(v)
        e = math.floor(math.log2(abs(f)))            # exact for a float's own exponent
        while Fraction(2) ** e > abs(f): e -= 1
        while Fraction(2) ** (e + 1) <= abs(f): e += 1
        e_norm = max(e, -126)                          # float32 subnormals share the exponent -126
        ulp = Fraction(2) ** (e_norm - mantissa_bits)
        q = round(f / ulp) * ulp                       # Python rounds a Fraction half to even
        if q == 0:
            out.reshape(-1)[k] = math.copysign(0.0, v)
            continue
        eq = math.floor(math.log2(abs(q)))
        while Fraction(2) ** eq > abs(q): eq -= 1
        while Fraction(2) ** (eq + 1) <= abs(q): eq += 1
        if exponent_bits >= 8:                         # float32's own exponent range: nothing to clamp, subnormals stay
            out.reshape(-1)[k] = float(q)
        elif eq > max_exp:
            out.reshape(-1)[k] = math.copysign(math.inf, v)
        elif eq < min_exp:
            out.reshape(-1)[k] = math.copysign(0.0, v)
        else:
            out.reshape(-1)[k] = float(q)
    return out


def _unary_module(name, body_line, in_t, out_t, decorated=False):
    """One-op module in the form jax.jit(f).lower(x).as_text() prints; `decorated` adds the location
    aliases and trailing loc(...) that as_text(debug_info=True) prints."""
    if not decorated:
        return (f"module @jit_{name} attributes {{mhlo.num_partitions = 1 : i32, mhlo.num_replicas = 1 : i32}} {{\n"
                f"  func.func public @main(%arg0: {in_t}) -> ({out_t} {{jax.result_info = \"result\"}}) {{\n"
                f"    %0 = {body_line}\n"
                f"    return %0 : {out_t}\n  }}\n}}\n")
    return (f"#loc1 = loc(\"x\")\n"
            f"module @jit_{name} attributes {{mhlo.num_partitions = 1 : i32, mhlo.num_replicas = 1 : i32}} {{\n"
            f"  func.func public @main(%arg0: {in_t} loc(\"x\")) -> ({out_t} {{jax.result_info = \"result\"}}) {{\n"
            f"    %0 = {body_line} loc(#loc3)\n"
            f"    return %0 : {out_t} loc(#loc)\n  }} loc(#loc)\n}} loc(#loc)\n"
            f"#loc = loc(unknown)\n#loc2 = loc(\"/tmp/f.py\":3:11 to :58)\n"
            f"#loc3 = loc(\"jit(f)/reduce_precision\"(#loc2))\n")


# reduce_precision (tests/configs/misc.py:153-167): sixteen normal draws at e5m10, which is what a round trip through
# IEEE half precision gives for values in half's normal range, plus ties, overflow by rounding and the format's limits
rp_x = np.concatenate([np.random.default_rng(42).standard_normal(16).astype(np.float32),
                       np.array([1 + 2.0**-11, 1 + 3 * 2.0**-11, 65504.0, 65519.0, 65520.0, -65520.0, 2.0**-14, 1e5], np.float32)])
rp_want = reduce_precision_exact(rp_x, 5, 10)
with np.errstate(over="ignore"):
    assert np.array_equal(rp_want, rp_x.astype(np.float16).astype(np.float32)), "e5m10 must equal a half-precision round trip"
add_text("reduce_precision_e5m10_pretty", _unary_module("reduce_precision", "stablehlo.reduce_precision %arg0, format = e5m10 : tensor<24xf32>", "tensor<24xf32>", "tensor<24xf32>"),
         [rp_x], rp_want, "tests/configs/misc.py:153-158")
add_text("reduce_precision_e5m10_generic", _unary_module("reduce_precision", '"stablehlo.reduce_precision"(%arg0) <{exponent_bits = 5 : i32, mantissa_bits = 10 : i32}> : (tensor<24xf32>) -> tensor<24xf32>', "tensor<24xf32>", "tensor<24xf32>"),
         [rp_x], rp_want, "tests/configs/misc.py:153-158")
add_text("reduce_precision_e5m10_with_locations", _unary_module("reduce_precision", "stablehlo.reduce_precision %arg0, format = e5m10 : tensor<24xf32>", "tensor<24xf32>", "tensor<24xf32>", decorated=True),
         [rp_x], rp_want, "tests/configs/misc.py:153-158")
# the reference's edge vector at e3m5 (largest exponent 3, smallest normal exponent -2), expectations written out by hand,
# followed by values at the format's limits: 15.75 is the largest e3m5 number, 15.875 is a tie that rounds up into the
# next binade and overflows, 0.25 is the smallest normal, 0.2 is below it, 1 + 2^-6 and 1 + 3 * 2^-6 are ties
rp_edge = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-38, -1e-38, 1.0, -1.0, 15.75, 15.875, -16.0, 0.25, 0.2, -0.2, 1 + 2.0**-6, 1 + 3 * 2.0**-6], np.float32)
rp_edge_want = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 0.0, -0.0, 1.0, -1.0, 15.75, np.inf, -np.inf, 0.25, 0.0, -0.0, 1.0, 1.0625], np.float32)
assert np.array_equal(reduce_precision_exact(rp_edge, 3, 5).view(np.uint32)[[k for k in range(17) if k != 4]], rp_edge_want.view(np.uint32)[[k for k in range(17) if k != 4]])
add_text("reduce_precision_e3m5_edge_pretty", _unary_module("reduce_precision_edge", "stablehlo.reduce_precision %arg0, format = e3m5 : tensor<17xf32>", "tensor<17xf32>", "tensor<17xf32>"),
         [rp_edge], rp_edge_want, "tests/configs/misc.py:159-167")
add_text("reduce_precision_e3m5_edge_generic", _unary_module("reduce_precision_edge", '"stablehlo.reduce_precision"(%arg0) <{exponent_bits = 3 : i32, mantissa_bits = 5 : i32}> : (tensor<17xf32>) -> tensor<17xf32>', "tensor<17xf32>", "tensor<17xf32>"),
         [rp_edge], rp_edge_want, "tests/configs/misc.py:159-167")
# e8m23 keeps float32 as it is, e8m7 is a bfloat16 round trip (ties to even on the upper 16 bits)
rp_b = np.array([1.0, 1 + 2.0**-8, 1 + 3 * 2.0**-8, 3.14159274, -2.71828175, 3.38e38, 1e-39], np.float32)
rp_b_bits = rp_b.view(np.uint32).astype(np.uint64)
rp_b_want = (((rp_b_bits + 0x7FFF + ((rp_b_bits >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32)
assert np.array_equal(reduce_precision_exact(rp_b, 8, 7), rp_b_want)
add_text("reduce_precision_e8m7_is_bf16", _unary_module("reduce_precision_bf16", "stablehlo.reduce_precision %arg0, format = e8m7 : tensor<7xf32>", "tensor<7xf32>", "tensor<7xf32>"),
         [rp_b], rp_b_want, "src/pjrt_plugin/ops/arithmetic.cc:430-492")
add_text("reduce_precision_e8m23_identity", _unary_module("reduce_precision_id", "stablehlo.reduce_precision %arg0, format = e8m23 : tensor<7xf32>", "tensor<7xf32>", "tensor<7xf32>"),
         [rp_b], rp_b, "src/pjrt_plugin/ops/arithmetic.cc:430-492")

# is_finite on every class of float (tests/configs/unary.py: jnp.isfinite)
fin_x = np.array([0.0, -0.0, 1.5, -3e38, np.inf, -np.inf, np.nan, 1e-45, -1e-40], np.float32)
add_text("is_finite_classes", _unary_module("is_finite", "stablehlo.is_finite %arg0 : (tensor<9xf32>) -> tensor<9xi1>", "tensor<9xf32>", "tensor<9xi1>"),
         [fin_x], np.array([True, True, True, True, False, False, False, True, True]), "src/pjrt_plugin/ops/arithmetic.cc:535-560")

# popcnt / count_leading_zeros against Python's own integer methods (arithmetic.cc:585-607)
bits32 = np.array([0, 1, -1, 255, 2**30, -2**31, 16777217, 0x55555555, 0x0000FFFF, 65536, 7, -2], np.int32)
pop32 = np.array([bin(int(v) & 0xFFFFFFFF).count("1") for v in bits32], np.int32)
clz32 = np.array([32 - (int(v) & 0xFFFFFFFF).bit_length() for v in bits32], np.int32)
add_text("popcnt_i32", _unary_module("popcnt", "stablehlo.popcnt %arg0 : tensor<12xi32>", "tensor<12xi32>", "tensor<12xi32>"), [bits32], pop32, "src/pjrt_plugin/ops/arithmetic.cc:585-607")
add_text("count_leading_zeros_i32", _unary_module("clz", "stablehlo.count_leading_zeros %arg0 : tensor<12xi32>", "tensor<12xi32>", "tensor<12xi32>"), [bits32], clz32, "src/pjrt_plugin/ops/arithmetic.cc:585-607")
bitsu32 = bits32.view(np.uint32)
add_text("popcnt_ui32", _unary_module("popcnt_u", "stablehlo.popcnt %arg0 : tensor<12xui32>", "tensor<12xui32>", "tensor<12xui32>"), [bitsu32], pop32.astype(np.uint32), "src/pjrt_plugin/ops/arithmetic.cc:585-607")
add_text("count_leading_zeros_ui32", _unary_module("clz_u", "stablehlo.count_leading_zeros %arg0 : tensor<12xui32>", "tensor<12xui32>", "tensor<12xui32>"), [bitsu32], clz32.astype(np.uint32), "src/pjrt_plugin/ops/arithmetic.cc:585-607")
bits64 = np.array([0, 1, -1, 2**40, 2**62, -2**63, 2**32 - 1, 2**32, 0x5555555555555555], np.int64)
add_text("popcnt_i64", _unary_module("popcnt64", "stablehlo.popcnt %arg0 : tensor<9xi64>", "tensor<9xi64>", "tensor<9xi64>"), [bits64],
         np.array([bin(int(v) & (2**64 - 1)).count("1") for v in bits64], np.int64), "src/pjrt_plugin/ops/arithmetic.cc:585-607")
add_text("count_leading_zeros_i64", _unary_module("clz64", "stablehlo.count_leading_zeros %arg0 : tensor<9xi64>", "tensor<9xi64>", "tensor<9xi64>"), [bits64],
         np.array([64 - (int(v) & (2**64 - 1)).bit_length() for v in bits64], np.int64), "src/pjrt_plugin/ops/arithmetic.cc:585-607")

# stablehlo.composite: the module text and the input of the reference's raw-client test (tests/test_ops.py:214-281),
# expectation numpy's arcsin / sinh at the test's own tolerance
COMPOSITE_BODIES = {
    "chlo.asin": ("""    %cst = stablehlo.constant dense<1.000000e+00> : tensor<4xf32>
    %0 = stablehlo.multiply %arg0, %arg0 : tensor<4xf32>
    %1 = stablehlo.subtract %cst, %0 : tensor<4xf32>
    %2 = stablehlo.sqrt %1 : tensor<4xf32>
    %3 = stablehlo.atan2 %arg0, %2 : tensor<4xf32>
    return %3 : tensor<4xf32>
""", np.arcsin),
    "chlo.sinh": ("""    %0 = stablehlo.exponential %arg0 : tensor<4xf32>
    %1 = stablehlo.negate %arg0 : tensor<4xf32>
    %2 = stablehlo.exponential %1 : tensor<4xf32>
    %3 = stablehlo.subtract %0, %2 : tensor<4xf32>
    %cst = stablehlo.constant dense<2.000000e+00> : tensor<4xf32>
    %4 = stablehlo.divide %3, %cst : tensor<4xf32>
    return %4 : tensor<4xf32>
""", np.sinh),
}
comp_x = np.array([0.0, 0.5, -0.5, 0.9], np.float32)
for cname, (body, fn) in COMPOSITE_BODIES.items():
    text = (f"\nmodule @test {{\n  func.func private @{cname}.impl(%arg0: tensor<4xf32>) -> tensor<4xf32> {{\n{body}\n  }}\n"
            f"  func.func @main(%arg0: tensor<4xf32>) -> tensor<4xf32> {{\n"
            f"    %0 = stablehlo.composite \"{cname}\" %arg0 {{decomposition = @{cname}.impl}} : (tensor<4xf32>) -> tensor<4xf32>\n"
            f"    return %0 : tensor<4xf32>\n  }}\n}}\n")
    add_text("composite_" + cname.replace(".", "_"), text, [comp_x], fn(comp_x.astype(np.float64)).astype(np.float32), "tests/test_ops.py:214-281",
             tol=dict(rtol=1e-5, atol=1e-5))
# the same ops reached directly: chlo pretty form and the custom_call spelling (ops/control_flow.cc:53-63)
un_x = np.array([0.0, 0.5, -0.5, 0.9], np.float32)
for nm, fn in [("asin", np.arcsin), ("acos", np.arccos), ("atan", np.arctan), ("sinh", np.sinh), ("cosh", np.cosh), ("asinh", np.arcsinh), ("atanh", np.arctanh)]:
    add_text("chlo_" + nm, _unary_module(nm, f"chlo.{nm} %arg0 : tensor<4xf32> -> tensor<4xf32>", "tensor<4xf32>", "tensor<4xf32>"), [un_x],
             fn(un_x.astype(np.float64)).astype(np.float32), "src/pjrt_plugin/ops/control_flow.cc:53-63", tol=dict(rtol=1e-5, atol=1e-5))
add_text("chlo_acosh", _unary_module("acosh", "chlo.acosh %arg0 : tensor<4xf32> -> tensor<4xf32>", "tensor<4xf32>", "tensor<4xf32>"), [un_x + 2],
         np.arccosh((un_x + 2).astype(np.float64)).astype(np.float32), "src/pjrt_plugin/ops/control_flow.cc:53-63", tol=dict(rtol=1e-5, atol=1e-5))
# erf at points with textbook values (erf(0)=0, erf(0.5)=0.5204998778, erf(1)=0.8427007929, erf(-2)=-0.9953222650) and its inverse
erf_x = np.array([0.0, 0.5, 1.0, -2.0], np.float32)
erf_want = np.array([0.0, 0.5204998778, 0.8427007929, -0.9953222650], np.float32)
add_text("custom_call_mhlo_erf", _unary_module("erf", "stablehlo.custom_call @mhlo.erf(%arg0) : (tensor<4xf32>) -> tensor<4xf32>", "tensor<4xf32>", "tensor<4xf32>"), [erf_x], erf_want,
         "src/pjrt_plugin/ops/control_flow.cc:53-63", tol=dict(rtol=1e-5, atol=1e-5))
add_text("chlo_erf_inv", _unary_module("erf_inv", "chlo.erf_inv %arg0 : tensor<4xf32> -> tensor<4xf32>", "tensor<4xf32>", "tensor<4xf32>"), [erf_want], erf_x,
         "src/pjrt_plugin/ops/control_flow.cc:53-63", tol=dict(rtol=2e-5, atol=2e-5))
# several named results on one op (the form jax prints for rng_bit_generator and top_k)
tk_x = np.array([3.0, 1.0, 4.0, 1.0, 5.0, 9.0, 2.0, 6.0], np.float32)
add_text("top_k_named_results", ("module @jit_topk {\n  func.func public @main(%arg0: tensor<8xf32>) -> (tensor<3xf32>, tensor<3xi32>) {\n"
                                 "    %values, %indices = chlo.top_k(%arg0, k = 3) : tensor<8xf32> -> (tensor<3xf32>, tensor<3xi32>)\n"
                                 "    return %values, %indices : tensor<3xf32>, tensor<3xi32>\n  }\n}\n"),
         [tk_x], [np.array([9.0, 6.0, 5.0], np.float32), np.array([5, 7, 4], np.int32)], "src/pjrt_plugin/ops/sort_fft_complex.cc:40-82")

out = Path(__file__).with_name("cases.json")
out.write_text(json.dumps(cases, indent=0))
print(f"wrote {len(cases)} cases to {out}")
