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

out = Path(__file__).with_name("cases.json")
out.write_text(json.dumps(cases, indent=0))
print(f"wrote {len(cases)} cases to {out}")
