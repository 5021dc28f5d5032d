"""Seeded random shapes on the GPU against the CPU oracle, sizes drawn log-uniformly so that the launch-shape rules of
every generator are crossed (one pass or two, one wavefront or a workgroup per row, vector or scalar lanes, the small
product kernels, the wide MFMA tiles, the convolution core for large fp32 products):

* reductions of rank 1 to 4 tensors over any subset of dims (sum, max, min, sum of squares, up to three sharing one
  pass, a fused elementwise input, a per-output scaling and rsqrt, and the result read back at the input's shape);
* products M x N x K up to 1500 x 1500 x 2000, float32 and bfloat16, either operand transposed, up to two batch dims,
  with a bias, an activation or an addend behind them.
Integer results and max / min are exact; float sums meet |got - want| <= tol (sqrt(n) + |want|), n the number of terms,
tol 2e-5 (float32) or 2e-2 (bfloat16)."""
import math
import random

import numpy as np
import pytest

from conftest import closeness
from shlo_oracle import Oracle, round_bf16

pytestmark = pytest.mark.gpu

REDUCE_SEEDS = list(range(8100, 8140))
PRODUCT_SEEDS = list(range(8200, 8240))


def _logu(rnd, lo, hi):
    return max(lo, min(hi, int(round(math.exp(rnd.uniform(math.log(lo), math.log(hi)))))))


def build_reduce(seed):
    from jax_mps_amd.shlo.builder import Builder
    rnd = random.Random(seed)
    b = Builder(f"random_reduce_{seed}")
    dt = rnd.choice(["f32", "f32", "f32", "i32"])
    rank = rnd.choice([1, 2, 2, 3, 4])
    shape = [_logu(rnd, 1, 3000) for _ in range(rank)]
    while int(np.prod(shape)) > 3_000_000:
        q = rnd.randrange(rank)
        shape[q] = max(1, shape[q] // 2)
    shape = tuple(shape)
    x, y = b.arg(shape, dt), b.arg(shape, dt)
    dims = sorted(rnd.sample(range(rank), rnd.randint(1, rank)))
    terms = int(np.prod([shape[d] for d in dims]))
    src = rnd.random()
    if src < 0.4: v = x
    elif src < 0.6: v = b.mul(x, y)
    elif src < 0.8: v = b.select(b.compare(y, 0, "GT"), x, b.full_like(x, 0))
    else: v = b.sub(x, b.mul(y, 2) if dt == "i32" else b.mul(y, 0.5))
    kept = [d for d in range(rank) if d not in dims]
    outs = []
    for kind in rnd.sample(["sum", "max", "min", "sumsq"], rnd.randint(1, 3)):
        if kind == "sum": r = b.reduce_sum(v, dims)
        elif kind == "max": r = b.reduce_max(v, dims)
        elif kind == "min": r = b.reduce_min(v, dims)
        else: r = b.reduce_sum(b.mul(v, v), dims)
        if dt == "f32" and kind in ("sum", "sumsq") and rnd.random() < 0.5:
            r = b.mul(r, 1.0 / terms)
            if rnd.random() < 0.4:
                r = b.rsqrt(b.add(b.abs(r), 1e-3))
        outs.append((r, kind))
    if rnd.random() < 0.3 and kept:
        outs.append((b.sub(v, b.broadcast_in_dim(outs[0][0], shape, kept)), "back"))
    b.ret(*[o[0] for o in outs])
    rng = np.random.default_rng(seed)
    ins = [rng.uniform(-1, 1, shape).astype(np.float32) for _ in range(2)] if dt == "f32" else [rng.integers(-1000, 1000, shape).astype(np.int32) for _ in range(2)]
    return b.text(), ins, [dt, dt], terms, [o[1] for o in outs]


def build_product(seed):
    from jax_mps_amd.shlo.builder import Builder
    rnd = random.Random(seed)
    b = Builder(f"random_product_{seed}")
    dt = rnd.choice(["f32", "f32", "bf16"])
    M, N, K = _logu(rnd, 1, 1500), _logu(rnd, 1, 1500), _logu(rnd, 1, 2000)
    if rnd.random() < 0.3:
        M, N, K = [v // 8 * 8 + 8 for v in (M, N, K)]
    bs = [rnd.choice([1, 2, 3, 5]) for _ in range(rnd.choice([0, 0, 0, 1, 2]))]
    while M * N * K * max(1, int(np.prod(bs))) > 4e8:
        M = max(1, M // 2)
    lhs_t, rhs_t = rnd.random() < 0.35, rnd.random() < 0.35
    shapes = [tuple(bs) + ((K, M) if lhs_t else (M, K)), tuple(bs) + ((N, K) if rhs_t else (K, N))]
    a, w = b.arg(shapes[0], dt), b.arg(shapes[1], dt)
    nb = len(bs)
    y = b.dot_general(a, w, ([nb + (0 if lhs_t else 1)], [nb + (1 if rhs_t else 0)]), (list(range(nb)), list(range(nb))))
    if rnd.random() < 0.3:
        shapes.append((N,))
        y = b.add(y, b.broadcast_in_dim(b.arg((N,), dt), y.shape, [len(y.shape) - 1]))
    act = rnd.random()
    if act < 0.2: y = b.maximum(y, 0.0)
    elif act < 0.3: y = b.tanh(y)
    elif act < 0.4: y = b.mul(b.mul(y, 0.5), b.add(b.tanh(b.mul(b.add(y, b.mul(b.mul(b.mul(y, y), y), 0.044715)), 0.7978845608)), 1.0))
    elif act < 0.5:
        shapes.append(tuple(y.shape))
        y = b.add(y, b.arg(tuple(y.shape), dt))
    b.ret(y)
    rng = np.random.default_rng(seed)
    return b.text(), [rng.uniform(-1, 1, s).astype(np.float32) for s in shapes], dt, K


def all_programs():
    """(name, text) of every program of this file, for whoever compiles kernels ahead of time."""
    return [(f"random_reduce_{s}", build_reduce(s)[0]) for s in REDUCE_SEEDS] + [(f"random_product_{s}", build_product(s)[0]) for s in PRODUCT_SEEDS]


@pytest.mark.parametrize("seed", REDUCE_SEEDS)
def test_random_reduction(client, seed):
    from jax_mps_amd import runner
    text, ins, dts, terms, kinds = build_reduce(seed)
    print("seed", seed, ins[0].shape, flush=True)
    exe = client.compile_and_load(text)
    got = [runner.download(o) for o in exe.execute(runner.upload(client, ins, dts))]
    want = Oracle(text).run(*ins)
    assert len(got) == len(want)
    for k, (g, w, kind) in enumerate(zip(got, want, kinds)):
        g, w = np.asarray(g), np.asarray(w)
        assert g.shape == w.shape
        if dts[0] == "i32" or kind in ("max", "min"):
            assert np.array_equal(g.astype(w.dtype), w), f"seed {seed}, output {k} ({kind}) differs"
        else:
            s = max(1.0, terms ** 0.5)
            ratio = closeness(g.astype(np.float64) / s, w.astype(np.float64) / s, 2e-5, 2e-5)
            assert ratio <= 1.0, f"seed {seed}, output {k} ({kind}): {ratio:.3f} x the bound"


@pytest.mark.parametrize("seed", PRODUCT_SEEDS)
def test_random_product(client, seed):
    from jax_mps_amd import runner
    text, ins, dt, K = build_product(seed)
    print("seed", seed, dt, [a.shape for a in ins], flush=True)
    exe = client.compile_and_load(text)
    got = runner.download(exe.execute(runner.upload(client, ins, [dt] * len(ins)))[0])
    want = Oracle(text).run(*([round_bf16(a) for a in ins] if dt == "bf16" else ins))[0]
    s = max(1.0, K ** 0.5)
    tol = 2e-5 if dt == "f32" else 2e-2
    ratio = closeness(np.asarray(got, dtype=np.float64) / s, np.asarray(want, dtype=np.float64) / s, tol, tol)
    assert ratio <= 1.0, f"seed {seed}: {ratio:.3f} x the bound"
