"""Seeded random programs on the GPU against the CPU oracle.  Each program is a few dozen fused-op candidates drawn at
random (elementwise arithmetic, tanh, reversals, transposes, slices and concatenations, row and column reductions
broadcast back, reshapes, small products), a third of them with a counted loop in the middle whose body is drawn the
same way.  They exercise what no hand-written case pins down: which values the planner stores, which kernels share a
launch, how loop carries are threaded.  No compare-and-select pairs (a decision that flips on the last bit is not an
error) and inputs in [-1, 1]; every output must meet |got - want| <= 2e-5 + 2e-5 |want|."""
import random

import numpy as np
import pytest

from conftest import closeness
from shlo_oracle import Oracle

pytestmark = pytest.mark.gpu

SEEDS = list(range(4100, 4140))


def build(seed):
    from jax_mps_amd.shlo.builder import Builder
    rnd = random.Random(seed)
    b = Builder(f"random_{seed}")
    R, C = rnd.choice([(8, 16), (64, 64), (4, 1024), (128, 32), (33, 7)])
    vals = [b.arg((R, C), "f32"), b.arg((R, C), "f32")]

    def grow(vals, steps):
        for _ in range(steps):
            k = rnd.random()
            x, y = rnd.choice(vals[-6:]), rnd.choice(vals[-6:])
            if k < 0.22:
                v = b.add(x, y)
            elif k < 0.32:
                v = b.mul(x, b.tanh(y))
            elif k < 0.42:
                v = b.reverse(x, [rnd.choice([0, 1])])
            elif k < 0.50:
                v = b.transpose(b.transpose(x, [1, 0]), [1, 0])
            elif k < 0.60 and R % 2 == 0:
                v = b.concatenate([b.slice(x, [0, 0], [R // 2, C]), b.slice(y, [R // 2, 0], [R, C])], 0)
            elif k < 0.68:
                v = b.broadcast_in_dim(b.div(b.reduce_sum(x, [0]), float(R)), (R, C), [1])
            elif k < 0.76:
                v = b.broadcast_in_dim(b.reduce_max(x, [1]), (R, C), [0])
            elif k < 0.84:
                v = b.maximum(x, b.mul(y, 0.5))
            elif k < 0.90:
                v = b.reshape(b.reshape(x, (R * C,)), (R, C))
            elif k < 0.95 and R == C:
                v = b.mul(b.matmul(x, y), 1.0 / C)
            else:
                v = b.tanh(b.mul(x, 0.7))
            vals.append(v)
        return vals

    vals = grow(vals, rnd.randint(3, 25))
    if rnd.random() < 0.35:
        zero = b.constant(0, "i32")
        trips = rnd.choice([1, 2, 5])

        def body(i, p, q):
            vs = grow([p, q], rnd.randint(2, 8))
            return [b.add(i, 1), b.tanh(vs[-1]), b.mul(b.add(vs[-2], q), 0.5)]
        r = b.while_loop([zero, vals[-1], vals[-2]], lambda i, p, q: b.compare(i, trips, "LT"), body)
        vals += [r[1], r[2]]
        vals = grow(vals, rnd.randint(0, 5))
    b.ret(*vals[-3:])
    rng = np.random.default_rng(seed)
    return b.text(), [rng.uniform(-1, 1, (R, C)).astype(np.float32) for _ in range(2)]


@pytest.mark.parametrize("seed", SEEDS)
def test_random_program(client, seed):
    from jax_mps_amd import runner
    text, ins = build(seed)
    print("seed", seed, flush=True)
    exe = client.compile_and_load(text)
    got = [runner.download(o) for o in exe.execute(runner.upload(client, ins, ["f32", "f32"]))]
    want = Oracle(text).run(*ins)
    assert len(got) == len(want)
    for k, (g, w) in enumerate(zip(got, want)):
        ratio = closeness(g, w, 2e-5, 2e-5)
        assert ratio <= 1.0, f"seed {seed}, output {k}: {ratio:.3f} x the bound"
