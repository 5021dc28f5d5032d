"""Seeded random scans on the GPU against the CPU oracle: a counted loop over a sequence xs[T, B, n] that reads a slice
at an index drawn from (i, T - 1 - i, i + c clamped at the end, i * 1), multiplies it and the carried state by weights,
and optionally stacks states with dynamic_update_slice, reads the stack back, sums a product into a carried
accumulator, carries the sequence unchanged, or runs fewer or more iterations than the sequence is long.  These are
the shapes the loop rules of the planner act on (products that leave the loop, slices addressed by the host, carries that
alternate between two halves, accumulating products); every output must meet |got - want| <= 2e-5 + 2e-5 |want|."""
import random

import numpy as np
import pytest

from conftest import closeness
from shlo_oracle import Oracle

pytestmark = pytest.mark.gpu

SEEDS = list(range(5200, 5230))


def build(seed):
    from jax_mps_amd.shlo.builder import Builder
    rnd = random.Random(seed)
    T, B = rnd.choice([2, 3, 7, 12]), rnd.choice([1, 4, 6, 16])
    NI, NH = rnd.choice([8, 20, 32]), rnd.choice([8, 16, 24])
    b = Builder(f"scan_{seed}")
    xs, w, u = b.arg((T, B, NI), "f32"), b.arg((NI, NH), "f32"), b.arg((NH, NH), "f32")
    zero = b.constant(0, "i32")
    trips = rnd.choice([T, T, T, max(1, T - 1), T + 2])

    def idx(i):
        k = rnd.random()
        if k < 0.4:
            return i
        if k < 0.7:
            return b.sub(b.constant(T - 1, "i32"), i)
        if k < 0.85:
            return b.add(i, rnd.choice([1, 2]))
        return b.mul(i, 1)
    use_stack, use_acc, carry_xs = rnd.random() < 0.6, rnd.random() < 0.6, rnd.random() < 0.3
    read_stack_back = use_stack and rnd.random() < 0.5
    init, names = [zero, b.zeros((B, NH))], ["i", "h"]
    if use_stack:
        init.append(b.zeros((T, B, NH))); names.append("hs")
    if use_acc:
        init.append(b.zeros((NI, NH))); names.append("acc")
    if carry_xs:
        init.append(xs); names.append("xs")

    def body(*c):
        d = dict(zip(names, c))
        i, h, seq = d["i"], d["h"], d.get("xs", xs)
        ix = idx(i)
        x_t = b.reshape(b.dynamic_slice(seq, [ix, zero, zero], [1, B, NI]), (B, NI))
        z = b.add(b.matmul(x_t, w), b.matmul(h, u))
        if read_stack_back:
            z = b.add(z, b.mul(b.reshape(b.dynamic_slice(d["hs"], [idx(i), zero, zero], [1, B, NH]), (B, NH)), 0.3))
        h2 = b.tanh(z)
        out = [b.add(i, 1), h2]
        if use_stack:
            src = h if rnd.random() < 0.5 else h2
            out.append(b.dynamic_update_slice(d["hs"], b.reshape(src, (1, B, NH)), [ix if rnd.random() < 0.7 else i, zero, zero]))
        if use_acc:
            g = b.mul(h2, b.sub(1.0, b.mul(h2, h2)))
            out.append(b.add(d["acc"], b.dot_general(x_t, g, ([0], [0]))))
        if carry_xs:
            out.append(seq)
        return out
    r = b.while_loop(init, lambda *c: b.compare(c[0], trips, "LT"), body)
    rets = [r[1]]
    if use_stack:
        rets.append(r[2])
    if use_acc:
        rets.append(r[names.index("acc")])
    b.ret(*rets)
    rng = np.random.default_rng(seed)
    ins = [rng.uniform(-1, 1, (T, B, NI)).astype(np.float32), rng.uniform(-0.4, 0.4, (NI, NH)).astype(np.float32),
           rng.uniform(-0.4, 0.4, (NH, NH)).astype(np.float32)]
    return b.text(), ins


@pytest.mark.parametrize("seed", SEEDS)
def test_random_scan(client, seed):
    from jax_mps_amd import runner
    text, ins = build(seed)
    print("seed", seed, flush=True)
    exe = client.compile_and_load(text)
    got = [runner.download(o) for o in exe.execute(runner.upload(client, ins, ["f32"] * 3))]
    want = Oracle(text).run(*ins)
    assert len(got) == len(want)
    for k, (g, w) in enumerate(zip(got, want)):
        ratio = closeness(g, w, 2e-5, 2e-5)
        assert ratio <= 1.0, f"seed {seed}, output {k}: {ratio:.3f} x the bound"
