"""Seeded random multilayer programs with their gradients on the GPU against the CPU oracle: a few layers drawn from
linear + bias, ReLU / GELU / tanh, layer norm, softmax, gated units (h * logistic(h @ W)), half swaps, row-max and
column-mean shifts, products on the transposed activations, row shifts by padding, and a softmax cross-entropy against
soft labels on top; the outputs are the loss and the gradient of every parameter (jax.grad form: transposed products,
broadcast sums, masks).  These are the programs that exposed a sum written by a product step being recomputed by its
readers.  Every output must meet |got - want| <= 1e-4 (s + |want|), s the output's largest magnitude (for a gradient
at least a hundredth of the largest gradient magnitude, so that a gradient that is zero but for rounding is measured
against the others); the seeds are those whose oracle result does not itself move by more than a third of that bound
between float32 and float64 accumulation."""
import random

import numpy as np
import pytest

from shlo_oracle import Oracle

pytestmark = pytest.mark.gpu

TOL = 1e-4
ILL_CONDITIONED = {7005}
SEEDS = [s for s in range(7000, 7060) if s not in ILL_CONDITIONED]


def build(seed):
    from jax_mps_amd.shlo.builder import Builder, relu, softmax, layer_norm, gelu_tanh, log_softmax
    rnd = random.Random(seed)
    b = Builder(f"random_network_{seed}")
    rows, width = rnd.choice([4, 16, 33, 64]), rnd.choice([8, 24, 64, 128])
    shapes, params = [], []

    def P(*shape, scale=None):
        p = b.arg(shape, "f32")
        shapes.append((tuple(shape), scale if scale is not None else (1.0 / max(1, shape[0])) ** 0.5))
        params.append(p)
        return p
    h = P(rows, width, scale=1.0)
    for _ in range(rnd.randint(2, 7)):
        m, d = h.shape
        k = rnd.random()
        if k < 0.25:
            dn = rnd.choice([8, 24, 64, 128])
            h = b.add(b.matmul(h, P(d, dn)), P(dn, scale=0.1))
        elif k < 0.40: h = rnd.choice([relu, gelu_tanh])(b, h) if rnd.random() < 0.7 else b.tanh(h)
        elif k < 0.50: h = layer_norm(b, h, P(d, scale=1.0), P(d, scale=0.1), 1e-5)
        elif k < 0.58: h = softmax(b, h)
        elif k < 0.66: h = b.mul(h, b.logistic(b.matmul(h, P(d, d))))
        elif k < 0.72 and d % 2 == 0: h = b.concatenate([b.slice(h, [0, d // 2], [m, d]), b.mul(b.slice(h, [0, 0], [m, d // 2]), 2.0)], 1)
        elif k < 0.78: h = b.sub(h, b.broadcast_in_dim(b.reduce_max(h, [1]), (m, d), [0]))
        elif k < 0.84: h = b.add(h, b.broadcast_in_dim(b.mean(h, [0]), (m, d), [1]))
        elif k < 0.90: h = b.transpose(b.matmul(b.transpose(h, [1, 0]), P(m, m)), [1, 0])
        elif k < 0.95: h = b.pad(b.slice(h, [1, 0], [m, d]), 0.0, [1, 0], [0, 0])
        else: h = b.exp(b.mul(h, 0.1))
    lp = log_softmax(b, b.matmul(h, P(h.shape[1], 7)))
    loss = b.neg(b.mean(b.reduce_sum(b.mul(lp, P(rows, 7, scale=0.3)), [1]), [0]))
    b.ret(loss, *b.grad(loss, params))
    rng = np.random.default_rng(seed)
    return b.text(), [(rng.uniform(-1, 1, s) * sc * 1.7).astype(np.float32) for s, sc in shapes]


def ratios(got, want):
    """Per output: max |got - want| / (TOL (s + |want|))."""
    largest = max([float(np.max(np.abs(np.asarray(w, dtype=np.float64)))) for w in want[1:]] + [1e-30])
    out = []
    for k, (g, w) in enumerate(zip(got, want)):
        g, w = np.asarray(g, dtype=np.float64), np.asarray(w, dtype=np.float64)
        s = max(1e-30, float(np.max(np.abs(w))), 1e-2 * largest if k else 0.0)
        out.append(float(np.max(np.abs(g - w) / (TOL * s + TOL * np.abs(w)))))
    return out


@pytest.mark.parametrize("seed", SEEDS)
def test_random_network(client, seed):
    from jax_mps_amd import runner
    text, ins = build(seed)
    print("seed", seed, flush=True)
    exe = client.compile_and_load(text)
    got = [runner.download(o) for o in exe.execute(runner.upload(client, ins, ["f32"] * len(ins)))]
    want = Oracle(text).run(*ins)
    assert len(got) == len(want)
    worst = ratios(got, want)
    assert max(worst) <= 1.0, f"seed {seed}: output {int(np.argmax(worst))} is {max(worst):.2f} x the bound"
