"""The eleven distinct convolution layers of the batch-128 ResNet18 train step, each at its exact benchmark shape
and in the three forms the step launches: forward (with the column sums batch norm takes from it), data gradient
and filter gradient, written by the same emitter rules as the step itself (`Builder.conv` and its VJP), so the
(M, N, K), the tile, the split of K, the packed residue classes and the statistics epilogue are the ones the timed
step uses.  Every output is non-zero random data against the CPU oracle (float64 accumulation).

Bar: |got - want| <= 1e-5 + 1e-5 |want| per element (the reference's rule, tests/test_ops.py:91-105).  Inputs are
uniform(-1, 1) / K^(1/4) per operand, K the contraction length of the form that reads them, so that sums stay of
order one and float32 accumulation noise stays below the bound (K reaches 131 072 in the filter gradients).  The
forward form draws from uniform(-0.5, 1.5) instead: its outputs then have a mean well away from zero, so the 131 072
terms of a per-feature sum do not cancel and the relative part of the rule is what judges the statistics (a sum that
cancels to near zero would be judged against 1e-5 absolute, which no float32 summation of that many terms meets)."""
import numpy as np
import pytest

from conftest import closeness
from shlo_oracle import Oracle

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(600)]

BATCH = 128
# name, input size, in features, out features, window, stride
LAYERS = [
    ("stem-3x3-3to64-32", 32, 3, 64, 3, 1),
    ("s1-3x3-64to64-32", 32, 64, 64, 3, 1),
    ("s2-3x3-64to128-s2", 32, 64, 128, 3, 2),
    ("s2-3x3-128to128-16", 16, 128, 128, 3, 1),
    ("s2-1x1-64to128-s2", 32, 64, 128, 1, 2),
    ("s3-3x3-128to256-s2", 16, 128, 256, 3, 2),
    ("s3-3x3-256to256-8", 8, 256, 256, 3, 1),
    ("s3-1x1-128to256-s2", 16, 128, 256, 1, 2),
    ("s4-3x3-256to512-s2", 8, 256, 512, 3, 2),
    ("s4-3x3-512to512-4", 4, 512, 512, 3, 1),
    ("s4-1x1-256to512-s2", 8, 256, 512, 1, 2),
]
FORMS = ("fwd", "dgrad", "wgrad")
CASES = [(f"{name}-{form}", form, size, cin, cout, k, stride, 9100 + 10 * i + j)
         for i, (name, size, cin, cout, k, stride) in enumerate(LAYERS) for j, form in enumerate(FORMS)
         if not (form == "dgrad" and cin == 3)]          # the step takes no gradient of the image


def _same_padding(n_in, k, stride):
    out = -(-n_in // stride)
    tot = max((out - 1) * stride + k - n_in, 0)
    return out, (tot // 2, tot - tot // 2)


def build(form, size, cin, cout, k, stride, seed, batch=BATCH):
    """(module text, inputs, names of the outputs).  The forward module returns the convolution and its per-feature
    sum and sum of squares (what batch norm reads); the gradient modules return what `Builder.grad` derives for the
    input or the filter from an upstream gradient argument."""
    from jax_mps_amd.shlo.builder import Builder
    rng = np.random.default_rng(seed)
    out, pad = _same_padding(size, k, stride)
    b = Builder("resnet_layer_" + form)
    X = b.arg((batch, size, size, cin))
    W = b.arg((k, k, cin, cout))
    x_len, w_len, g_len = {"fwd": (k * k * cin,) * 2 + (1,), "dgrad": (1, k * k * cout, k * k * cout),
                           "wgrad": (batch * out * out, 1, batch * out * out)}[form]

    shift = 0.5 if form == "fwd" else 0.0

    def draw(shape, contraction):
        return ((rng.uniform(-1, 1, shape) + shift) / contraction ** 0.25).astype(np.float32)
    x, w = draw(X.shape, x_len), draw(W.shape, w_len)
    y = b.conv(X, W, strides=(stride, stride), padding=(pad, pad))
    if form == "fwd":
        b.ret(y, b.reduce_sum(y, [0, 1, 2]), b.reduce_sum(b.mul(y, y), [0, 1, 2]))
        return b.text(), [x, w], ["y", "sum", "sum of squares"]
    G = b.arg(y.shape)
    g = draw(G.shape, g_len)
    (d,) = b.grad(y, [X if form == "dgrad" else W], seed=G)
    b.ret(d)
    return b.text(), [x, w, g], ["dx" if form == "dgrad" else "dw"]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_resnet_layer(client, case):
    from jax_mps_amd import runner
    name, *spec = case
    text, ins, names = build(*spec)
    print("case", name, spec, flush=True)
    exe = client.compile_and_load(text)
    got = [runner.download(o) for o in exe.execute(runner.upload(client, ins, ["f32"] * len(ins)))]
    want = Oracle(text).run(*ins)
    for n, g, w in zip(names, got, want):
        w = np.asarray(w)
        assert g.shape == w.shape
        # (the data gradient of a 1x1 window with stride 2 is zero at three positions of four)
        assert np.abs(w).max() > 1e-3 and (w != 0).mean() > 0.24, f"{name} {n}: the expectation is (nearly) all zero"
        ratio = closeness(g, w, 1e-5, 1e-5)
        print(f"  {n}: {ratio:.3f} x the bound, max |want| {np.abs(w).max():.3g}", flush=True)
        assert ratio <= 1.0, f"{name} {n}: {ratio:.3f} x the bound"
