"""Seeded sweep of convolution shapes on the GPU against the CPU oracle: forward, data-gradient (input dilation,
reversed filter with its feature dims swapped) and filter-gradient (batch and feature swapped, window dilation)
forms at random sizes, strides, paddings and feature counts that are multiples of 16 and of 4, which is what the
vector-loader kernel takes; every result must meet |got - want| <= 1e-5 + 1e-5 |want| (inputs in [-1, 1] / sqrt(K)
so that the float32 accumulation noise stays below the bound)."""
import numpy as np
import pytest

from conftest import closeness
from shlo_oracle import Oracle

pytestmark = pytest.mark.gpu


def _cases():
    rng = np.random.default_rng(20240607)
    out = []
    for i in range(36):
        form = ("fwd", "dgrad", "wgrad")[i % 3]
        b = int(rng.integers(1, 9))
        h, w = int(rng.integers(3, 15)), int(rng.integers(3, 15))
        cin = 16 * int(rng.integers(1, 5))
        cout = 16 * int(rng.integers(1, 9)) if form == "dgrad" else 4 * int(rng.integers(1, 33))
        k0, k1 = (int(rng.choice([1, 2, 3, 5])) for _ in range(2))
        s0, s1 = (int(rng.choice([1, 1, 2, 3])) for _ in range(2))
        p = [[int(rng.integers(0, k0)), int(rng.integers(0, k0))], [int(rng.integers(0, k1)), int(rng.integers(0, k1))]]
        out.append((f"{form}-{i}", form, b, h, w, cin, cout, k0, k1, s0, s1, p, 7000 + i))
    return out


def _build(form, b, h, w, cin, cout, k0, k1, s0, s1, p, seed):
    from jax_mps_amd.shlo.builder import Builder
    rng = np.random.default_rng(seed)
    bld = Builder("conv_shape")
    oh = (h + p[0][0] + p[0][1] - k0) // s0 + 1
    ow = (w + p[1][0] + p[1][1] - k1) // s1 + 1
    if oh < 1 or ow < 1:
        return None
    if form == "fwd":
        x = bld.arg((b, h, w, cin), "f32"); f = bld.arg((k0, k1, cin, cout), "f32")
        bld.ret(bld.conv(x, f, strides=(s0, s1), padding=p))
        shapes, K = [(b, h, w, cin), (k0, k1, cin, cout)], k0 * k1 * cin
    elif form == "dgrad":
        # gradient of the forward convolution with respect to its input: g is dilated by the stride, the filter is
        # reversed and read with its feature dims swapped, the padding mirrors the forward one
        g = bld.arg((b, oh, ow, cout), "f32"); f = bld.arg((k0, k1, cin, cout), "f32")
        pad = []
        for d, (n, k, s, o) in enumerate(((h, k0, s0, oh), (w, k1, s1, ow))):
            lo = k - 1 - p[d][0]
            hi = n + k - 1 - ((o - 1) * s + 1) - lo
            pad.append([lo, hi])
        if cout % 16:
            return None          # the contracted feature is the forward one's output feature here
        bld.ret(bld.conv(g, bld.reverse(f, [0, 1]), strides=(1, 1), padding=pad, lhs_dilation=(s0, s1), dn=("b01f", "01oi", "b01f")))
        shapes, K = [(b, oh, ow, cout), (k0, k1, cin, cout)], k0 * k1 * cout
    else:
        # gradient with respect to the filter: batch is contracted, the window is g's extent dilated by the stride
        if b % 16:
            b = 16 * ((b + 15) // 16)
        x = bld.arg((b, h, w, cin), "f32"); g = bld.arg((b, oh, ow, cout), "f32")
        hi0 = (oh - 1) * s0 + k0 - h - p[0][0]
        hi1 = (ow - 1) * s1 + k1 - w - p[1][0]
        bld.ret(bld.conv(x, g, strides=(1, 1), padding=[[p[0][0], hi0], [p[1][0], hi1]], rhs_dilation=(s0, s1), dn=("f01b", "i01o", "01bf")))
        shapes, K = [(b, h, w, cin), (b, oh, ow, cout)], b * oh * ow
    ins = [(rng.uniform(-1, 1, s) / np.sqrt(np.sqrt(K))).astype(np.float32) for s in shapes]
    return bld.text(), ins


CASES = _cases()


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_convolution_shape(client, case):
    from jax_mps_amd import runner
    name, form, *rest = case
    built = _build(form, *rest)
    if built is None:
        pytest.skip("degenerate shape for this form")
    text, ins = built
    print("case", name, rest, flush=True)
    exe = client.compile_and_load(text)
    got = runner.download(exe.execute(runner.upload(client, ins, ["f32", "f32"]))[0])
    want = Oracle(text).run(*ins)[0]
    assert got.shape == np.asarray(want).shape
    ratio = closeness(got, want, 1e-5, 1e-5)
    assert ratio <= 1.0, f"{name}: {ratio:.3f} x the bound"
