"""A convolution whose result is read much later runs on a second stream next to the steps in between; the step that
reads it waits for it.  The program below has such a convolution followed by a chain of kernels over other data that
allocate and release temporaries the whole time (so that a missing wait or a buffer reused too early would show),
and reads the convolution's result only at the end; every one of several executions must match the oracle."""
import numpy as np
import pytest

from conftest import closeness
from shlo_oracle import Oracle

pytestmark = pytest.mark.gpu


def _program():
    from jax_mps_amd.shlo.builder import Builder
    b = Builder("distant_consumer")
    x = b.arg((16, 24, 24, 32), "f32")
    g = b.arg((16, 24, 24, 64), "f32")
    t = b.arg((16, 24, 24, 64), "f32")
    # filter-gradient form: nothing needs it until the last line
    dw = b.conv(x, g, strides=(1, 1), padding=((1, 1), (1, 1)), dn=("f01b", "i01o", "01bf"))
    h = t
    for k in range(10):
        # each round materialises a reduction and a new tensor of the same size: temporaries come and go
        m = b.reduce_sum(h, [0, 1, 2])
        h = b.add(b.mul(h, 0.5), b.broadcast_in_dim(b.mul(m, 1e-4), h.shape, [3]))
        h = b.maximum(h, b.mul(g, float(k) * 0.01))
    s = b.reduce_sum(h, [0, 1, 2])                                  # [64]
    out = b.add(dw, b.broadcast_in_dim(s, dw.shape, [3]))         # the first reader of the convolution's result
    b.ret(out, h)
    return b.text()


def test_distant_consumer_waits_for_the_second_stream(client):
    from jax_mps_amd import runner
    text = _program()
    rng = np.random.default_rng(5)
    ins = [rng.uniform(0.05, 1.0, s).astype(np.float32) / 8 for s in ((16, 24, 24, 32), (16, 24, 24, 64), (16, 24, 24, 64))]
    exe = client.compile_and_load(text)
    want = Oracle(text).run(*ins)
    bufs = runner.upload(client, ins, ["f32"] * 3)
    for call in range(8):
        print("execute", call, flush=True)
        got = [runner.download(o) for o in exe.execute(bufs)]
        for k, (g, w) in enumerate(zip(got, want)):
            ratio = closeness(g, w, 1e-5, 1e-5)
            assert ratio <= 1.0, f"call {call} output {k}: {ratio:.3f} x the bound"
