"""The 256 x 256 tile of the bf16 GEMM (eight wavefronts per workgroup) on shapes that exercise its edges: ragged M and
N, both layouts of the right-hand side (k-contiguous, and [K][N] rows read in place through transposing LDS reads),
bias epilogue, bf16 and f32 results, a batch dim, and K of one and of many 64-wide slabs.  The dispatcher only picks
this tile on its own for large products, so the tests force it (MI355X_GEMM_WIDE=2 is read at every call)."""
import os

import numpy as np
import pytest

from conftest import closeness
from shlo_oracle import Oracle, round_bf16

pytestmark = pytest.mark.gpu

# name, lhs shape, rhs shape, contracting dims (lhs, rhs), batch dims, bias, out dtype
CASES = [
    ("nt-ragged", (500, 256), (328, 256), ([1], [1]), ((), ()), False, "bf16"),
    ("nn-ragged-bias", (500, 192), (192, 328), ([1], [0]), ((), ()), True, "bf16"),
    ("nn-exact-one-slab", (512, 64), (64, 512), ([1], [0]), ((), ()), True, "bf16"),
    ("nt-f32-result", (300, 128), (264, 128), ([1], [1]), ((), ()), False, "f32"),
    ("nn-batched", (3, 260, 128), (3, 128, 272), ([2], [1]), ([0], [0]), False, "bf16"),
    ("nn-long-k", (256, 1024), (1024, 256), ([1], [0]), ((), ()), True, "bf16"),
]


def build(lhs, rhs, contract, batch, bias, out):
    from jax_mps_amd.shlo.builder import Builder
    b = Builder("gemm_wide")
    A, B = b.arg(lhs, "bf16"), b.arg(rhs, "bf16")
    y = b.dot_general(A, B, contract, batch, out_dtype=out)
    args = [A, B]
    if bias:
        v = b.arg((y.shape[-1],), out)
        y = b.add(y, b.broadcast_in_dim(v, y.shape, [len(y.shape) - 1]))
        args.append(v)
    b.ret(y)
    return b.text(), [a.shape for a in args], [a.dtype for a in args]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_wide_tile(client, case):
    from jax_mps_amd import runner
    name, *spec = case
    text, shapes, dtypes = build(*spec)
    rng = np.random.default_rng(abs(hash(name)) % 1000)
    ins = [rng.standard_normal(s).astype(np.float32) for s in shapes]
    print("case", name, spec, flush=True)
    exe = client.compile_and_load(text)
    bufs = runner.upload(client, ins, dtypes)
    os.environ["MI355X_GEMM_WIDE"] = "0"
    try:
        narrow = runner.download(exe.execute(bufs)[0])
        os.environ["MI355X_GEMM_WIDE"] = "2"
        got = runner.download(exe.execute(bufs)[0])
    finally:
        del os.environ["MI355X_GEMM_WIDE"]
    want = Oracle(text).run(*[round_bf16(a) if d == "bf16" else a for a, d in zip(ins, dtypes)])[0]
    tol = 2e-2 if spec[-1] == "bf16" else 1e-5 * max(1.0, float(np.abs(want).max()))
    ratio = closeness(got, want, 2e-2 if spec[-1] == "bf16" else 1e-5, tol)
    assert ratio <= 1.0, f"{name}: {ratio:.3f} x the bound"
    # same products in the same order within a tile column: the two tilings agree to the last bit of the rounded result
    assert closeness(got, narrow, 2e-2 if spec[-1] == "bf16" else 1e-5, tol) <= 1.0
