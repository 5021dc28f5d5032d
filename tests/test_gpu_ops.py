"""Per-op parity on the GPU: every case of op_cases.py runs through PJRT_Client_Compile /
PJRT_LoadedExecutable_Execute / PJRT_Buffer_ToHostBuffer and is compared with the CPU oracle.

Bar: bit-exact for integer, boolean, index and data-movement results; for float arithmetic the reference's
elementwise rule |got - want| <= tol + tol |want| (tests/test_ops.py:91-105) with tol = 1e-5 for f32 and
2e-2 for bf16."""
import numpy as np
import pytest

import op_cases
from conftest import closeness
from shlo_oracle import Oracle, round_bf16

pytestmark = pytest.mark.gpu

F32_TOL = 1e-5
BF16_TOL = 2e-2
F16_TOL = 2e-3    # two units in the last place of an 11-bit significand
# cases the plan compiler rejects (none at present; the error texts are checked in test_frontend.py)
UNSUPPORTED = set()
# cases held to a looser elementwise bound than the dtype's, each with its reason
LOOSER = {
    # Sums of K products whose magnitudes add up to S ~ 750 (K = 3000 terms of products of uniform(-1, 1) values) or
    # S ~ 500 (K = 384 terms of uniform(-2, 2) values) while the sum itself can be near 0: float32 accumulation, in
    # any order, is good to a few 2^-24 S ~ 3e-5 absolute, which an element near 0 cannot meet at 1e-5.
    "dot-large-k": 4e-5,
    "dot-sum-two-products-bias": 4e-5,
}


@pytest.mark.parametrize("name", [n for n in op_cases.case_names() if n not in UNSUPPORTED])
def test_op_case(client, name):
    from jax_mps_amd import runner
    c = op_cases.get_case(name)
    print("case", name, flush=True)
    exe = client.compile_and_load(c.text)
    bufs = runner.upload(client, c.inputs, c.dtypes)
    got = [runner.download(b) for b in exe.execute(bufs)]
    ins = [round_bf16(a) if d == "bf16" else a for a, d in zip(c.inputs, c.dtypes)]
    oracle = Oracle(c.text)
    want = oracle.run(*ins)
    assert len(got) == len(want)
    for k, (g, w, (shape, dt)) in enumerate(zip(got, want, oracle.result_types)):
        assert g.shape == tuple(shape)
        if dt in ("f32", "bf16", "f16") and not c.exact:
            tol = BF16_TOL if "bf16" in c.dtypes or dt == "bf16" else F16_TOL if "f16" in c.dtypes or dt == "f16" else F32_TOL
            tol = LOOSER.get(name, tol)
            ratio = closeness(g, w, tol, tol)
            assert ratio <= 1.0, f"{name} output {k}: {ratio:.3f} x the bound |d| <= {tol} + {tol} |want|"
        else:
            gw = g.view(np.uint32) if g.dtype == np.float32 else g
            ww = np.asarray(w).astype(g.dtype)
            ww = ww.view(np.uint32) if ww.dtype == np.float32 else ww
            if g.dtype == np.float32:
                # NaN payloads may differ; everything else must match bit for bit
                nan = np.isnan(g) & np.isnan(np.asarray(w, dtype=np.float32))
                assert np.array_equal(gw[~nan], ww[~nan]), f"{name} output {k} differs"
            else:
                assert np.array_equal(gw, ww), f"{name} output {k} differs"
