"""The HIP path against the committed golden vectors, through the PJRT C API (bit-exact)."""
import numpy as np
import pytest

from test_oracle_golden import CASES, load_expected, load_inputs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_plugin_matches_golden(client, case):
    from jax_mps_amd import runner
    print("golden", case["name"], flush=True)
    exe = client.compile_and_load(case["text"])
    bufs = runner.upload(client, load_inputs(case), [i["dtype"] for i in case["inputs"]])
    got = [runner.download(b) for b in exe.execute(bufs)]
    for g, w in zip(got, load_expected(case)):
        assert g.shape == w.shape
        if "tol" in case:
            np.testing.assert_allclose(g, w, rtol=case["tol"]["rtol"], atol=case["tol"]["atol"])
        else:
            assert np.array_equal(g, w.astype(g.dtype), equal_nan=True), (case["name"], g, w)
