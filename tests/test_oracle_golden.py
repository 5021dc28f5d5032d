"""The CPU oracle against the committed golden vectors (tests/golden/cases.json): literal cases of the
reference's own tests with expectations computed by independent closed forms."""
import json
from pathlib import Path

import numpy as np
import pytest

from shlo_oracle import Oracle

CASES = json.loads((Path(__file__).parent / "golden" / "cases.json").read_text())
_NP = {"f32": np.float32, "i32": np.int32, "i64": np.int64, "ui32": np.uint32, "ui64": np.uint64, "i1": np.bool_, "i8": np.int8, "ui8": np.uint8}


def load_inputs(case):
    return [np.array(i["data"], dtype=_NP[i["dtype"]]).reshape(i["shape"]) for i in case["inputs"]]


def load_expected(case):
    return [np.array(e["data"], dtype=np.dtype(e["dtype"])).reshape(e["shape"]) for e in case["expected"]]


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_oracle_matches_golden(case):
    got = Oracle(case["text"]).run(*load_inputs(case))
    want = load_expected(case)
    assert len(got) == len(want)
    for g, w in zip(got, want):
        assert g.shape == w.shape
        assert g.dtype == w.dtype
        if "tol" in case:   # transcendental results: the reference's own bound (tests/test_ops.py:91-105)
            np.testing.assert_allclose(g, w, rtol=case["tol"]["rtol"], atol=case["tol"]["atol"])
        else:
            assert np.array_equal(g, w, equal_nan=True), (case["name"], g, w)
