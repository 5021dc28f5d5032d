"""The MLIR bytecode (VHLO portable artifact) input of PJRT_Client_Compile (reference:
src/pjrt_plugin/stablehlo_parser.cc:263-285, deserializePortableArtifact).  No artifact written by jaxlib exists
offline, so the artifacts come from tests/vhlo_writer.py: parity with jaxlib's bytes is unpinned; what these tests
pin is that a module survives text -> bytecode -> reader -> text with the same meaning, in every container
variant the format allows (versions 1-6, isolated and inline function regions, packed and byte-wide booleans)."""
import subprocess
import tempfile
from pathlib import Path

import numpy as np
import pytest

import op_cases
from jax_mps_amd.programs import configs
from shlo_oracle import Oracle, round_bf16
from vhlo_writer import to_vhlo_bytecode, varint

ROOT = Path(__file__).resolve().parents[1]
TOOL = ROOT / "jax-mps_amd" / "mi355x-aot"

# op cases the writer can express (it covers the ops of the benchmark programs and the common data-movement,
# control-flow and window ops; chlo ops are not part of a vhlo artifact)
CASES = ["binary-add", "compare-f32-LT", "compare-totalorder", "select", "convert-f32-i32", "while-nested", "while-scan-cumsum",
         "while-dynamic-collatz-27", "case-index-1", "case-inside-counted-loop", "dot-sum-two-products-bias", "int-shifts",
         "while-swapped-carries", "maxpool-3x3-s2-pad1", "maxpool-grad-ties", "round-half", "unary-specials", "bool-logic",
         "all-reduce-one-device-pmean", "all-reduce-one-device-two-operands", "partition-id-axis-index-zero",
         "token-created-merged-and-returned", "token-argument-returned-as-is", "token-carried-by-a-loop",
         "while-hoist-two-loops-share-the-whole-product", "scatter-add-updates-masked-by-the-range-check",
         # custom calls whose JSON backend_config (quotes inside a string attribute) must survive
         "fused-sdpa-padding-mask-f32", "fused-rope-partial-traditional-f32", "fused-layer-norm-bwd-f32"]


def _to_text(bytecode: bytes, *flags) -> subprocess.CompletedProcess:
    with tempfile.NamedTemporaryFile("wb", suffix=".mlirbc", delete=False) as f:
        f.write(bytecode)
        path = f.name
    r = subprocess.run([str(TOOL), *flags, path], capture_output=True, text=True)
    Path(path).unlink()
    return r


def _same_meaning(text, inputs, dtypes, **writer_options):
    r = _to_text(to_vhlo_bytecode(text, **writer_options), "--bytecode-to-text")
    assert r.returncode == 0, r.stderr[-800:]
    ins = [round_bf16(a) if d == "bf16" else a for a, d in zip(inputs, dtypes)]
    want = Oracle(text).run(*ins)
    got = Oracle(r.stdout).run(*ins)
    assert len(got) == len(want)
    for g, w in zip(got, want):
        assert g.dtype == w.dtype and g.shape == w.shape
        assert np.array_equal(g, w, equal_nan=True)


def test_prefix_varints():
    assert varint(0) == b"\x01" and varint(127) == b"\xff" and varint(128) == b"\x02\x02"
    assert varint(1 << 63)[0] == 0 and len(varint(1 << 63)) == 9


@pytest.mark.parametrize("name", list(configs.ALL))
def test_benchmark_programs_survive_the_round_trip(name):
    p = configs.ALL[name](**configs.SMALL[name])
    _same_meaning(p.text, p.inputs, p.input_dtypes)


@pytest.mark.parametrize("name", CASES)
def test_op_cases_survive_the_round_trip(name):
    c = op_cases.get_case(name)
    _same_meaning(c.text, c.inputs, c.dtypes)


def test_every_op_case_the_writer_can_express_survives_the_round_trip():
    """All per-op cases in one sweep (the list above is the subset that runs one test each): a case either is outside
    what the writer expresses (chlo ops: not part of a vhlo artifact) or comes back from the reader with the same meaning."""
    skipped = []
    for name in op_cases.case_names():
        c = op_cases.get_case(name)
        try:
            to_vhlo_bytecode(c.text)
        except Exception:
            skipped.append(name)
            continue
        with np.errstate(all="ignore"):
            _same_meaning(c.text, c.inputs, c.dtypes)
    assert len(skipped) <= 12 and all("chlo" in op_cases.get_case(n).text for n in skipped), skipped


@pytest.mark.parametrize("options", [dict(version=1), dict(version=2, isolated_funcs=True), dict(version=3), dict(version=4),
                                     dict(version=5, isolated_funcs=True), dict(version=6, pack_bools=False), dict(version=6, isolated_funcs=True),
                                     dict(version=5, module_properties=True), dict(version=6, isolated_funcs=True, module_properties=True)],
                         ids=lambda o: "-".join(f"{k}={v}" for k, v in o.items()))
def test_container_variants(options):
    p = configs.build_lstm(**configs.SMALL["lstm"])            # loops, nested regions, constants, dots
    _same_meaning(p.text, p.inputs, p.input_dtypes, **options)
    c = op_cases.get_case("bool-logic")
    _same_meaning(c.text, c.inputs, c.dtypes, **options)


def test_bytecode_plans_like_its_text():
    p = configs.build_resnet18(**configs.SMALL["resnet18"])
    a = _to_text(to_vhlo_bytecode(p.text), "--no-compile")
    with tempfile.NamedTemporaryFile("w", suffix=".mlir", delete=False) as f:
        f.write(p.text)
    b = subprocess.run([str(TOOL), "--no-compile", f.name], capture_output=True, text=True)
    Path(f.name).unlink()
    assert a.returncode == 0 and b.returncode == 0, a.stderr[-500:]
    assert a.stdout.split(":", 1)[1] == b.stdout.split(":", 1)[1]       # same ops, steps, kernels, arena


def test_device_counts_and_replica_groups_travel():
    """The module's device counts (builtin attributes of builtin.module) and the shape of replica_groups reach the
    compiler from bytecode too: the multi-device errors fire as they do for text."""
    c = op_cases.get_case("partition-id-axis-index-zero")
    r = _to_text(to_vhlo_bytecode(c.text), "--bytecode-to-text")
    assert "module attributes {mhlo.num_partitions = 1 : i32, mhlo.num_replicas = 1 : i32} {" in r.stdout
    r = _to_text(to_vhlo_bytecode(c.text.replace("mhlo.num_partitions = 1", "mhlo.num_partitions = 8")))
    assert r.returncode != 0 and "multi-partition execution is not supported" in r.stderr
    c = op_cases.get_case("all-reduce-one-device-pmean")
    r = _to_text(to_vhlo_bytecode(c.text.replace("dense<0> : tensor<1x1xi64>", "dense<[[0, 1]]> : tensor<1x2xi64>")))
    assert r.returncode != 0 and "multi-device all_reduce is not supported" in r.stderr
    r = _to_text(to_vhlo_bytecode(c.text.replace("dense<0> : tensor<1x1xi64>", "dense<[[0], [1]]> : tensor<2x1xi64>")))
    assert r.returncode == 0, r.stderr


def test_donation_attributes_travel():
    text = ("module { func.func public @main(%w: tensor<8xf32> {tf.aliasing_output = 0 : i32}, %g: tensor<8xf32>) -> tensor<8xf32> {\n"
            " %0 = stablehlo.subtract %w, %g : tensor<8xf32>\n return %0 : tensor<8xf32> } }")
    from vhlo_writer import Writer
    w = Writer(text)
    w.arg_attrs_override = {("main", 0): [("tf.aliasing_output", w.a_int(0, "i32"))]}
    r = _to_text(w.write(), "--bytecode-to-text")
    assert r.returncode == 0, r.stderr
    assert "tf.aliasing_output = 0 : i32" in r.stdout


def test_unknown_encoding_of_a_used_attribute_is_a_compile_error():
    """An attribute an op's meaning depends on, written with an attribute code the reader does not know, must stop the
    compile with an error that names the attribute and the op: never a silently defaulted comparison."""
    from vhlo_writer import Writer

    class FutureWriter(Writer):
        def a_enum(self, code, names, value):
            key = super().a_enum(code, names, value)
            return (key[0], key[1], 250, key[3]) if "LT" in names else key     # comparison_direction in an encoding of the future
    c = op_cases.get_case("compare-f32-LT")
    r = _to_text(FutureWriter(c.text).write(), "--no-compile")
    assert r.returncode == 1, r.stdout
    assert "comparison_direction" in r.stderr and "vhlo.compare" in r.stderr and "attribute code 250" in r.stderr, r.stderr[-400:]


@pytest.mark.parametrize("damage", ["truncate", "bad_magic_version", "bad_section"])
def test_damaged_files_are_compile_errors_not_crashes(damage):
    good = to_vhlo_bytecode(configs.build_mlp(**configs.SMALL["mlp"]).text)
    if damage == "truncate":
        blobs = [good[:n] for n in (5, 40, len(good) // 2, len(good) - 3)]
    elif damage == "bad_magic_version":
        blobs = [good[:4] + varint(9) + good[5:]]
    else:
        blobs = [good[:30] + bytes([0x7F]) + good[31:], good.replace(b"vhlo\x00", b"vhlx\x00")]
    for b in blobs:
        r = _to_text(b, "--no-compile")
        assert r.returncode == 1 and ("bytecode" in r.stderr or "parse error" in r.stderr), r.stderr[-300:]


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(configs.ALL))
def test_plugin_runs_bytecode_like_text(client, name):
    """PJRT_Client_Compile with the artifact in place of the text: identical results, bit for bit."""
    from jax_mps_amd import runner
    p = configs.ALL[name](**configs.SMALL[name])
    bufs = runner.upload(client, p.inputs, p.input_dtypes)
    want = [runner.download(o) for o in client.compile_and_load(p.text).execute(bufs)]
    got = [runner.download(o) for o in client.compile_and_load(to_vhlo_bytecode(p.text)).execute(bufs)]
    assert len(got) == len(want)
    for g, w in zip(got, want):
        assert np.array_equal(g, w, equal_nan=True)
