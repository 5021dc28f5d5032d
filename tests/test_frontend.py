"""Front end and planner on the CPU: the ahead-of-time tool parses and plans StableHLO text (no GPU),
including the generic op form, counted-loop detection and the unsupported-op diagnostics."""
import subprocess
import tempfile
from pathlib import Path

import pytest

import op_cases
from jax_mps_amd.programs import configs

ROOT = Path(__file__).resolve().parents[1]
TOOL = ROOT / "jax-mps_amd" / "mi355x-aot"


def plan(text, *flags):
    with tempfile.NamedTemporaryFile("wb", suffix=".mlir", delete=False) as f:
        f.write(text if isinstance(text, bytes) else text.encode())
        path = f.name
    r = subprocess.run([str(TOOL), "--no-compile", *flags, path], capture_output=True, text=True)
    Path(path).unlink()
    return r


def test_tool_is_built():
    assert TOOL.exists(), "run __graft_entry__.build() first"


def test_every_op_case_plans():
    bad = []
    for c in op_cases.all_cases():
        r = plan(c.text)
        if r.returncode != 0:
            bad.append((c.name, r.stderr[-300:]))
    assert not bad, bad


def test_unsupported_ops_are_named():
    r = plan("module { func.func public @main(%a: tensor<4xf32>) -> tensor<4xf32> {\n %0 = stablehlo.fft %a : tensor<4xf32>\n return %0 : tensor<4xf32> } }")
    assert r.returncode != 0 and ("fft" in r.stderr)
    r = plan("module { func.func public @main(%a: tensor<4xf64>) -> tensor<4xf64> {\n return %a : tensor<4xf64> } }")
    assert r.returncode == 0   # f64 values may pass through; arithmetic on them is generated as double


def test_bytecode_is_rejected_with_a_clear_message():
    r = plan(b"ML\xefR" + b"\x00" * 16)
    assert r.returncode != 0 and "bytecode" in r.stderr


def test_counted_loop_detection():
    r = plan(op_cases.get_case("while-130-iterations").text, "--dump-plan")
    assert "while while trip 130" in r.stdout
    r = plan(op_cases.get_case("while-zero-trip").text, "--dump-plan")
    assert "trip 0" in r.stdout
    r = plan(op_cases.get_case("while-value-dependent").text, "--dump-plan")
    assert "trip -1" in r.stdout
    r = plan(op_cases.get_case("while-traced-bound").text, "--dump-plan")
    assert "trip -1" in r.stdout


def test_lstm_scan_updates_in_place():
    p = configs.build_lstm(**configs.SMALL["lstm"])
    r = plan(p.text, "--dump-plan")
    assert r.returncode == 0
    assert "while while trip 7" in r.stdout
    assert "dynamic_update_slice operand copy" not in r.stdout     # residual stacks are written in place


def test_generic_op_form_and_helper_functions():
    text = '''
module @m {
  func.func public @main(%arg0: tensor<4x3xf32>, %arg1: tensor<2xi32>) -> (tensor<2x3xf32>) {
    %0 = "stablehlo.reshape"(%arg1) : (tensor<2xi32>) -> tensor<2x1xi32>
    %1 = "stablehlo.gather"(%arg0, %0) <{dimension_numbers = #stablehlo.gather<offset_dims = [1], collapsed_slice_dims = [0], start_index_map = [0], index_vector_dim = 1>, indices_are_sorted = false, slice_sizes = array<i64: 1, 3>}> : (tensor<4x3xf32>, tensor<2x1xi32>) -> tensor<2x3xf32>
    %2 = "stablehlo.transpose"(%1) <{permutation = array<i64: 1, 0>}> : (tensor<2x3xf32>) -> tensor<3x2xf32>
    %3 = "stablehlo.broadcast_in_dim"(%2) <{broadcast_dimensions = array<i64: 0, 1>}> : (tensor<3x2xf32>) -> tensor<3x2xf32>
    %4 = func.call @double(%3) : (tensor<3x2xf32>) -> tensor<3x2xf32>
    %5 = "stablehlo.dot_general"(%1, %4) <{dot_dimension_numbers = #stablehlo.dot<lhs_contracting_dimensions = [1], rhs_contracting_dimensions = [0]>}> : (tensor<2x3xf32>, tensor<3x2xf32>) -> tensor<2x2xf32>
    %6 = "stablehlo.compare"(%5, %5) <{comparison_direction = #stablehlo<comparison_direction GE>}> : (tensor<2x2xf32>, tensor<2x2xf32>) -> tensor<2x2xi1>
    %7 = "stablehlo.slice"(%1) <{limit_indices = array<i64: 2, 3>, start_indices = array<i64: 0, 0>, strides = array<i64: 1, 1>}> : (tensor<2x3xf32>) -> tensor<2x3xf32>
    return %7 : tensor<2x3xf32>
  }
  func.func private @double(%a: tensor<3x2xf32>) -> tensor<3x2xf32> {
    %0 = stablehlo.add %a, %a : tensor<3x2xf32>
    return %0 : tensor<3x2xf32>
  }
}'''
    r = plan(text, "--dump-plan")
    assert r.returncode == 0, r.stderr


@pytest.mark.parametrize("name", list(configs.ALL))
def test_benchmark_programs_plan(name):
    p = configs.ALL[name](**configs.SMALL[name])
    r = plan(p.text)
    assert r.returncode == 0, r.stderr[-500:]
