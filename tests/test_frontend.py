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


def test_malformed_bytecode_is_rejected_with_a_clear_message():
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


def test_dynamic_loops_and_cases_in_loops_stay_on_the_device():
    """A data-dependent while runs under a device flag with conditional carry commits; a case inside a loop runs all
    of its branches with result copies selected on the device; neither needs a host read per iteration."""
    r = plan(op_cases.get_case("while-dynamic-collatz-27").text, "--dump-plan")
    assert "flag-init loop flag" in r.stdout and "while while trip -1 on-device" in r.stdout
    assert "flag-and loop flag &= condition" in r.stdout and "loop carry update if-alive" in r.stdout
    r = plan(op_cases.get_case("while-dynamic-scan-stops-early").text, "--dump-plan")
    assert "dynamic_update_slice operand copy" in r.stdout      # no in-place update of a carry that a queued-ahead iteration could spoil
    r = plan(op_cases.get_case("case-inside-counted-loop").text, "--dump-plan")
    assert "case case all-branches" in r.stdout and r.stdout.count("case result if-selected") == 3
    r = plan(op_cases.get_case("case-index-1").text, "--dump-plan")
    assert "all-branches" not in r.stdout                        # outside loops one branch runs, chosen on the host


def test_missing_required_attributes_are_compile_errors():
    text = 'module { func.func public @main(%a: tensor<4xf32>) -> tensor<4xf32> {\n %0 = "stablehlo.reduce_precision"(%a) : (tensor<4xf32>) -> tensor<4xf32>\n return %0 : tensor<4xf32> } }'
    r = plan(text)
    assert r.returncode != 0 and "exponent_bits" in r.stderr
    text = 'module { func.func public @main(%a: tensor<4xf32>) -> tensor<4x2xf32> {\n %0 = "stablehlo.broadcast_in_dim"(%a) : (tensor<4xf32>) -> tensor<4x2xf32>\n return %0 : tensor<4x2xf32> } }'
    r = plan(text)
    assert r.returncode != 0 and "dims" in r.stderr


def test_collectives_and_ids_of_more_than_one_device_are_compile_errors():
    """One device only: an all_reduce whose replica groups hold more than one member, a partition_id in a module of
    several partitions and a replica_id in a module of several replicas fail at compile time with the reference's
    messages (src/pjrt_plugin/ops/collectives.cc:22-33, 58-66) instead of computing on one device's share."""
    good = op_cases.get_case("all-reduce-one-device-two-operands").text
    assert plan(good).returncode == 0
    r = plan(good.replace("dense<0> : tensor<1x1xi64>", "dense<[[0, 1]]> : tensor<1x2xi64>"))
    assert r.returncode != 0 and "multi-device all_reduce is not supported" in r.stderr
    r = plan(good.replace("dense<0> : tensor<1x1xi64>", "dense<[0, 1]> : tensor<2xi64>"))
    assert r.returncode != 0 and "multi-device all_reduce is not supported" in r.stderr
    assert plan(good.replace("dense<0> : tensor<1x1xi64>", "dense<[[0], [1]]> : tensor<2x1xi64>")).returncode == 0   # groups of one
    ids = op_cases.get_case("partition-id-axis-index-zero").text
    assert plan(ids).returncode == 0
    r = plan(ids.replace("mhlo.num_partitions = 1", "mhlo.num_partitions = 2"))
    assert r.returncode != 0 and "multi-partition execution is not supported" in r.stderr
    r = plan(ids.replace("mhlo.num_replicas = 1", "mhlo.num_replicas = 4"))
    assert r.returncode != 0 and "replica" in r.stderr
    r = plan(ids.replace("stablehlo.partition_id : tensor<ui32>", "stablehlo.partition_id : tensor<1xui32>").replace("(tensor<ui32>) -> tensor<i32>", "(tensor<1xui32>) -> tensor<i32>"))
    assert r.returncode != 0 and "scalar" in r.stderr


def test_tokens_travel_as_scalar_placeholders():
    """Tokens order side effects and carry no data; the plan holds no step for create_token or after_all and the
    token results of main are f32 scalars (reference: src/pjrt_plugin/ops/control_flow.cc:2266-2288)."""
    r = plan(op_cases.get_case("token-created-merged-and-returned").text, "--dump-plan")
    assert r.returncode == 0, r.stderr
    assert "token" not in r.stdout and "after_all" not in r.stdout
    r = plan(op_cases.get_case("token-carried-by-a-loop").text, "--dump-plan")
    assert r.returncode == 0 and "while while trip 3" in r.stdout


def test_relu_rides_in_a_small_product_and_its_mask_reads_the_activation():
    """maximum(x, 0) after a small fp32 product is applied while the product is stored; the backward mask compare(x, 0, GT)
    is taken from the activation, so the value before it is never written.  A second reader of that value, or a product
    too large for the small-product kernel, keeps the separate kernel."""
    r = plan(op_cases.get_case("dot-bias-relu-f32-small-mask-from-activation").text, "--dump-plan")
    assert "+ bias + relu" in r.stdout and "maximum" not in r.stdout
    r = plan(op_cases.get_case("dot-bias-relu-f32-small-value-before-also-read").text, "--dump-plan")
    assert "+ relu" not in r.stdout and "maximum" in r.stdout
    r = plan(op_cases.get_case("dot-relu-f32-igemm-not-small").text, "--dump-plan")
    assert "+ relu" not in r.stdout
    r = plan(configs.ALL["mlp"]().text, "--dump-plan")
    assert r.stdout.count("+ bias + relu") == 1 and " 7 steps" in r.stdout


def test_products_of_sequence_slices_leave_the_loop():
    """x[i] . W inside a counted loop, x and W untouched by the loop, is one product over all of x ahead of the loop; two loops
    that need the same whole product share it.  A loop far shorter than the sequence, or a sequence whose selected dim and
    other free dims are apart in memory, keeps its products."""
    r = plan(op_cases.get_case("while-hoist-product-of-sequence-slice").text, "--dump-plan")
    ahead, body = r.stdout.split("while while trip 12")
    assert "dot_general tensor<12x6x20xf32> x tensor<20x16xf32>" in ahead
    assert "dot_general tensor<6x16xf32> x tensor<16x16xf32>" in body and "20x16" not in body
    for name in ("while-hoist-reversed-index", "while-hoist-index-clamped-at-the-end", "while-hoist-sequence-carried-unchanged"):
        r = plan(op_cases.get_case(name).text, "--dump-plan")
        assert "dot_general tensor<12x6x20xf32> x tensor<20x16xf32>" in r.stdout.split("while while trip")[0], name
    r = plan(op_cases.get_case("while-hoist-slice-of-a-middle-dim").text, "--dump-plan")
    assert "dot_general tensor<6x12x20xf32> x tensor<20x16xf32>" in r.stdout.split("while while trip")[0]
    r = plan(op_cases.get_case("while-hoist-slice-is-the-right-operand").text, "--dump-plan")
    assert "dot_general tensor<16x20xf32> x tensor<9x6x20xf32>" in r.stdout.split("while while trip")[0]
    r = plan(op_cases.get_case("while-hoist-two-loops-share-the-whole-product").text, "--dump-plan")
    assert r.stdout.count("dot_general tensor<12x6x20xf32> x tensor<20x16xf32>") == 1 and r.stdout.count("tensor<12x6x16xf32> x tensor<16x16xf32>") == 1
    assert r.stdout.count("+ tensor") == 2        # the two weight gradients are summed into their carries by the products themselves
    for name in ("while-short-loop-over-long-sequence-keeps-its-products", "while-slice-is-the-right-operand-free-dims-apart"):
        r = plan(op_cases.get_case(name).text, "--dump-plan")
        assert "dot_general" not in r.stdout.split("while while trip")[0], name
    r = plan(configs.ALL["lstm"]().text, "--dump-plan")
    loops = r.stdout.split("while while trip 100")
    assert len(loops) == 3
    forward = loops[1].split("\ngemm ")[0]
    assert forward.count("\n  gemm ") == 1 and forward.count("\n  kernel ") == 2        # (one of the two is the unused condition)
    backward = loops[2].split("\nkernel ")[0]
    assert backward.count("\n  gemm-group ") == 1 and backward.count("\n  gemm ") == 0 and backward.count("\n  kernel ") == 2


def test_updates_masked_by_the_scatter_s_own_range_check_are_read_unmasked():
    """select(index in range, u, 0) ahead of a whole-row scatter with that index only rewrites rows the scatter drops anyway:
    no kernel computes it.  A narrower check, or a check of another index, changes rows the scatter keeps and stays."""
    for name in ("scatter-add-updates-masked-by-the-range-check", "scatter-max-updates-masked-by-the-range-check"):
        r = plan(op_cases.get_case(name).text, "--dump-plan")
        assert r.returncode == 0 and "fusion:select" not in r.stdout, name
    for name in ("scatter-add-updates-masked-by-a-narrower-check", "scatter-add-updates-masked-by-another-index"):
        r = plan(op_cases.get_case(name).text, "--dump-plan")
        assert r.returncode == 0 and "fusion:select" in r.stdout, name
    r = plan(configs.ALL["embedding"]().text, "--dump-plan")
    assert " 2 steps" in r.stdout and "arena 0.22 MiB" in r.stdout        # the masked copy of the 25 MB of updates is gone


def test_a_value_read_at_ever_more_positions_is_stored():
    """v + reverse(v), forty times over, would be one kernel evaluating the first value at 2^40 positions; the planner stores a
    value once a kernel would evaluate it at more than 32 positions, so the program compiles at once into a handful of kernels."""
    import time
    t0 = time.time()
    r = plan(op_cases.get_case("elementwise-chain-read-at-mirrored-positions-40-links").text, "--dump-plan")
    assert r.returncode == 0 and time.time() - t0 < 20
    steps = int(r.stdout.rsplit("->", 1)[1].split("steps")[0])
    assert 5 <= steps <= 12


def test_a_column_reduction_stores_the_value_it_reads_first():
    """A large elementwise value that has to exist in memory and is first read by a column reduction gets no kernel of its
    own: the reduction's pass over the data writes it.  A product that reads it earlier keeps the separate kernel."""
    r = plan(op_cases.get_case("reduce-column-stores-its-input-two-passes").text, "--dump-plan")
    assert r.stdout.count("storing select") == 2 and "fusion:select" not in r.stdout        # the pass over the data and the fold
    r = plan(op_cases.get_case("reduce-column-small-input-stored-by-one-pass").text, "--dump-plan")
    assert r.stdout.count("storing select") == 1 and "fusion:select" not in r.stdout        # one launch: narrow column tiles give it a few dozen workgroups
    r = plan(op_cases.get_case("reduce-column-tiny-input-keeps-its-own-kernel").text, "--dump-plan")
    assert "storing" not in r.stdout        # below 16 384 elements the value is recomputed or keeps its kernel
    r = plan(op_cases.get_case("reduce-column-input-read-by-a-product-first").text, "--dump-plan")
    assert "storing" not in r.stdout
    r = plan(configs.build_resnet18().text, "--dump-plan")
    assert r.stdout.count("storing select") == 34 and "fusion:select" not in r.stdout        # 17 batch-norm backward passes, two launches each


def test_location_aliases_result_lists_and_composites_parse():
    text = """#loc1 = loc("x")
module @jit_f attributes {mhlo.num_partitions = 1 : i32} {
  func.func private @chlo.sinh.impl(%arg0: tensor<4xf32> loc(unknown)) -> tensor<4xf32> {
    %0 = stablehlo.exponential %arg0 : tensor<4xf32> loc(#loc2)
    %1 = stablehlo.negate %arg0 : tensor<4xf32> loc(#loc2)
    %2 = stablehlo.exponential %1 : tensor<4xf32> loc(#loc2)
    %3 = stablehlo.subtract %0, %2 : tensor<4xf32> loc(#loc2)
    return %3 : tensor<4xf32> loc(#loc)
  } loc(#loc)
  func.func public @main(%arg0: tensor<4xf32> loc("x"), %arg1: tensor<8xf32> loc("y")) -> (tensor<4xf32>, tensor<3xf32>, tensor<3xi32>) {
    %0 = stablehlo.composite "chlo.sinh" %arg0 {decomposition = @chlo.sinh.impl, version = 1 : i32} : (tensor<4xf32>) -> tensor<4xf32> loc(#loc3)
    %values, %indices = chlo.top_k(%arg1, k = 3) : tensor<8xf32> -> (tensor<3xf32>, tensor<3xi32>) loc(#loc3)
    return %0, %values, %indices : tensor<4xf32>, tensor<3xf32>, tensor<3xi32> loc(#loc)
  } loc(#loc)
} loc(#loc)
#loc = loc(unknown)
#loc2 = loc("/tmp/f.py":3:11 to :58)
#loc3 = loc("jit(f)/sinh"(#loc2))
"""
    r = plan(text, "--dump-plan")
    assert r.returncode == 0, r.stderr


def test_shardy_declarations_hex_constants_and_argument_attributes_parse():
    """What jax prints around a single-device program when the Shardy partitioner is on (module-level sdy.mesh, #sdy.sharding
    argument attributes), large constants as hex strings, boolean lists, layout / donor attributes, @Sharding custom calls
    and optimization barriers: all accepted, as the reference lets unregistered dialects pass (stablehlo_parser.cc:74-75)."""
    text = """#loc = loc(unknown)
module @jit_f attributes {jax.uses_shape_polymorphism = false, mhlo.num_partitions = 1 : i32, mhlo.num_replicas = 1 : i32} {
  sdy.mesh @mesh = <["x"=1]>
  func.func public @main(%arg0: tensor<3xf32> {mhlo.layout_mode = "default", sdy.sharding = #sdy.sharding<@mesh, [{"x"}]>} loc(unknown), %arg1: tensor<2x4xf32> {jax.buffer_donor = true}) -> (tensor<3xf32> {jax.result_info = "[0]", mhlo.layout_mode = "default"}, tensor<2xi1>, tensor<1x2xf32>) {
    %cst = stablehlo.constant dense<"0x0000803F0000004000004040"> : tensor<3xf32> loc(#loc)
    %c = stablehlo.constant dense<[true, false]> : tensor<2xi1> loc(#loc)
    %c_0 = stablehlo.constant dense<true> : tensor<i1>
    %cst_2 = stablehlo.constant dense<1.500000e+00> : tensor<3xf32>
    %0 = stablehlo.add %arg0, %cst : tensor<3xf32> loc(#loc)
    %1 = stablehlo.multiply %0, %cst_2 : tensor<3xf32>
    %2 = stablehlo.broadcast_in_dim %c_0, dims = [] : (tensor<i1>) -> tensor<2xi1>
    %3 = stablehlo.and %c, %2 : tensor<2xi1>
    %c_3 = stablehlo.constant dense<1> : tensor<i32>
    %c_4 = stablehlo.constant dense<0> : tensor<i32>
    %4 = stablehlo.dynamic_slice %arg1, %c_4, %c_3, sizes = [1, 2] : (tensor<2x4xf32>, tensor<i32>, tensor<i32>) -> tensor<1x2xf32>
    %5 = stablehlo.custom_call @Sharding(%4) {backend_config = "", mhlo.sharding = "{replicated}"} : (tensor<1x2xf32>) -> tensor<1x2xf32>
    %6 = stablehlo.optimization_barrier %5 : tensor<1x2xf32>
    return %1, %3, %6 : tensor<3xf32>, tensor<2xi1>, tensor<1x2xf32> loc(#loc)
  } loc(#loc)
} loc(#loc)
"""
    r = plan(text)
    assert r.returncode == 0, r.stderr
    # the hex string holds 1, 2, 3: the oracle reads the same text and adds it to the argument
    import numpy as np
    from shlo_oracle import Oracle
    plain = text.replace('  sdy.mesh @mesh = <["x"=1]>\n', "").replace(', sdy.sharding = #sdy.sharding<@mesh, [{"x"}]>', "")   # (the oracle reads no Shardy)
    got = Oracle(plain).run(np.array([10, 20, 30], np.float32), np.arange(8, dtype=np.float32).reshape(2, 4))
    assert np.array_equal(got[0], np.array([16.5, 33.0, 49.5], np.float32)) and np.array_equal(got[1], [True, False]) and np.array_equal(got[2], [[1.0, 2.0]])


def test_convolution_delivers_batch_norm_statistics():
    """The column sum and sum of squares of an unsplit convolution's output come from its accumulators: the pass over
    the output is gone and only the fold of the per-tile sums remains; a convolution that splits K, or a reduction
    of another kind, keeps its own pass over the output."""
    r = plan(op_cases.get_case("conv-statistics-from-accumulators").text, "--dump-plan")
    assert "+ column statistics" in r.stdout and r.stdout.count("kernel ") == 1 and "fold of convolution statistics" in r.stdout
    r = plan(op_cases.get_case("conv-statistics-split-k-stays-unfused").text, "--dump-plan")
    assert "column statistics" not in r.stdout and "reduce" in r.stdout      # (small enough for single-pass reductions, which share a launch)
    r = plan(op_cases.get_case("conv-statistics-max-stays-unfused").text, "--dump-plan")
    assert "column statistics" not in r.stdout
    p = configs.build_resnet18()
    r = plan(p.text, "--dump-plan")
    assert r.stdout.count("+ column statistics") >= 14      # every unsplit forward convolution that feeds a batch norm


def test_distant_convolutions_take_the_second_stream():
    """A convolution nothing reads for several steps is marked for the second stream and its first reader waits for it;
    the filter gradients of the ResNet step are such convolutions, and a program with a loop forks nothing."""
    import test_gpu_second_stream
    r = plan(test_gpu_second_stream._program(), "--dump-plan")
    lines = r.stdout.splitlines()
    assert "[second stream #0]" in lines[0] and lines[0].startswith("conv ")
    assert any("[waits for #0]" in l for l in lines[1:]) and sum("[second stream" in l for l in lines) == 1
    r = plan(configs.build_resnet18().text, "--dump-plan")
    assert r.stdout.count("[second stream #") >= 13 and r.stdout.count("[waits for #") == r.stdout.count("[second stream #")
    r = plan(configs.build_lstm(**configs.SMALL["lstm"]).text, "--dump-plan")
    assert "[second stream" not in r.stdout


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


def test_fused_op_custom_calls_are_expanded_or_refused_by_name():
    """custom_call @mps.<op> (the reference's Python primitives, src/jax_plugins/mps/ops.py) is rewritten into plain
    StableHLO before planning; the bf16 attention call at a shape the attention kernel takes becomes one launch of it;
    a malformed call, an undeclared result type and an unknown target are compile errors that name the target."""
    r = plan(op_cases.get_case("fused-sdpa-encoder-heads-bf16").text, "--dump-plan")
    assert r.returncode == 0 and "attention tensor<2x12x128x64xbf16> masked" in r.stdout and "1 steps" in r.stdout, r.stdout[-400:]
    # JAX's own spelling of a quote inside a string attribute is \22; the plainer \" is read as well
    text = op_cases.get_case("fused-rms-norm-f32").text
    assert "\\22eps\\22" in text
    assert plan(text.replace("\\22", '\\"')).returncode == 0
    assert plan(text.replace("@mps.rms_norm", "@mi355x.rms_norm")).returncode == 0
    r = plan(text.replace("@mps.rms_norm", "@mps.rms_norm_bwd"))
    assert r.returncode != 0 and "mps.rms_norm_bwd" in r.stderr and "expected 3 inputs and 2 outputs" in r.stderr
    r = plan(text.replace("-> tensor<6x33x96xf32>", "-> tensor<6x33x95xf32>"))
    assert r.returncode != 0 and "mps.rms_norm" in r.stderr and "declared" in r.stderr
    r = plan(text.replace("@mps.rms_norm", "@mps.quantized_matmul"))
    assert r.returncode != 0 and "mps.quantized_matmul" in r.stderr
