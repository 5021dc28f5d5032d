"""The five benchmark programs on the GPU against the CPU oracle (reduced sizes the oracle
finishes in seconds), plus size-independent properties at the full benchmark sizes."""
import numpy as np
import pytest

from conftest import closeness
from shlo_oracle import Oracle, round_bf16

pytestmark = pytest.mark.gpu


def _run_both(client, program):
    from jax_mps_amd import runner
    cp = runner.CompiledProgram(program, client)
    got = cp.run_once()
    ins = [round_bf16(a) if d == "bf16" else a for a, d in zip(program.inputs, program.input_dtypes)]
    want = Oracle(program.text).run(*ins)
    return got, want


def _worst(program, got, want, tol=1e-5):
    """Worst ratio to the reference's elementwise rule |got - want| <= tol + tol |want| (tests/test_ops.py:91-105)
    over the float outputs (<= 1 passes); integer outputs must be equal."""
    worst, where = 0.0, None
    for n, g, w in zip(program.output_names, got, want):
        if np.asarray(w).dtype.kind in "iub":
            assert np.array_equal(g, w), n
            continue
        e = closeness(g, w, tol, tol)
        if e > worst:
            worst, where = e, n
    return worst, where


@pytest.mark.parametrize("size", ["SMALL", "MEDIUM"])
def test_mlp_train_step(client, size):
    from jax_mps_amd.programs import configs
    p = configs.build_mlp(**getattr(configs, size)["mlp"])
    got, want = _run_both(client, p)
    worst, where = _worst(p, got, want)
    assert worst <= 1.0, (where, worst)


def test_mlp_100_steps_loss_trajectory(client):
    """Config 1 as BASELINE states it: 100 SGD steps, loss and parameters against the oracle."""
    from jax_mps_amd import runner
    from jax_mps_amd.programs import configs
    p = configs.build_mlp(batch=64, d_in=96, d_hidden=64)
    cp = runner.CompiledProgram(p, client)
    oracle = Oracle(p.text)
    state = list(p.inputs)
    for step in range(100):
        outs = cp.step()
        ref = oracle.run(*state)
        for k, i in p.feedback.items():
            state[i] = ref[k]
        if step % 20 == 19 or step == 0:
            loss = float(runner.download(outs[-1]))
            assert abs(loss - float(ref[-1])) <= 1e-5 * abs(float(ref[-1])) + 1e-6, (step, loss, float(ref[-1]))
    for k in range(4):
        assert closeness(runner.download(cp.state[k]), state[k]) <= 1.0


@pytest.mark.parametrize("size", ["SMALL", "MEDIUM"])
def test_embedding_gather_scatter_bit_exact(client, size):
    from jax_mps_amd.programs import configs
    p = configs.build_embedding(**getattr(configs, size)["embedding"])
    got, want = _run_both(client, p)
    table, idx, g = p.inputs
    assert np.array_equal(got[0].view(np.uint32), table[idx].view(np.uint32))
    assert np.array_equal(got[0].view(np.uint32), want[0].view(np.uint32))
    # sequential accumulation in update order, independent of the oracle's scatter
    seq = np.zeros_like(table)
    np.add.at(seq, idx, g)
    assert np.array_equal(got[1].view(np.uint32), seq.view(np.uint32))
    assert np.array_equal(got[1].view(np.uint32), want[1].view(np.uint32))


def test_embedding_full_size_properties(client):
    """Config 2 at full size (50,000 x 768 table, 8,192 Zipf indices)."""
    from jax_mps_amd import runner
    from jax_mps_amd.programs import configs
    p = configs.build_embedding()
    cp = runner.CompiledProgram(p, client)
    rows, dtable = cp.run_once()
    table, idx, g = p.inputs
    assert np.array_equal(rows.view(np.uint32), table[idx].view(np.uint32))
    seq = np.zeros_like(table)
    np.add.at(seq, idx, g)
    assert np.array_equal(dtable.view(np.uint32), seq.view(np.uint32))
    # untouched rows stay exactly zero; column sums agree with the upstream gradient's
    untouched = np.ones(table.shape[0], bool)
    untouched[idx] = False
    assert not dtable[untouched].any()
    np.testing.assert_allclose(dtable.sum(0, dtype=np.float64), g.sum(0, dtype=np.float64), rtol=1e-4, atol=1e-3)
    # determinism: a second run gives the same bits
    rows2, dtable2 = cp.run_once()
    assert np.array_equal(dtable.view(np.uint32), dtable2.view(np.uint32))


@pytest.mark.parametrize("size", ["SMALL", "MEDIUM"])
def test_resnet18_train_step(client, size):
    from jax_mps_amd.programs import configs
    p = configs.build_resnet18(**getattr(configs, size)["resnet18"])
    got, want = _run_both(client, p)
    assert closeness(got[-1], want[-1]) <= 1.0
    worst, where = _worst(p, got, want)
    print(f"resnet18 {size}: worst closeness {worst:.3f} at {where}", flush=True)
    assert worst <= 1.0, (where, worst)


def test_resnet18_forward_only(client):
    from jax_mps_amd.programs import configs
    p = configs.build_resnet18(batch=8, image=16, width=16, train=False, zero_bn2_scale=False)
    got, want = _run_both(client, p)
    worst, where = _worst(p, got, want)
    assert worst <= 1.0, (where, worst)


@pytest.mark.parametrize("size", ["SMALL", "MEDIUM"])
@pytest.mark.parametrize("dtype,tol", [("f32", 1e-5), ("bf16", 2e-2)])
def test_distilbert_forward(client, size, dtype, tol):
    from jax_mps_amd.programs import configs
    p = configs.build_distilbert(dtype=dtype, **getattr(configs, size)["distilbert"])
    got, want = _run_both(client, p)
    if dtype == "bf16":
        # The plugin keeps fused bf16 chains in float32 and rounds where a tensor is stored; the oracle rounds after
        # every op.  Both are held to the 2e-2 rule against the unrounded evaluation of the same formulas; against
        # each other a single element may land a few percent outside it (the roundings fall at different places).
        ins = [round_bf16(a) if d == "bf16" else a for a, d in zip(p.inputs, p.input_dtypes)]
        exact = Oracle(p.text, round_intermediates=False).run(*ins)
        assert _worst(p, got, exact, tol)[0] <= 1.0 and _worst(p, want, exact, tol)[0] <= 1.0
        assert _worst(p, got, want, tol)[0] <= 1.25
        return
    worst, where = _worst(p, got, want, tol)
    assert worst <= 1.0, (where, worst)


@pytest.mark.parametrize("size", ["SMALL", "MEDIUM"])
def test_lstm_scan_adam(client, size):
    from jax_mps_amd.programs import configs
    p = configs.build_lstm(**getattr(configs, size)["lstm"])
    got, want = _run_both(client, p)
    worst, where = _worst(p, got, want)
    print(f"lstm {size}: worst closeness {worst:.3f} at {where}", flush=True)
    assert worst <= 1.0, (where, worst)


def test_lstm_ten_steps(client):
    from jax_mps_amd import runner
    from jax_mps_amd.programs import configs
    p = configs.build_lstm(**configs.SMALL["lstm"])
    cp = runner.CompiledProgram(p, client)
    oracle = Oracle(p.text)
    state = list(p.inputs)
    for _ in range(10):
        outs = cp.step()
        ref = oracle.run(*state)
        for k, i in p.feedback.items():
            state[i] = ref[k]
    assert int(runner.download(cp.state[15])) == 10
    assert closeness(runner.download(outs[-1]), ref[-1]) <= 1.0


def test_dynamic_loop_reads_its_flag_once_per_chunk(client):
    """A loop of 178 data-dependent iterations (Collatz from 871): the host reads the loop's device flag after chunks
    of 4, 4, 8, 16, 32, 64, 64 queued iterations, seven round trips in all, not one per iteration (the reference
    evaluates the condition on the host every iteration: ops/control_flow.cc:504-536).  The next call starts with a
    chunk as long as the loop ran before, so a loop that repeats its trip count costs one round trip."""
    import op_cases
    from jax_mps_amd import runner
    c = op_cases.get_case("while-dynamic-collatz-871")
    exe = client.compile_and_load(c.text)
    bufs = runner.upload(client, c.inputs, c.dtypes)
    outs = exe.execute(bufs)
    assert [int(runner.download(o)) for o in outs] == [1, 178]
    assert exe.cost_analysis()["loop.host_syncs"] == 7
    for _ in range(3):       # replayed from one captured graph of 179 iterations
        outs = exe.execute(bufs)
        assert [int(runner.download(o)) for o in outs] == [1, 178]
    assert exe.cost_analysis()["loop.host_syncs"] == 10
    outs = exe.execute(runner.upload(client, [np.int32(1)], c.dtypes))      # zero iterations: everything queued runs past the end
    assert [int(runner.download(o)) for o in outs] == [1, 0]
    outs = exe.execute(runner.upload(client, [np.int32(27)], c.dtypes))
    assert [int(runner.download(o)) for o in outs] == [1, 111]


def test_error_paths(client):
    """Failures surface as PJRT errors with a code, never as crashes (reference: tests/test_ops.py:284-302)."""
    from jax_mps_amd import pjrt
    with pytest.raises(pjrt.PjrtError) as e:
        client.compile_and_load("module { func.func public @main(%a: tensor<4xf32>) -> tensor<4xf32> { %0 = stablehlo.fft %a : tensor<4xf32>\n return %0 : tensor<4xf32> } }")
    assert "unsupported" in str(e.value).lower() or "parse" in str(e.value).lower()
    with pytest.raises(pjrt.PjrtError):
        client.buffer_from_pyval(np.zeros(4, np.float64))
    exe = client.compile_and_load("module { func.func public @main(%a: tensor<4xf32>) -> tensor<4xf32> { %0 = stablehlo.add %a, %a : tensor<4xf32>\n return %0 : tensor<4xf32> } }")
    with pytest.raises(pjrt.PjrtError) as e:
        exe.execute([client.buffer_from_pyval(np.zeros(5, np.float32))])
    assert "type" in str(e.value)
    out = exe.execute([client.buffer_from_pyval(np.arange(4, dtype=np.float32))])[0]
    assert np.array_equal(out.to_numpy(), 2 * np.arange(4, dtype=np.float32))
    stats = client.memory_stats()
    assert stats["bytes_in_use"] > 0 and stats["bytes_limit"] > 2**36


def test_serialize_round_trip(client):
    """PJRT_Executable_Serialize -> PJRT_Executable_DeserializeAndLoad gives an executable with the same results
    (the reference leaves both unimplemented: pjrt_executable.cc:101-107, 269-271)."""
    from jax_mps_amd import pjrt, runner
    from jax_mps_amd.programs import configs
    p = configs.build_mlp(**configs.SMALL["mlp"])
    cp = runner.CompiledProgram(p, client)
    want = cp.run_once()
    blob = cp.exe.serialize()
    assert blob.startswith(b"MI355X-PJRT-EXE") and p.text.encode() in blob
    exe2 = client.deserialize_and_load(blob)
    got = [runner.download(o) for o in exe2.execute(cp.state)]
    assert len(got) == len(want)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)
    with pytest.raises(pjrt.PjrtError) as e:
        client.deserialize_and_load(b"not an executable")
    assert e.value.code == 3   # INVALID_ARGUMENT
    with pytest.raises(pjrt.PjrtError):
        client.deserialize_and_load(blob[:-5])


def test_strided_host_buffer(client):
    x = np.arange(24, dtype=np.float32).reshape(4, 6).T   # non-contiguous host view
    buf = client.buffer_from_pyval(x)
    assert np.array_equal(buf.to_numpy(), x)
    assert buf.shape() == (6, 4)
