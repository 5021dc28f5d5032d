"""Whole-plan graph replay (opt-in: MI355X_PLAN_GRAPHS=1 when the program is compiled): a loop-free plan whose buffer
addresses repeat from call to call is captured once per address set and then costs one graph launch per execute.
Every replay is checked against the launch-by-launch result of the same program, with eager work and
synchronisations between the replays (other programs run, results are read back), because a graph that holds a
node it should not hold shows on later replays, not on the first."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _compile(client, text, graphs):
    if graphs:
        os.environ["MI355X_PLAN_GRAPHS"] = "1"
    try:
        return client.compile_and_load(text)
    finally:
        os.environ.pop("MI355X_PLAN_GRAPHS", None)


def test_train_state_threaded_through_graph_replays(client):
    """MLP train steps with donated state: the addresses alternate between two sets, so the third call captures and
    later calls replay; losses and final parameters are bit-identical to the launch-by-launch run."""
    from jax_mps_amd import runner
    from jax_mps_amd.programs import configs
    p = configs.build_mlp(**configs.MEDIUM["mlp"])

    def run(graphs, steps=12):
        exe = _compile(client, p.text, graphs)
        state = runner.upload(client, p.inputs, p.input_dtypes)
        losses = []
        for _ in range(steps):
            outs = exe.execute(state, donate=True)
            for k, i in p.feedback.items():
                state[i] = outs[k]
            losses.append(runner.download(outs[-1]))        # a read-back (synchronisation) between replays
        return losses, [runner.download(state[i]) for i in p.feedback.values()], exe.cost_analysis()
    eager_losses, eager_params, ca0 = run(False)
    graph_losses, graph_params, ca1 = run(True)
    assert ca0.get("plan.graph_launches", 0) == 0
    assert ca1["plan.graph_launches"] >= 6, ca1
    for a, b in zip(eager_losses, graph_losses):
        assert np.array_equal(a, b)
    for a, b in zip(eager_params, graph_params):
        assert np.array_equal(a, b)


def test_forked_convolutions_inside_a_graph(client):
    """The program of the second-stream test (a filter gradient forked onto the second stream, joined by its late
    reader) replayed from a graph: the fork and the join become edges of the graph."""
    import test_gpu_second_stream as t
    from conftest import closeness
    from jax_mps_amd import runner
    from shlo_oracle import Oracle
    text = t._program()
    rng = np.random.default_rng(5)
    ins = [rng.uniform(0.05, 1.0, s).astype(np.float32) / 8 for s in ((16, 24, 24, 32), (16, 24, 24, 64), (16, 24, 24, 64))]
    want = Oracle(text).run(*ins)
    exe = _compile(client, text, True)
    other = client.compile_and_load(text)                      # eager work between the replays
    bufs = runner.upload(client, ins, ["f32"] * 3)
    keep = None
    for call in range(8):
        outs = exe.execute(bufs)
        got = [runner.download(o) for o in outs]
        keep = outs if call % 2 else None                       # holding results now and then changes which blocks the next call gets
        for k, (g, w) in enumerate(zip(got, want)):
            assert closeness(g, w, 1e-5, 1e-5) <= 1.0, (call, k)
        other.execute(bufs)
    assert exe.cost_analysis()["plan.graph_launches"] >= 1
    del keep
