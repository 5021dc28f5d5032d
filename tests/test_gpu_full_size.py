"""The five benchmark programs at their full benchmark sizes, through the PJRT C API, against the CPU oracle
(float64 accumulation) on the same seeded inputs.

Bar: integer outputs bit-exact; float32 outputs elementwise |got - want| <= 1e-5 + 1e-5 |want| (the reference's own
rule, tests/test_ops.py:91-105); bfloat16 outputs |got - want| <= 2e-2 + 2e-2 |want|.  Where a program's
arithmetic cannot meet the float32 rule for a stated reason, the bound used is written next to the assertion."""
import time

import numpy as np
import pytest

from conftest import closeness
from shlo_oracle import Oracle, round_bf16

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(900)]


def _oracle_inputs(p):
    return [round_bf16(a) if d == "bf16" else a for a, d in zip(p.inputs, p.input_dtypes)]


def _compare(p, got, want, rtol, atol, bounds=None):
    """Worst closeness ratio per output; `bounds` maps an output-name prefix to its own (rtol, atol)."""
    worst, where = 0.0, None
    for n, g, w in zip(p.output_names, got, want):
        if np.asarray(w).dtype.kind in "iub":
            assert np.array_equal(g, w), n
            continue
        r, a = rtol, atol
        for prefix, (br, ba) in (bounds or {}).items():
            if n.startswith(prefix):
                r, a = br, ba
        c = closeness(g, w, r, a)
        if c > worst:
            worst, where = c, n
    return worst, where


def test_mlp_full_size_100_steps(client):
    """Config 1 as stated: batch 256, 784 -> 512 -> 10, lr 0.01, 100 SGD steps; loss at every step and the final
    parameters against the oracle run on its own trajectory."""
    from jax_mps_amd import runner
    from jax_mps_amd.programs import configs
    p = configs.build_mlp()
    cp = runner.CompiledProgram(p, client)
    oracle = Oracle(p.text)
    state = list(p.inputs)
    worst_loss = 0.0
    for step in range(100):
        outs = cp.step()
        ref = oracle.run(*state)
        for k, i in p.feedback.items():
            state[i] = ref[k]
        worst_loss = max(worst_loss, closeness(runner.download(outs[-1]), ref[-1]))
    print(f"mlp full size: worst loss closeness over 100 steps {worst_loss:.3f}", flush=True)
    assert worst_loss <= 1.0
    for k, i in p.feedback.items():
        c = closeness(runner.download(cp.state[i]), state[i])
        assert c <= 1.0, (p.output_names[k], c)


def test_resnet18_full_size_train_step(client):
    """Config 3 as stated: batch 128, 32x32x3, one SGD-momentum step: loss, every updated parameter, momentum and
    batch statistic."""
    from jax_mps_amd import runner
    from jax_mps_amd.programs import configs
    p = configs.build_resnet18()
    cp = runner.CompiledProgram(p, client)
    got = cp.run_once()
    print("resnet18 b128: plugin done, running the oracle", flush=True)
    t0 = time.time()
    want = Oracle(p.text).run(*p.inputs)
    print(f"resnet18 b128: oracle took {time.time() - t0:.0f} s", flush=True)
    assert closeness(got[-1], want[-1]) <= 1.0, (float(got[-1]), float(want[-1]))
    worst, where = _compare(p, got, want, 1e-5, 1e-5)
    print(f"resnet18 b128: worst closeness {worst:.3f} at {where}", flush=True)
    assert worst <= 1.0, (where, worst)


def test_distilbert_full_size_one_layer(client):
    """One encoder layer of config 4 at its full dimensions (embedding gather, LayerNorm, 4096 x 768 projections,
    12 heads of 128 x 128 attention, 3072-wide GELU feed-forward): every kernel the benchmarked pass launches, at the
    tile and launch shapes it launches them with.

    Elementwise within 2e-2 + 2e-2 |want| of the unrounded evaluation of the program's formulas (float64 arithmetic on
    the bf16 inputs).  Against the oracle that rounds to bf16 after every op the same rule holds for all but a few
    of the 3.1 M elements (a dozen roundings separate the two orders of evaluation even in one layer; the worst
    element is 1.02 x the rule away, while that oracle is itself further from the unrounded evaluation than the
    plugin is), so the bound there is 1.25 x the rule with at most 1e-5 of the elements beyond 1 x."""
    from jax_mps_amd import runner
    from jax_mps_amd.programs import configs
    p = configs.build_distilbert(layers=1)
    cp = runner.CompiledProgram(p, client)
    got = cp.run_once()
    ins = _oracle_inputs(p)
    exact = Oracle(p.text, round_intermediates=False).run(*ins)
    want = Oracle(p.text).run(*ins)
    c_exact = closeness(got[0], exact[0], 2e-2, 2e-2)
    c_want = closeness(got[0], want[0], 2e-2, 2e-2)
    c_oracle = closeness(want[0], exact[0], 2e-2, 2e-2)
    r = np.abs(got[0].astype(np.float64) - want[0]) / (2e-2 + 2e-2 * np.abs(want[0].astype(np.float64)))
    print(f"distilbert one full-size layer: vs unrounded {c_exact:.3f}, vs per-op-rounded oracle {c_want:.3f} "
          f"(beyond the rule: {(r > 1).mean():.2e}), oracle vs unrounded {c_oracle:.3f}", flush=True)
    assert c_exact <= 1.0, c_exact
    assert c_want <= 1.25 and (r > 1).mean() <= 1e-5, (c_want, (r > 1).mean())


def test_distilbert_full_size_forward(client):
    """Config 4 as stated: 6 layers, d_model 768, 12 heads, FFN 3072, vocabulary 30522, batch 32 x seq 128, bf16.

    Through six layers the elementwise 2e-2 rule cannot hold between two correct bf16 evaluations: every stored
    bf16 tensor carries a rounding error of up to 2^-9 relative, the residual stream carries it from layer to layer,
    and the oracle (which rounds after every op, as the program's types say) and the plugin (which keeps fused chains
    in float32 and rounds where a tensor is stored) round at different places.  Measured on these inputs: the
    per-op-rounded oracle itself lies up to 1.84 x the rule away from the unrounded evaluation of the same formulas,
    the plugin 1.34 x, and the two differ by 2.6 x at the worst of 3.1 M elements (mean difference 0.008 at values up
    to 5.7).  Asserted here: (a) 99 % of the elements meet the 2e-2 rule and none is beyond 3 x it; (b) the north
    star's aggregate form max |diff| / max |want| <= 2.5e-2; (c) the plugin is at least as close to the unrounded
    evaluation as the oracle is, in the mean and at the 99.99th percentile.  The one-layer test above holds the
    kernels themselves to the elementwise rule."""
    from jax_mps_amd import runner
    from jax_mps_amd.programs import configs
    p = configs.build_distilbert()
    cp = runner.CompiledProgram(p, client)
    got = cp.run_once()[0].astype(np.float64)
    ins = _oracle_inputs(p)
    t0 = time.time()
    want = Oracle(p.text).run(*ins)[0].astype(np.float64)
    exact = Oracle(p.text, round_intermediates=False).run(*ins)[0].astype(np.float64)
    print(f"distilbert full size: both oracle runs took {time.time() - t0:.0f} s", flush=True)

    def ratio(a, b):
        return np.abs(a - b) / (2e-2 + 2e-2 * np.abs(b))
    r = ratio(got, want)
    print(f"distilbert full size: vs oracle max {r.max():.3f}, beyond the rule {(r > 1).mean():.2e}; "
          f"max|diff|/max|want| {np.abs(got - want).max() / np.abs(want).max():.4f}", flush=True)
    assert r.max() <= 3.0 and (r > 1).mean() <= 1e-2, (r.max(), (r > 1).mean())
    assert np.abs(got - want).max() <= 2.5e-2 * np.abs(want).max()
    rg, ro = ratio(got, exact), ratio(want, exact)
    print(f"distilbert full size: vs unrounded evaluation: plugin mean {rg.mean():.4f} p99.99 {np.quantile(rg, 0.9999):.3f}; "
          f"oracle mean {ro.mean():.4f} p99.99 {np.quantile(ro, 0.9999):.3f}", flush=True)
    assert rg.mean() <= ro.mean() and np.quantile(rg, 0.9999) <= np.quantile(ro, 0.9999)


@pytest.mark.parametrize("steps", [1, 10])
def test_lstm_full_size_adam(client, steps):
    """Config 5 as stated: seq 100, batch 64, input 128, hidden 256, Adam; loss and every parameter and moment
    after 1 and after 10 steps (the oracle follows its own trajectory)."""
    from jax_mps_amd import runner
    from jax_mps_amd.programs import configs
    p = configs.build_lstm()
    cp = runner.CompiledProgram(p, client)
    oracle = Oracle(p.text)
    state = list(p.inputs)
    for _ in range(steps):
        outs = cp.step()
        ref = oracle.run(*state)
        for k, i in p.feedback.items():
            state[i] = ref[k]
    got = [runner.download(o) for o in outs]
    worst, where = _compare(p, got, ref, 1e-5, 1e-5)
    print(f"lstm full size, {steps} step(s): worst closeness {worst:.3f} at {where}", flush=True)
    assert worst <= 1.0, (where, worst)
