"""The five benchmark programs at their full benchmark sizes, through the PJRT C API, against the CPU oracle
(float64 accumulation) on the same seeded inputs.

Bar: integer outputs bit-exact; float32 outputs elementwise |got - want| <= 1e-5 + 1e-5 |want| (the reference's own
rule, tests/test_ops.py:91-105); bfloat16 outputs |got - want| <= 2e-2 + 2e-2 |want|.  Where a program's
arithmetic cannot meet the float32 rule for a stated reason, the bound used is written next to the assertion."""
import os
import time
from contextlib import contextmanager

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


def _no_gradient_is_zero(p, want):
    """Every float momentum output (momentum starts at zero, so after a step it is the gradient) must hold data: an
    all-zero expectation would accept whatever the backward kernels wrote into it only by accident of being zero too."""
    dead = [n for n, w in zip(p.output_names, want) if n.startswith("mom.") and not np.any(np.asarray(w))]
    assert not dead, f"{len(dead)} gradient outputs of the oracle are all zero: {dead[:4]}"
    thin = [n for n, w in zip(p.output_names, want) if n.startswith("mom.") and (np.asarray(w) != 0).mean() < 0.5]
    assert not thin, thin


def test_resnet18_full_size_two_train_steps(client):
    """Config 3 as stated: batch 128, 32x32x3, SGD with momentum: loss, every updated parameter, momentum and batch
    statistic (165 outputs) under |got - want| <= 1e-5 + 1e-5 |want|, for two chained steps.

    The reference model starts the second batch norm of every block at scale 0 (examples/resnet/model.py:39-40), which
    makes the gradient entering every residual branch exactly zero on the first step: the filter and data gradients of
    the sixteen 3x3 block convolutions are compared 0 against 0 there.  The second step starts from the state the
    plugin itself produced (those scales are no longer 0), the oracle evaluates that same state, and no gradient it
    expects may be all zero."""
    from jax_mps_amd import runner
    from jax_mps_amd.programs import configs
    p = configs.build_resnet18()
    cp = runner.CompiledProgram(p, client)
    oracle = Oracle(p.text)
    state = list(p.inputs)
    for step in (1, 2):
        got = [runner.download(o) for o in cp.step()]
        print(f"resnet18 b128 step {step}: plugin done, running the oracle", flush=True)
        t0 = time.time()
        want = oracle.run(*state)
        print(f"resnet18 b128 step {step}: oracle took {time.time() - t0:.0f} s", flush=True)
        assert closeness(got[-1], want[-1]) <= 1.0, (float(got[-1]), float(want[-1]))
        worst, where = _compare(p, got, want, 1e-5, 1e-5)
        zero = sum(1 for n, w in zip(p.output_names, want) if n.startswith("mom.") and not np.any(np.asarray(w)))
        print(f"resnet18 b128 step {step}: worst closeness {worst:.3f} at {where}; {zero} all-zero gradients expected",
              flush=True)
        assert worst <= 1.0, (where, worst)
        for k, i in p.feedback.items():          # the next step starts from what the plugin produced
            state[i] = got[k]
    _no_gradient_is_zero(p, want)


def build_resnet18_with_relu_decisions(**kw):
    """The ResNet18 train step with two extra outputs per ReLU: the activation and the mask its gradient uses
    (`compare GT` of the `maximum`'s VJP).  Returns (program, number of ReLUs); the extra outputs follow the loss,
    activations first."""
    from jax_mps_amd.programs import configs
    from jax_mps_amd.shlo.builder import Builder
    acts, masks = [], []
    relu0, compare0, ret0 = configs.relu, Builder.compare, Builder.ret

    def relu(b, x):
        y = relu0(b, x)
        acts.append(y)
        return y

    def compare(self, a, b, direction, kind=None):
        m = compare0(self, a, b, direction, kind)
        if direction == "GT" and len(m.shape) == 4:
            masks.append(m)
        return m

    def ret(self, *vals):
        assert len(masks) == len(acts)
        return ret0(self, *vals, *acts, *reversed(masks))      # the backward pass meets the ReLUs last to first
    configs.relu, Builder.compare, Builder.ret = relu, compare, ret
    try:
        p = configs.build_resnet18(**kw)
    finally:
        configs.relu, Builder.compare, Builder.ret = relu0, compare0, ret0
    return p, len(acts)


def test_resnet18_full_size_train_step_every_scale_one(client):
    """Config 3 at batch 128 with every batch-norm scale starting at 1, so that on the very first step every
    convolution's filter and data gradient is dense non-zero data.

    Started like this the network is ill-conditioned for an elementwise comparison of gradients between any two
    float32 evaluations: of its 71.3 M ReLU inputs a few lie within rounding noise of zero (measured: 22 elements,
    all below 5.2e-6 where activations reach 11), the two sides take different branches there, and one such element
    is about 1 / sqrt(elements of the layer) of that layer's whole gradient signal, which then spreads backwards
    (measured: 0.3 % relative difference in every filter gradient, up to 42 x the bound).  So the test pins the
    decisions: the program also returns every ReLU's activation and gradient mask; each activation tensor must agree
    to max |diff| <= 1e-5 max |want| (these are hidden values seventeen normalised layers deep, not outputs of the
    step; their noise is relative to the layer's scale, not to each element), decisions may differ only at elements
    whose activation is below that same bound on both sides, the oracle then evaluates the backward pass with the
    masks the plugin used, and all 165 outputs of the step must meet |got - want| <= 1e-5 + 1e-5 |want| with no
    gradient all zero."""
    from conftest import rel_err
    from jax_mps_amd import runner
    p, n_relu = build_resnet18_with_relu_decisions(zero_bn2_scale=False)
    exe = client.compile_and_load(p.text)
    got = [runner.download(o) for o in exe.execute(runner.upload(client, p.inputs, p.input_dtypes))]
    n_out = len(p.output_names)
    first_mask = n_out + n_relu
    print("resnet18 b128, scales one: plugin done, running the oracle", flush=True)
    oracle = Oracle(p.text)
    want = oracle.run(*p.inputs, pinned={first_mask + k: got[first_mask + k] for k in range(n_relu)})
    flips, worst_act = 0, 0.0
    for k in range(n_relu):
        worst_act = max(worst_act, rel_err(got[n_out + k], want[n_out + k]) / 1e-5)
        differ = oracle.replaced[first_mask + k].astype(bool) != got[first_mask + k].astype(bool)
        flips += int(differ.sum())
        if differ.any():
            # where the two sides decide differently, one activation is 0 and the other within the bound of 0
            bound = 1e-5 * np.abs(want[n_out + k]).max()
            assert max(np.abs(got[n_out + k][differ]).max(), np.abs(want[n_out + k][differ]).max()) <= bound
    total = sum(got[n_out + k].size for k in range(n_relu))
    print(f"resnet18 b128, scales one: activations at {worst_act:.3f} of 1e-5 max |want|; {flips} of {total} ReLU "
          f"decisions differ", flush=True)
    assert worst_act <= 1.0 and flips <= total * 1e-5
    assert closeness(got[n_out - 1], want[n_out - 1]) <= 1.0
    worst, where = _compare(p, got[:n_out], want[:n_out], 1e-5, 1e-5)
    print(f"resnet18 b128, scales one: worst closeness {worst:.3f} at {where}", flush=True)
    assert worst <= 1.0, (where, worst)
    _no_gradient_is_zero(p, want[:n_out])


@contextmanager
def strict_bf16():
    """Programs compiled inside this block round every bf16 op as the program's types say (the switch is read at
    every PJRT_Client_Compile; programs compiled outside keep their fused float32 chains)."""
    os.environ["MI355X_STRICT_BF16"] = "1"
    try:
        yield
    finally:
        del os.environ["MI355X_STRICT_BF16"]


def _rule_bf16(a, b):
    return np.abs(a.astype(np.float64) - b) / (2e-2 + 2e-2 * np.abs(b.astype(np.float64)))


@pytest.mark.parametrize("layers", [1, 2, 6])
def test_distilbert_full_size_strict_rounding(client, layers):
    """Config 4 at its full dimensions with the rounding points of the program itself: every bf16-typed op rounds its
    result (MI355X_STRICT_BF16=1; the GELU-in-epilogue and one-launch attention fusions, which move a rounding point,
    are off with it).  Against the oracle that rounds after every op the elementwise rule
    |got - want| <= 2e-2 + 2e-2 |want| must hold outright for one and for two layers (measured at three: one element
    of 3.1 M at 1.18 x the rule, mean 0.056).

    Through six layers it cannot hold between two correct evaluations that round at the same places but accumulate
    their sums differently: a sum that lands near a bf16 rounding boundary rounds the other way (4 % of the elements
    differ by one bf16 step after one layer), the next layer's roundings decorrelate from there, and the two results
    drift towards two independent draws of the rounding noise.  That is measured here, not argued: the oracle itself
    is run a second time with float32 instead of float64 accumulation and nothing else changed.  CPU figures at six
    layers for that pair: worst element 1.72 x the rule, mean 0.129, 6.6e-5 of the elements beyond it; the plugin
    against the float64 oracle: 1.69 x, 0.130, 6.9e-5.  Asserted for six layers: the pair of oracles does exceed the
    rule (so the rule is unattainable there), and the plugin is no further from the float64 oracle than 1.1 x what
    the float32-accumulating oracle is, at the worst element, in the mean and in the fraction beyond the rule."""
    from jax_mps_amd import runner
    from jax_mps_amd.programs import configs
    p = configs.build_distilbert(layers=layers)
    with strict_bf16():
        cp = runner.CompiledProgram(p, client)
    got = cp.run_once()[0]
    ins = _oracle_inputs(p)
    want = Oracle(p.text).run(*ins)[0]
    r = _rule_bf16(got, want)
    print(f"distilbert {layers} full-size layer(s), strict rounding: worst element at {r.max():.3f} of the rule, "
          f"mean {r.mean():.4f}, beyond it {(r > 1).mean():.2e}", flush=True)
    if layers < 6:
        assert r.max() <= 1.0, r.max()
        return
    pair = _rule_bf16(Oracle(p.text, accum="f32").run(*ins)[0], want)
    print(f"distilbert {layers} full-size layers: float32- against float64-accumulating oracle: worst element at "
          f"{pair.max():.3f} of the rule, mean {pair.mean():.4f}, beyond it {(pair > 1).mean():.2e}", flush=True)
    assert pair.max() > 1.0, "the rule holds between the two oracles: hold the plugin to it as well"
    assert r.max() <= 1.1 * pair.max() and r.mean() <= 1.1 * pair.mean() and (r > 1).mean() <= 1.1 * (pair > 1).mean()


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
