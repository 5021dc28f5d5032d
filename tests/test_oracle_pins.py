"""Pins of the CPU oracle that the golden vectors leave open: library routines (torch CPU conv2d /
conv_transpose2d, numpy einsum), brute force on tiny inputs, IEEE identities, and torch autograd for
the five benchmark programs (which also pins the StableHLO emitter's VJP rules)."""
import importlib
import math

import numpy as np
import pytest


class _Lazy:
    """Module imported at first use.  torch ships its own HIP runtime; importing it while pytest collects would put
    that runtime into the process before the plugin library loads, also in runs that select no test of this file."""

    def __init__(self, name):
        self._name, self._module = name, None

    def __getattr__(self, attr):
        if self._module is None:
            self._module = importlib.import_module(self._name)
        return getattr(self._module, attr)


torch = _Lazy("torch")
F = _Lazy("torch.nn.functional")

import op_cases
from jax_mps_amd.programs import configs
from jax_mps_amd.shlo.builder import Builder
from shlo_oracle import Oracle, round_bf16, f32_to_bf16_bits, bf16_bits_to_f32


def run(fn, *inputs, dtypes=None):
    b = Builder("pin")
    dts = dtypes or ["f32" if np.asarray(a).dtype.kind == "f" else "i32" for a in inputs]
    args = [b.arg(np.asarray(a).shape, d) for a, d in zip(inputs, dts)]
    out = fn(b, *args)
    out = out if isinstance(out, (list, tuple)) else [out]
    b.ret(*out)
    return Oracle(b.text()).run(*inputs)


def rnd(seed, *shape):
    return np.random.default_rng(seed).uniform(-1, 1, size=shape).astype(np.float32)


# ------------------------------------------------------------------ convolution
@pytest.mark.parametrize("stride,pad,rdil", [(1, 1, 1), (2, 1, 1), (2, 0, 1), (1, 2, 2), (2, 3, 2)])
def test_conv_forward_vs_torch(stride, pad, rdil):
    x, w = rnd(1, 2, 9, 10, 3), rnd(2, 3, 3, 3, 5)
    got = run(lambda b, a, k: b.conv(a, k, strides=(stride, stride), padding=((pad, pad), (pad, pad)), rhs_dilation=(rdil, rdil)), x, w)[0]
    want = F.conv2d(torch.tensor(x).double().permute(0, 3, 1, 2), torch.tensor(w).double().permute(3, 2, 0, 1), stride=stride, padding=pad, dilation=rdil)
    np.testing.assert_allclose(got, want.permute(0, 2, 3, 1).numpy(), rtol=1e-6, atol=1e-6)


def test_conv_asymmetric_and_negative_padding_vs_torch():
    x, w = rnd(3, 1, 8, 8, 2), rnd(4, 3, 3, 2, 4)
    got = run(lambda b, a, k: b.conv(a, k, padding=((2, -1), (0, 1))), x, w)[0]
    xt = torch.tensor(x).double().permute(0, 3, 1, 2)
    xt = F.pad(xt, (0, 1, 2, 0))[:, :, :-1, :]          # pad W by (0,1), H by (2,0), then crop one row at the bottom
    want = F.conv2d(xt, torch.tensor(w).double().permute(3, 2, 0, 1))
    np.testing.assert_allclose(got, want.permute(0, 2, 3, 1).numpy(), rtol=1e-6, atol=1e-6)


def test_conv_lhs_dilation_is_transposed_conv():
    # lhs dilation by s with padding k-1 and a flipped kernel == conv_transpose2d with stride s
    x, w = rnd(5, 2, 5, 5, 3), rnd(6, 3, 3, 3, 4)
    got = run(lambda b, a, k: b.conv(a, b.reverse(k, [0, 1]), padding=((2, 2), (2, 2)), lhs_dilation=(2, 2)), x, w)[0]
    want = F.conv_transpose2d(torch.tensor(x).double().permute(0, 3, 1, 2), torch.tensor(w).double().permute(2, 3, 0, 1), stride=2)
    np.testing.assert_allclose(got, want.permute(0, 2, 3, 1).numpy(), rtol=1e-6, atol=1e-6)


def test_conv_groups_vs_torch():
    x, w = rnd(7, 2, 7, 7, 8), rnd(8, 3, 3, 4, 6)
    got = run(lambda b, a, k: b.conv(a, k, padding=((1, 1), (1, 1)), feature_group_count=2), x, w)[0]
    want = F.conv2d(torch.tensor(x).double().permute(0, 3, 1, 2), torch.tensor(w).double().permute(3, 2, 0, 1), padding=1, groups=2)
    np.testing.assert_allclose(got, want.permute(0, 2, 3, 1).numpy(), rtol=1e-6, atol=1e-6)


def test_conv_brute_force_general_dimension_numbers():
    # NCHW input, OIHW kernel, stride (2,1), rhs dilation (1,2), padding ((1,0),(2,1)): seven nested loops
    x, w = rnd(9, 2, 3, 6, 7), rnd(10, 4, 3, 2, 3)
    got = run(lambda b, a, k: b.conv(a, k, strides=(2, 1), padding=((1, 0), (2, 1)), rhs_dilation=(1, 2), dn=("bf01", "oi01", "bf01")), x, w)[0]
    N, C, H, W = x.shape
    O, _, KH, KW = w.shape
    OH = (H + 1 + 0 - ((KH - 1) * 1 + 1)) // 2 + 1
    OW = (W + 2 + 1 - ((KW - 1) * 2 + 1)) // 1 + 1
    want = np.zeros((N, O, OH, OW))
    for n in range(N):
        for o in range(O):
            for oh in range(OH):
                for ow in range(OW):
                    for c in range(C):
                        for kh in range(KH):
                            for kw in range(KW):
                                ih, iw = oh * 2 - 1 + kh, ow - 2 + kw * 2
                                if 0 <= ih < H and 0 <= iw < W:
                                    want[n, o, oh, ow] += float(x[n, c, ih, iw]) * float(w[o, c, kh, kw])
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)


def test_conv_batch_group_count_brute_force():
    x, w = rnd(11, 6, 5, 5, 2), rnd(12, 3, 3, 2, 6)
    got = run(lambda b, a, k: b.conv(a, k, padding=((1, 1), (1, 1)), batch_group_count=3), x, w)[0]
    # group g uses batch rows [2g, 2g+2) and output features [2g, 2g+2)
    want = np.zeros((2, 5, 5, 6))
    for g in range(3):
        xs = torch.tensor(x[2 * g:2 * g + 2]).double().permute(0, 3, 1, 2)
        ws = torch.tensor(w[..., 2 * g:2 * g + 2]).double().permute(3, 2, 0, 1)
        want[..., 2 * g:2 * g + 2] = F.conv2d(xs, ws, padding=1).permute(0, 2, 3, 1).numpy()
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)


# ------------------------------------------------------------------ dot_general
@pytest.mark.parametrize("spec,contract,batch,sa,sb", [
    ("ik,kj->ij", ([1], [0]), ((), ()), (5, 7), (7, 3)),
    ("ki,kj->ij", ([0], [0]), ((), ()), (7, 5), (7, 3)),
    ("ik,jk->ij", ([1], [1]), ((), ()), (5, 7), (3, 7)),
    ("bik,bkj->bij", ([2], [1]), ([0], [0]), (4, 5, 7), (4, 7, 3)),
    ("btnh,bsnh->bnts", ([3], [3]), ([0, 2], [0, 2]), (2, 5, 3, 4), (2, 6, 3, 4)),
    ("ijk,jkl->il", ([1, 2], [0, 1]), ((), ()), (3, 4, 5), (4, 5, 6)),
    ("k,k->", ([0], [0]), ((), ()), (9,), (9,)),
])
def test_dot_general_vs_einsum(spec, contract, batch, sa, sb):
    a, b_ = rnd(20, *sa), rnd(21, *sb)
    got = run(lambda b, x, y: b.dot_general(x, y, contract, batch), a, b_)[0]
    want = np.einsum(spec, a.astype(np.float64), b_.astype(np.float64))
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)


# ------------------------------------------------------------------ reductions / elementwise identities
def test_reduce_vs_numpy():
    x = rnd(30, 6, 7, 8)
    for dims in ([0], [1], [2], [0, 2], [0, 1, 2]):
        got = run(lambda b, a: b.reduce_sum(a, dims), x)[0]
        np.testing.assert_allclose(got, x.astype(np.float64).sum(tuple(dims)), rtol=1e-6, atol=1e-6)
    assert np.array_equal(run(lambda b, a: b.reduce_max(a, [1]), x)[0], x.max(1))
    assert np.array_equal(run(lambda b, a: b.reduce_min(a, [0, 2]), x)[0], x.min((0, 2)))


def test_argmax_first_occurrence():
    x = np.array([[1, 3, 3, 0], [2, 2, 2, 2], [0, -1, 5, 5]], np.float32)
    assert np.array_equal(run(lambda b, a: b.argmax(a, 1), x)[0], np.array([1, 0, 2], np.int32))


def test_bf16_rounding_is_nearest_even():
    # 1 + 2^-8 lies exactly between two bf16 values: ties go to the even mantissa
    x = np.array([1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8, 1 + 2.0 ** -7, 3.0e38, -1e-40], np.float32)
    r = round_bf16(x)
    assert r[0] == 1.0 and r[1] == np.float32(1 + 2.0 ** -6) and r[2] == x[2]
    assert np.array_equal(bf16_bits_to_f32(f32_to_bf16_bits(x)), r)
    assert np.isinf(round_bf16(np.array([3.4e38], np.float32))[0])


def test_convert_float_to_int_saturates():
    x = np.array([3e9, -3e9, np.nan, 1.9, -1.9], np.float32)
    assert np.array_equal(run(lambda b, a: b.convert(a, "i32"), x)[0], np.array([2**31 - 1, -2**31, 0, 1, -1], np.int32))


def test_integer_division_against_exact_integers():
    """Quotient truncated toward zero and remainder with the dividend's sign, both wrapped to the type (the most negative
    value divided by -1 is itself), a zero divisor giving all ones and the dividend: every pair of int8 and uint8 values
    and the corners of the 64-bit types against Python's unbounded integers (reference: arithmetic.cc:46-83, 496-513)."""
    def exact(x, y, bits, signed):
        if y == 0:
            return (-1 if signed else 2 ** bits - 1), x
        q = abs(x) // abs(y)
        q = -q if (x < 0) != (y < 0) else q
        r = x - q * y
        if signed:
            q = (q + 2 ** (bits - 1)) % 2 ** bits - 2 ** (bits - 1)
        return q, r
    for dt, name, signed in ((np.int8, "i8", True), (np.uint8, "ui8", False)):
        v = np.arange(np.iinfo(dt).min, np.iinfo(dt).max + 1).astype(dt)
        a, b_ = [m.ravel() for m in np.meshgrid(v, v, indexing="ij")]
        q = run(lambda b, x, y: b.div(x, y), a, b_, dtypes=[name, name])[0]
        r = run(lambda b, x, y: b.remainder(x, y), a, b_, dtypes=[name, name])[0]
        want = [exact(int(x), int(y), 8, signed) for x, y in zip(a, b_)]
        assert np.array_equal(q.astype(np.int64), np.array([w[0] for w in want])) and np.array_equal(r.astype(np.int64), np.array([w[1] for w in want]))
    lo, hi = np.iinfo(np.int64).min, np.iinfo(np.int64).max
    a = np.array([lo, lo, lo, lo, lo + 1, hi, hi, 7, -7, lo], np.int64)
    b_ = np.array([lo + 1, -1, 2 ** 62 - 1, lo, -1, -1, lo, -2, 2, 0], np.int64)
    q = run(lambda b, x, y: b.div(x, y), a, b_, dtypes=["i64", "i64"])[0]
    r = run(lambda b, x, y: b.remainder(x, y), a, b_, dtypes=["i64", "i64"])[0]
    want = [exact(int(x), int(y), 64, True) for x, y in zip(a, b_)]
    assert [int(t) for t in q] == [w[0] for w in want] and [int(t) for t in r] == [w[1] for w in want]
    a = np.array([2 ** 64 - 1, 2 ** 64 - 5, 12, 2 ** 63, 9], np.uint64)
    b_ = np.array([2 ** 64 - 1, 2 ** 64 - 1, 2 ** 64 - 1, 3, 0], np.uint64)
    q = run(lambda b, x, y: b.div(x, y), a, b_, dtypes=["ui64", "ui64"])[0]
    r = run(lambda b, x, y: b.remainder(x, y), a, b_, dtypes=["ui64", "ui64"])[0]
    want = [exact(int(x), int(y), 64, False) for x, y in zip(a, b_)]
    assert [int(t) for t in q] == [w[0] for w in want] and [int(t) for t in r] == [w[1] for w in want]


def test_round_half_away_is_the_reference_s_formula():
    """sign(x) * floor(|x| + 0.5) evaluated in float32 (arithmetic.cc:316-327): exact halves go away from zero, and where the
    sum is not a float32 it rounds before the floor (the predecessor of 0.5 gives 1, an odd integer above 2^23 its even
    neighbour), checked against the same formula in exact rational arithmetic with one rounding of the sum."""
    from fractions import Fraction
    xs = np.array([0.5, 1.5, 2.5, -0.5, -2.5, 0.49999997, -0.49999997, 8388609.0, -8404769.0, 16777215.0, 4194303.5, 0.25, -7.75, 1e-45], np.float32)
    got = run(lambda b, x: b._unary("round_nearest_afz", x), xs)[0]
    want = []
    for x in xs:
        s = float(np.float32(float(abs(Fraction(float(x))) + Fraction(1, 2))))   # the one rounding: the sum to float32
        want.append(math.copysign(math.floor(s), float(x)))
    assert np.array_equal(got, np.array(want, np.float32))
    assert got[5] == 1.0 and got[7] == 8388610.0


def test_total_order_compare():
    a = np.array([-0.0, 0.0], np.float32)
    b_ = np.array([0.0, -0.0], np.float32)
    assert np.array_equal(run(lambda b, x, y: b.compare(x, y, "LT", "TOTALORDER"), a, b_)[0], np.array([True, False]))
    assert np.array_equal(run(lambda b, x, y: b.compare(x, y, "LT"), a, b_)[0], np.array([False, False]))


def test_scatter_is_sequential_in_update_order():
    # float addition is not associative: only the in-order fold gives this exact value
    rng = np.random.default_rng(40)
    idx = rng.integers(0, 7, size=500).astype(np.int32)
    upd = (rng.standard_normal((500, 3)) * 10 ** rng.uniform(-3, 3, size=(500, 1))).astype(np.float32)
    op = rng.standard_normal((7, 3)).astype(np.float32)
    c = op_cases._row_scatter("add")
    got = run(c, op, idx, upd)[0]
    want = op.copy()
    for i, u in zip(idx, upd):
        want[i] = want[i] + u
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_bf16_scatter_rounds_after_every_application():
    # the body adds two bf16 scalars, so each application rounds: a float32 accumulation rounded once at the end differs
    c = op_cases.get_case("scatter-add-very-long-run-bf16")
    x, idx, upd = [round_bf16(a) if d == "bf16" else a for a, d in zip(c.inputs, c.dtypes)]
    got = Oracle(c.text).run(x, idx, upd)[0]
    want, once = x.copy(), x.copy()
    for i, u in zip(idx, upd):
        want[i] = round_bf16((want[i] + u).astype(np.float32))
        once[i] = once[i] + u
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert not np.array_equal(want, round_bf16(once))      # the case tells the two rules apart


# ------------------------------------------------------------------ the five programs vs torch autograd
def test_mlp_program_vs_torch():
    p = configs.build_mlp(**configs.SMALL["mlp"])
    out = Oracle(p.text).run(*p.inputs)
    w1, b1, w2, b2, x, y = [torch.tensor(a) for a in p.inputs]
    ps = [t.double().requires_grad_(True) for t in (w1, b1, w2, b2)]
    loss = F.cross_entropy(torch.relu(x.double() @ ps[0] + ps[1]) @ ps[2] + ps[3], y.long())
    loss.backward()
    assert abs(float(out[-1]) - loss.item()) < 1e-6
    for t, o in zip(ps, out):
        np.testing.assert_allclose(o, (t - 0.01 * t.grad).detach().numpy(), rtol=1e-5, atol=1e-6)


def _torch_resnet(p, width):
    """Loss and gradients of the program's network from torch autograd in float64 (oracle/torch_resnet.py)."""
    import torch_resnet
    specs = configs.resnet18_param_specs(width, 10)
    n = len(specs)
    P = {nm: torch.tensor(a, dtype=torch.float64, requires_grad=True) for (nm, _, _), a in zip(specs, p.inputs[:n])}
    x = torch.tensor(p.inputs[-2], dtype=torch.float64).permute(0, 3, 1, 2)
    y = torch.tensor(p.inputs[-1]).long()
    loss = torch_resnet.forward(P, x, y, width)
    loss.backward()
    return specs, P, loss


def test_resnet18_program_vs_torch():
    p = configs.build_resnet18(batch=4, image=8, width=8, zero_bn2_scale=False)
    out = Oracle(p.text).run(*p.inputs)
    specs, P, loss = _torch_resnet(p, 8)
    assert abs(float(out[-1]) - loss.item()) < 2e-5
    n = len(specs)
    nstat = len(p.inputs) - 2 - 2 * n
    for i, (nm, _, _) in enumerate(specs):
        g = P[nm].grad.numpy()
        mom = out[n + nstat + i]          # new momentum = grad (old momentum is zero)
        assert np.abs(mom - g).max() <= 2e-5 * (np.abs(g).max() + 1e-12), nm
        np.testing.assert_allclose(out[i], p.inputs[i] - 0.1 * g, rtol=0, atol=3e-6 * (np.abs(g).max() + 1))


def test_torch_train_step_is_the_program(tmp_path):
    """The torch-CPU train step that bench.py times as its host baseline computes the benchmark program: two chained
    steps in float64 against the oracle's, every parameter, running statistic, momentum and the loss."""
    import torch_resnet
    p = configs.build_resnet18(**configs.SMALL["resnet18"])      # batch 8, 16x16, width 8, every scale one
    specs = configs.resnet18_param_specs(8, 10)
    ts = torch_resnet.TrainStep(p, specs, 8, dtype=torch.float64)
    oracle = Oracle(p.text)
    state = list(p.inputs)
    n = len(specs)
    for step in range(2):
        out = oracle.run(*state)
        for k, i in p.feedback.items():
            state[i] = out[k]
        loss = ts.step()
        # the oracle's state is float32 between steps, torch's stays float64
        assert abs(loss - float(out[-1])) < (2e-5 if step == 0 else 2e-4)
    for i, nm in enumerate(ts.names):
        np.testing.assert_allclose(out[i], ts.P[nm].detach().numpy(), rtol=0, atol=2e-5 * (np.abs(out[i]).max() + 1), err_msg=nm)
    for k, r in enumerate(ts.running):
        np.testing.assert_allclose(out[n + k], r.numpy(), rtol=1e-4, atol=1e-5)
    n_stats = len(ts.running)
    for i, nm in enumerate(ts.names):
        mom = out[n + n_stats + i]
        np.testing.assert_allclose(mom, ts.M[nm].numpy(), rtol=0, atol=1e-4 * (np.abs(mom).max() + 1e-12), err_msg=nm)


def test_embedding_program_vs_numpy():
    p = configs.build_embedding(**configs.SMALL["embedding"])
    rows, dtable = Oracle(p.text).run(*p.inputs)
    table, idx, g = p.inputs
    assert np.array_equal(rows, table[idx])
    want = np.zeros_like(table)
    for i, u in zip(idx, g):
        want[i] = want[i] + u
    assert np.array_equal(dtable.view(np.uint32), want.view(np.uint32))


def test_lstm_program_vs_torch():
    kw = configs.SMALL["lstm"]
    p = configs.build_lstm(**kw)
    out = Oracle(p.text).run(*p.inputs)
    H, T, B = kw["hidden"], kw["seq"], kw["batch"]
    wi, wh, b, wo, bo = [torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in p.inputs[:5]]
    xs = torch.tensor(p.inputs[-2], dtype=torch.float64)
    y = torch.tensor(p.inputs[-1]).long()
    h = torch.zeros(B, H, dtype=torch.float64)
    c = torch.zeros(B, H, dtype=torch.float64)
    for t in range(T):
        z = xs[t] @ wi + h @ wh + b
        i, f, g, o = torch.sigmoid(z[:, :H]), torch.sigmoid(z[:, H:2 * H]), torch.tanh(z[:, 2 * H:3 * H]), torch.sigmoid(z[:, 3 * H:])
        c = f * c + i * g
        h = o * torch.tanh(c)
    loss = F.cross_entropy(h @ wo + bo, y)
    loss.backward()
    assert abs(float(out[-1]) - loss.item()) < 1e-6
    for k, t in enumerate((wi, wh, b, wo, bo)):
        g = t.grad.numpy()
        m = 0.1 * g
        np.testing.assert_allclose(out[5 + k], m, rtol=0, atol=2e-6 * np.abs(m).max())
        step = (m / 0.1) / (np.sqrt(g * g) + 1e-8)     # bias-corrected Adam direction at step 1
        np.testing.assert_allclose(out[k], t.detach().numpy() - 1e-3 * step, rtol=0, atol=2e-5)
    assert int(out[15]) == 1


def test_distilbert_program_vs_torch():
    kw = dict(configs.SMALL["distilbert"])
    p = configs.build_distilbert(dtype="f32", **kw)
    out = Oracle(p.text).run(*p.inputs)[0]
    A = {n: torch.tensor(a, dtype=torch.float64) for n, a in zip(p.input_names, p.inputs)}
    ids = torch.tensor(p.inputs[-2]).long()
    B, T, D, Hh = kw["batch"], kw["seq"], kw["d_model"], kw["heads"]

    def ln(x, s, b):
        m = x.mean(-1, keepdim=True)
        v = ((x * x).mean(-1, keepdim=True) - m * m).clamp(min=0)
        return (x - m) * torch.rsqrt(v + 1e-12) * s + b
    x = ln(A["word_emb"][ids] + A["pos_emb"][torch.arange(T)][None], A["emb_ln.scale"], A["emb_ln.bias"])
    for l in range(kw["layers"]):
        pf = f"layer{l}."
        qkv = (x @ A[pf + "qkv.kernel"] + A[pf + "qkv.bias"]).reshape(B, T, 3, Hh, D // Hh)
        q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
        pr = torch.softmax(torch.einsum("btnh,bsnh->bnts", q, k) / math.sqrt(D // Hh), -1)
        enc = torch.einsum("bnts,bsnh->btnh", pr, v).reshape(B, T, D)
        x = ln(x + enc @ A[pf + "out.kernel"] + A[pf + "out.bias"], A[pf + "sa_ln.scale"], A[pf + "sa_ln.bias"])
        ff = F.gelu(x @ A[pf + "ffn1.kernel"] + A[pf + "ffn1.bias"], approximate="tanh") @ A[pf + "ffn2.kernel"] + A[pf + "ffn2.bias"]
        x = ln(x + ff, A[pf + "out_ln.scale"], A[pf + "out_ln.bias"])
    np.testing.assert_allclose(out, x.numpy(), rtol=0, atol=5e-6)
    # bf16 module: within bf16 resolution of the f32 result
    pb = configs.build_distilbert(dtype="bf16", **kw)
    ins = [round_bf16(a) if d == "bf16" else a for a, d in zip(pb.inputs, pb.input_dtypes)]
    outb = Oracle(pb.text).run(*ins)[0]
    assert np.abs(outb - x.numpy()).max() <= 2e-2 * np.abs(x.numpy()).max()


def test_all_op_cases_run_on_the_oracle():
    for c in op_cases.all_cases():
        ins = [round_bf16(a) if d == "bf16" else a for a, d in zip(c.inputs, c.dtypes)]
        out = Oracle(c.text).run(*ins)
        assert len(out) >= 1, c.name


def test_threefry2x32_known_answer_vectors():
    """Random123 KATs (the vectors JAX's own tests use): key (0,0) ctr (0,0) -> 6b200159 99ba4efe; all ones -> 1cb996fc bb002be7;
    key (13198a2e, 03707344) ctr (243f6a88, 85a308d3) -> c4923a9c 483df7a0.  Pins ui32 add / xor / shifts of the oracle."""
    import op_cases
    c = op_cases.get_case("threefry2x32-known-answers")
    out = Oracle(c.text).run(*c.inputs)
    assert np.array_equal(out[0], op_cases.THREEFRY_KAT["out0"])
    assert np.array_equal(out[1], op_cases.THREEFRY_KAT["out1"])


def test_sort_against_numpy_stable_sorts():
    """The oracle's sort (comparator on all pairs, no sorting routine) against numpy: np.sort for values, stable
    np.argsort for key/value and descending ties (JAX's descending sort is a stable sort under GT, so equal keys keep
    their original order), np.lexsort for two keys, total order for NaN and signed zero."""
    import op_cases
    def run(name):
        c = op_cases.get_case(name)
        ins = [round_bf16(a) if d == "bf16" else a for a, d in zip(c.inputs, c.dtypes)]
        return ins, Oracle(c.text).run(*ins)
    for name, axis in (("sort-1d", 0), ("sort-1d-odd-length", 0), ("sort-2d-axis0", 0), ("sort-3d-axis1", 1), ("sort-int32", 1), ("sort-bool", 1), ("sort-4096", 1), ("sort-long-slice-in-memory", 0)):
        ins, out = run(name)
        assert np.array_equal(out[0], np.sort(ins[0], axis=axis, kind="stable")), name
    ins, out = run("sort-descending")
    assert np.array_equal(out[0], -np.sort(-ins[0], axis=1, kind="stable"))
    ins, out = run("sort-uint8")
    assert np.array_equal(out[0], np.sort(ins[0], axis=1)[:, ::-1])
    ins, out = run("sort-nan-and-signed-zero-total-order")
    want = np.array([[-np.inf, -1.0, -0.0, 0.0, 2.0, 2.0, 3.0, np.inf, np.nan, np.nan]], np.float32)
    assert np.array_equal(out[0].view(np.uint32), want.view(np.uint32))       # -0.0 before +0.0, NaNs last
    ins, out = run("sort-key-val-stable-ties")
    order = np.argsort(ins[0], axis=1, kind="stable")
    assert np.array_equal(out[0], np.take_along_axis(ins[0], order, 1)) and np.array_equal(out[1], np.take_along_axis(ins[1], order, 1))
    ins, out = run("sort-argsort-descending-ties")
    order = np.argsort(-ins[0], axis=1, kind="stable")
    assert np.array_equal(out[1], order.astype(np.int32)) and np.array_equal(out[0], np.take_along_axis(ins[0], order, 1))
    ins, out = run("sort-long-key-val-in-memory")
    order = np.argsort(-ins[0], axis=0, kind="stable")
    assert np.array_equal(out[0], np.take_along_axis(ins[0], order, 0)) and np.array_equal(out[1], np.take_along_axis(ins[1], order, 0))
    ins, out = run("sort-two-keys-lexicographic")
    order = np.lexsort((ins[1], ins[0]))                                       # last key is the primary one; lexsort is stable
    assert all(np.array_equal(o, i[order]) for o, i in zip(out, ins))
    ins, out = run("sort-custom-comparator-abs")
    order = np.argsort(np.abs(ins[0]), axis=1, kind="stable")
    assert np.array_equal(out[0], np.take_along_axis(ins[0], order, 1))
    ins, out = run("sort-bf16-keys")
    order = np.argsort(ins[0], axis=1, kind="stable")
    assert np.array_equal(out[1], np.take_along_axis(ins[1], order, 1))


def test_top_k_against_numpy():
    """top_k of the oracle (rank counting) against a stable numpy argsort of the negated values, and the literal tie /
    NaN expectations: equal values come out in ascending position, NaN ranks above +inf (total order)."""
    import op_cases
    for name in ("top-k-1d", "top-k-2d-k5", "top-k-4d", "top-k-equals-size", "top-k-ties-lowest-index-first", "top-k-int32", "top-k-vocabulary-row"):
        c = op_cases.get_case(name)
        vals, idx = Oracle(c.text).run(*c.inputs)
        x = c.inputs[0]
        k = vals.shape[-1]
        order = np.argsort(-x.astype(np.float64), axis=-1, kind="stable")[..., :k]
        assert np.array_equal(idx, order.astype(np.int32)), name
        assert np.array_equal(vals, np.take_along_axis(x, order, -1)), name
    c = op_cases.get_case("top-k-nan-first")
    vals, idx = Oracle(c.text).run(*c.inputs)
    assert np.array_equal(idx, np.array([[1, 8, 5, 0]], np.int32)) and np.isnan(vals[0, :2]).all() and vals[0, 2] == np.inf and vals[0, 3] == 3.0


def test_rng_bit_generator_state_rule_and_bits():
    """State: key unchanged, counter += ceil(output bytes / 16) (reference: src/pjrt_plugin/ops/control_flow.cc:2343-2355),
    wrapping at 2^64.  Bits: the oracle's threefry helper reproduces the Random123 known answers, element i of a draw is
    threefry(key halves; (i, counter low half)), and the stream looks uniform (bit balance, byte chi-square)."""
    import op_cases
    import shlo_oracle
    kat = op_cases.THREEFRY_KAT
    x0, x1 = shlo_oracle.threefry2x32(kat["key0"], kat["key1"], kat["ctr0"], kat["ctr1"])
    assert np.array_equal(x0, kat["out0"]) and np.array_equal(x1, kat["out1"])
    for name, nbytes in (("rng-bits-u32", 4000), ("rng-bits-u64", 129 * 8), ("rng-bits-u8", 50), ("rng-bits-u32-2d-default", 7 * 33 * 4)):
        c = op_cases.get_case(name)
        state, bits = Oracle(c.text).run(*c.inputs)
        assert state[0] == c.inputs[0][0] and int(state[1]) == int(c.inputs[0][1]) + (nbytes + 15) // 16, name
    c = op_cases.get_case("rng-bits-chained")
    s2, b1, b2 = Oracle(c.text).run(*c.inputs)
    assert int(s2[0]) == 7 and int(s2[1]) == 7            # key untouched; counter (2^64 - 1) + 4 + 4 wraps to 7
    assert not np.array_equal(b1, b2)                      # the second draw uses the advanced counter
    c = op_cases.get_case("rng-bits-u32")
    _, bits = Oracle(c.text).run(*c.inputs)
    k0, k1 = np.uint32(0x89ABCDEF), np.uint32(0x01234567)
    want, _ = shlo_oracle.threefry2x32(k0, k1, np.arange(1000, dtype=np.uint32), np.full(1000, 41, np.uint32))
    assert np.array_equal(bits, want)
    ones = np.unpackbits(bits.view(np.uint8)).mean()
    assert abs(ones - 0.5) < 0.01
    counts = np.bincount(bits.view(np.uint8), minlength=256)
    chi2 = ((counts - counts.mean()) ** 2 / counts.mean()).sum()
    assert chi2 < 340                                      # 255 degrees of freedom: P(chi2 > 340) < 3e-4
    c = op_cases.get_case("rng-uniform-floats")
    u = Oracle(c.text).run(*c.inputs)[0]
    assert u.min() >= 0.0 and u.max() < 1.0 and abs(u.mean() - 0.5) < 0.02 and abs(u.var() - 1 / 12) < 0.01


def test_pooling_against_torch():
    """reduce_window (max / sum) and select_and_scatter (gradient of max pooling, first maximum wins) against
    torch.nn.functional.max_pool2d / avg_pool2d and torch autograd, NHWC <-> NCHW."""
    import torch
    from jax_mps_amd.shlo.builder import Builder
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 9, 8, 3)).astype(np.float32)
    pad = [(0, 0), (1, 1), (1, 1), (0, 0)]
    b = Builder()
    b.ret(b.reduce_window(b.arg(x.shape), float("-inf"), "max", (1, 3, 3, 1), (1, 2, 2, 1), pad))
    t = torch.nn.functional.max_pool2d(torch.tensor(x).permute(0, 3, 1, 2), 3, 2, 1).permute(0, 2, 3, 1).numpy()
    assert np.array_equal(Oracle(b.text()).run(x)[0], t)
    b = Builder()
    b.ret(b.reduce_window(b.arg(x.shape), 0.0, "add", (1, 2, 2, 1), (1, 2, 2, 1)))
    t = 4 * torch.nn.functional.avg_pool2d(torch.tensor(x).permute(0, 3, 1, 2), 2, 2).permute(0, 2, 3, 1).numpy()
    assert np.allclose(Oracle(b.text()).run(x)[0], t, rtol=1e-6, atol=1e-6)
    xt = torch.tensor(x).permute(0, 3, 1, 2).clone().requires_grad_(True)
    y = torch.nn.functional.max_pool2d(xt, 3, 2, 1)
    g = torch.tensor(rng.standard_normal(tuple(y.shape)).astype(np.float32))
    y.backward(g)
    b = Builder()
    b.ret(b.select_and_scatter(b.arg(x.shape), b.arg((2, 5, 4, 3)), 0.0, (1, 3, 3, 1), (1, 2, 2, 1), pad))
    got = Oracle(b.text()).run(x, g.permute(0, 2, 3, 1).numpy().copy())[0]
    assert np.allclose(got, xt.grad.permute(0, 2, 3, 1).numpy(), rtol=1e-6, atol=1e-6)


# ------------------------------------------------------------------ fused-op custom calls (oracle's `fused_*`) vs torch / closed forms
def _fused_oracle(name):
    c = op_cases.get_case(name)
    ins = [round_bf16(a) if d == "bf16" else a for a, d in zip(c.inputs, c.dtypes)]
    return ins, Oracle(c.text).run(*ins)


def _t64(a, grad=False):
    return torch.tensor(np.asarray(a, np.float64), requires_grad=grad)


def _torch_sdpa(q, k, v, mask, scale):
    g = q.shape[1] // k.shape[1]
    return F.scaled_dot_product_attention(q, k.repeat_interleave(g, 1), v.repeat_interleave(g, 1), attn_mask=mask, scale=scale)


@pytest.mark.parametrize("name, scale", [("fused-sdpa-padding-mask-f32", 0.25), ("fused-sdpa-grouped-heads-f32", 0.25), ("fused-sdpa-full-mask-f32", 0.3),
                                         ("fused-sdpa-additive-bias-f32", 0.25)])
def test_fused_sdpa_vs_torch(name, scale):
    (q, k, v, m), out = _fused_oracle(name)
    mask = torch.tensor(m) if m.dtype == np.bool_ else _t64(m)
    want = _torch_sdpa(_t64(q), _t64(k), _t64(v), mask, scale).numpy()
    np.testing.assert_allclose(out[0], want, rtol=2e-6, atol=2e-6)


@pytest.mark.parametrize("name", ["fused-sdpa-causal-f32", "fused-sdpa-causal-longer-keys-f32"])
def test_fused_sdpa_causal_vs_torch(name):
    """Query t sees keys 0 .. t + (S - T): with as many keys as queries this is torch's is_causal; with more keys the
    window is aligned to the last key (the newest query sees everything), written here as an explicit mask."""
    (q, k, v), out = _fused_oracle(name)
    T, S = q.shape[2], k.shape[2]
    if T == S:
        want = F.scaled_dot_product_attention(_t64(q), _t64(k), _t64(v), is_causal=True, scale=0.25).numpy()
    else:
        mask = torch.tensor(np.tril(np.ones((T, S), bool), k=S - T))
        want = _torch_sdpa(_t64(q), _t64(k), _t64(v), mask, 0.25).numpy()
    np.testing.assert_allclose(out[0], want, rtol=2e-6, atol=2e-6)


@pytest.mark.parametrize("name, causal", [("fused-sdpa-bwd-f32", False), ("fused-sdpa-bwd-grouped-heads-f32", False), ("fused-sdpa-causal-bwd-f32", True)])
def test_fused_sdpa_backward_vs_autograd(name, causal):
    ins, out = _fused_oracle(name)
    q, k, v = (_t64(a, True) for a in ins[:3])
    if causal:
        y = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=0.25)
    else:
        y = _torch_sdpa(q, k, v, torch.tensor(ins[3]), 0.25)
    y.backward(_t64(ins[-1]))
    for got, t in zip(out, (q, k, v)):
        np.testing.assert_allclose(got, t.grad.numpy(), rtol=2e-5, atol=2e-6)


def test_fused_norms_vs_torch():
    (x, w), out = _fused_oracle("fused-rms-norm-f32")
    np.testing.assert_allclose(out[0], F.rms_norm(_t64(x), (x.shape[-1],), _t64(w), eps=1e-6).numpy(), rtol=2e-6, atol=2e-6)
    (x, w, g), out = _fused_oracle("fused-rms-norm-bwd-f32")
    tx, tw = _t64(x, True), _t64(w, True)
    F.rms_norm(tx, (x.shape[-1],), tw, eps=1e-6).backward(_t64(g))
    np.testing.assert_allclose(out[0], tx.grad.numpy(), rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(out[1], tw.grad.numpy(), rtol=2e-5, atol=2e-5)
    (x, w, b), out = _fused_oracle("fused-layer-norm-f32")
    np.testing.assert_allclose(out[0], F.layer_norm(_t64(x), (x.shape[-1],), _t64(w), _t64(b), eps=1e-5).numpy(), rtol=2e-6, atol=2e-6)
    (x, w, b, g), out = _fused_oracle("fused-layer-norm-bwd-f32")
    tx, tw, tb = _t64(x, True), _t64(w, True), _t64(b, True)
    F.layer_norm(tx, (x.shape[-1],), tw, tb, eps=1e-5).backward(_t64(g))
    for got, t in zip(out, (tx, tw, tb)):
        np.testing.assert_allclose(got, t.grad.numpy(), rtol=2e-5, atol=2e-5)


def test_fused_gelu_vs_torch():
    (x,), out = _fused_oracle("fused-gelu-f32")
    np.testing.assert_allclose(out[0], F.gelu(_t64(x), approximate="tanh").numpy(), rtol=2e-6, atol=2e-7)
    (x, g), out = _fused_oracle("fused-gelu-bwd-f32")
    tx = _t64(x, True)
    F.gelu(tx, approximate="tanh").backward(_t64(g))
    np.testing.assert_allclose(out[0], tx.grad.numpy(), rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("name, dims, base, scale, traditional", [("fused-rope-f32", 32, 10000.0, 1.0, False),
                                                                  ("fused-rope-partial-traditional-f32", 16, 500.0, 0.5, True)])
def test_fused_rope_is_a_complex_rotation(name, dims, base, scale, traditional):
    """Each rotated pair (a, b) is the complex number a + ib multiplied by exp(i * position * frequency): written with
    numpy's complex arithmetic, which shares nothing with the oracle's cos / sin form."""
    (x, offset), out = _fused_oracle(name)
    x = x.astype(np.float64)
    T, half = x.shape[-2], dims // 2
    theta = ((np.arange(T) + int(offset)) * scale)[:, None] * base ** (-2.0 * np.arange(half) / dims)[None, :]
    want = x.copy()
    if traditional:
        z = (x[..., 0:dims:2] + 1j * x[..., 1:dims:2]) * np.exp(1j * theta)
        want[..., 0:dims:2], want[..., 1:dims:2] = z.real, z.imag
    else:
        z = (x[..., :half] + 1j * x[..., half:dims]) * np.exp(1j * theta)
        want[..., :half], want[..., half:dims] = z.real, z.imag
    np.testing.assert_allclose(out[0], want, rtol=2e-6, atol=2e-6)
    # position 0 with no offset leaves the row as it is; features past `dims` pass through
    if int(offset) == 0:
        np.testing.assert_array_equal(out[0][..., 0, :], x[..., 0, :].astype(np.float32))
    np.testing.assert_array_equal(out[0][..., dims:], x[..., dims:].astype(np.float32))


def test_fused_rope_backward_inverts_the_rotation():
    """rope is orthogonal per pair, so its vjp is the inverse rotation: rope_bwd(x, offset, rope(g)) == g."""
    (x, offset, g), out = _fused_oracle("fused-rope-bwd-f32")
    o = Oracle(op_cases.get_case("fused-rope-bwd-f32").text)
    cfg = {"dims": 24, "traditional": False, "base": 10000.0, "rope_scale": 1.0}
    forward = o.fused_rope([g, offset], cfg)[0]
    back = o.fused_rope_bwd([x, offset, forward], cfg)[0]
    np.testing.assert_allclose(back, g, rtol=1e-12, atol=1e-12)
    # and it is the transpose of the forward map: <rope(u), g> == <u, rope_bwd(g)>
    u = np.random.default_rng(0).standard_normal(g.shape)
    assert abs((o.fused_rope([u, offset], cfg)[0] * g).sum() - (u * out[0].astype(np.float64)).sum()) < 1e-4
