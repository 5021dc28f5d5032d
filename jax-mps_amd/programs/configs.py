"""The five benchmark programs as StableHLO modules plus their synthetic inputs.

Each `build_*` returns a `Program`: the module text that goes to
PJRT_Client_Compile, the host arrays that go to PJRT_Client_BufferFromHostBuffer
(generated with numpy.random.default_rng(seed) so that every backend sees the
same bits), and the names of inputs/outputs.  Model structure follows the
reference's examples: ResNet18 from examples/resnet/model.py:6-163, the
DistilBERT-shaped encoder from examples/distilbert/model.py:21-94, the
scan-trained RNN step from benchmarks/bench_rnn_training.py:63-90.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Sequence, Tuple

import numpy as np

from ..shlo.builder import (Builder, Val, gelu_tanh, layer_norm, log_softmax, one_hot, relu, softmax,
                            softmax_cross_entropy_int, f32_to_bf16_bits)


@dataclass
class Program:
    name: str
    text: str
    inputs: List[np.ndarray]
    input_names: List[str]
    output_names: List[str]
    input_dtypes: List[str]
    output_types: List[Tuple[Tuple[int, ...], str]]
    # indices: output k feeds input feedback[k] on the next step (train-state threading)
    feedback: Dict[int, int] = field(default_factory=dict)
    meta: Dict[str, object] = field(default_factory=dict)


def _finish(name: str, b: Builder, inputs, in_names, out_names, feedback=None, meta=None) -> Program:
    # train state threaded from step to step is donated, as jax.jit(step, donate_argnums=...) would declare it
    for k, i in (feedback or {}).items():
        b.donate(b._main_args[i], k)
    return Program(name, b.text(), list(inputs), list(in_names), list(out_names), [d for _, d in b.arg_types],
                   list(b.result_types), dict(feedback or {}), dict(meta or {}))


# ----------------------------------------------------------------------------
# 1. two-layer MLP, SGD
# ----------------------------------------------------------------------------
def build_mlp(batch=256, d_in=784, d_hidden=512, n_cls=10, lr=0.01, seed=0) -> Program:
    rng = np.random.default_rng(seed)
    w1 = (rng.standard_normal((d_in, d_hidden)) * math.sqrt(2.0 / (d_in + d_hidden))).astype(np.float32)
    w2 = (rng.standard_normal((d_hidden, n_cls)) * math.sqrt(2.0 / (d_hidden + n_cls))).astype(np.float32)
    b1 = np.zeros(d_hidden, np.float32)
    b2 = np.zeros(n_cls, np.float32)
    x = rng.standard_normal((batch, d_in)).astype(np.float32)
    y = rng.integers(0, n_cls, size=(batch,)).astype(np.int32)

    b = Builder("jit_mlp_train_step")
    W1, B1, W2, B2 = b.arg(w1.shape), b.arg(b1.shape), b.arg(w2.shape), b.arg(b2.shape)
    X, Y = b.arg(x.shape), b.arg(y.shape, "i32")
    h = relu(b, b.add(b.matmul(X, W1), B1))
    logits = b.add(b.matmul(h, W2), B2)
    loss = softmax_cross_entropy_int(b, logits, Y)
    grads = b.grad(loss, [W1, B1, W2, B2])
    new = [b.sub(p, b.mul(g, lr)) for p, g in zip([W1, B1, W2, B2], grads)]
    b.ret(*new, loss)
    return _finish("mlp_sgd", b, [w1, b1, w2, b2, x, y], ["w1", "b1", "w2", "b2", "x", "y"],
                   ["w1", "b1", "w2", "b2", "loss"], feedback={0: 0, 1: 1, 2: 2, 3: 3},
                   meta=dict(batch=batch, flops_per_step=6 * batch * (d_in * d_hidden + d_hidden * n_cls)))


# ----------------------------------------------------------------------------
# 2. embedding gather + scatter-add gradient
# ----------------------------------------------------------------------------
def zipf_indices(rng, n, vocab, s=1.1):
    p = 1.0 / np.arange(1, vocab + 1, dtype=np.float64) ** s
    cdf = np.cumsum(p / p.sum())
    ranks = np.searchsorted(cdf, rng.random(n), side="left")
    perm = rng.permutation(vocab)
    return perm[np.minimum(ranks, vocab - 1)].astype(np.int32)


def build_embedding(vocab=50000, dim=768, n_idx=8192, seed=1) -> Program:
    rng = np.random.default_rng(seed)
    table = (rng.standard_normal((vocab, dim)) * 0.02).astype(np.float32)
    idx = zipf_indices(rng, n_idx, vocab)
    g = rng.standard_normal((n_idx, dim)).astype(np.float32)

    b = Builder("jit_embedding_fwd_bwd")
    T, I, G = b.arg(table.shape), b.arg(idx.shape, "i32"), b.arg(g.shape)
    rows = b.take_rows(T, I)
    (dT,) = b.grad(rows, [T], seed=G)
    b.ret(rows, dT)
    return _finish("embedding", b, [table, idx, g], ["table", "idx", "upstream"], ["rows", "dtable"],
                   meta=dict(gather_bytes=n_idx * (4 + 2 * dim * 4), scatter_bytes=vocab * dim * 4 + n_idx * dim * 4 + n_idx * 4))


# ----------------------------------------------------------------------------
# 3. ResNet18 (CIFAR variant) train step, SGD momentum
# ----------------------------------------------------------------------------
def _batch_norm_train(b: Builder, x: Val, scale: Val, bias: Val, ra_mean: Val, ra_var: Val, momentum=0.9, eps=1e-5):
    """flax.nnx.BatchNorm in training mode: batch statistics over (N,H,W) as E[x],
    E[x^2]; var = max(0, E[x^2]-E[x]^2); running averages updated with `momentum`."""
    axes = [0, 1, 2]
    mean = b.mean(x, axes)
    mean2 = b.mean(b.mul(x, x), axes)
    var = b.maximum(b.sub(mean2, b.mul(mean, mean)), 0.0)
    y = b.sub(x, b.broadcast_in_dim(mean, x.shape, [3]))
    mul = b.mul(b.rsqrt(b.add(var, eps)), scale)
    y = b.mul(y, b.broadcast_in_dim(mul, x.shape, [3]))
    y = b.add(y, b.broadcast_in_dim(bias, x.shape, [3]))
    sm, sv = b.stop_gradient(mean), b.stop_gradient(var)
    new_mean = b.add(b.mul(ra_mean, momentum), b.mul(sm, 1.0 - momentum))
    new_var = b.add(b.mul(ra_var, momentum), b.mul(sv, 1.0 - momentum))
    return y, new_mean, new_var


def resnet18_param_specs(width=64, n_cls=10, in_ch=3):
    """[(name, shape, kind)] in a fixed order; kind in conv/bn_scale/bn_bias/dense_w/dense_b."""
    specs = []

    def conv(name, k, cin, cout):
        specs.append((name + ".kernel", (k, k, cin, cout), "conv"))

    def bn(name, c, zero_scale=False):
        specs.append((name + ".scale", (c,), "bn_scale0" if zero_scale else "bn_scale"))
        specs.append((name + ".bias", (c,), "bn_bias"))

    conv("conv_init", 3, in_ch, width)
    bn("bn_init", width)
    cin = width
    for stage, mult in enumerate((1, 2, 4, 8), start=1):
        cout = width * mult
        for blk in (1, 2):
            stride = 2 if (stage > 1 and blk == 1) else 1
            p = f"stage{stage}_block{blk}"
            conv(p + ".conv1", 3, cin, cout); bn(p + ".bn1", cout)
            conv(p + ".conv2", 3, cout, cout); bn(p + ".bn2", cout, zero_scale=True)
            if cin != cout or stride != 1:
                conv(p + ".conv_proj", 1, cin, cout); bn(p + ".bn_proj", cout)
            cin = cout
    specs.append(("dense.kernel", (cin, n_cls), "dense_w"))
    specs.append(("dense.bias", (n_cls,), "dense_b"))
    return specs


def build_resnet18(batch=128, image=32, width=64, n_cls=10, lr=0.1, momentum=0.9, seed=2, zero_bn2_scale=True,
                   train=True) -> Program:
    rng = np.random.default_rng(seed)
    specs = resnet18_param_specs(width, n_cls)
    params, stats = [], []
    for name, shape, kind in specs:
        if kind == "conv":
            fan_in = shape[0] * shape[1] * shape[2]
            params.append((rng.standard_normal(shape) * math.sqrt(2.0 / fan_in)).astype(np.float32))
        elif kind == "bn_scale":
            params.append(np.ones(shape, np.float32))
        elif kind == "bn_scale0":
            params.append(np.zeros(shape, np.float32) if zero_bn2_scale else np.ones(shape, np.float32))
        elif kind == "dense_w":
            params.append((rng.standard_normal(shape) * math.sqrt(1.0 / shape[0])).astype(np.float32))
        else:
            params.append(np.zeros(shape, np.float32))
    bn_names = [n[:-6] for n, _, k in specs if k.startswith("bn_scale")]
    for n in bn_names:
        c = [s for nn, s, _ in specs if nn == n + ".scale"][0]
        stats.append(np.zeros(c, np.float32))
        stats.append(np.ones(c, np.float32))
    x = rng.standard_normal((batch, image, image, 3)).astype(np.float32)
    y = rng.integers(0, n_cls, size=(batch,)).astype(np.int32)

    b = Builder("jit_resnet18_train_step")
    P = [b.arg(p.shape) for p in params]
    S = [b.arg(s.shape) for s in stats]
    M = [b.arg(p.shape) for p in params] if train else []
    X, Y = b.arg(x.shape), b.arg(y.shape, "i32")
    pidx = {n: i for i, (n, _, _) in enumerate(specs)}
    sidx = {n: 2 * i for i, n in enumerate(bn_names)}
    new_stats: List[Val] = [None] * len(S)

    def conv(name, h, stride):
        w = P[pidx[name + ".kernel"]]
        k = w.shape[0]
        # SAME padding as flax computes it: total = max((ceil(in/stride)-1)*stride + k - in, 0)
        n_in = h.shape[1]
        out = -(-n_in // stride)
        tot = max((out - 1) * stride + k - n_in, 0)
        pad = (tot // 2, tot - tot // 2)
        return b.conv(h, w, strides=(stride, stride), padding=(pad, pad))

    def bn(name, h):
        i = sidx[name]
        yv, nm, nv = _batch_norm_train(b, h, P[pidx[name + ".scale"]], P[pidx[name + ".bias"]], S[i], S[i + 1])
        new_stats[i], new_stats[i + 1] = nm, nv
        return yv

    h = relu(b, bn("bn_init", conv("conv_init", X, 1)))
    cin = width
    for stage, mult in enumerate((1, 2, 4, 8), start=1):
        cout = width * mult
        for blk in (1, 2):
            stride = 2 if (stage > 1 and blk == 1) else 1
            p = f"stage{stage}_block{blk}"
            r = h
            yv = relu(b, bn(p + ".bn1", conv(p + ".conv1", h, stride)))
            yv = bn(p + ".bn2", conv(p + ".conv2", yv, 1))
            if cin != cout or stride != 1:
                r = bn(p + ".bn_proj", conv(p + ".conv_proj", r, stride))
            h = relu(b, b.add(r, yv))
            cin = cout
    pooled = b.mean(h, [1, 2])
    logits = b.add(b.matmul(pooled, P[pidx["dense.kernel"]]), P[pidx["dense.bias"]])
    loss = softmax_cross_entropy_int(b, logits, Y)
    in_names = [n for n, _, _ in specs] + [f"{n}.{k}" for n in bn_names for k in ("mean", "var")]
    if not train:
        b.ret(logits, loss)
        return _finish("resnet18_fwd", b, params + stats + [x, y], in_names + ["x", "y"], ["logits", "loss"])
    grads = b.grad(loss, P)
    new_m = [b.add(g, b.mul(m, momentum)) for g, m in zip(grads, M)]
    new_p = [b.sub(p, b.mul(m, lr)) for p, m in zip(P, new_m)]
    b.ret(*new_p, *new_stats, *new_m, loss)
    momenta = [np.zeros_like(p) for p in params]
    in_names = in_names + ["mom." + n for n, _, _ in specs] + ["x", "y"]
    out_names = in_names[:-2] + ["loss"]
    nstate = len(P) + len(S) + len(M)
    macs = _resnet_macs(specs, batch, image)
    return _finish("resnet18_train", b, params + stats + momenta + [x, y], in_names, out_names,
                   feedback={i: i for i in range(nstate)},
                   meta=dict(batch=batch, fwd_flops=2 * macs["fwd"], step_flops=2 * macs["step"], n_params=len(P)))


def _resnet_macs(specs, batch, image):
    fwd = 0
    step = 0
    size = image
    first = True
    for name, shape, kind in specs:
        if kind != "conv":
            continue
        k, _, cin, cout = shape
        if ".conv1" in name and "stage1" not in name and "block1" in name:
            size //= 2
        out = size
        m = batch * out * out * k * k * cin * cout
        fwd += m
        step += 3 * m if not first else 2 * m   # no input gradient for the image itself
        first = False
    d = [s for n, s, k in specs if k == "dense_w"][0]
    fwd += batch * d[0] * d[1]
    step += 3 * batch * d[0] * d[1]
    return dict(fwd=fwd, step=step)


# ----------------------------------------------------------------------------
# 4. DistilBERT-shaped encoder forward, bf16
# ----------------------------------------------------------------------------
def build_distilbert(batch=32, seq=128, layers=6, d_model=768, heads=12, d_ff=3072, vocab=30522, max_pos=512,
                     eps=1e-12, seed=3, dtype="bf16") -> Program:
    rng = np.random.default_rng(seed)

    def w(*shape):
        return (rng.standard_normal(shape) * 0.02).astype(np.float32)
    names, arrays = [], []

    def add(n, a):
        names.append(n); arrays.append(a)
    add("word_emb", w(vocab, d_model)); add("pos_emb", w(max_pos, d_model))
    add("emb_ln.scale", np.ones(d_model, np.float32)); add("emb_ln.bias", np.zeros(d_model, np.float32))
    for l in range(layers):
        p = f"layer{l}."
        add(p + "qkv.kernel", w(d_model, 3 * d_model)); add(p + "qkv.bias", np.zeros(3 * d_model, np.float32))
        add(p + "out.kernel", w(d_model, d_model)); add(p + "out.bias", np.zeros(d_model, np.float32))
        add(p + "sa_ln.scale", np.ones(d_model, np.float32)); add(p + "sa_ln.bias", np.zeros(d_model, np.float32))
        add(p + "ffn1.kernel", w(d_model, d_ff)); add(p + "ffn1.bias", np.zeros(d_ff, np.float32))
        add(p + "ffn2.kernel", w(d_ff, d_model)); add(p + "ffn2.bias", np.zeros(d_model, np.float32))
        add(p + "out_ln.scale", np.ones(d_model, np.float32)); add(p + "out_ln.bias", np.zeros(d_model, np.float32))
    ids = rng.integers(0, vocab, size=(batch, seq)).astype(np.int32)
    mask = np.ones((batch, seq), np.int32)

    b = Builder("jit_distilbert_forward")
    A = {n: b.arg(a.shape, dtype) for n, a in zip(names, arrays)}
    IDS, MASK = b.arg(ids.shape, "i32"), b.arg(mask.shape, "i32")
    hd = d_model // heads

    def linear(x, name):
        k, bias = A[name + ".kernel"], A[name + ".bias"]
        y = b.dot_general(x, k, ([x.ndim - 1], [0]))
        return b.add(y, b.broadcast_in_dim(bias, y.shape, [y.ndim - 1]))

    pos = b.iota((1, seq), 1, "i32")
    x = b.add(b.take_rows(A["word_emb"], IDS), b._bcast_np(b.take_rows(A["pos_emb"], pos), (batch, seq, d_model)))
    x = layer_norm(b, x, A["emb_ln.scale"], A["emb_ln.bias"], eps)
    mb = b.compare(b.reshape(MASK, (batch, 1, 1, seq)), 0, "NE")
    for l in range(layers):
        p = f"layer{l}."
        qkv = b.reshape(linear(x, p + "qkv"), (batch, seq, 3, heads, hd))
        q, k_, v = (b.reshape(b.slice(qkv, [0, 0, i, 0, 0], [batch, seq, i + 1, heads, hd]), (batch, seq, heads, hd)) for i in range(3))
        # jax.nn.dot_product_attention (XLA path): f32 logits, scale, mask, softmax in f32, cast, PV
        logits = b.dot_general(q, k_, ([3], [3]), ([0, 2], [0, 2]), out_dtype="f32")      # B N T S
        logits = b.mul(logits, 1.0 / math.sqrt(hd))
        big_neg = float(-0.7 * np.finfo(np.float32).max)
        logits = b.select(b.broadcast_in_dim(mb, logits.shape, [0, 1, 2, 3]) if mb.shape != logits.shape else mb,
                          logits, b.full_like(logits, big_neg))
        probs = b.convert(softmax(b, logits, -1), dtype)
        enc = b.dot_general(probs, v, ([3], [1]), ([0, 1], [0, 2]))                       # B N T H
        enc = b.reshape(b.transpose(enc, [0, 2, 1, 3]), (batch, seq, d_model))
        x = layer_norm(b, b.add(x, linear(enc, p + "out")), A[p + "sa_ln.scale"], A[p + "sa_ln.bias"], eps)
        ff = linear(gelu_tanh(b, linear(x, p + "ffn1")), p + "ffn2")
        x = layer_norm(b, b.add(x, ff), A[p + "out_ln.scale"], A[p + "out_ln.bias"], eps)
    b.ret(x)
    ins = [a for a in arrays] + [ids, mask]
    tok = batch * seq
    flops = layers * (2 * tok * d_model * 3 * d_model + 2 * tok * d_model * d_model + 4 * tok * d_model * d_ff
                      + 4 * batch * heads * seq * seq * hd)
    return _finish("distilbert_fwd", b, ins, names + ["input_ids", "attention_mask"], ["hidden"], meta=dict(flops=flops))


# ----------------------------------------------------------------------------
# 5. LSTM through a scan (stablehlo.while), Adam
# ----------------------------------------------------------------------------
def build_lstm(seq=100, batch=64, d_in=128, hidden=256, n_cls=10, lr=1e-3, b1=0.9, b2=0.999, eps=1e-8, seed=4) -> Program:
    rng = np.random.default_rng(seed)

    def glorot(*shape):
        return (rng.standard_normal(shape) * math.sqrt(2.0 / (shape[0] + shape[1]))).astype(np.float32)
    wi, wh = glorot(d_in, 4 * hidden), glorot(hidden, 4 * hidden)
    bias = np.zeros(4 * hidden, np.float32)
    wo, bo = glorot(hidden, n_cls), np.zeros(n_cls, np.float32)
    params = [wi, wh, bias, wo, bo]
    xs = rng.standard_normal((seq, batch, d_in)).astype(np.float32)
    y = rng.integers(0, n_cls, size=(batch,)).astype(np.int32)
    mu = [np.zeros_like(p) for p in params]
    nu = [np.zeros_like(p) for p in params]
    count = np.zeros((), np.int32)

    b = Builder("jit_lstm_train_step")
    P = [b.arg(p.shape) for p in params]
    MU = [b.arg(p.shape) for p in params]
    NU = [b.arg(p.shape) for p in params]
    CNT = b.arg((), "i32")
    XS, Y = b.arg(xs.shape), b.arg(y.shape, "i32")
    WI, WH, BI, WO, BO = P
    H = hidden

    def cell(x_t, h, c, wi_, wh_, bi_):
        z = b.add(b.add(b.matmul(x_t, wi_), b.matmul(h, wh_)), b.broadcast_in_dim(bi_, (batch, 4 * H), [1]))
        i = b.logistic(b.slice(z, [0, 0], [batch, H]))
        f = b.logistic(b.slice(z, [0, H], [batch, 2 * H]))
        g = b.tanh(b.slice(z, [0, 2 * H], [batch, 3 * H]))
        o = b.logistic(b.slice(z, [0, 3 * H], [batch, 4 * H]))
        c2 = b.add(b.mul(f, c), b.mul(i, g))
        h2 = b.mul(o, b.tanh(c2))
        return h2, c2

    zero_i = b.constant(0, "i32")
    h0 = b.zeros((batch, H))
    c0 = b.zeros((batch, H))
    hs0 = b.zeros((seq, batch, H))      # h_{t-1} for every step (residuals of the scan)
    cs0 = b.zeros((seq, batch, H))

    def fwd_cond(i, h, c, hs, cs):
        return b.compare(i, seq, "LT")

    def fwd_body(i, h, c, hs, cs):
        x_t = b.reshape(b.dynamic_slice(XS, [i, zero_i_in(), zero_i_in()], [1, batch, d_in]), (batch, d_in))
        hs2 = b.dynamic_update_slice(hs, b.reshape(h, (1, batch, H)), [i, zero_i_in(), zero_i_in()])
        cs2 = b.dynamic_update_slice(cs, b.reshape(c, (1, batch, H)), [i, zero_i_in(), zero_i_in()])
        h2, c2 = cell(x_t, h, c, WI, WH, BI)
        return [b.add(i, 1), h2, c2, hs2, cs2]

    def zero_i_in():
        return b.constant(0, "i32")

    _, hT, cT, hs, cs = b.while_loop([zero_i, h0, c0, hs0, cs0], fwd_cond, fwd_body)
    logits = b.add(b.matmul(hT, WO), BO)
    loss = softmax_cross_entropy_int(b, logits, Y)
    d_hT, d_wo, d_bo = b.grad(loss, [hT, WO, BO])

    # reverse scan: recompute the cell from saved (h_{t-1}, c_{t-1}, x_t) and pull cotangents back
    def bwd_cond(i, dh, dc, dwi, dwh, dbi):
        return b.compare(i, seq, "LT")

    def bwd_body(i, dh, dc, dwi, dwh, dbi):
        t = b.sub(seq - 1, i)
        z0 = zero_i_in()
        x_t = b.reshape(b.dynamic_slice(XS, [t, z0, z0], [1, batch, d_in]), (batch, d_in))
        h_p = b.reshape(b.dynamic_slice(hs, [t, z0, z0], [1, batch, H]), (batch, H))
        c_p = b.reshape(b.dynamic_slice(cs, [t, z0, z0], [1, batch, H]), (batch, H))
        h2, c2 = cell(x_t, h_p, c_p, WI, WH, BI)
        obj = b.add(b.reduce_sum(b.mul(h2, dh), [0, 1]), b.reduce_sum(b.mul(c2, dc), [0, 1]))
        g_h, g_c, g_wi, g_wh, g_bi = b.grad(obj, [h_p, c_p, WI, WH, BI])
        return [b.add(i, 1), g_h, g_c, b.add(dwi, g_wi), b.add(dwh, g_wh), b.add(dbi, g_bi)]

    init = [b.constant(0, "i32"), d_hT, b.zeros((batch, H)), b.zeros(wi.shape), b.zeros(wh.shape), b.zeros(bias.shape)]
    _, _, _, d_wi, d_wh, d_bi = b.while_loop(init, bwd_cond, bwd_body)
    grads = [d_wi, d_wh, d_bi, d_wo, d_bo]

    # optax.adam: bias-corrected moments
    cnt = b.add(CNT, 1)
    cf = b.convert(cnt, "f32")
    bc1 = b.sub(1.0, b.power(b.constant(b1, "f32"), cf))
    bc2 = b.sub(1.0, b.power(b.constant(b2, "f32"), cf))
    new_p, new_mu, new_nu = [], [], []
    for p, g, m, v in zip(P, grads, MU, NU):
        m2 = b.add(b.mul(m, b1), b.mul(g, 1.0 - b1))
        v2 = b.add(b.mul(v, b2), b.mul(b.mul(g, g), 1.0 - b2))
        mh = b.div(m2, b._bcast_np(bc1, m2.shape))
        vh = b.div(v2, b._bcast_np(bc2, v2.shape))
        upd = b.div(mh, b.add(b.sqrt(vh), eps))
        new_p.append(b.sub(p, b.mul(upd, lr)))
        new_mu.append(m2); new_nu.append(v2)
    b.ret(*new_p, *new_mu, *new_nu, cnt, loss)
    pn = ["wi", "wh", "b", "wo", "bo"]
    in_names = pn + ["mu." + n for n in pn] + ["nu." + n for n in pn] + ["count", "xs", "y"]
    out_names = in_names[:-2] + ["loss"]
    flops = seq * 3 * 2 * batch * (d_in + hidden) * 4 * hidden
    return _finish("lstm_adam", b, params + mu + nu + [count, xs, y], in_names, out_names,
                   feedback={i: i for i in range(16)}, meta=dict(flops=flops))


ALL = {
    "mlp": build_mlp,
    "embedding": build_embedding,
    "resnet18": build_resnet18,
    "distilbert": build_distilbert,
    "lstm": build_lstm,
}


# Reduced instances of the five programs: sizes the CPU oracle finishes in seconds.
SMALL = {
    "mlp": dict(batch=8, d_in=12, d_hidden=16),
    "embedding": dict(vocab=50, dim=8, n_idx=32),
    # batch statistics need a few dozen elements per channel to be well conditioned: the last stage of an 8 x 16 x 16
    # batch still has 8 x 2 x 2 = 32 (a 4 x 8 x 8 batch leaves 4, and float32 summation order then moves the
    # normalised values by 1e-4)
    "resnet18": dict(batch=8, image=16, width=8, zero_bn2_scale=False),
    "distilbert": dict(batch=2, seq=8, layers=2, d_model=16, heads=4, d_ff=32, vocab=50, max_pos=16),
    "lstm": dict(seq=7, batch=4, d_in=6, hidden=8),
}
# Mid-size instances: large enough to span several workgroup tiles, still seconds on the oracle.
MEDIUM = {
    "mlp": dict(batch=96, d_in=200, d_hidden=130),
    "embedding": dict(vocab=5000, dim=768, n_idx=2048),
    "resnet18": dict(batch=8, image=16, width=16, zero_bn2_scale=False),
    "distilbert": dict(batch=2, seq=40, layers=2, d_model=128, heads=4, d_ff=256, vocab=300, max_pos=64),
    "lstm": dict(seq=12, batch=16, d_in=40, hidden=72),
}


def to_device_bytes(arr: np.ndarray, dtype: str) -> np.ndarray:
    """Host array in the element type the module declares (bf16 as uint16 bit patterns)."""
    if dtype == "bf16":
        return f32_to_bf16_bits(np.asarray(arr, np.float32))
    a = np.asarray(arr)
    return a if a.flags.c_contiguous else a.copy(order="C")
