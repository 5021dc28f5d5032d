"""The ResNet18 (CIFAR variant) SGD-momentum train step of the benchmark restated on torch's CPU backend
(oneDNN convolutions, autograd): test and benchmark infrastructure only, never part of the product path.

Two uses: (1) in float64 it pins the StableHLO emitter's program and the numpy oracle against an independent
autograd (tests/test_oracle_pins.py); (2) in float32 it is the host-CPU baseline `bench.py` times next to the GPU
(the numpy interpreter is a poor stand-in for a CPU framework; torch-CPU is the closest thing to JAX's CPU backend
that exists on the benchmark machine).  Model structure: the reference's examples/resnet/model.py:6-163 (3x3 stem,
no max-pool, stages 64/128/256/512 of two basic blocks, projection shortcut where the shape changes, flax-style
batch norm with batch statistics E[x], E[x^2] and running averages at momentum 0.9)."""
from __future__ import annotations

import torch
import torch.nn.functional as F


def _conv(w_hwio, h, stride):
    w = w_hwio.permute(3, 2, 0, 1)
    k = w.shape[2]
    n_in = h.shape[2]
    out = -(-n_in // stride)
    tot = max((out - 1) * stride + k - n_in, 0)          # SAME padding as flax computes it
    lo, hi = tot // 2, tot - tot // 2
    if lo == hi:
        return F.conv2d(h, w, stride=stride, padding=lo)
    return F.conv2d(F.pad(h, (lo, hi, lo, hi)), w, stride=stride)


def forward(P, x_nchw, y, width, stats_out=None, eps=1e-5):
    """Loss of the train-mode network.  `P` maps parameter names (programs/configs.py::resnet18_param_specs) to
    tensors; `stats_out`, when given, receives (name, batch mean, batch variance) per batch-norm layer."""
    def bn(name, h):
        m = h.mean((0, 2, 3))
        v = torch.clamp((h * h).mean((0, 2, 3)) - m * m, min=0)
        if stats_out is not None:
            stats_out.append((name, m.detach(), v.detach()))
        mul = torch.rsqrt(v + eps) * P[name + ".scale"]
        return (h - m[None, :, None, None]) * mul[None, :, None, None] + P[name + ".bias"][None, :, None, None]

    h = torch.relu(bn("bn_init", _conv(P["conv_init.kernel"], x_nchw, 1)))
    cin = width
    for stage, mult in enumerate((1, 2, 4, 8), 1):
        cout = width * mult
        for blk in (1, 2):
            stride = 2 if (stage > 1 and blk == 1) else 1
            pn = f"stage{stage}_block{blk}"
            r = h
            yv = torch.relu(bn(pn + ".bn1", _conv(P[pn + ".conv1.kernel"], h, stride)))
            yv = bn(pn + ".bn2", _conv(P[pn + ".conv2.kernel"], yv, 1))
            if cin != cout or stride != 1:
                r = bn(pn + ".bn_proj", _conv(P[pn + ".conv_proj.kernel"], r, stride))
            h = torch.relu(r + yv)
            cin = cout
    return F.cross_entropy(h.mean((2, 3)) @ P["dense.kernel"] + P["dense.bias"], y)


class TrainStep:
    """State and step of the benchmark's train program (`configs.build_resnet18`) on torch-CPU."""

    def __init__(self, program, specs, width, dtype=torch.float32, lr=0.1, momentum=0.9):
        n = len(specs)
        self.names = [nm for nm, _, _ in specs]
        self.width, self.lr, self.momentum = width, lr, momentum
        self.P = {nm: torch.tensor(a, dtype=dtype, requires_grad=True) for nm, a in zip(self.names, program.inputs[:n])}
        self.M = {nm: torch.zeros_like(p) for nm, p in self.P.items()}
        n_stats = len(program.inputs) - 2 - 2 * n
        self.running = [torch.tensor(a, dtype=dtype) for a in program.inputs[n:n + n_stats]]
        self.x = torch.tensor(program.inputs[-2], dtype=dtype).permute(0, 3, 1, 2).contiguous()
        self.y = torch.tensor(program.inputs[-1]).long()

    def step(self) -> float:
        stats = []
        loss = forward(self.P, self.x, self.y, self.width, stats)
        grads = torch.autograd.grad(loss, [self.P[nm] for nm in self.names])
        with torch.no_grad():
            for nm, g in zip(self.names, grads):
                self.M[nm].mul_(self.momentum).add_(g)
                self.P[nm].sub_(self.lr * self.M[nm])
            for k, (_, m, v) in enumerate(stats):
                self.running[2 * k].mul_(0.9).add_(0.1 * m)
                self.running[2 * k + 1].mul_(0.9).add_(0.1 * v)
        return float(loss.detach())
