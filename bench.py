"""Benchmark: jitted ResNet18 (CIFAR variant) train steps per second, batch 128, fp32, SGD momentum,
on one MI355X through the plugin's PJRT C API, plus fused-op HBM bandwidth.

Prints ONE JSON line.  `value` is steps/s with all inputs resident in HBM; `roofline` is the
convolution kernels' achieved fp32 matrix throughput (algorithmic flops / HIP-event time on the
compute stream, collected by the plugin and read back through PJRT_Executable_GetCostAnalysis);
`cpu_baseline` is the same train step on the host cores for a bounded sample: torch's CPU backend (oneDNN)
with the numpy oracle's rate next to it.
"""
import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for p in (str(ROOT), str(ROOT / "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)

import numpy as np  # noqa: E402

PEAK_HBM_GBS = 8000.0
PEAK_F32_MFMA_TFLOPS = 157.3


_FUSED_SPECS = {}     # name -> ((shape, dtype), ...) of the module's arguments


def fused_op_modules():
    """The fused-op bandwidth shapes (elementwise / reduce chains of the reference's benchmark configs,
    tests/configs/benchmark.py:14-45, and of the ResNet18 / DistilBERT programs)."""
    from jax_mps_amd.shlo.builder import Builder, gelu_tanh, layer_norm, softmax

    def mod(name, fn, *specs):
        b = Builder("fused_" + name)
        args = [b.arg(s, d) for s, d in specs]
        out = fn(b, *args)
        b.ret(*(out if isinstance(out, (list, tuple)) else [out]))
        _FUSED_SPECS[name] = specs
        return name, b.text()

    n = 10_000_000
    c = 64
    act = (128, 32, 32, c)
    return [
        mod("add_10M_f32", lambda b, x, y: b.add(x, y), ((n,), "f32"), ((n,), "f32")),
        mod("exp_10M_f32", lambda b, x: b.exp(x), ((n,), "f32")),
        mod("sum_10M_f32", lambda b, x: b.reduce_sum(x, [0]), ((n,), "f32")),
        mod("softmax_10000x1000_f32", lambda b, x: softmax(b, x, -1), ((10000, 1000), "f32")),
        mod("bn_apply_relu_128x32x32x64_f32",
            lambda b, x, s, t: b.maximum(b.add(b.mul(x, b.broadcast_in_dim(s, act, [3])), b.broadcast_in_dim(t, act, [3])), 0.0),
            (act, "f32"), ((c,), "f32"), ((c,), "f32")),
        mod("bn_stats_128x32x32x64_f32", lambda b, x: [b.reduce_sum(x, [0, 1, 2]), b.reduce_sum(b.mul(x, x), [0, 1, 2])], (act, "f32")),
        mod("layernorm_4096x768_bf16", lambda b, x, s, t: layer_norm(b, x, s, t, 1e-12), ((4096, 768), "bf16"), ((768,), "bf16"), ((768,), "bf16")),
        mod("bias_gelu_4096x3072_bf16", lambda b, x, t: gelu_tanh(b, b.add(x, b.broadcast_in_dim(t, (4096, 3072), [1]))), ((4096, 3072), "bf16"), ((3072,), "bf16")),
    ]


_FUSED_BYTES = {   # algorithmic bytes: distinct inputs + outputs, broadcast operands at their own size
    "add_10M_f32": 120e6, "exp_10M_f32": 80e6, "sum_10M_f32": 40e6, "softmax_10000x1000_f32": 80e6,
    "bn_apply_relu_128x32x32x64_f32": 2 * 128 * 32 * 32 * 64 * 4, "bn_stats_128x32x32x64_f32": 128 * 32 * 32 * 64 * 4,
    "layernorm_4096x768_bf16": 2 * 4096 * 768 * 2, "bias_gelu_4096x3072_bf16": 2 * 4096 * 3072 * 2,
}


LOSS_CHECK_STEPS = 3         # losses of the first steps are compared with the CPU baseline's (as many as it ran)
LOSS_CHECK_RTOL = 1e-4       # float32 losses after float32 accumulation in a different order on each side
FUSED_REPEAT = 64           # launches of each fused kernel between one pair of HIP events ...
FUSED_ROTATE_BYTES = 640e6  # ... cycling through copies of all its buffers that together hold this much: more than
                            # twice the 256 MB memory-side cache, so every launch reads its operands from HBM


def bench_fused_ops(client, iters=10):
    from jax_mps_amd import pjrt, runner
    out = []
    rng = np.random.default_rng(7)
    for name, text in fused_op_modules():
        ins = [rng.standard_normal(shape).astype(np.float32) for shape, _ in _FUSED_SPECS[name]]
        dts = [d for _, d in _FUSED_SPECS[name]]
        exe = client.compile_and_load(text)
        bufs = runner.upload(client, ins, dts)
        for _ in range(3):
            r = exe.execute(bufs)
        r[0].block_until_ready()
        t0 = time.perf_counter()
        for _ in range(iters):
            r = exe.execute(bufs)
        r[0].block_until_ready()
        dt = (time.perf_counter() - t0) / iters
        ca = exe.cost_analysis()
        # device time of the kernels themselves: HIP events around FUSED_REPEAT back-to-back launches of each
        # kernel of the program (the event pair alone costs a few microseconds, as much as a small kernel)
        kms = sum(v for k, v in ca.items() if k.endswith(".time_ms"))
        kcount = sum(v for k, v in ca.items() if k.endswith(".count"))
        steps = int(ca.get("steps", 0))
        passes = kcount / max(steps, 1)                       # how many times the whole program was timed
        dev = (kms / passes) * 1e-3 if kcount else dt
        gbs = _FUSED_BYTES[name] / dev / 1e9
        out.append({"op": name, "GB/s": round(gbs, 1), "frac_of_peak": round(gbs / PEAK_HBM_GBS, 4), "us": round(dev * 1e6, 2),
                    "launches": steps, "us_per_call_wall": round(dt * 1e6 / FUSED_REPEAT, 2)})
    return out


def _numpy_port_baseline(budget_s, batch):
    """The numpy oracle (float32 BLAS accumulation) on whole train steps of the benchmark workload."""
    from jax_mps_amd.programs import configs
    from shlo_oracle import Oracle
    p = configs.build_resnet18(batch=batch)
    o = Oracle(p.text, accum="f32")
    state = list(p.inputs)
    losses = []
    n, t0 = 0, time.perf_counter()
    while True:
        out = o.run(*state)
        for k, i in p.feedback.items():
            state[i] = out[k]
        losses.append(float(out[-1]))
        n += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s or n >= 50:
            break
    return {"value": round(n / dt, 5), "unit": "steps/s", "cores": os.cpu_count(), "kind": "port", "engine": "numpy", "losses": losses,
            "sample": f"{n} ResNet18 train step(s) at batch {batch} in {dt:.1f} s (numpy/BLAS float32 interpreter of the same module)"}


def _torch_cpu_baseline(budget_s, batch):
    """The same train step on torch's CPU backend (oneDNN convolutions, autograd; oracle/torch_resnet.py): the
    closest thing to a CPU framework backend on the benchmark machine, where no jax is installed.  None when
    torch is not importable."""
    try:
        import torch
        import torch_resnet
    except ImportError:
        return None
    from jax_mps_amd.programs import configs
    threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or (os.cpu_count() or 1))
    torch.set_num_threads(threads)
    p = configs.build_resnet18(batch=batch)
    ts = torch_resnet.TrainStep(p, configs.resnet18_param_specs(64, 10), 64)
    losses = [ts.step()]                      # first step: also warms the oneDNN primitive caches
    n, t0 = 0, time.perf_counter()
    while True:
        losses.append(ts.step())
        n += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s or n >= 200:
            break
    return {"value": round(n / dt, 4), "unit": "steps/s", "cores": threads, "kind": "port", "engine": f"torch-cpu {torch.__version__}",
            "losses": losses,
            "sample": f"{n} ResNet18 train step(s) at batch {batch} in {dt:.1f} s after one untimed step "
                      f"(torch CPU backend, float32, {threads} threads)"}


def cpu_baseline(budget_s=10.0, batch=128):
    """Host-CPU baseline on a bounded sample of the benchmark workload: the torch-CPU train step when torch is
    importable (the record's `numpy_port` then holds the numpy oracle's rate next to it), else the numpy oracle."""
    port = _numpy_port_baseline(budget_s, batch)
    tc = _torch_cpu_baseline(budget_s, batch)
    if tc is None:
        return port
    tc["numpy_port"] = {k: port[k] for k in ("value", "unit", "cores", "sample")}
    tc["numpy_losses"] = port["losses"]
    return tc


# HBM bytes per conv_igemm_f32 launch of this workload: rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE, each scaled by
# what the same counter reads for a 256 MiB copy (profiles/conv_igemm_f32_resnet18_b128_hbm_traffic.md).
CONV_HBM_BYTES_PER_LAUNCH = 117.5e6


# Algorithmic work of the other four benchmark programs (the figures the design notes quote): flops of the MFMA
# part for the GEMM-bound one, bytes for the HBM-bound one, launches for the two that are bound by launch latency.
def time_config(client, name, steps, warmup):
    from jax_mps_amd import runner
    from jax_mps_amd.programs import configs
    p = configs.ALL[name]()
    cp = runner.CompiledProgram(p, client)
    for _ in range(warmup):
        outs = cp.step()
    outs[-1].block_until_ready()
    t0 = time.perf_counter()
    for _ in range(steps):
        outs = cp.step()
    outs[-1].block_until_ready()
    dt = (time.perf_counter() - t0) / steps
    ca = cp.exe.cost_analysis()
    rec = {"config": name, "ms_per_step": round(dt * 1e3, 4), "steps_per_s": round(1 / dt, 1), "plan_steps": int(ca.get("steps", 0))}
    if name == "distilbert":
        rec["roofline"] = {"bound": "mfma", "unit": "TFLOP/s", "achieved": round(p.meta["flops"] / dt / 1e12, 1), "peak": 2500.0,
                           "frac": round(p.meta["flops"] / dt / 2.5e15, 4), "note": "whole forward pass (GEMM flops / wall time), bf16"}
    elif name == "embedding":
        nbytes = 50.4e6 + 178.8e6      # gather: indices + rows read + rows written; scatter-add: dense result + updates + indices
        rec["roofline"] = {"bound": "hbm", "unit": "GB/s", "achieved": round(nbytes / dt / 1e9, 1), "peak": PEAK_HBM_GBS,
                           "frac": round(nbytes / dt / 1e9 / PEAK_HBM_GBS, 4), "note": "gather + sorted scatter-add of 8192 Zipf rows"}
    else:
        rec["note"] = "launch-latency bound: us per plan step = %.2f" % (dt * 1e6 / max(rec["plan_steps"], 1)) if name == "mlp" else \
            "launch-latency bound: 2 x 100 loop iterations replayed from HIP graphs"
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-fused", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true")
    ap.add_argument("--config", default=None, help="time only this benchmark program (mlp, embedding, distilbert, lstm) and print its record")
    ap.add_argument("--fused-only", action="store_true", help="time only the fused-op bandwidth shapes and print their records")
    ap.add_argument("--one-stream", action="store_true",
                    help="keep every launch on one stream (no filter gradients on the second stream): kernel traces then show each kernel alone")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a 256 MiB device copy (kernel copy_vec16) a few times: the known-size reference for scaling FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build drives exactly one GPU (one PJRT device); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.one_stream:
        os.environ["MI355X_SECOND_STREAM"] = "0"
    os.environ.setdefault("MI355X_TIMING", "conv")     # HIP-event timing of the convolution launches only,
    every = int(os.environ.setdefault("MI355X_TIMING_EVERY", "10"))  # on one step in ten: the events cost ~5 us per launch, and a timed step runs every launch in order on one stream
    from jax_mps_amd import pjrt, runner
    from jax_mps_amd.programs import configs
    client = pjrt.get_client()
    if args.fused_only:
        os.environ["MI355X_TIMING"] = "all"
        os.environ["MI355X_TIMING_EVERY"] = "1"
        os.environ["MI355X_TIMING_REPEAT"] = str(FUSED_REPEAT)
        os.environ["MI355X_TIMING_ROTATE_BYTES"] = str(int(FUSED_ROTATE_BYTES))
        print(json.dumps({"fused_ops": bench_fused_ops(client)}))
        return
    if args.config:
        os.environ.pop("MI355X_TIMING", None)
        print(json.dumps(time_config(client, args.config, args.steps, args.warmup)))
        return
    p = configs.build_resnet18()
    cp = runner.CompiledProgram(p, client)
    first_losses = []                                  # loss buffers of the first steps, read back after the timed region
    for _ in range(args.warmup):
        outs = cp.step()
        if len(first_losses) < LOSS_CHECK_STEPS:
            first_losses.append(outs[-1])
    if args.warmup:
        outs[-1].block_until_ready()
    before = cp.exe.cost_analysis()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        outs = cp.step()
        if len(first_losses) < LOSS_CHECK_STEPS:
            first_losses.append(outs[-1])
    outs[-1].block_until_ready()
    dt = time.perf_counter() - t0
    after = cp.exe.cost_analysis()
    loss = float(runner.download(outs[-1]))
    assert np.isfinite(loss), loss
    first_losses = [float(runner.download(b)) for b in first_losses]
    conv_ms = after.get("conv.time_ms", 0.0) - before.get("conv.time_ms", 0.0)
    conv_n = after.get("conv.count", 0.0) - before.get("conv.count", 0.0)
    conv_flops = p.meta["step_flops"] - 6 * 128 * 512 * 10      # dense head is a GEMM step, not a convolution
    timed_steps = sum(1 for i in range(args.warmup, args.warmup + args.steps) if i % every == 0)   # execute calls the plugin sampled
    achieved = conv_flops * timed_steps / (conv_ms * 1e-3) / 1e12 if conv_ms > 0 else None
    line = {
        "metric": "jitted train steps/sec (ResNet18 b128, 1 MI355X); fused-op HBM GB/s vs peak",
        "value": round(args.steps / dt, 3), "unit": "steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt / args.steps * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "resnet18_cifar_train_step_batch128_fp32_sgd_momentum", "steps_per_launch_sequence": int(after.get("steps", 0)),
                   "final_loss": round(loss, 5)},
        "roofline": {"bound": "mfma", "kernel": "convolution (all launches of one step)", "achieved": None if achieved is None else round(achieved, 3),
                     "peak": PEAK_F32_MFMA_TFLOPS, "unit": "TFLOP/s", "frac": None if achieved is None else round(achieved / PEAK_F32_MFMA_TFLOPS, 4),
                     "traffic": CONV_HBM_BYTES_PER_LAUNCH, "launches_per_step": conv_n / max(timed_steps, 1), "timed_steps": timed_steps, "avg_launch_us": round(conv_ms * 1e3 / conv_n, 2) if conv_n else None,
                     "algorithmic_flops_per_step": conv_flops},
    }
    if args.copy_calibration:
        from jax_mps_amd.shlo.builder import Builder
        b = Builder("copy_calibration")
        x = b.arg((64 * 1024 * 1024,), "f32")
        b.ret(x)                                   # an argument returned as a result is one copy_vec16 launch of 256 MiB
        exe = client.compile_and_load(b.text())
        buf = client.buffer_from_pyval(np.zeros(64 * 1024 * 1024, np.float32))
        for _ in range(5):
            o = exe.execute([buf])
        o[0].block_until_ready()
        line["copy_calibration"] = {"kernel": "copy_vec16", "bytes_read": 256 * 1024 * 1024, "bytes_written": 256 * 1024 * 1024, "launches": 5}
    if not args.no_other_configs:
        os.environ.pop("MI355X_TIMING", None)      # timing events would keep counted loops off their captured graphs
        line["other_configs"] = [time_config(client, n, 50, 5) for n in ("mlp", "embedding", "distilbert", "lstm")]
    if not args.no_fused:
        os.environ["MI355X_TIMING"] = "all"
        os.environ["MI355X_TIMING_EVERY"] = "1"
        os.environ["MI355X_TIMING_REPEAT"] = str(FUSED_REPEAT)
        os.environ["MI355X_TIMING_ROTATE_BYTES"] = str(int(FUSED_ROTATE_BYTES))
        line["fused_ops"] = bench_fused_ops(client)
    ok = True
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline()
        line["speedup_vs_cpu_baseline"] = round(line["value"] / line["cpu_baseline"]["value"], 1)
        # the same steps from the same initial state on both sides: the losses must agree to float32 accumulation noise
        want = line["cpu_baseline"].pop("losses")[:len(first_losses)]
        others = line["cpu_baseline"].pop("numpy_losses", [])[:len(first_losses)]
        got = first_losses[:len(want)]
        rel = max(abs(g - w) / max(abs(w), 1e-30) for ws in (want, others) for g, w in zip(got, ws))
        ok = rel <= LOSS_CHECK_RTOL
        line["loss_check"] = {"steps": len(want), "gpu": [round(g, 6) for g in got], "cpu": [round(w, 6) for w in want],
                              "max_rel_diff": float("%.3g" % rel), "rtol": LOSS_CHECK_RTOL, "ok": ok}
    print(json.dumps(line))
    if not ok:
        print("bench.py: the GPU losses of the first steps differ from the CPU baseline's beyond the stated tolerance", file=sys.stderr)
        sys.exit(1)


if __name__ == "__main__":
    main()
