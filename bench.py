#!/usr/bin/env python3
"""Benchmark of the scanet training step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload lenet|mlp|lstm|wide_mlp|optim] [--no-extras]

One "step" is one pass of the hot path over one batch of synthetic input that is already
resident in HBM when the timed region starts.  The headline value is train samples/s of the
LeNet-style CNN (the second configuration of the baseline list); with extras on (default) the
same JSON line also carries the other configurations: the small MLP, the LSTM, the wide bf16
MLP (GEMM roofline) and the 100 M-element optimizer / 8-replica averaging sweep (HBM roofline).

`roofline.achieved` = algorithmic work per launch of the dominant kernel divided by that
kernel's average launch duration, measured here with HIP events on the stream the kernels are
launched on (the library brackets every launch when profiling is enabled).
`cpu_baseline` times the CPU oracle (oracle/) on this box's host cores on a bounded sample.
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0          # MI355X HBM3E
PEAK_FP32_MFMA = 157.3         # TFLOP/s dense
PEAK_BF16_MFMA = 2500.0        # TFLOP/s dense
SEED = 20251125


def lenet_layers(S, pool_stride=1):
    ps = (pool_stride, pool_stride)
    return (S.Conv2D(32, activation=S.ReLU()) >> S.Pool2D(strides=ps) >> S.Conv2D(64, activation=S.ReLU())
            >> S.Pool2D(strides=ps) >> S.Flatten >> S.Dense(10, S.Softmax))


def glorot(rng, shape):
    fan_in, fan_out = int(np.prod(shape[:-1])), shape[-1]
    lim = np.sqrt(6.0 / (fan_in + fan_out))
    return rng.uniform(-lim, lim, shape).astype(np.float32)


def init_params(cm, rng):
    out = {}
    for path, shape, _ in cm.params:
        leaf = path.rsplit("/", 1)[-1]
        if leaf in ("beta", "gamma", "moving_mean", "moving_variance"):      # BatchNorm.scala:68-71
            out[path] = np.ones(shape, np.float32) if leaf in ("gamma", "moving_variance") else np.zeros(shape, np.float32)
        elif len(shape) == 1:
            out[path] = np.ones(shape, np.float32) if "forget/1/" in path else np.zeros(shape, np.float32)
        else:
            out[path] = glorot(rng, shape)
    return out


def one_hot(rng, rows, classes):
    return np.eye(classes, dtype=np.float32)[rng.integers(0, classes, rows)]


def kernel_table(ctx):
    rep = ctx.profile_report()
    return {k: {"total_ms": v[0], "launches": v[1], "avg_us": 1e3 * v[0] / max(v[1], 1)} for k, v in rep.items()}


def gemm_flops(name):
    """2 M N K of the bracketed shape in a kernel label (the implicit GEMM's own, possibly padded, shape)."""
    m = re.search(r"\[(\d+)x(\d+)x(\d+)\]", name)
    if not m:
        return None
    M, N, K = (int(v) for v in m.groups())
    return 2.0 * M * N * K


def _out_size(pad, size, k, s):
    from scanet3_amd import _lib as L
    return -(-size // s) if pad == L.PAD_SAME else -(-(size - k + 1) // s)


def model_work(layers, in_shape, batch):
    """Algorithmic flops of one training step and of its matrix kernels, from the layer list alone.

    Returns (flops per step, {kernel label: algorithmic flops per launch}).  Per layer (B = batch):
      Dense in->out ........ 2 B in out for each of forward, weight gradient and (not for the first layer) input gradient
      Conv2D ................ 2 B Ho Wo Cout kh kw Cin for each of the same three; the input-gradient kernel's label carries
                              the padded implicit GEMM B H W x Cin x kh kw Cout, which counts border taps that do not exist
      LSTM (T steps) ........ forward 2 B 4H (F + H) per step, hidden gradient 2 B H 4H per step but the first,
                              weight gradient 2 (F + H) 4H (T B), input gradient 2 B F 4H per step unless first layer
      SimpleRNN ............. the same with one gate
    Element-wise work (activations, pooling, softmax, optimizer) is not counted: the roofline here is the matrix one."""
    from scanet3_amd import _lib as L
    shape = tuple(in_shape)
    total, labels, first = 0.0, {}, True
    for l in layers:
        if l.kind == L.LAYER_DENSE:
            f = 2.0 * batch * shape[0] * l.units
            total += f * (2 if first else 3)
            labels[f"[{batch}x{l.units}x{shape[0]}]"] = f
            labels[f"[{shape[0]}x{l.units}x{batch}]"] = f
            labels[f"[{shape[0] + 1}x{l.units}x{batch}]"] = f            # with the bias-gradient row riding along
            labels[f"[{batch}x{shape[0]}x{l.units}]"] = f
            shape, first = (l.units,), False
        elif l.kind == L.LAYER_CONV2D:
            h, w, cin = shape
            ho, wo = _out_size(l.padding, h, l.kernel[0], l.strides[0]), _out_size(l.padding, w, l.kernel[1], l.strides[1])
            k = l.kernel[0] * l.kernel[1] * cin
            f = 2.0 * batch * ho * wo * l.units * k
            total += f * (2 if first else 3)
            labels[f"[{batch * ho * wo}x{l.units}x{k}]"] = f
            labels[f"[{k}x{l.units}x{batch * ho * wo}]"] = f
            labels[f"[{batch * h * w}x{cin}x{l.kernel[0] * l.kernel[1] * l.units}]"] = f
            shape, first = (ho, wo, l.units), False
        elif l.kind == L.LAYER_POOL2D:
            h, w, c = shape
            shape = (_out_size(l.padding, h, l.kernel[0], l.strides[0]), _out_size(l.padding, w, l.kernel[1], l.strides[1]), c)
        elif l.kind == L.LAYER_FLATTEN:
            shape = (int(np.prod(shape)),)
        elif l.kind in (L.LAYER_LSTM, L.LAYER_SIMPLE_RNN):
            T, F = shape
            H, G = l.units, (4 if l.kind == L.LAYER_LSTM else 1)
            fwd, dh, wg, dx = 2.0 * batch * G * H * (F + H), 2.0 * batch * H * G * H, 2.0 * (F + H) * G * H * T * batch, 2.0 * batch * F * G * H
            total += T * fwd + (T - 1) * dh + wg + (0 if first else T * dx)
            labels[f"[{batch}x{G * H}x{F + H}]"] = fwd
            labels[f"[{batch * T}x{G * H}x{F + H}]"] = T * fwd             # every forward step in one launch
            labels[f"[{batch}x{G * H}x{H}]"] = 2.0 * batch * G * H * H       # the recurrent half alone (input half hoisted)
            labels[f"[{batch * T}x{G * H}x{F}]"] = 2.0 * batch * T * G * H * F
            labels[f"[{batch}x{H}x{G * H}]"] = dh
            labels[f"[{batch * (T - 1)}x{H}x{G * H}]"] = (T - 1) * dh      # every backward product in one launch
            labels[f"[{batch}x{H}x{H}]"] = dh
            labels[f"[{F + H}x{G * H}x{T * batch}]"] = wg
            labels[f"[{F + H + 1}x{G * H}x{T * batch}]"] = wg
            shape, first = ((T, H) if l.return_sequence else (H,)), False
    return total, labels


def algorithmic_flops(name, labels):
    """Algorithmic flops of one launch of the kernel labelled `name` (None when it is not a matrix kernel)."""
    m = re.search(r"\[\d+x\d+x\d+\]", name)
    if not m:
        return None
    return labels.get(m.group(0), gemm_flops(name))


def run_model_workload(S, ctx, name, layers, loss, in_shape, batch, alg, make_xy, n_batches, steps, warmup, flags=0):
    """Times `steps` training steps (forward, loss, backward, update) cycling over n_batches resident batches."""
    rng = np.random.default_rng(SEED)
    cm = S.CompiledModel(ctx, [l.desc() for l in layers.layers], loss.kind, in_shape, batch, flags)
    rep = cm.replica(alg)
    rep.set_params(init_params(cm, rng))
    X, Y = make_xy(rng, batch * n_batches)
    Xb, Yb = ctx.to_device(X), ctx.to_device(Y)
    xs, ys = batch * cm.in_elems, batch * cm.out_elems
    it = 0

    def step():
        nonlocal it
        b = it % n_batches
        it += 1
        rep.step(Xb.offset(b * xs), Yb.offset(b * ys), it)

    for _ in range(warmup):
        step()
    ctx.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    ctx.sync()
    dt = time.perf_counter() - t0
    # the same steps fed from pinned HOST memory (batch i+1 copied while batch i trains): the PCIe-inclusive rate
    Xp, Yp = ctx.pinned_array(X.shape), ctx.pinned_array(Y.shape)
    Xp[...] = X
    Yp[...] = Y
    epochs = max(1, steps // n_batches)
    rep.train_epoch_host(Xp, Yp, batch, it, want_loss=False)
    t1 = time.perf_counter()
    for e in range(epochs):
        rep.train_epoch_host(Xp, Yp, batch, it + (e + 1) * n_batches, want_loss=False)
    dt_host = time.perf_counter() - t1
    it += (epochs + 1) * n_batches
    host_fed = {"samples_per_s": batch * n_batches * epochs / dt_host, "ms_per_step": 1e3 * dt_host / (epochs * n_batches),
                "bytes_per_step": 4 * batch * (cm.in_elems + cm.out_elems)}
    # second, instrumented pass: per-kernel durations from HIP events on the library's stream
    ctx.profile_reset()
    ctx.profile(True)
    prof_steps = max(3, min(steps, 20))
    for _ in range(prof_steps):
        step()
    ctx.profile(False)
    kernels = kernel_table(ctx)
    for k in kernels.values():
        k["per_step_us"] = 1e3 * k["total_ms"] / prof_steps
    last_loss = rep.loss(Xb.offset(0), Yb.offset(0))
    n_params = sum(int(np.prod(s)) for _, s, _ in cm.params)
    step_flops, labels = model_work(layers.layers, in_shape, batch)
    for kname, k in kernels.items():
        k["flops_per_launch"] = algorithmic_flops(kname, labels)
    rep.close()
    cm.close()
    Xb.free()
    Yb.free()
    return {"workload": name, "samples_per_s": batch * steps / dt, "ms_per_step": 1e3 * dt / steps, "steps": steps,
            "batch": batch, "params": n_params, "loss_after": last_loss, "kernels": kernels, "host_fed": host_fed,
            "flops_per_step": step_flops}


def dominant_gemm_roofline(kernels, peak_tflops, shared=()):
    """Roofline entry for the matrix-core kernel that takes the most time: ALGORITHMIC flops of one launch (model_work)
    divided by the launch's average duration (HIP events on the library's stream).  `shared`: label prefixes of launches
    that run beside another stream's kernels (their event times include that sharing): left out of the choice."""
    best = None
    for name, k in kernels.items():
        fl = k.get("flops_per_launch")
        if fl is None or any(name.startswith(p) for p in shared):
            continue
        if best is None or k["total_ms"] > best[1]["total_ms"]:
            best = (name, k, fl)
    if best is None:
        return None
    name, k, fl = best
    ach = fl / (k["avg_us"] * 1e-6) / 1e12
    return {"kernel": name, "bound": "mfma", "achieved": ach, "peak": peak_tflops, "unit": "TFLOP/s", "frac": ach / peak_tflops,
            "avg_launch_us": k["avg_us"], "flops_per_launch": fl, "traffic": measured_traffic(name)}


def whole_step_roofline(res, peak_tflops):
    """Every matrix flop the step has to do divided by the step's wall time (launch gaps, element-wise kernels and the
    optimizer all count against it)."""
    ach = res["flops_per_step"] / (res["ms_per_step"] * 1e-3) / 1e12
    return {"bound": "mfma", "achieved": ach, "peak": peak_tflops, "unit": "TFLOP/s", "frac": ach / peak_tflops,
            "flops_per_step": res["flops_per_step"], "ms_per_step": res["ms_per_step"]}


def bench_lenet(S, ctx, steps, warmup, pool_stride=1):
    return run_model_workload(
        S, ctx, f"LeNet-style CNN 28x28x1, batch 100, Adam 1e-3, fp32, pool stride {pool_stride}", lenet_layers(S, pool_stride),
        S.CategoricalCrossentropy, (28, 28, 1), 100, S.Adam(1e-3),
        lambda rng, n: (rng.random((n, 28, 28, 1), np.float32), one_hot(rng, n, 10)), 100, steps, warmup)


def bench_mlp(S, ctx, steps, warmup):
    return run_model_workload(
        S, ctx, "MLP 784->50 sigmoid->10 softmax, batch 1000, Adam 0.01, fp32", S.Dense(50, S.Sigmoid) >> S.Dense(10, S.Softmax),
        S.CategoricalCrossentropy, (784,), 1000, S.Adam(0.01),
        lambda rng, n: (rng.random((n, 784), np.float32), one_hot(rng, n, 10)), 30, steps, warmup)


def bench_lstm(S, ctx, steps, warmup):
    return run_model_workload(
        S, ctx, "LSTM(256)->Dense(1,tanh), batch 512, T 64, F 32, Adam, MSE, fp32", S.LSTM(256) >> S.Dense(1, S.Tanh),
        S.MeanSquaredError, (64, 32), 512, S.Adam(),
        lambda rng, n: (rng.standard_normal((n, 64, 32)).astype(np.float32), rng.uniform(-1, 1, (n, 1)).astype(np.float32)),
        4, steps, warmup)


def bench_cnn_bn(S, ctx, steps, warmup):
    """The CNN the reference trains on MNIST (test models/CNNSpec.scala:22-35), BatchNorm(fused = Some(true)) as there."""
    layers = (S.Conv2D(32, activation=S.ReLU()) >> S.BatchNorm(fused=True) >> S.Pool2D(strides=(2, 2))
              >> S.Conv2D(64, activation=S.ReLU()) >> S.Pool2D(strides=(2, 2)) >> S.Activate(S.ReLU()) >> S.Flatten
              >> S.Dense(64, S.ReLU()) >> S.Dense(10, S.Softmax))
    r = run_model_workload(
        S, ctx, "CNN with BatchNorm 28x28x1 (Conv32-BN-Pool/2-Conv64-Pool/2-Dense64-Dense10), batch 1000, Adam, fp32", layers,
        S.CategoricalCrossentropy, (28, 28, 1), 1000, S.Adam(),
        lambda rng, n: (rng.random((n, 28, 28, 1), np.float32), one_hot(rng, n, 10)), 4, steps, warmup)
    # the batch-norm kernels stream a [1000*26*26, 32] activation: bytes each pass has to move / its measured time
    elems = 1000 * 26 * 26 * 32
    passes = {"batchnorm_mean": 1, "batchnorm_variance": 1, "batchnorm_apply": 2, "batchnorm_gradient_sums": 2,
              "batchnorm_input_gradient": 3}
    r["batchnorm_hbm"] = {k: {"bytes": 4 * elems * p, "avg_us": r["kernels"][k]["avg_us"],
                              "GBps": 4 * elems * p / (r["kernels"][k]["avg_us"] * 1e-6) / 1e9,
                              "frac_of_peak": 4 * elems * p / (r["kernels"][k]["avg_us"] * 1e-6) / 1e9 / PEAK_HBM_GBS}
                          for k, p in passes.items() if k in r["kernels"]}
    return r


def bench_simple_rnn(S, ctx, steps, warmup):
    return run_model_workload(
        S, ctx, "SimpleRNN(256)->Dense(1,tanh), batch 512, T 64, F 32, Adam, MSE, fp32", S.SimpleRNN(256) >> S.Dense(1, S.Tanh),
        S.MeanSquaredError, (64, 32), 512, S.Adam(),
        lambda rng, n: (rng.standard_normal((n, 64, 32)).astype(np.float32), rng.uniform(-1, 1, (n, 1)).astype(np.float32)),
        4, steps, warmup)


def bench_wide_mlp(S, ctx, steps, warmup, bf16=True):
    from scanet3_amd import _lib as L
    return run_model_workload(
        S, ctx, "MLP 4096->4096 relu->4096 relu->1000 softmax, batch 8192, Adam 1e-3, " + ("bf16 MFMA / fp32 acc" if bf16 else "fp32"),
        S.Dense(4096, S.ReLU()) >> S.Dense(4096, S.ReLU()) >> S.Dense(1000, S.Softmax),
        S.CategoricalCrossentropy, (4096,), 8192, S.Adam(1e-3),
        lambda rng, n: (rng.standard_normal((n, 4096)).astype(np.float32), one_hot(rng, n, 1000)), 4, steps, warmup,
        flags=L.FLAG_GEMM_BF16 if bf16 else 0)


# HBM bytes per launch from `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` (two runs, each scaled by what the same counter
# reads for a one-input average = a plain copy of known size; summaries under profiles/).  A figure belongs to the kernel
# source it was measured on: every entry carries the SHA-1 of that source file, and `measured_traffic` returns None
# (JSON null) when the file has changed since.
CSRC = os.path.join(ROOT, "scanet3_amd", "csrc")
MEASURED_TRAFFIC = {
    # kernel label (or optimizer name): (bytes per launch, source file, sha1 of the file when measured)
    # rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE (one run each), KiB per dispatch, scaled by what the same counters read
    # for a plain copy of 400 MB (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0); the summaries are under profiles/
    "conv2d_forward[52900x64x288]": (22.3e6, "conv_ring_kernels.hip", "9ad35c60088e844b2f3f3f3c28cbad9fe520c83f"),
    "conv2d_input_gradient[62500x32x576]": (22.3e6, "conv_ring_kernels.hip", "9ad35c60088e844b2f3f3f3c28cbad9fe520c83f"),
    "conv2d_filter_gradient_tap_rows[288x64x52900]": (28.2e6, "conv_wgrad_kernels.hip", "86fd829667595ab42abdb3131518e7142ff50eba"),
    "gemm_bf16_256x256_bf16out[8192x4096x4096]": (474.8e6, "gemm_bf16.hip", "a403cf021cd20e0154725176d99f33018b440f94"),
    "gemm_bf16_256x256[4096x4096x8192]": (494.7e6, "gemm_bf16.hip", "a403cf021cd20e0154725176d99f33018b440f94"),
    "gemm_bf16_256x256_handover[8192x4096x4096]": (486.2e6, "gemm_bf16.hip", "a403cf021cd20e0154725176d99f33018b440f94"),
    "gemm_bf16_256x256_handover[8192x4096x1000]": (187.9e6, "gemm_bf16.hip", "a403cf021cd20e0154725176d99f33018b440f94"),
    "gemm_bf16_128x128[4096x1000x8192]": (214.9e6, "gemm_bf16.hip", "a403cf021cd20e0154725176d99f33018b440f94"),
    "gemm_bf16_128x256[8192x1000x4096]": (171.4e6, "gemm_bf16.hip", "a403cf021cd20e0154725176d99f33018b440f94"),
    "lstm_sequence_forward[32768x1024x288]": (249.9e6, "lstm_kernels.hip", "6d2dbe90ac02733993f507dc6304b11f1f3acfbd"),
    "lstm_sequence_backward_and_weight_gradient[512x1024x34560]": (520.3e6, "lstm_kernels.hip", "6d2dbe90ac02733993f507dc6304b11f1f3acfbd"),
    "rnn_sequence_forward[32768x256x288]": (74.8e6, "lstm_kernels.hip", "6d2dbe90ac02733993f507dc6304b11f1f3acfbd"),
    "rnn_sequence_backward_and_weight_gradient[512x256x34560]": (116.8e6, "lstm_kernels.hip", "6d2dbe90ac02733993f507dc6304b11f1f3acfbd"),
    "conv2d_forward[121000x64x288]": (53.3e6, "conv_ring_kernels.hip", "9ad35c60088e844b2f3f3f3c28cbad9fe520c83f"),
    "conv2d_input_gradient[169000x32x576]": (53.3e6, "conv_ring_kernels.hip", "9ad35c60088e844b2f3f3f3c28cbad9fe520c83f"),
    "conv2d_filter_gradient_tap_rows[288x64x121000]": (60.9e6, "conv_wgrad_kernels.hip", "86fd829667595ab42abdb3131518e7142ff50eba"),
    "mlp2_rows_forward_backward[1000x50x784]": (5.4e6, "mlp2_kernels.hip", "ebb1ef9fa9d2339b26bc579ca878dfb04138a92b"),
    "mlp2_weight_gradients_and_optimizer[784x50x1000]": (9.8e6, "mlp2_kernels.hip", "ebb1ef9fa9d2339b26bc579ca878dfb04138a92b"),
    "lstm_weight_gradient_rows[289x1024x32768]": (474.3e6, "lstm_wgrad_kernels.hip", "070ad64002f0fb967fbd759a0aabe0851ddfb7e3"),
    "lstm_weight_gradient_rows[289x256x32768]": (147.1e6, "lstm_wgrad_kernels.hip", "070ad64002f0fb967fbd759a0aabe0851ddfb7e3"),
    "gradient_sums_and_optimizer": (23.6e6, "optim_kernels.hip", "6b4919f35f7d5a085e20f3257517e6a0a096a7b4"),
    "adam": (2.800e9, "optim_kernels.hip", "6b4919f35f7d5a085e20f3257517e6a0a096a7b4"),
    "average": (0.900e9, "optim_kernels.hip", "6b4919f35f7d5a085e20f3257517e6a0a096a7b4"),
}


def _sha1(path):
    import hashlib
    try:
        with open(path, "rb") as f:
            return hashlib.sha1(f.read()).hexdigest()
    except OSError:
        return None


def measured_traffic(key):
    entry = MEASURED_TRAFFIC.get(key)
    if entry is None:
        return None
    nbytes, source, sha = entry
    return nbytes if _sha1(os.path.join(CSRC, source)) == sha else None


OPT_BYTES = {"sgd": 20, "adagrad": 20, "rmsprop": 20, "adadelta": 28, "adam": 28, "nadam": 28, "adamax": 28, "amsgrad": 36}


def bench_optim(S, ctx, steps, warmup, n=100_000_000, k=8, n_avg=25_000_000):
    """One fused update per optimizer over n float32 parameters, then the mean of k replicas of n_avg."""
    rng = np.random.default_rng(SEED + 5)
    block = 1 << 20
    reps = -(-n // block)
    w = np.tile((rng.standard_normal(block) * 0.02).astype(np.float32), reps)[:n]
    g = np.tile((rng.standard_normal(block) * 1e-3).astype(np.float32), reps)[:n]
    wb, gb = ctx.to_device(w), ctx.to_device(g)
    states = [ctx.alloc(n) for _ in range(3)]
    algs = [("sgd", S.SGD()), ("adagrad", S.AdaGrad()), ("adadelta", S.AdaDelta()), ("rmsprop", S.RMSProp()), ("adam", S.Adam()),
            ("nadam", S.Nadam()), ("adamax", S.Adamax()), ("amsgrad", S.AMSGrad())]
    out = {}
    ctx.profile_reset()
    for name, desc in algs:
        ns = {20: 1, 28: 2, 36: 3}[OPT_BYTES[name]]
        for s in states[:ns]:
            s.fill(desc.init_acc)
        wb.copy_from(w)
        it = 0
        for _ in range(warmup):          # warm-up steps also move the state off its degenerate initial value
            it += 1
            ctx.optimizer_update(desc, wb, gb, states[:ns], it)
        ctx.sync()
        ctx.profile(True)
        t0 = time.perf_counter()
        for _ in range(steps):
            it += 1
            ctx.optimizer_update(desc, wb, gb, states[:ns], it)
        ctx.sync()
        dt = time.perf_counter() - t0
        ctx.profile(False)
        kern = ctx.profile_report()[f"optimizer_{name}"]
        avg_s = kern[0] / kern[1] * 1e-3
        out[name] = {"bytes_per_elem": OPT_BYTES[name], "ms_per_step": 1e3 * dt / steps, "kernel_avg_us": avg_s * 1e6,
                     "GBps": OPT_BYTES[name] * n / avg_s / 1e9, "frac_of_peak": OPT_BYTES[name] * n / avg_s / 1e9 / PEAK_HBM_GBS,
                     "elems_per_s": n / avg_s}
    # a plain copy of the same 100 M elements (the mean of ONE input: n floats in, n out) is what this box's memory
    # system gives a streaming kernel; the update kernels are to be read against it as well as against the 8 TB/s peak
    for _ in range(warmup):
        ctx.average([wb], states[0])
    ctx.sync()
    ctx.profile_reset()
    ctx.profile(True)
    for _ in range(steps):
        ctx.average([wb], states[0])
    ctx.profile(False)
    kern = ctx.profile_report()["average_replicas"]
    avg_s = kern[0] / kern[1] * 1e-3
    out["copy_100M"] = {"n": n, "bytes_per_elem": 8, "kernel_avg_us": avg_s * 1e6, "GBps": 8 * n / avg_s / 1e9,
                        "frac_of_peak": 8 * n / avg_s / 1e9 / PEAK_HBM_GBS}
    for name, _ in algs:
        out[name]["frac_of_copy"] = out[name]["GBps"] / out["copy_100M"]["GBps"]
    ctx.profile_reset()
    for b in states + [wb, gb]:
        b.free()
    # averaging
    base = (rng.standard_normal(block) * 0.02).astype(np.float32)
    reps_bufs = []
    for r in range(k):
        reps_bufs.append(ctx.to_device(np.tile(np.roll(base, r * 17), -(-n_avg // block))[:n_avg]))
    dst = ctx.alloc(n_avg)
    for _ in range(warmup):
        ctx.average(reps_bufs, dst)
    ctx.sync()
    ctx.profile_reset()
    ctx.profile(True)
    t0 = time.perf_counter()
    for _ in range(steps):
        ctx.average(reps_bufs, dst)
    ctx.sync()
    dt = time.perf_counter() - t0
    ctx.profile(False)
    kern = ctx.profile_report()["average_replicas"]
    avg_s = kern[0] / kern[1] * 1e-3
    bpe = 4 * (k + 1)
    out["average"] = {"k": k, "n": n_avg, "bytes_per_elem": bpe, "ms_per_step": 1e3 * dt / steps, "kernel_avg_us": avg_s * 1e6,
                      "GBps": bpe * n_avg / avg_s / 1e9, "frac_of_peak": bpe * n_avg / avg_s / 1e9 / PEAK_HBM_GBS}
    # mean of ONE input = a plain copy of known size (n_avg floats in, n_avg out): the reference point that
    # hardware byte counters of the kernels above are scaled by
    ctx.profile_reset()
    ctx.profile(True)
    for _ in range(steps):
        ctx.average(reps_bufs[:1], dst)
    ctx.profile(False)
    kern = ctx.profile_report()["average_replicas"]
    avg_s = kern[0] / kern[1] * 1e-3
    out["copy_k1"] = {"k": 1, "n": n_avg, "bytes_per_elem": 8, "kernel_avg_us": avg_s * 1e6, "GBps": 8 * n_avg / avg_s / 1e9,
                      "frac_of_peak": 8 * n_avg / avg_s / 1e9 / PEAK_HBM_GBS}
    for b in reps_bufs + [dst]:
        b.free()
    # seeded initializer draws (TensorFlow-compatible Philox streams): 4 bytes written per element
    from scanet3_amd import _lib as L
    rbuf = ctx.alloc(n)
    for label, dist in (("random_uniform", L.RANDOM_UNIFORM), ("random_normal", L.RANDOM_NORMAL),
                        ("random_truncated_normal", L.RANDOM_TRUNCATED_NORMAL)):
        ctx.random_fill(rbuf, dist, 7)
        ctx.sync()
        ctx.profile_reset()
        ctx.profile(True)
        for _ in range(steps):
            ctx.random_fill(rbuf, dist, 7, 0.1, -0.05)
        ctx.profile(False)
        kern = ctx.profile_report()[label]
        avg_s = kern[0] / kern[1] * 1e-3
        out[label] = {"n": n, "bytes_per_elem": 4, "kernel_avg_us": avg_s * 1e6, "GBps": 4 * n / avg_s / 1e9,
                      "frac_of_peak": 4 * n / avg_s / 1e9 / PEAK_HBM_GBS, "elems_per_s": n / avg_s}
    rbuf.free()
    return {"workload": f"fused optimizer updates over {n} fp32 params + average of {k} x {n_avg}", "n": n, "results": out}


def cpu_baseline_lenet(pool_stride=1, budget_s=15.0):
    """The oracle's LeNet step on the host cores; bounded to about `budget_s` seconds."""
    from oracle import scanet_oracle as O
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = os.cpu_count() or 1
    ps = (pool_stride, pool_stride)
    model = O.Model([O.Conv2D(32, activation=O.ACT_RELU), O.Pool2D(strides=ps), O.Conv2D(64, activation=O.ACT_RELU),
                     O.Pool2D(strides=ps), O.Flatten(), O.Dense(10, O.ACT_SOFTMAX)], O.LOSS_CCE)
    rng = np.random.default_rng(SEED)
    batch = 100
    params = {p: (glorot(rng, s) if len(s) > 1 else np.zeros(s, np.float32)) for p, s in model.param_defs((batch, 28, 28, 1))}
    alg = O.Adam(1e-3)
    state = O.init_opt_state(alg, params)
    x = rng.random((batch, 28, 28, 1), np.float32)
    y = one_hot(rng, batch, 10)
    params, state, _, _ = O.train_step(model, alg, x, y, params, state, 1)      # warm-up
    n, t0 = 0, time.perf_counter()
    while True:
        n += 1
        params, state, _, _ = O.train_step(model, alg, x, y, params, state, n + 1)
        if time.perf_counter() - t0 > budget_s or n >= 200:
            break
    dt = time.perf_counter() - t0
    out = {"value": batch * n / dt, "unit": "samples/s", "cores": int(threads), "kind": "port",
           "sample": f"{n} LeNet training steps of batch {batch} (numpy oracle, BLAS threads = {threads})"}
    out["torch_cpu"] = torch_cpu_lenet(pool_stride, budget_s=10.0)
    return out


def torch_cpu_lenet(pool_stride=1, budget_s=10.0):
    """The same LeNet training step through torch on the host cores (oneDNN convolutions, autograd, torch's Adam): a
    framework-grade CPU figure beside the numpy port.  NOT the reference (that is TensorFlow-Java, which this image
    does not hold) and not op-order faithful; torch is imported here and nowhere else.  None if torch cannot be imported."""
    try:
        import torch
        import torch.nn.functional as F
    except Exception:
        return None
    torch.manual_seed(SEED)
    batch = 100
    w1 = torch.nn.Parameter(torch.empty(32, 1, 3, 3).uniform_(-0.1, 0.1))
    w2 = torch.nn.Parameter(torch.empty(64, 32, 3, 3).uniform_(-0.05, 0.05))
    side = 28 - 2
    side = (side - 2) // pool_stride + 1
    side = side - 2
    side = (side - 2) // pool_stride + 1
    w3 = torch.nn.Parameter(torch.empty(side * side * 64, 10).uniform_(-0.01, 0.01))
    b3 = torch.nn.Parameter(torch.zeros(10))
    opt = torch.optim.Adam([w1, w2, w3, b3], lr=1e-3, eps=1e-7)
    x = torch.rand(batch, 1, 28, 28)
    y = torch.randint(0, 10, (batch,))

    def step():
        opt.zero_grad(set_to_none=True)
        h = F.max_pool2d(F.relu(F.conv2d(x, w1)), 2, pool_stride)
        h = F.max_pool2d(F.relu(F.conv2d(h, w2)), 2, pool_stride)
        loss = F.cross_entropy(h.flatten(1) @ w3 + b3, y)
        loss.backward()
        opt.step()

    for _ in range(3):
        step()
    n, t0 = 0, time.perf_counter()
    while True:
        n += 1
        step()
        if time.perf_counter() - t0 > budget_s or n >= 2000:
            break
    dt = time.perf_counter() - t0
    return {"value": batch * n / dt, "unit": "samples/s", "cores": int(torch.get_num_threads()), "kind": "torch-cpu, not the reference",
            "sample": f"{n} LeNet training steps of batch {batch} (torch {torch.__version__} on CPU: conv2d / max_pool2d / autograd / Adam)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="lenet", choices=["lenet", "mlp", "lstm", "wide_mlp", "optim", "cnn_bn", "simple_rnn"])
    ap.add_argument("--pool-stride", type=int, default=1, help="LeNet pool stride (reference default 1)")
    ap.add_argument("--no-extras", action="store_true", help="skip the other configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import scanet3_amd as S
    ctx = S.Context(0)
    dev_name, hbm, cu = ctx.device_info()
    steps, warmup = args.steps, args.warmup

    def run(which, st, wu):
        if which == "lenet":
            return bench_lenet(S, ctx, st, wu, args.pool_stride)
        if which == "mlp":
            return bench_mlp(S, ctx, st, wu)
        if which == "lstm":
            return bench_lstm(S, ctx, st, wu)
        if which == "wide_mlp":
            return bench_wide_mlp(S, ctx, st, wu)
        if which == "cnn_bn":
            return bench_cnn_bn(S, ctx, st, wu)
        if which == "simple_rnn":
            return bench_simple_rnn(S, ctx, st, wu)
        return bench_optim(S, ctx, st, wu)

    main_res = run(args.workload, steps, warmup)
    line = {"metric": "train samples/sec on 1 GPU", "unit": "samples/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "data": "synthetic", "dtype": "f32",
            "device": dev_name}
    if args.workload == "optim":
        adam = main_res["results"]["adam"]
        line.update({"metric": "fused Adam update, elements/s over 100M fp32 params", "unit": "elements/s",
                     "value": adam["elems_per_s"], "ms_per_step": adam["ms_per_step"],
                     "config": {"workload": main_res["workload"]},
                     "roofline": {"kernel": "optimizer_adam", "bound": "hbm", "achieved": adam["GBps"], "peak": PEAK_HBM_GBS,
                                  "unit": "GB/s", "frac": adam["frac_of_peak"], "traffic": measured_traffic("adam")},
                     "optimizers": main_res["results"]})
    else:
        peak = PEAK_BF16_MFMA if args.workload == "wide_mlp" else PEAK_FP32_MFMA
        line.update({"value": main_res["samples_per_s"], "ms_per_step": main_res["ms_per_step"],
                     "dtype": "bf16" if args.workload == "wide_mlp" else "f32",
                     "config": {"workload": main_res["workload"], "batch": main_res["batch"], "params": main_res["params"]},
                     "roofline": dominant_gemm_roofline(main_res["kernels"], peak, ("gemm_bf16_256x256[",) if args.workload == "wide_mlp" else ()),
                     "roofline_whole_step": whole_step_roofline(main_res, peak),
                     "host_fed": main_res["host_fed"],
                     "kernels_us_per_step": {k: round(v["per_step_us"], 2) for k, v in
                                             sorted(main_res["kernels"].items(), key=lambda kv: -kv[1]["total_ms"])[:12]}})
        if "batchnorm_hbm" in main_res:
            line["batchnorm_hbm"] = main_res["batchnorm_hbm"]
    if not args.no_extras:
        extras = {}
        for which, st, wu in (("mlp", 100, 10), ("lstm", 50, 5), ("wide_mlp", 20, 3), ("optim", 10, 3), ("lenet", 50, 5),
                               ("cnn_bn", 30, 3), ("simple_rnn", 30, 3)):
            if which == args.workload:
                continue
            try:
                r = run(which, st, wu)
            except Exception as e:        # an extra must never hide the headline number
                extras[which] = {"error": str(e)}
                continue
            if which == "optim":
                extras[which] = r
            else:
                peak = PEAK_BF16_MFMA if which == "wide_mlp" else PEAK_FP32_MFMA
                extras[which] = {"workload": r["workload"], "samples_per_s": r["samples_per_s"], "ms_per_step": r["ms_per_step"],
                                 "steps": r["steps"], "loss_after": r["loss_after"], "host_fed": r["host_fed"],
                                 # (the bf16 MLP's weight-gradient products share the chip with the optimizer launches of the layers above)
                                 "roofline": dominant_gemm_roofline(r["kernels"], peak, ("gemm_bf16_256x256[",) if which == "wide_mlp" else ()),
                                 "roofline_whole_step": whole_step_roofline(r, peak),
                                 "kernels_us_per_step": {k: round(v["per_step_us"], 2) for k, v in
                                                         sorted(r["kernels"].items(), key=lambda kv: -kv[1]["total_ms"])[:8]}}
                if "batchnorm_hbm" in r:
                    extras[which]["batchnorm_hbm"] = r["batchnorm_hbm"]
        line["other_configs"] = extras
        # the two rooflines the memory-bound and the GEMM-bound configurations are judged on
        rl = {}
        opt = extras.get("optim") or (main_res if args.workload == "optim" else None)
        if opt and "results" in opt:
            for k in ("adam", "average"):
                v = opt["results"][k]
                rl["optimizer_adam_100M" if k == "adam" else "average_8x25M"] = {
                    "bound": "hbm", "achieved": v["GBps"], "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": v["frac_of_peak"],
                    "traffic": measured_traffic(k)}
        wide = extras.get("wide_mlp")
        if wide and wide.get("roofline"):
            rl["wide_mlp_gemm_bf16"] = wide["roofline"]
        line["rooflines"] = rl
    ctx.close()
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline_lenet(args.pool_stride)
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
