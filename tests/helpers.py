"""Shared helpers of the parity tests: one model spec builds both the oracle model and the
HIP-side layer list, so both sides see identical layers, parameters and data."""
from __future__ import annotations

from typing import Dict, List, Tuple

import numpy as np

from oracle import scanet_oracle as O

f32 = np.float32


def build_pair(spec: List[tuple], loss: str):
    """spec entries: ("dense", units, act[, reg, lam]) | ("conv", filters, kernel, strides, pad, act, bias)
    | ("pool", window, strides, pad[, "avg"]) | ("flatten",) | ("lstm", units[, bias[, seq[, regs]]]) | ("simple_rnn", units[, act[, bias[, seq[, regs]]]]) | ("batchnorm", momentum, epsilon[, "fused" or None[, regs]]) | ("activate", act) | ("bias", features)
    Returns (oracle Model, scanet3_amd layer composition, scanet3_amd loss)."""
    import scanet3_amd as S
    acts_o = {"identity": O.ACT_IDENTITY, "sigmoid": O.ACT_SIGMOID, "tanh": O.ACT_TANH, "relu": O.ACT_RELU,
              "softmax": O.ACT_SOFTMAX}
    acts_s = {"identity": S.Identity, "sigmoid": S.Sigmoid, "tanh": S.Tanh, "relu": S.ReLU(), "softmax": S.Softmax}
    pads_o = {"valid": O.PAD_VALID, "same": O.PAD_SAME}
    pads_s = {"valid": S.Valid, "same": S.Same}
    regs_o = {"none": O.REG_NONE, "l1": O.REG_L1, "l2": O.REG_L2}
    ol, sl = [], None

    def regs(entry, at):
        """Optional trailing tuple of (kind, lambda) pairs -> (oracle pairs, library Regularizations)."""
        given = entry[at] if len(entry) > at else ()
        o = [(regs_o[k], lam) for k, lam in given]
        s_ = [S.Zero if k == "none" else (S.L1(lam) if k == "l1" else S.L2(lam)) for k, lam in given]
        return o, s_

    def add(layer):
        nonlocal sl
        sl = layer if sl is None else (sl >> layer)

    for e in spec:
        k = e[0]
        if k == "dense":
            units, act = e[1], e[2]
            reg, lam = (e[3], e[4]) if len(e) > 3 else ("none", 0.0)
            ol.append(O.Dense(units, acts_o[act], reg=regs_o[reg], reg_lambda=lam))
            sreg = S.Zero if reg == "none" else (S.L1(lam) if reg == "l1" else S.L2(lam))
            add(S.Dense(units, acts_s[act], reg=sreg))
        elif k == "conv":
            _, filters, kernel, strides, pad, act, bias = e
            if isinstance(pad, tuple):      # explicit paddings (top, bottom, left, right)
                ol.append(O.Conv2D(filters, kernel, strides, O.PAD_EXPLICIT, acts_o[act], bias=bias, explicit=pad))
                add(S.Conv2D(filters, kernel, strides, S.Explicit(pad[0:2], pad[2:4]), acts_s[act], bias=bias))
            else:
                ol.append(O.Conv2D(filters, kernel, strides, pads_o[pad], acts_o[act], bias=bias))
                add(S.Conv2D(filters, kernel, strides, pads_s[pad], acts_s[act], bias=bias))
        elif k == "pool":
            _, window, strides, pad = e[:4]
            if len(e) > 4 and e[4] == "avg":    # the kernel function's Reduce.Avg, not the reference layer's behaviour
                ol.append(O.Pool2D(window, strides, pads_o[pad], reduce="Avg", as_reference_layer=False))
                add(S.Pool2D(window, strides, pads_s[pad], reduce=S.ReduceAvg, as_reference_layer=False))
            else:
                ol.append(O.Pool2D(window, strides, pads_o[pad]))
                add(S.Pool2D(window, strides, pads_s[pad]))
        elif k == "flatten":
            ol.append(O.Flatten())
            add(S.Flatten)
        elif k == "lstm":     # ("lstm", units[, bias[, return_sequence]])
            bias = e[2] if len(e) > 2 else True
            seq = e[3] if len(e) > 3 else False
            ro, rs = regs(e, 4)           # ((kernel), (recurrent), (bias)) regularizers
            names_o, names_s = ("kernel_reg", "recurrent_reg", "bias_reg"), ("kernelReg", "recurrentReg", "biasReg")
            ol.append(O.LSTM(e[1], bias=bias, return_sequence=seq, **dict(zip(names_o, ro))))
            add(S.LSTM(e[1], bias=bias, returnSequence=seq, **dict(zip(names_s, rs))))
        elif k == "simple_rnn":  # ("simple_rnn", units[, act[, bias[, return_sequence]]])
            act = e[2] if len(e) > 2 else "tanh"
            bias = e[3] if len(e) > 3 else True
            seq = e[4] if len(e) > 4 else False
            ro, rs = regs(e, 5)
            names_o, names_s = ("kernel_reg", "recurrent_reg", "bias_reg"), ("kernelReg", "recurrentReg", "biasReg")
            ol.append(O.SimpleRNN(e[1], acts_o[act], bias=bias, return_sequence=seq, **dict(zip(names_o, ro))))
            add(S.SimpleRNN(e[1], acts_s[act], bias=bias, returnSequence=seq, **dict(zip(names_s, rs))))
        elif k == "batchnorm":   # ("batchnorm", momentum, epsilon[, "fused"]): the generic form (fused = Some(false)) unless asked
            fused = len(e) > 3 and e[3] == "fused"   # rank-4 input only: the layer's default there (fused = None)
            ro, rs = regs(e, 4)           # ((beta regularizer),)
            ol.append(O.BatchNorm(e[1], e[2], fused=fused, **({"beta_reg": ro[0]} if ro else {})))
            add(S.BatchNorm(momentum=e[1], epsilon=e[2], fused=None if fused else False, **({"betaRegularizer": rs[0]} if rs else {})))
        elif k == "activate":
            ol.append([O.Layer("activate", activation=acts_o[e[1]])])
            add(S.Activate(acts_s[e[1]]))
        elif k == "bias":
            ol.append([O.Layer("bias", units=e[1])])
            add(S.Bias(e[1]))
        else:
            raise ValueError(k)
    losses_o = {"mse": O.LOSS_MSE, "bce": O.LOSS_BCE, "cce": O.LOSS_CCE}
    losses_s = {"mse": S.MeanSquaredError, "bce": S.BinaryCrossentropy, "cce": S.CategoricalCrossentropy}
    return O.Model(ol, losses_o[loss]), sl, losses_s[loss]


def glorot_params(model: O.Model, in_shape, rng: np.random.Generator, scale: float = 1.0) -> Dict[str, np.ndarray]:
    """Xavier-uniform weights, zero biases (forget-gate bias one), from the harness' own generator."""
    out = {}
    for path, shape in model.param_defs(in_shape):
        leaf = path.rsplit("/", 1)[-1]
        if leaf in O.BN_PARAMS:      # gamma and the moving variance start at one (BatchNorm.scala:68-71)
            out[path] = np.ones(shape, f32) if leaf in ("gamma", "moving_variance") else np.zeros(shape, f32)
        elif len(shape) == 1:
            out[path] = np.ones(shape, f32) if "forget/1/" in path else np.zeros(shape, f32)
        else:
            fan_in = int(np.prod(shape[:-1]))
            fan_out = shape[-1]
            lim = np.sqrt(6.0 / (fan_in + fan_out)) * scale
            out[path] = rng.uniform(-lim, lim, shape).astype(f32)
    return out


def one_hot(rng, rows, classes):
    return np.eye(classes, dtype=f32)[rng.integers(0, classes, rows)]


ATOL_FRACTION = 0.25


def rel_err(a: np.ndarray, b: np.ndarray, atol_fraction: float = ATOL_FRACTION) -> float:
    """Mixed elementwise error of `a` against the reference tensor `b`: max_i |a_i - b_i| / (|b_i| + f * max|b|).

    `rel_err(a, b) <= tol` therefore means |a_i - b_i| <= tol * |b_i| + f * tol * max|b| for every element: relative to
    the element itself, plus an absolute floor of a quarter of the tolerance at the tensor's scale (an entry that is
    small because its terms cancel carries the rounding error of those terms, not of its own size)."""
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    if a.size != b.size:
        raise AssertionError(f"size mismatch: {a.shape} vs {b.shape}")
    a = a.reshape(b.shape)
    if b.size == 0:
        return 0.0
    floor = atol_fraction * max(float(np.max(np.abs(b))), 1e-30)
    return float(np.max(np.abs(a - b) / (np.abs(b) + floor)))


def norm_err(a: np.ndarray, b: np.ndarray) -> float:
    """max |a-b| relative to the largest magnitude of the reference tensor b (a yardstick for noise estimates)."""
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    denom = max(float(np.max(np.abs(b))), 1e-30)
    return float(np.max(np.abs(a - b))) / denom


OPT_PAIRS = None


def optimizer_pairs():
    """[(name, oracle Algorithm, HIP optimizer descriptor)] with the reference's defaults."""
    import scanet3_amd as S
    return [
        ("sgd", O.SGD(), S.SGD()),
        ("sgd_momentum", O.SGD(0.01, 0.9), S.SGD(0.01, 0.9)),
        ("sgd_nesterov", O.SGD(0.01, 0.9, True), S.SGD(0.01, 0.9, True)),
        ("adagrad", O.AdaGrad(), S.AdaGrad()),
        ("adadelta", O.AdaDelta(), S.AdaDelta()),
        ("rmsprop", O.RMSProp(), S.RMSProp()),
        ("adam", O.Adam(), S.Adam()),
        ("nadam", O.Nadam(), S.Nadam()),
        ("adamax", O.Adamax(), S.Adamax()),
        ("amsgrad", O.AMSGrad(), S.AMSGrad()),
    ]
