"""CPU oracle for scanet's compiled training/inference step (TEST INFRASTRUCTURE ONLY).

This module is a numpy restatement, op for op and in the reference's evaluation
order, of the graph that scanet3 lowers to TensorFlow for one training step:
layers, losses, hand-derived backward passes that follow the reference's
``localGrad`` rules, the eight optimizer algorithms, the per-partition step
loop and the parameter averaging.  It is the checker for the HIP library and
nothing else: only tests, the smoke entry and the benchmark's CPU-baseline leg
import it.  The shipped package never does.

Every function works in the dtype of its inputs (float32 on the hot path,
float64 when a test wants a high-precision check of the mathematics).

What pins each part (see tests/test_oracle_golden.py):
  * dense / bias / sigmoid forward, BinaryCrossentropy gradients ... reference goldens
  * softmax rows, tanh, relu, exp, log, sigmoid points ........... reference goldens
  * conv2d (same/valid/explicit, stride 1/2), both conv grads ..... reference goldens + brute force + torch
  * max pool (same/valid, stride 1/2), max-pool grad with ties .... reference goldens + brute force
  * average pool and its gradient (padding cells not counted) ..... reference goldens + brute force + numeric gradient
  * SimpleRNN and LSTM forward ................................... reference goldens
  * LSTM / conv / pool / softmax+CCE backward .................... float64 numerical gradients + torch autograd
  * BatchNorm (generic form): training output, next moving
    statistics, frozen output ................................... reference goldens
  * BatchNorm backward through the batch statistics .............. float64 numerical gradients (rank 2 and rank 4)
  * FusedBatchNormV3 / GradV3 as TensorFlow defines them .......... the generic form's goldens (same y), numpy's unbiased
    variance, float64 numerical gradients when handed the true statistics
  * decayingAvg / boost / sqrtZeroSafe ........................... reference goldens
  * optimizer trajectories ....................................... reference convergence thresholds + closed forms
Parity unpinned (only running TensorFlow-CPU could pin them): last-ulp
behaviour of TF's Exp/Tanh/Sigmoid/Log/Pow, summation order inside TF's
MatMul/Conv2D/Sum, averaging of more than one replica and the multi-partition
iteration counter (no reference test runs with more than one partition), and
the WIRING of the FusedBatchNormV3 branch BatchNorm takes for rank-4 input
unless `fused = Some(false)` (`batchnorm_fused_forward/backward`): which of
the op's outputs reach the moving statistics and the gradient op is read off
math/nn/AllKernels.scala:437-448, and what TensorFlow's CPU kernel puts into
those outputs is restated from its published source (TF 2.10,
core/kernels/fused_batch_norm_op.cc); no reference test holds values for it.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

F32 = np.float32

# --------------------------------------------------------------------------- #
# scalar helpers (src/main/scala/scanet/math/alg/AllKernels.scala:491-549)
# --------------------------------------------------------------------------- #


def _c(x, like):
    """A constant cast to the dtype of `like` (reference: `x.const.cast[T]`)."""
    return np.asarray(like).dtype.type(x)


def pow_scalar(base, exponent, dtype=F32):
    """`Pow(rate, iter.cast[Float])` on scalars, rounded once to `dtype`.

    AllKernels.scala:546-549 (`boost`).  Evaluated in float64 and rounded, which
    is the correctly rounded float32 power.
    """
    return np.dtype(dtype).type(float(np.dtype(dtype).type(base)) ** float(exponent))


def sqr(x):
    """`sqr = Pow(x, 2)` (AllKernels.scala:648); x*x is the correctly rounded value."""
    return x * x


def decaying_avg(avg, nxt, decay):
    """`decay * avg + (1 - decay) * next` (AllKernels.scala:541-544)."""
    d = _c(decay, avg)
    one = _c(1.0, avg)
    return d * avg + (one - d) * nxt


def boost(x, rate, it):
    """`x / (1 - rate^iter)` (AllKernels.scala:546-549)."""
    dt = np.asarray(x).dtype
    return x / (dt.type(1.0) - pow_scalar(rate, it, dt))


def sqrt_zero_safe(x, eps):
    """`sqrt(x + eps)` (AllKernels.scala:491-492)."""
    return np.sqrt(x + _c(eps, x))


def to_bf16(x):
    """float32 values rounded to the nearest bfloat16 (ties to even), returned as float32.

    Used only by the bf16 Dense mode, which has no counterpart in the reference (its arithmetic is
    float32 throughout): the HIP library's bf16 GEMMs are checked against float32 products of
    operands rounded this way."""
    a = np.ascontiguousarray(x, dtype=np.float32)
    u = a.view(np.uint32)
    r = ((u >> 16) & 1) + np.uint32(0x7FFF)
    return ((u + r) & np.uint32(0xFFFF0000)).view(np.float32)


def rint(x):
    """TF `Rint`: round half to even (AllKernels.scala:339-345)."""
    return np.rint(x)


# --------------------------------------------------------------------------- #
# activations (models/Activation.scala:32-83; grads math/alg/AllKernels.scala)
# --------------------------------------------------------------------------- #


def sigmoid(x):
    one = _c(1.0, x)
    return one / (one + np.exp(-x))


def sigmoid_grad(x, dy):
    """AllKernels.scala:397-404: recomputes s, grad = s*(1-s), then * parent."""
    s = sigmoid(x)
    return (s * (_c(1.0, x) - s)) * dy


def tanh_grad(x, dy):
    """AllKernels.scala:414-420: (1 - tanh(x)^2) * parent."""
    return (_c(1.0, x) - sqr(np.tanh(x))) * dy


def relu(x, threshold=0.0):
    """Activation.scala:79-82: Maximum(threshold, x)."""
    return np.maximum(_c(threshold, x), x)


def relu_grad(x, dy, threshold=0.0):
    """Maximum's grad to its right input: (left < right) strict (AllKernels.scala:297-302)."""
    return (_c(threshold, x) < x).astype(x.dtype) * dy


def softmax(x):
    """Activation.scala:63-69: e = exp(x); e / sum(e, axis 1).  No max subtraction."""
    e = np.exp(x)
    s = e.sum(axis=1, dtype=x.dtype)
    return e / s[:, None]


def softmax_grad(x, dp):
    """Chain of Div / Sum / Exp local gradients (AllKernels.scala:196-201,214-227,237-244)."""
    e = np.exp(x)
    s = e.sum(axis=1, dtype=x.dtype)[:, None]
    de_div = dp / s
    ds = ((-e * dp) / sqr(s)).sum(axis=1, dtype=x.dtype)[:, None]
    de = de_div + ds            # Sum's grad broadcasts ds over the row
    return e * de


ACT_IDENTITY, ACT_SIGMOID, ACT_TANH, ACT_RELU, ACT_SOFTMAX = 0, 1, 2, 3, 4


def activate(kind, x, param=0.0):
    if kind == ACT_IDENTITY:
        return x
    if kind == ACT_SIGMOID:
        return sigmoid(x)
    if kind == ACT_TANH:
        return np.tanh(x)
    if kind == ACT_RELU:
        return relu(x, param)
    if kind == ACT_SOFTMAX:
        return softmax(x)
    raise ValueError(f"unknown activation {kind}")


def activate_grad(kind, x, dy, param=0.0):
    if kind == ACT_IDENTITY:
        return dy
    if kind == ACT_SIGMOID:
        return sigmoid_grad(x, dy)
    if kind == ACT_TANH:
        return tanh_grad(x, dy)
    if kind == ACT_RELU:
        return relu_grad(x, dy, param)
    if kind == ACT_SOFTMAX:
        return softmax_grad(x, dy)
    raise ValueError(f"unknown activation {kind}")


# --------------------------------------------------------------------------- #
# losses (models/Loss.scala:18-57)
# --------------------------------------------------------------------------- #

LOSS_IDENTITY, LOSS_MSE, LOSS_BCE, LOSS_CCE = 0, 1, 2, 3


def loss_value(kind, p, y):
    dt = p.dtype
    if kind == LOSS_IDENTITY:
        return p
    if kind == LOSS_MSE:                      # Loss.scala:18-24
        return sqr(p - y).mean(dtype=dt)
    if kind == LOSS_BCE:                      # Loss.scala:26-42
        one, eps = dt.type(1.0), dt.type(1e-8)
        left = y * np.log(p + eps)
        right = (one - y) * np.log(one - (p - eps))
        return (-left - right).mean(dtype=dt)
    if kind == LOSS_CCE:                      # Loss.scala:44-57
        eps = dt.type(1e-8)
        num = dt.type(y.shape[0])
        return -((y * np.log(p + eps)).sum(dtype=dt)) / num
    raise ValueError(f"unknown loss {kind}")


def loss_grad(kind, p, y):
    """d loss / d predicted, following the reference's localGrad chain."""
    dt = p.dtype
    if kind == LOSS_MSE:
        # Mean: ones/size ; Pow: (d^(2-1) * 2) * parent ; Minus: +parent
        size = dt.type(p.size)
        g = np.ones_like(p) * dt.type(1.0) / size
        d = p - y
        return (d * dt.type(2.0)) * g
    if kind == LOSS_BCE:
        one, eps = dt.type(1.0), dt.type(1e-8)
        size = dt.type(p.size)
        g = np.ones_like(p) * dt.type(1.0) / size
        # (left.negate - right): d left = -g ; d right = -g
        # left = y * log(p+eps): d log = y * (-g); d p = that / (p+eps)
        dp_left = (y * (-g)) / (p + eps)
        # right = (1-y) * log(1 - (p-eps)): d log = (1-y)*(-g); d(1-(p-eps)) = that/(1-(p-eps)); d p = -that
        dp_right = -(((one - y) * (-g)) / (one - (p - eps)))
        return dp_left + dp_right
    if kind == LOSS_CCE:
        eps = dt.type(1e-8)
        num = dt.type(y.shape[0])
        g = -(dt.type(1.0) / num)             # Div then Negate
        return (y * g) / (p + eps)
    raise ValueError(f"no gradient for loss {kind}")


# --------------------------------------------------------------------------- #
# convolution / pooling (math/nn/AllKernels.scala)
# --------------------------------------------------------------------------- #

PAD_VALID, PAD_SAME, PAD_EXPLICIT = 0, 1, 2


def out_size(padding, inp, window, stride, explicit=(0, 0)):
    """Padding.size (nn/AllKernels.scala:39-89)."""
    if padding == PAD_SAME:
        return int(math.ceil(inp / stride))
    if padding == PAD_VALID:
        return int(math.ceil((inp - window + 1) / stride))
    return int(math.ceil((inp + explicit[0] + explicit[1] - window) / stride)) + 1


def pads_for(padding, inp, window, stride, explicit=(0, 0)):
    """(before, after) zero padding TensorFlow applies along one spatial axis."""
    if padding == PAD_VALID:
        return 0, 0
    if padding == PAD_EXPLICIT:
        return explicit
    out = out_size(PAD_SAME, inp, window, stride)
    total = max((out - 1) * stride + window - inp, 0)
    return total // 2, total - total // 2


def _geometry(xshape, kh, kw, strides, padding, explicit):
    n, h, w, c = xshape
    sh, sw = strides
    eh, ew = (explicit[0], explicit[1]), (explicit[2], explicit[3])
    ho = out_size(padding, h, kh, sh, eh)
    wo = out_size(padding, w, kw, sw, ew)
    pt, pb = pads_for(padding, h, kh, sh, eh)
    pl, pr = pads_for(padding, w, kw, sw, ew)
    # make the padded plane large enough for every window that is read
    need_h = (ho - 1) * sh + kh
    need_w = (wo - 1) * sw + kw
    pb = max(pb, need_h - h - pt)
    pr = max(pr, need_w - w - pl)
    return ho, wo, pt, pb, pl, pr


def _patches(xp, kh, kw, sh, sw, ho, wo):
    """[N, Ho, Wo, kh, kw, C] view-copy of the sliding windows of a padded input."""
    win = np.lib.stride_tricks.sliding_window_view(xp, (kh, kw), axis=(1, 2))
    win = win[:, ::sh, ::sw][:, :ho, :wo]           # [N, Ho, Wo, C, kh, kw]
    return win.transpose(0, 1, 2, 4, 5, 3)


def conv2d(x, w, strides=(1, 1), padding=PAD_VALID, explicit=(0, 0, 0, 0)):
    """TF `Conv2D`, NHWC, filter [kh, kw, Cin, Cout], cross-correlation (nn/AllKernels.scala:143-209)."""
    kh, kw, cin, cout = w.shape
    ho, wo, pt, pb, pl, pr = _geometry(x.shape, kh, kw, strides, padding, explicit)
    xp = np.pad(x, ((0, 0), (pt, pb), (pl, pr), (0, 0)))
    p = _patches(xp, kh, kw, strides[0], strides[1], ho, wo)
    out = p.reshape(-1, kh * kw * cin) @ w.reshape(kh * kw * cin, cout)
    return out.reshape(x.shape[0], ho, wo, cout)


def conv2d_grad_filter(x, wshape, dy, strides=(1, 1), padding=PAD_VALID, explicit=(0, 0, 0, 0)):
    """TF `Conv2DBackpropFilter` (nn/AllKernels.scala:211-235)."""
    kh, kw, cin, cout = wshape
    ho, wo, pt, pb, pl, pr = _geometry(x.shape, kh, kw, strides, padding, explicit)
    xp = np.pad(x, ((0, 0), (pt, pb), (pl, pr), (0, 0)))
    p = _patches(xp, kh, kw, strides[0], strides[1], ho, wo)
    g = p.reshape(-1, kh * kw * cin).T @ dy.reshape(-1, cout)
    return g.reshape(kh, kw, cin, cout)


def conv2d_grad_input(xshape, w, dy, strides=(1, 1), padding=PAD_VALID, explicit=(0, 0, 0, 0)):
    """TF `Conv2DBackpropInput` (nn/AllKernels.scala:237-261)."""
    kh, kw, cin, cout = w.shape
    n, h, wd, _ = xshape
    sh, sw = strides
    ho, wo, pt, pb, pl, pr = _geometry(xshape, kh, kw, strides, padding, explicit)
    dp = dy.reshape(-1, cout) @ w.reshape(kh * kw * cin, cout).T
    dp = dp.reshape(n, ho, wo, kh, kw, cin)
    dxp = np.zeros((n, h + pt + pb, wd + pl + pr, cin), dtype=dy.dtype)
    for r in range(kh):
        for q in range(kw):
            dxp[:, r:r + sh * ho:sh, q:q + sw * wo:sw, :] += dp[:, :, :, r, q, :]
    return dxp[:, pt:pt + h, pl:pl + wd, :]


def max_pool(x, window=(2, 2), strides=(1, 1), padding=PAD_VALID, return_arg=False):
    """TF `MaxPoolV2`, NHWC (nn/AllKernels.scala:270-303). Padding cells never win."""
    kh, kw = window
    ho, wo, pt, pb, pl, pr = _geometry(x.shape, kh, kw, strides, padding, (0, 0, 0, 0))
    xp = np.pad(x, ((0, 0), (pt, pb), (pl, pr), (0, 0)), constant_values=-np.inf)
    p = _patches(xp, kh, kw, strides[0], strides[1], ho, wo)       # [N,Ho,Wo,kh,kw,C]
    flat = p.reshape(p.shape[0], ho, wo, kh * kw, p.shape[-1])
    arg = flat.argmax(axis=3)                                      # first max, row-major window order
    out = np.take_along_axis(flat, arg[:, :, :, None, :], axis=3)[:, :, :, 0, :]
    if return_arg:
        return out, arg
    return out


def max_pool_grad(x, dy, window=(2, 2), strides=(1, 1), padding=PAD_VALID):
    """TF `MaxPoolGradV2`: each window's gradient goes to its first maximum (nn/AllKernels.scala:305-324)."""
    kh, kw = window
    sh, sw = strides
    n, h, wd, c = x.shape
    ho, wo, pt, pb, pl, pr = _geometry(x.shape, kh, kw, strides, padding, (0, 0, 0, 0))
    _, arg = max_pool(x, window, strides, padding, return_arg=True)
    dxp = np.zeros((n, h + pt + pb, wd + pl + pr, c), dtype=dy.dtype)
    for r in range(kh):
        for q in range(kw):
            dxp[:, r:r + sh * ho:sh, q:q + sw * wo:sw, :] += dy * (arg == r * kw + q)
    return dxp[:, pt:pt + h, pl:pl + wd, :]


def _window_cells(shape, window, strides, padding):
    """Number of cells of each pooling window that lie inside the input: [Ho, Wo]."""
    kh, kw = window
    n, h, wd, _ = shape
    ho, wo, pt, pb, pl, pr = _geometry(shape, kh, kw, strides, padding, (0, 0, 0, 0))
    y0 = np.arange(ho) * strides[0] - pt
    x0 = np.arange(wo) * strides[1] - pl
    rows = np.minimum(y0 + kh, h) - np.maximum(y0, 0)
    cols = np.minimum(x0 + kw, wd) - np.maximum(x0, 0)
    return rows[:, None] * cols[None, :]


def avg_pool(x, window=(2, 2), strides=(1, 1), padding=PAD_VALID):
    """TF `AvgPool`, NHWC (nn/AllKernels.scala:326-353): the mean over the window's cells inside the input (padding
    cells are not counted)."""
    kh, kw = window
    ho, wo, pt, pb, pl, pr = _geometry(x.shape, kh, kw, strides, padding, (0, 0, 0, 0))
    xp = np.pad(x, ((0, 0), (pt, pb), (pl, pr), (0, 0)))
    p = _patches(xp, kh, kw, strides[0], strides[1], ho, wo)       # [N,Ho,Wo,kh,kw,C]
    total = np.zeros(p.shape[:3] + p.shape[5:], dtype=x.dtype)
    for r in range(kh):
        for q in range(kw):
            total = total + p[:, :, :, r, q, :]
    cells = _window_cells(x.shape, window, strides, padding).astype(x.dtype)
    return total / cells[None, :, :, None]


def avg_pool_grad(xshape, dy, window=(2, 2), strides=(1, 1), padding=PAD_VALID):
    """TF `AvgPoolGrad` (nn/AllKernels.scala:355-381): every cell of a window gets the window's gradient times
    1 / (its cells inside the input)."""
    kh, kw = window
    sh, sw = strides
    n, h, wd, c = xshape
    ho, wo, pt, pb, pl, pr = _geometry(xshape, kh, kw, strides, padding, (0, 0, 0, 0))
    share = (dy.dtype.type(1) / _window_cells(xshape, window, strides, padding).astype(dy.dtype))[None, :, :, None]
    part = dy * share
    dxp = np.zeros((n, h + pt + pb, wd + pl + pr, c), dtype=dy.dtype)
    for r in range(kh):
        for q in range(kw):
            dxp[:, r:r + sh * ho:sh, q:q + sw * wo:sw, :] += part
    return dxp[:, pt:pt + h, pl:pl + wd, :]


# --------------------------------------------------------------------------- #
# layers (models/layer/*.scala) -- the flattened `Composed` list
# --------------------------------------------------------------------------- #

REG_NONE, REG_L1, REG_L2 = 0, 1, 2


@dataclass
class Layer:
    """One entry of the flattened layer list of `Composed` (layer/Composed.scala:89-99)."""
    kind: str                       # dense | bias | activate | flatten | conv2d | pool2d | lstm | simple_rnn | batchnorm
    units: int = 0
    activation: int = ACT_IDENTITY
    act_param: float = 0.0
    kernel: Tuple[int, int] = (3, 3)
    strides: Tuple[int, int] = (1, 1)
    padding: int = PAD_VALID
    explicit: Tuple[int, int, int, int] = (0, 0, 0, 0)   # conv2d with PAD_EXPLICIT: top, bottom, left, right (AllKernels.scala:67-100)
    reg: int = REG_NONE             # dense / bias; lstm / simple_rnn: kernelReg; batchnorm: betaRegularizer
    reg_lambda: float = 0.0
    recurrent_reg: int = REG_NONE   # lstm / simple_rnn: recurrentReg and biasReg (RNN.scala:120-122,233-235)
    recurrent_lambda: float = 0.0
    bias_reg: int = REG_NONE
    bias_lambda: float = 0.0
    bias: bool = True               # lstm / simple_rnn only
    rnn_activation: int = ACT_TANH  # simple_rnn cell activation / lstm `activation`
    return_sequence: bool = False   # lstm / simple_rnn: every step's output, (batch, time, units) (RNN.scala:27,75-77)
    stateful: bool = False          # lstm / simple_rnn: the cell state after one batch is the start of the next (RNN.scala:27,34,66-67)
    momentum: float = 0.99          # batchnorm (BatchNorm.scala:66-67)
    epsilon: float = 1e-3
    fused: bool = False             # batchnorm: the FusedBatchNormV3 branch as the reference wires it (rank-4 input)
    pool_avg: bool = False          # pool2d: mean of the window (kernel-level `Reduce.Avg`) instead of its maximum

    # ---- parameter definitions, in flat-buffer order ---------------------- #
    def params(self, in_shape) -> List[Tuple[str, Tuple[int, ...]]]:
        if self.kind == "dense":        # Dense.scala:50-55
            return [("weights", (in_shape[1], self.units))]
        if self.kind == "bias":         # Bias.scala:29-30
            return [("weights", (self.units,))]
        if self.kind == "conv2d":       # Conv2D.scala:84-90
            return [("weights", (self.kernel[0], self.kernel[1], in_shape[3], self.units))]
        if self.kind == "lstm":         # RNN.scala:285-305 (gate order forget,input,gate,output)
            f, h = in_shape[2], self.units
            # `if (stateful) state ++ weights else weights` (RNN.scala:32-35); states (batch, units), Zeros, no aggregation (:302-303)
            out = [("cell_state", (in_shape[0], h)), ("hidden_state", (in_shape[0], h))] if self.stateful else []
            for gate in ("forget", "input", "gate", "output"):
                out.append((f"{gate}/0/kernel_weights", (f, h)))
                out.append((f"{gate}/0/recurrent_weights", (h, h)))
                if self.bias:
                    out.append((f"{gate}/1/weights", (h,)))
            return out
        if self.kind == "simple_rnn":   # RNN.scala:170-206
            f, h = in_shape[2], self.units
            out = [("0/state", (in_shape[0], h))] if self.stateful else []     # RNN.scala:188: `State -> ParamDef(outputShape(input), Zeros)`
            out += [("0/kernel_weights", (f, h)), ("0/recurrent_weights", (h, h))]
            if self.bias:
                out.append(("1/weights", (h,)))
            return out
        if self.kind == "batchnorm":    # BatchNorm.scala:80-98: normalised axis keeps its size, every other becomes 1
            shape = (1,) * (len(in_shape) - 1) + (in_shape[-1],)
            return [(name, shape) for name in BN_PARAMS]
        return []

    def out_shape(self, s):
        if self.kind == "dense":
            return (s[0], self.units)
        if self.kind in ("bias", "activate", "batchnorm"):
            return tuple(s)
        if self.kind == "flatten":      # Flatten.scala:12-18
            return (s[0], int(np.prod(s[1:])))
        if self.kind == "conv2d":
            return (s[0], out_size(self.padding, s[1], self.kernel[0], self.strides[0], self.explicit[0:2]),
                    out_size(self.padding, s[2], self.kernel[1], self.strides[1], self.explicit[2:4]), self.units)
        if self.kind == "pool2d":
            return (s[0], out_size(self.padding, s[1], self.kernel[0], self.strides[0]),
                    out_size(self.padding, s[2], self.kernel[1], self.strides[1]), s[3])
        if self.kind in ("lstm", "simple_rnn"):    # RNN.scala:84-90
            return (s[0], s[1], self.units) if self.return_sequence else (s[0], self.units)
        raise ValueError(self.kind)


def Dense(units, activation=ACT_IDENTITY, act_param=0.0, reg=REG_NONE, reg_lambda=0.0, bias=True):
    """`Dense(..)` expands to Dense ?>> Bias ?>> Activate (Dense.scala:30-40)."""
    out = [Layer("dense", units=units, reg=reg, reg_lambda=reg_lambda)]
    if bias:
        out.append(Layer("bias", units=units, reg=reg, reg_lambda=reg_lambda))
    if activation != ACT_IDENTITY:
        out.append(Layer("activate", activation=activation, act_param=act_param))
    return out


def Conv2D(filters, kernel=(3, 3), strides=(1, 1), padding=PAD_VALID, activation=ACT_IDENTITY,
           act_param=0.0, bias=False, explicit=(0, 0, 0, 0)):
    """Conv2D.scala:54-68: defaults Valid, stride 1, no bias; `explicit` = (top, bottom, left, right) with PAD_EXPLICIT."""
    out = [Layer("conv2d", units=filters, kernel=kernel, strides=strides, padding=padding, explicit=tuple(explicit))]
    if bias:
        out.append(Layer("bias", units=filters))
    if activation != ACT_IDENTITY:
        out.append(Layer("activate", activation=activation, act_param=act_param))
    return out


def Pool2D(window=(2, 2), strides=(1, 1), padding=PAD_VALID, reduce="Max", as_reference_layer=True):
    """Pool2D.scala:28-42.  `build` (:36-42) calls `pool2D` without `reduce`, so the reference's layer max-pools
    whatever it was given; `as_reference_layer=False` gives the layer the kernel function's `Reduce.Avg` instead."""
    avg = reduce == "Avg" and not as_reference_layer
    return [Layer("pool2d", kernel=window, strides=strides, padding=padding, pool_avg=avg)]


def Flatten():
    return [Layer("flatten")]


def LSTM(units, bias=True, return_sequence=False, kernel_reg=(REG_NONE, 0.0), recurrent_reg=(REG_NONE, 0.0), bias_reg=(REG_NONE, 0.0),
         stateful=False):
    return [Layer("lstm", units=units, bias=bias, return_sequence=return_sequence, stateful=stateful, reg=kernel_reg[0], reg_lambda=kernel_reg[1],
                  recurrent_reg=recurrent_reg[0], recurrent_lambda=recurrent_reg[1], bias_reg=bias_reg[0], bias_lambda=bias_reg[1])]


def SimpleRNN(units, activation=ACT_TANH, bias=True, return_sequence=False, kernel_reg=(REG_NONE, 0.0), recurrent_reg=(REG_NONE, 0.0),
              bias_reg=(REG_NONE, 0.0), stateful=False):
    return [Layer("simple_rnn", units=units, bias=bias, rnn_activation=activation, return_sequence=return_sequence, stateful=stateful,
                  reg=kernel_reg[0], reg_lambda=kernel_reg[1], recurrent_reg=recurrent_reg[0], recurrent_lambda=recurrent_reg[1],
                  bias_reg=bias_reg[0], bias_lambda=bias_reg[1])]


BN_PARAMS = ("beta", "gamma", "moving_mean", "moving_variance")   # BatchNorm.scala:92-97,170-173
BN_STATE = ("moving_mean", "moving_variance")                      # not trainable: replaced by the layer, not by the optimizer


def BatchNorm(momentum=0.99, epsilon=1e-3, fused=False, beta_reg=(REG_NONE, 0.0)):
    """`BatchNorm(axes = Seq(-1))` (BatchNorm.scala:64-76).  fused=False: the generic `batchNorm` form
    (math/nn/AllKernels.scala:663-684), which the layer takes for `fused = Some(false)` and for any input that is not
    rank 4.  fused=True: the FusedBatchNormV3 branch it takes for rank-4 input otherwise, wired as the reference
    wires it (`batchnorm_fused_forward`)."""
    return [Layer("batchnorm", momentum=momentum, epsilon=epsilon, fused=fused, reg=beta_reg[0], reg_lambda=beta_reg[1])]


RNN_STATE = ("state", "cell_state", "hidden_state")                # RNN.scala:167,253-254


def is_state_path(path: str) -> bool:
    """Parameters with `trainable = false`: MovingMean / MovingVariance (BatchNorm.scala:96-97) and the carried state of
    a stateful RNN (RNN.scala:188,302-303; `ParamDef.trainable` defaults to false)."""
    return path.rsplit("/", 1)[-1] in BN_STATE + RNN_STATE


def is_unaggregated_path(path: str) -> bool:
    """Parameters whose ParamDef has `aggregation = None`: `aggregateParams` re-initialises them instead of averaging
    (Optimizer.scala:205-210).  Only the RNN states (Zeros) are such."""
    return path.rsplit("/", 1)[-1] in RNN_STATE


def batchnorm_forward(x, params, pre, l: Layer, training: bool):
    """math/nn/AllKernels.scala:663-684 in its op order; returns (y, cache, next_state).

    training: moments over every axis but the last (alg/AllKernels.scala:505-513, biased variance);
    frozen: the moving statistics.  next_state = decayingAvg(moving, batch, momentum) (BatchNorm.scala:146-149,
    alg/AllKernels.scala:541-544), present only when training."""
    dt = x.dtype
    gamma, beta = params[pre + "gamma"], params[pre + "beta"]
    axes = tuple(range(x.ndim - 1))
    if training:
        n = dt.type(np.prod([x.shape[a] for a in axes]))
        mean = x.sum(axis=axes, keepdims=True, dtype=dt) / n
        var = sqr(x - mean).sum(axis=axes, keepdims=True, dtype=dt) / n
    else:
        mean, var = params[pre + "moving_mean"], params[pre + "moving_variance"]
    r = dt.type(1.0) / np.sqrt(var + dt.type(l.epsilon))
    inv = r * gamma
    y = ((x * inv) - (mean * inv)) + beta
    nxt = {}
    if training:
        mom = dt.type(l.momentum)
        nxt[pre + "moving_mean"] = mom * params[pre + "moving_mean"] + (dt.type(1.0) - mom) * mean
        nxt[pre + "moving_variance"] = mom * params[pre + "moving_variance"] + (dt.type(1.0) - mom) * var
    return y, (x, mean, r, gamma, training), nxt


def batchnorm_backward(dy, cache, pre, grads):
    """Reverse mode through `((x*inv) - (mean*inv)) + beta`, inv = rsqrt(var+eps)*gamma, with mean and var
    functions of x when training."""
    x, mean, r, gamma, training = cache
    dt = dy.dtype
    axes = tuple(range(x.ndim - 1))
    xc = x - mean
    s1 = dy.sum(axis=axes, keepdims=True, dtype=dt)
    s2 = (dy * xc).sum(axis=axes, keepdims=True, dtype=dt)
    grads[pre + "beta"] = s1
    grads[pre + "gamma"] = s2 * r
    inv = r * gamma
    if not training:
        return dy * inv
    n = dt.type(np.prod([x.shape[a] for a in axes]))
    return inv * (dy - s1 / n - xc * (r * r * s2 / n))


# ---- the FusedBatchNormV3 form (rank-4 input unless `fused = Some(false)`, BatchNorm.scala:98-130) ------------------ #
def fused_batch_norm(x, scale, offset, mean_in, var_in, eps, training):
    """The six outputs of TensorFlow's `FusedBatchNormV3` on the CPU, NHWC, exponential_avg_factor = 1 (the op the
    reference builds at nn/AllKernels.scala:399-421): (y, batch_mean, batch_variance, reserve_space_1,
    reserve_space_2, reserve_space_3).

    training: batch_mean = mean over all axes but the last; y = (x - mean) * (rsqrt(var + eps) * scale) + offset with
    the biased variance; `batch_variance` (the value meant for the running average) is the UNBIASED variance
    var * n / max(n - 1, 1); reserve_space_1 / 2 keep the mean and the biased variance for the gradient.
    inference: the given population statistics everywhere."""
    dt = x.dtype
    c = x.shape[-1]
    x2 = x.reshape(-1, c)
    n = x2.shape[0]
    scale, offset = scale.reshape(c), offset.reshape(c)
    if training:
        mean = x2.sum(axis=0, dtype=dt) / dt.type(n)
        xc = x2 - mean
        var = (xc * xc).sum(axis=0, dtype=dt) / dt.type(n)
        y = xc * ((dt.type(1.0) / np.sqrt(var + dt.type(eps))) * scale) + offset
        unbiased = var * (dt.type(n) / dt.type(max(n - 1, 1)))
        return y.reshape(x.shape), mean, unbiased, mean, var, np.zeros(0, dt)
    mean, var = mean_in.reshape(c), var_in.reshape(c)
    y = (x2 - mean) * ((dt.type(1.0) / np.sqrt(var + dt.type(eps))) * scale) + offset
    return y.reshape(x.shape), mean, var, mean, var, np.zeros(0, dt)


def fused_batch_norm_grad(dy, x, scale, reserve_1, reserve_2, eps):
    """`FusedBatchNormGradV3` on the CPU with is_training = true (nn/AllKernels.scala:503-531): it takes reserve_1 as
    the batch mean m and reserve_2 as the batch variance v and returns
        dx      = scale * rsqrt(v + eps) * (dy - mean(dy) - (x - m) * mean(dy * (x - m)) / (v + eps))
        dscale  = sum(dy * (x - m) * rsqrt(v + eps))
        doffset = sum(dy)."""
    dt = dy.dtype
    c = x.shape[-1]
    x2, dy2 = x.reshape(-1, c), dy.reshape(-1, c)
    n = dt.type(x2.shape[0])
    m, v, scale = reserve_1.reshape(c), reserve_2.reshape(c), scale.reshape(c)
    r = dt.type(1.0) / np.sqrt(v + dt.type(eps))
    xc = x2 - m
    s1 = dy2.sum(axis=0, dtype=dt)
    s2 = (dy2 * xc).sum(axis=0, dtype=dt)
    dx = (scale * r) * (dy2 - s1 / n - xc * (r * r * s2 / n))
    return dx.reshape(x.shape), s2 * r, s1


def batchnorm_fused_forward(x, params, pre, l: Layer, training: bool):
    """The layer's fused branch AS THE REFERENCE WIRES IT (BatchNorm.scala:117-130, nn/AllKernels.scala:437-448):
    `outputs` takes TF output 1 for batchMean AND for batchVariance, output 2 for reserveSpace1, 3 for reserveSpace2
    and 4 for reserveSpace3.  So the moving variance follows the batch MEAN, and the gradient op receives the
    unbiased batch variance where it expects the mean and the batch mean where it expects the variance.
    Returns (y, cache, next_state)."""
    dt = x.dtype
    outs = fused_batch_norm(x, params[pre + "gamma"], params[pre + "beta"], params[pre + "moving_mean"],
                            params[pre + "moving_variance"], l.epsilon, training)
    y = outs[0]
    batch_mean, batch_variance = outs[1], outs[1]
    reserve_1, reserve_2 = outs[2], outs[3]
    nxt = {}
    if training:
        mom = dt.type(l.momentum)
        shape = params[pre + "moving_mean"].shape
        nxt[pre + "moving_mean"] = mom * params[pre + "moving_mean"] + (dt.type(1.0) - mom) * batch_mean.reshape(shape)
        nxt[pre + "moving_variance"] = mom * params[pre + "moving_variance"] + (dt.type(1.0) - mom) * batch_variance.reshape(shape)
    return y, (x, reserve_1, reserve_2, params[pre + "gamma"], l.epsilon, training), nxt


def batchnorm_fused_backward(dy, cache, pre, grads):
    x, reserve_1, reserve_2, gamma, eps, training = cache
    if not training:
        raise NotImplementedError("the gradient of the frozen fused form is not on the training path")
    dx, dscale, doffset = fused_batch_norm_grad(dy, x, gamma, reserve_1, reserve_2, eps)
    grads[pre + "gamma"] = dscale.reshape(gamma.shape)
    grads[pre + "beta"] = doffset.reshape(gamma.shape)
    return dx


class Model:
    """A `Composed` model: flattened layers, index-prefixed parameter paths (Composed.scala:22-31)."""

    def __init__(self, layers: Sequence, loss: int = LOSS_MSE, bf16_dense: bool = False):
        self.bf16_dense = bf16_dense
        flat: List[Layer] = []
        for l in layers:
            flat.extend(l if isinstance(l, (list, tuple)) else [l])
        self.layers = flat
        self.loss = loss

    def _prefix(self, idx):
        return "" if len(self.layers) == 1 else f"{idx}/"

    def param_defs(self, in_shape) -> List[Tuple[str, Tuple[int, ...]]]:
        out, s = [], tuple(in_shape)
        for i, l in enumerate(self.layers):
            for name, shape in l.params(s):
                out.append((self._prefix(i) + name, shape))
            s = l.out_shape(s)
        return out

    def out_shape(self, in_shape):
        s = tuple(in_shape)
        for l in self.layers:
            s = l.out_shape(s)
        return s

    # ---- forward ---------------------------------------------------------- #
    def forward(self, x, params: Dict[str, np.ndarray], cache: Optional[list] = None, training: bool = False,
                next_state: Optional[dict] = None):
        """training = the model as `Optimizer` compiles it; False = frozen, as `LossModel.trained` hands it to
        `TrainedModel` (Model.scala:126-127).  Only stateful layers (BatchNorm) tell the two apart."""
        for i, l in enumerate(self.layers):
            pre = self._prefix(i)
            k = l.kind
            if k == "dense":
                w = params[pre + "weights"]
                if self.bf16_dense:
                    x, w = to_bf16(x), to_bf16(w)
                y = x @ w                                     # Dense.scala:57-61
                c = (x, w)
            elif k == "bias":
                y = x + params[pre + "weights"]               # Bias.scala:32-33
                c = None
            elif k == "activate":
                y = activate(l.activation, x, l.act_param)
                c = x
            elif k == "flatten":
                y = x.reshape(x.shape[0], -1)
                c = x.shape
            elif k == "conv2d":
                w = params[pre + "weights"]
                y = conv2d(x, w, l.strides, l.padding, l.explicit)
                c = (x, w)
            elif k == "pool2d":
                y = (avg_pool if l.pool_avg else max_pool)(x, l.kernel, l.strides, l.padding)
                c = x
            elif k == "lstm":
                y, c, nxt = lstm_forward(x, params, pre, l)
                if next_state is not None:
                    next_state.update(nxt)
            elif k == "simple_rnn":
                y, c, nxt = simple_rnn_forward(x, params, pre, l)
                if next_state is not None:
                    next_state.update(nxt)
            elif k == "batchnorm":
                y, c, nxt = (batchnorm_fused_forward if l.fused else batchnorm_forward)(x, params, pre, l, training)
                if next_state is not None:
                    next_state.update(nxt)
            else:
                raise ValueError(k)
            if cache is not None:
                cache.append(c)
            x = y
        return x

    # ---- penalty (Regularization.scala:30-44; Composed.scala:66-75) -------- #
    def regularized(self, training: bool = True):
        """(path, kind, lambda, times) of every penalty term of the model.

        Dense: reg(weights), always (Dense.scala:63-64).  Bias (also the ones inside Dense, Conv2D and the RNN cells):
        reg(weights) only while trainable (Bias.scala:35-36), so not in the frozen model a TrainedModel holds.
        SimpleRNNCell: kernelReg(kernel) + recurrentReg(recurrent), always (RNN.scala:198-199); an LSTM sums its four
        gate cells (:341-346).  BatchNorm: betaRegularizer(gamma) + betaRegularizer(gamma) while trainable
        (BatchNorm.scala:158-160; gammaRegularizer is never used)."""
        out = []
        for i, l in enumerate(self.layers):
            pre = self._prefix(i)
            if l.kind == "dense":
                out.append((pre + "weights", l.reg, l.reg_lambda, 1))
            elif l.kind == "bias" and training:
                out.append((pre + "weights", l.reg, l.reg_lambda, 1))
            elif l.kind in ("lstm", "simple_rnn"):
                for g in ([f"{gate}/" for gate in GATES] if l.kind == "lstm" else [""]):
                    out.append((pre + g + "0/kernel_weights", l.reg, l.reg_lambda, 1))
                    out.append((pre + g + "0/recurrent_weights", l.recurrent_reg, l.recurrent_lambda, 1))
                    if l.bias and training:
                        out.append((pre + g + "1/weights", l.bias_reg, l.bias_lambda, 1))
            elif l.kind == "batchnorm" and training:
                out.append((pre + "gamma", l.reg, l.reg_lambda, 2))
        return [t for t in out if t[1] != REG_NONE]

    def penalty(self, params, training: bool = True):
        dt = next(iter(params.values())).dtype if params else np.dtype(F32)
        total = dt.type(0.0)
        for path, kind, lam, times in self.regularized(training):
            w = params[path]
            if kind == REG_L2:
                term = dt.type(lam) * sqr(w).sum(dtype=dt) / dt.type(2.0)
            else:
                term = dt.type(lam) * np.abs(w).sum(dtype=dt) / dt.type(2.0)
            for _ in range(times):
                total = total + term
        return total

    def loss_of(self, x, y, params, training: bool = False):
        """LossModel.buildStateful (Model.scala:92-99): loss(model(x), y) + penalty."""
        p = self.forward(x, params, training=training)
        return loss_value(self.loss, p, y) + self.penalty(params, training)

    # ---- backward: gradients w.r.t. every weight -------------------------- #
    def grad(self, x, y, params):
        """LossModel.grad (Model.scala:107-119): returns (loss, {path: gradient})."""
        loss, grads, _ = self.grad_stateful(x, y, params)
        return loss, grads

    def grad_stateful(self, x, y, params):
        """LossModel.gradStateful (Model.scala:113-119): (loss, {weight path: gradient}, {state path: next value})."""
        cache: list = []
        next_state: dict = {}
        p = self.forward(x, params, cache, training=True, next_state=next_state)
        loss = loss_value(self.loss, p, y) + self.penalty(params)
        dy = np.ones_like(p) if self.loss == LOSS_IDENTITY else loss_grad(self.loss, p, y)
        grads: Dict[str, np.ndarray] = {}
        for i in range(len(self.layers) - 1, -1, -1):
            l, c, pre = self.layers[i], cache[i], self._prefix(i)
            k = l.kind
            if k == "dense":
                xi, w = c
                if self.bf16_dense:
                    dy = to_bf16(dy)
                grads[pre + "weights"] = xi.T @ dy            # AllKernels.scala:382-388
                dy = dy @ w.T
            elif k == "bias":
                axes = tuple(range(dy.ndim - 1))
                grads[pre + "weights"] = dy.sum(axis=axes, dtype=dy.dtype)   # Plus grad: Sum over broadcast axes
            elif k == "activate":
                dy = activate_grad(l.activation, c, dy, l.act_param)
            elif k == "flatten":
                dy = dy.reshape(c)
            elif k == "conv2d":
                xi, w = c
                grads[pre + "weights"] = conv2d_grad_filter(xi, w.shape, dy, l.strides, l.padding, l.explicit)
                dy = conv2d_grad_input(xi.shape, w, dy, l.strides, l.padding, l.explicit) if i > 0 else None
            elif k == "pool2d":
                dy = (avg_pool_grad(c.shape, dy, l.kernel, l.strides, l.padding) if l.pool_avg
                      else max_pool_grad(c, dy, l.kernel, l.strides, l.padding))
            elif k == "lstm":
                dy = lstm_backward(dy, c, params, pre, l, grads, need_dx=i > 0)
            elif k == "simple_rnn":
                dy = simple_rnn_backward(dy, c, params, pre, l, grads, need_dx=i > 0)
            elif k == "batchnorm":
                dy = (batchnorm_fused_backward if l.fused else batchnorm_backward)(dy, c, pre, grads)
        for path, kind, lam_f, times in self.regularized(True):
            w = params[path]
            lam = w.dtype.type(lam_f)
            for _ in range(times):
                if kind == REG_L2:        # d/dw lambda * sum(w^2) / 2 through Pow's grad: (w^1 * 2) * (lambda/2)
                    grads[path] = grads[path] + (w * w.dtype.type(2.0)) * (lam / w.dtype.type(2.0))
                else:                     # Abs grad in the reference is |parent| (AllKernels.scala:330-335)
                    grads[path] = grads[path] + np.abs(np.ones_like(w) * (lam / w.dtype.type(2.0)))
        return loss, grads, next_state


# --------------------------------------------------------------------------- #
# recurrent layers (models/layer/RNN.scala)
# --------------------------------------------------------------------------- #

GATES = ("forget", "input", "gate", "output")


def lstm_forward(x, params, pre, l: Layer):
    """RNN.build + LSTMCell.build (RNN.scala:40-72, 320-338); returns (output, cache, next state).

    `stateful`: the first step starts from the `cell_state` / `hidden_state` parameters instead of zeros and the last
    step's c and h are the layer's next state (RNN.scala:66-72, 338)."""
    b, t_steps, _ = x.shape
    h_units = l.units
    dt = x.dtype
    c = params[pre + "cell_state"][:b] if l.stateful else np.zeros((b, h_units), dt)
    h = params[pre + "hidden_state"][:b] if l.stateful else np.zeros((b, h_units), dt)
    steps = []
    outs = []
    for t in range(t_steps):
        xt = x[:, t, :]
        z = {}
        for gate in GATES:
            zz = (xt @ params[f"{pre}{gate}/0/kernel_weights"]) + (h @ params[f"{pre}{gate}/0/recurrent_weights"])
            if l.bias:
                zz = zz + params[f"{pre}{gate}/1/weights"]
            z[gate] = zz
        f = sigmoid(z["forget"])
        i = sigmoid(z["input"])
        g = activate(l.rnn_activation, z["gate"])
        o = sigmoid(z["output"])
        c_new = c * f + i * g                     # RNN.scala:336
        h_new = o * activate(l.rnn_activation, c_new)   # RNN.scala:337
        steps.append((xt, h, c, z, f, i, g, o, c_new))
        c, h = c_new, h_new
        outs.append(h_new)
    out = np.stack(outs, axis=1) if l.return_sequence else h     # `joinAlong(outputs, 1)` or `outputs.last` (RNN.scala:74-77)
    nxt = {pre + "cell_state": c, pre + "hidden_state": h} if l.stateful else {}
    return out, (x.shape, steps), nxt


def lstm_backward(dout, cache, params, pre, l: Layer, grads, need_dx=False):
    """dout: gradient of the layer's output, (batch, units) or with `return_sequence` (batch, time, units): every
    step's output then adds its own gradient to the one carried back from the step after it."""
    xshape, steps = cache
    dt = dout.dtype
    b = xshape[0]
    seq = l.return_sequence
    dh = np.zeros((b, l.units), dt) if seq else dout
    dc = np.zeros((b, l.units), dt)
    acc = {}
    dx = np.zeros(xshape, dt) if need_dx else None
    for t in range(len(steps) - 1, -1, -1):
        xt, h_prev, c_prev, z, f, i, g, o, c_new = steps[t]
        if seq:
            dh = dh + dout[:, t, :]
        a = activate(l.rnn_activation, c_new)
        do = dh * a
        dc = dc + activate_grad(l.rnn_activation, c_new, dh * o)
        df = dc * c_prev
        di = dc * g
        dg = dc * i
        dc_prev = dc * f
        dz = {
            "forget": sigmoid_grad(z["forget"], df),
            "input": sigmoid_grad(z["input"], di),
            "gate": activate_grad(l.rnn_activation, z["gate"], dg),
            "output": sigmoid_grad(z["output"], do),
        }
        dh_prev = np.zeros_like(dh)
        for gate in GATES:
            kk, rr, bb = f"{pre}{gate}/0/kernel_weights", f"{pre}{gate}/0/recurrent_weights", f"{pre}{gate}/1/weights"
            acc[kk] = acc.get(kk, 0) + xt.T @ dz[gate]
            acc[rr] = acc.get(rr, 0) + h_prev.T @ dz[gate]
            if l.bias:
                acc[bb] = acc.get(bb, 0) + dz[gate].sum(axis=0, dtype=dt)
            dh_prev = dh_prev + dz[gate] @ params[rr].T
            if need_dx:
                dx[:, t, :] += dz[gate] @ params[kk].T
        dh, dc = dh_prev, dc_prev
    grads.update(acc)
    return dx


def simple_rnn_forward(x, params, pre, l: Layer):
    """RNN over `SimpleRNNCell ?>> Bias ?>> act` (RNN.scala:170-206).

    The cell's carried state is its own pre-bias, pre-activation output
    (`Params(State -> result)`, RNN.scala:195-196)."""
    b, t_steps, _ = x.shape
    dt = x.dtype
    wk, wr = params[pre + "0/kernel_weights"], params[pre + "0/recurrent_weights"]
    s = params[pre + "0/state"][:b] if l.stateful else np.zeros((b, l.units), dt)
    steps = []
    out = None
    outs = []
    for t in range(t_steps):
        xt = x[:, t, :]
        r = (xt @ wk) + (s @ wr)
        zz = r + params[pre + "1/weights"] if l.bias else r
        out = activate(l.rnn_activation, zz)
        outs.append(out)
        steps.append((xt, s, zz))
        s = r
    if l.return_sequence:
        out = np.stack(outs, axis=1)
    return out, (x.shape, steps), ({pre + "0/state": s} if l.stateful else {})


def simple_rnn_backward(dout, cache, params, pre, l: Layer, grads, need_dx=False):
    xshape, steps = cache
    dt = dout.dtype
    wk, wr = params[pre + "0/kernel_weights"], params[pre + "0/recurrent_weights"]
    dx = np.zeros(xshape, dt) if need_dx else None
    gk = np.zeros_like(wk)
    gr = np.zeros_like(wr)
    gb = np.zeros((l.units,), dt)
    # without `return_sequence` only the last step's output feeds the loss; earlier steps act through the state
    t_last = len(steps) - 1
    seq = l.return_sequence
    dr = np.zeros((xshape[0], l.units), dt)
    for t in range(t_last, -1, -1):
        xt, s_prev, zz = steps[t]
        if seq or t == t_last:
            dz = activate_grad(l.rnn_activation, zz, dout[:, t, :] if seq else dout)
            gb += dz.sum(axis=0, dtype=dt)
            dr = dr + dz
        gk += xt.T @ dr
        gr += s_prev.T @ dr
        if need_dx:
            dx[:, t, :] = dr @ wk.T
        dr = dr @ wr.T
    grads[pre + "0/kernel_weights"] = gk
    grads[pre + "0/recurrent_weights"] = gr
    if l.bias:
        grads[pre + "1/weights"] = gb
    return dx


# --------------------------------------------------------------------------- #
# optimizer algorithms (optimizers/*.scala)
# --------------------------------------------------------------------------- #

OPT_SGD, OPT_ADAGRAD, OPT_ADADELTA, OPT_RMSPROP, OPT_ADAM, OPT_NADAM, OPT_ADAMAX, OPT_AMSGRAD = range(8)


@dataclass
class Algorithm:
    kind: int
    rate: float = 0.001
    beta1: float = 0.9          # momentum (SGD) / rho (AdaDelta, RMSProp) / beta1
    beta2: float = 0.999
    epsilon: float = 1e-7
    init_acc: float = 0.0
    nesterov: bool = False

    @property
    def state_names(self) -> List[str]:
        return {
            OPT_SGD: ["velocity"], OPT_ADAGRAD: ["grad_acc"], OPT_ADADELTA: ["avg_grad", "avg_delta"],
            OPT_RMSPROP: ["avg_grad"], OPT_ADAM: ["momentum", "velocity"], OPT_NADAM: ["momentum", "velocity"],
            OPT_ADAMAX: ["momentum_1", "momentum_2"], OPT_AMSGRAD: ["momentum", "velocity", "corrected_velocity"],
        }[self.kind]

    def init_state(self, shape, dtype=F32) -> List[np.ndarray]:
        return [np.full(shape, self.init_acc, dtype) for _ in self.state_names]

    def build(self, g, state: List[np.ndarray], it: int):
        """`Algorithm.build(grad, params, iter): Delta` -> (delta, new_state)."""
        dt = g.dtype
        r, b1, b2, eps = dt.type(self.rate), dt.type(self.beta1), dt.type(self.beta2), dt.type(self.epsilon)
        one = dt.type(1.0)
        k = self.kind
        if k == OPT_SGD:                                  # SGD.scala:15-25
            v = (r * g) - (b1 * state[0])
            delta = (r * g) - (b1 * v) if self.nesterov else v
            return delta, [v]
        if k == OPT_ADAGRAD:                              # AdaGrad.scala:21-32
            acc = state[0] + sqr(g)
            rates = r / sqrt_zero_safe(acc, eps)
            return rates * g, [acc]
        if k == OPT_ADADELTA:                             # AdaDelta.scala:33-44
            avg_grad = decaying_avg(state[0], sqr(g), b1)
            delta = r * ((sqrt_zero_safe(state[1], eps) / sqrt_zero_safe(avg_grad, eps)) * g)
            avg_delta = decaying_avg(state[1], sqr(delta), b1)
            return delta, [avg_grad, avg_delta]
        if k == OPT_RMSPROP:                              # RMSProp.scala:24-32
            avg_grad = decaying_avg(state[0], sqr(g), b1)
            delta = (r / sqrt_zero_safe(avg_grad, eps)) * g
            return delta, [avg_grad]
        if k == OPT_ADAM:                                 # Adam.scala:29-41
            m = decaying_avg(state[0], g, b1)
            v = decaying_avg(state[1], sqr(g), b2)
            delta = (r / np.sqrt(boost(v, b2, it) + eps)) * boost(m, b1, it)
            return delta, [m, v]
        if k == OPT_NADAM:                                # Nadam.scala:37-49
            m = decaying_avg(state[0], g, b1)
            v = decaying_avg(state[1], sqr(g), b2)
            m_nest = (b1 * boost(m, b1, it)) + ((one - b1) * boost(g, b1, it))
            delta = m_nest / (np.sqrt(boost(v, b2, it)) + eps)
            return delta, [m, v]
        if k == OPT_ADAMAX:                               # Adamax.scala:41-52
            m1 = decaying_avg(state[0], g, b1)
            m2 = np.maximum(b2 * state[1], (one - b2) * np.abs(g))
            delta = r * boost(m1, b1, it) / (m2 + eps)
            return delta, [m1, m2]
        if k == OPT_AMSGRAD:                              # AMSGrad.scala:34-46
            m = decaying_avg(state[0], g, b1)
            v_cur = decaying_avg(state[1], sqr(g), b2)
            v = np.maximum(state[2], v_cur)
            delta = r * m / (np.sqrt(v) + eps)
            return delta, [m, v_cur, v]
        raise ValueError(k)


def SGD(rate=0.01, momentum=0.0, nesterov=False):
    return Algorithm(OPT_SGD, rate=rate, beta1=momentum, nesterov=nesterov)


def AdaGrad(rate=0.001, epsilon=1e-7):
    return Algorithm(OPT_ADAGRAD, rate=rate, epsilon=epsilon)


def AdaDelta(rate=1.0, rho=0.9, epsilon=1e-7):
    return Algorithm(OPT_ADADELTA, rate=rate, beta1=rho, epsilon=epsilon)


def RMSProp(rate=0.001, rho=0.9, epsilon=1e-7):
    return Algorithm(OPT_RMSPROP, rate=rate, beta1=rho, epsilon=epsilon)


def Adam(rate=0.001, beta1=0.9, beta2=0.999, epsilon=1e-7):
    return Algorithm(OPT_ADAM, rate=rate, beta1=beta1, beta2=beta2, epsilon=epsilon)


def Nadam(beta1=0.9, beta2=0.999, epsilon=1e-7, init_acc=0.001):
    return Algorithm(OPT_NADAM, rate=0.0, beta1=beta1, beta2=beta2, epsilon=epsilon, init_acc=init_acc)


def Adamax(rate=0.001, beta1=0.9, beta2=0.999, epsilon=1e-7, init_acc=0.001):
    return Algorithm(OPT_ADAMAX, rate=rate, beta1=beta1, beta2=beta2, epsilon=epsilon, init_acc=init_acc)


def AMSGrad(rate=0.001, beta1=0.9, beta2=0.999, epsilon=1e-7):
    return Algorithm(OPT_AMSGRAD, rate=rate, beta1=beta1, beta2=beta2, epsilon=epsilon)


# --------------------------------------------------------------------------- #
# the step, the per-partition loop and the averaging (optimizers/Optimizer.scala)
# --------------------------------------------------------------------------- #


def train_step(model: Model, alg: Algorithm, x, y, params, opt_state, it: int, minimizing=True):
    """`compileBackprop`'s function (Optimizer.scala:169-194): one update of every weight.

    Returns (new_params, new_opt_state, loss_before_update, grads)."""
    loss, grads, next_state = model.grad_stateful(x, y, params)
    new_params, new_state = {}, {}
    for path, w in params.items():
        if path in next_state:      # `nextWeights ++ nextState` (Optimizer.scala:142-144): state bypasses the algorithm
            new_params[path] = next_state[path]
            if path in opt_state:
                new_state[path] = opt_state[path]
            continue
        delta, st = alg.build(grads[path], opt_state[path], it)
        new_params[path] = w - delta if minimizing else w + delta    # Optimizer.scala:186
        new_state[path] = st
    return new_params, new_state, loss, grads


def init_opt_state(alg: Algorithm, params):
    return {p: alg.init_state(w.shape, w.dtype) for p, w in params.items()}


def optimize_on_partition(model, alg, X, Y, batch, global_iter, params, opt_state):
    """`optimizeOnPartition` (Optimizer.scala:106-161).

    Full batches only (Iterators.scala:90, `Skip`); iteration numbers are
    `global_iter + i + 1`; after the last batch the loss of that batch is
    evaluated once more with the updated parameters (Optimizer.scala:148).
    Returns (iterations, params, opt_state, loss)."""
    n_batches = X.shape[0] // batch
    if n_batches == 0:
        raise StopIteration("empty partition")          # batches.next() throws (Iterators.scala:80-81)
    for i in range(n_batches):
        xb, yb = X[i * batch:(i + 1) * batch], Y[i * batch:(i + 1) * batch]
        params, opt_state, _, _ = train_step(model, alg, xb, yb, params, opt_state, global_iter + i + 1)
    loss = model.loss_of(xb, yb, params, training=True)     # `lossModel.lossStateful`, not frozen (Optimizer.scala:148,163-167)
    return n_batches, params, opt_state, loss


def average_uniform(replicas: Sequence[np.ndarray]):
    """`Aggregation.Avg` over K inputs: AddN(inputs) / K (Aggregation.scala:16-19).

    AddN accumulates left to right in the element type."""
    acc = replicas[0].copy()
    for r in replicas[1:]:
        acc = acc + r
    return acc / acc.dtype.type(len(replicas))


def avg2(l, r):
    """The pairwise form `aggregateParams` applies (Optimizer.scala:205-210)."""
    return (l + r) / l.dtype.type(2.0)


def train(model, alg, partitions, batch, epochs, init_params, avg="uniform"):
    """`Optimizer.run` (Optimizer.scala:59-104) with the Spark partitions given explicitly.

    `partitions` is a list of (X, Y).  Every epoch each partition starts from
    the same broadcast parameters; results are averaged (parameters and
    optimizer state), losses averaged, iterations summed."""
    params = {k: v.copy() for k, v in init_params.items()}
    opt_state = init_opt_state(alg, params)
    global_iter = 0
    history = []
    for _ in range(epochs):
        results = [optimize_on_partition(model, alg, X, Y, batch, global_iter, params, opt_state)
                   for X, Y in partitions]
        if len(results) == 1:
            iters, params, opt_state, loss = results[0]
        else:
            iters = sum(r[0] for r in results)
            # tensors without an aggregation are re-initialised (Optimizer.scala:207-210): the RNN states, to zeros
            params = {p: np.zeros_like(params[p]) if is_unaggregated_path(p) else average_uniform([r[1][p] for r in results])
                      for p in params}
            opt_state = {p: [average_uniform([r[2][p][s] for r in results])
                             for s in range(len(alg.state_names))] for p in params}
            loss = float(np.mean([r[3] for r in results]))
        global_iter += iters
        history.append(float(loss))
    return params, opt_state, history


def error_sum(model, x, y, params, absolute=False):
    """`errorSum` of the regression estimators (estimators/package.scala:80-84): sum over every output element of
    (predicted - expected)^2 (MSE, :56-62) or |predicted - expected| (MAE, :64-70) for the frozen model."""
    d = model.forward(x, params) - y
    return (np.abs(d) if absolute else sqr(d)).sum(dtype=d.dtype)


def mean_error(model, X, Y, params, batch=1000, absolute=False):
    """`meanError` (estimators/package.scala:72-101): batch sums added in float, divided by the row count."""
    total = F32(0.0)
    for s in range(0, X.shape[0], batch):
        total = F32(total + error_sum(model, X[s:s + batch], Y[s:s + batch], params, absolute))
    return float(total / F32(X.shape[0]))


def r2_score(model, X, Y, params, batch=1000):
    """`R2Score` (estimators/package.scala:103-138), with its total sum of squares around the mean prediction."""
    pred = np.concatenate([model.forward(X[s:s + batch], params).reshape(-1) for s in range(0, X.shape[0], batch)]).astype(np.float64)
    exp = Y.reshape(-1).astype(np.float64)
    return float(F32(1.0 - ((pred - exp) ** 2).sum() / ((pred - pred.mean()) ** 2).sum()))


def count_correct(model, x, y, params):
    """`estimators.accuracy`'s per-batch count (estimators/package.scala:28-32):
    rows whose every rounded output equals the label."""
    p = rint(model.forward(x, params))
    matched = (y == p).astype(np.int32).sum(axis=1)
    return int((matched == model.out_shape(x.shape)[-1]).astype(np.int32).sum())


# --------------------------------------------------------------------------- #
# seeded initializers (models/Initializer.scala over math/rand/AllKernels.scala)
# --------------------------------------------------------------------------- #
# The reference draws with TensorFlow's RandomUniform / RandomStandardNormal / TruncatedNormal ops and their `seed`
# attribute (math/rand/AllKernels.scala:12-43).  TensorFlow is a dependency that does not ship with the reference
# (build.sbt:13, "org.tensorflow" % "tensorflow-core-platform" % "0.5.0", i.e. TensorFlow 2.10): what follows restates
# the published algorithm of those CPU kernels (tensorflow/core/lib/random/philox_random.h, random_distributions.h,
# kernels/random_op_cpu.h): Philox4x32-10 keyed by the op seed (seed2 = 0), counter = output group, four outputs per
# counter, uint32 -> [0,1) through the float mantissa, Box-Muller for normals, and for the truncated normal a
# rejection loop per group of four outputs that starts 256 counters after the previous group's start.
# Pinned by the values models/InitializerSpec.scala:23-66 records for seeds 1 and 2.

_M32 = np.uint64(0xFFFFFFFF)


def philox4x32_10(counter: np.ndarray, key: Tuple[int, int]) -> np.ndarray:
    """counter: uint32 [n, 4]; returns uint32 [n, 4] (philox_random.h: ten rounds, key raised between rounds)."""
    c = counter.astype(np.uint64)
    k0, k1 = np.uint64(key[0]), np.uint64(key[1])
    for rnd in range(10):
        if rnd:
            k0 = (k0 + np.uint64(0x9E3779B9)) & _M32
            k1 = (k1 + np.uint64(0xBB67AE85)) & _M32
        p0 = np.uint64(0xD2511F53) * c[:, 0]
        p1 = np.uint64(0xCD9E8D57) * c[:, 2]
        c = np.stack([(p1 >> np.uint64(32)) ^ c[:, 1] ^ k0, p1 & _M32, (p0 >> np.uint64(32)) ^ c[:, 3] ^ k1, p0 & _M32], axis=1)
    return c.astype(np.uint32)


def _philox_blocks(seed: int, first: np.ndarray) -> np.ndarray:
    """Outputs of the counters `first` (uint64 [n]) under PhiloxRandom(seed, 0): key = the seed's two halves."""
    ctr = np.zeros((first.shape[0], 4), np.uint32)
    ctr[:, 0] = (first & _M32).astype(np.uint32)
    ctr[:, 1] = (first >> np.uint64(32)).astype(np.uint32)
    return philox4x32_10(ctr, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))


def uint32_to_float(x: np.ndarray) -> np.ndarray:
    """random_distributions.h Uint32ToFloat: 23 mantissa bits under exponent 127, minus one."""
    return ((x & np.uint32(0x7FFFFF)) | np.uint32(127 << 23)).view(np.float32) - F32(1.0)


def box_muller(x0: np.ndarray, x1: np.ndarray):
    """random_distributions.h BoxMullerFloat."""
    u1 = np.maximum(uint32_to_float(x0), F32(1.0e-7))
    v1 = (2.0 * math.pi * uint32_to_float(x1).astype(np.float64)).astype(np.float32)     # `2.0f * M_PI * u` is a double product
    u2 = np.sqrt(F32(-2.0) * np.log(u1))
    return np.sin(v1) * u2, np.cos(v1) * u2


def tf_random_uniform(n: int, seed: int) -> np.ndarray:
    groups = np.arange((n + 3) // 4, dtype=np.uint64)
    return uint32_to_float(_philox_blocks(seed, groups).reshape(-1))[:n]


def tf_random_normal(n: int, seed: int) -> np.ndarray:
    r = _philox_blocks(seed, np.arange((n + 3) // 4, dtype=np.uint64))
    f0, f1 = box_muller(r[:, 0], r[:, 1])
    f2, f3 = box_muller(r[:, 2], r[:, 3])
    return np.stack([f0, f1, f2, f3], axis=1).reshape(-1)[:n]


def tf_truncated_normal(n: int, seed: int) -> np.ndarray:
    """Group g of four outputs reads single samples from counter 256 g on and keeps normals with |f| < 2."""
    out = np.empty(((n + 3) // 4) * 4, np.float32)
    for g in range((n + 3) // 4):
        got, block = 0, 0
        while got < 4:
            r = _philox_blocks(seed, np.array([256 * g + block], np.uint64))[0]
            block += 1
            for a, b in ((0, 1), (2, 3)):
                for f in box_muller(r[a:a + 1], r[b:b + 1]):
                    if got < 4 and abs(float(f[0])) < 2.0:
                        out[4 * g + got] = f[0]
                        got += 1
                if got >= 4:
                    break
    return out[:n]


def initializer_fans(shape) -> Tuple[int, int]:
    """Initializer.fans (Initializer.scala:16-25), including its `out :: in :: receptive` reading of rank > 2."""
    s = list(shape)
    if not s:
        return 1, 1
    if len(s) == 1:
        return s[0], s[0]
    if len(s) == 2:
        return s[0], s[1]
    size = int(np.prod(s[2:]))
    return size * s[1], size * s[0]


_TRUNC_COEF = F32(0.87962566103423978)     # Initializer.scala:30


def tf_rand(shape, dist: str, seed: int, scale=None, shift=None) -> np.ndarray:
    """`rand` (math/rand/AllKernels.scala:68-81): draw, then `* scale`, then `+ shift`, each only when given."""
    n = int(np.prod(shape)) if len(shape) else 1
    x = {"uniform": tf_random_uniform, "normal": tf_random_normal, "truncated": tf_truncated_normal}[dist](n, seed)
    if scale is not None:
        x = x * F32(scale)
    if shift is not None:
        x = x + F32(shift)
    return x.reshape(shape)


def initialize(name: str, shape, seed: int, **kw) -> np.ndarray:
    """The seeded initializers of models/Initializer.scala:48-219 by name."""
    shape = tuple(shape)
    fan_in, fan_out = initializer_fans(shape)
    sq = lambda v: F32(math.sqrt(float(F32(v))))            # `math.sqrt(6f / n).toFloat`
    if name == "RandomUniform":
        lo, hi = F32(kw.get("min", -0.05)), F32(kw.get("max", 0.05))
        return tf_rand(shape, "uniform", seed, hi - lo, lo)
    if name == "RandomNormal":
        return tf_rand(shape, "normal", seed, kw.get("std", 0.05), kw.get("mean", 0.0))
    if name == "RandomNormalTruncated":
        return tf_rand(shape, "truncated", seed, kw.get("std", 0.05), kw.get("mean", 0.0))
    if name in ("GlorotUniform", "HeUniform", "LecunUniform"):
        limit = {"GlorotUniform": sq(F32(6.0) / F32(fan_in + fan_out)), "HeUniform": sq(F32(6.0) / F32(fan_in)),
                 "LecunUniform": sq(F32(3.0) / F32(fan_in))}[name]
        return tf_rand(shape, "uniform", seed, F32(2.0) * limit, -limit)
    if name in ("GlorotNormal", "HeNormal", "LecunNormal"):
        std = {"GlorotNormal": sq(F32(2.0) / F32(fan_in + fan_out)), "HeNormal": sq(F32(2.0) / F32(fan_in)),
               "LecunNormal": sq(F32(1.0) / F32(fan_in))}[name] / _TRUNC_COEF
        return tf_rand(shape, "truncated", seed, std)
    if name == "Orthogonal":                                # Initializer.scala:202-219
        rows, cols = int(np.prod(shape[:-1])), shape[-1]
        a = tf_rand((max(rows, cols), min(rows, cols)), "normal", seed)
        q, r = np.linalg.qr(a)
        q = q * np.sign(np.diag(r))
        if rows < cols:
            q = q.T
        if kw.get("gain") is not None:
            q = q * F32(kw["gain"])
        return q.reshape(shape).astype(np.float32)
    raise ValueError(name)
