"""Host-side mirror of scanet's user-facing training DSL on top of the HIP library.

    model = Dense(50, Sigmoid) >> Dense(10, Softmax)
    trained = ds.train(model).loss(CategoricalCrossentropy).using(Adam(0.01)).batch(1000).epochs(10).run()
    accuracy(trained, test_ds)

Names, defaults and semantics follow the reference (paths under src/main/scala/scanet/):
layers models/layer/*.scala, activations models/Activation.scala, losses models/Loss.scala,
algorithms optimizers/*.scala, the builder optimizers/Optimizer.scala:267-310, the epoch
loop optimizers/Optimizer.scala:59-161 and `accuracy` estimators/package.scala:18-47.
The Spark partitions of the reference become K device-resident replicas that are averaged
on the GPU after every epoch.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field, replace
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import _lib as L
from .core import CompiledModel, Context, DeviceBuffer, Replica, average_replicas
from .formats import TensorBoard

# --------------------------------------------------------------------------- activations / losses / misc


@dataclass(frozen=True)
class Activation:
    kind: int
    param: float = 0.0
    name: str = ""

    @property
    def identity(self) -> bool:
        return self.kind == L.ACT_IDENTITY

    def __repr__(self):
        return self.name


Identity = Activation(L.ACT_IDENTITY, name="Identity")
Sigmoid = Activation(L.ACT_SIGMOID, name="Sigmoid")
Tanh = Activation(L.ACT_TANH, name="Tanh")
Softmax = Activation(L.ACT_SOFTMAX, name="Softmax")


def ReLU(threshold: float = 0.0) -> Activation:
    return Activation(L.ACT_RELU, float(threshold), f"ReLU({float(threshold)})")


@dataclass(frozen=True)
class Loss:
    kind: int
    name: str

    def __repr__(self):
        return self.name


MeanSquaredError = Loss(L.LOSS_MSE, "MeanSquaredError")
BinaryCrossentropy = Loss(L.LOSS_BINARY_CROSSENTROPY, "BinaryCrossentropy")
CategoricalCrossentropy = Loss(L.LOSS_CATEGORICAL_CROSSENTROPY, "CategoricalCrossentropy")
IdentityLoss = Loss(L.LOSS_IDENTITY, "Identity")


@dataclass(frozen=True)
class Regularization:
    kind: int = L.REG_NONE
    lam: float = 0.0


Zero = Regularization()


def L1(lam: float = 0.01) -> Regularization:
    return Regularization(L.REG_L1, lam)


def L2(lam: float = 0.01) -> Regularization:
    return Regularization(L.REG_L2, lam)


Valid, Same = L.PAD_VALID, L.PAD_SAME
_PAD_NAME = {Valid: "Valid", Same: "Same"}


@dataclass(frozen=True)
class Explicit:
    """`Padding.Explicit((pad_top, pad_bottom), (pad_left, pad_right))` (math/nn/AllKernels.scala:67-100); Conv2D only."""
    height: Tuple[int, int]
    width: Tuple[int, int]

    def __repr__(self):
        return f"Explicit({tuple(self.height)},{tuple(self.width)})"


# --------------------------------------------------------------------------- initializers (models/Initializer.scala)


def fans(shape: Sequence[int]) -> Tuple[int, int]:
    """Initializer.fans (Initializer.scala:16-25), including its rank > 2 rule `out :: in :: receptive`."""
    s = list(shape)
    if len(s) == 0:
        return 1, 1
    if len(s) == 1:
        return s[0], s[0]
    if len(s) == 2:
        return s[0], s[1]
    size = int(np.prod(s[2:]))
    return size * s[1], size * s[0]


_TRUNC_COEF = np.float32(0.87962566103423978)     # Initializer.scala:30


def _sqrt32(v) -> np.float32:
    return np.float32(math.sqrt(float(np.float32(v))))     # `math.sqrt(6f / n).toFloat`


@dataclass(frozen=True)
class Initializer:
    """models/Initializer.scala:28-219.  Random draws are made on the device by `sn_random_fill`, which produces the
    stream of the TensorFlow op the reference uses: a seeded initializer gives the reference's values.  Without a
    seed the reference lets TensorFlow pick one at random; here it is taken from the builder's generator."""
    name: str
    value: float = 0.0
    seed: Optional[int] = None
    args: Tuple[float, ...] = ()

    def build(self, shape, ctx: Context, rng: np.random.Generator) -> np.ndarray:
        shape = tuple(int(d) for d in shape)
        if self.name == "Zeros":
            return np.zeros(shape, np.float32)
        if self.name == "Ones":
            return np.ones(shape, np.float32)
        if self.name == "Const":
            return np.full(shape, self.value, np.float32)
        seed = int(self.seed) if self.seed is not None else int(rng.integers(1, 2 ** 31))
        fan_in, fan_out = fans(shape)
        f32 = np.float32
        if self.name == "RandomUniform":                      # Initializer.scala:48-53
            lo, hi = f32(self.args[0]), f32(self.args[1])
            return ctx.random(shape, L.RANDOM_UNIFORM, seed, float(hi - lo), float(lo))
        if self.name == "RandomNormal":                       # :55-60
            return ctx.random(shape, L.RANDOM_NORMAL, seed, self.args[1], self.args[0])
        if self.name == "RandomNormalTruncated":              # :62-70
            return ctx.random(shape, L.RANDOM_TRUNCATED_NORMAL, seed, self.args[1], self.args[0])
        if self.name in ("GlorotUniform", "HeUniform", "LecunUniform"):     # :83-90, 121-128, 159-166
            limit = {"GlorotUniform": _sqrt32(f32(6.0) / f32(fan_in + fan_out)), "HeUniform": _sqrt32(f32(6.0) / f32(fan_in)),
                     "LecunUniform": _sqrt32(f32(3.0) / f32(fan_in))}[self.name]
            return ctx.random(shape, L.RANDOM_UNIFORM, seed, float(f32(2.0) * limit), float(-limit))
        if self.name in ("GlorotNormal", "HeNormal", "LecunNormal"):        # :103-110, 140-147, 178-185
            std = {"GlorotNormal": _sqrt32(f32(2.0) / f32(fan_in + fan_out)), "HeNormal": _sqrt32(f32(2.0) / f32(fan_in)),
                   "LecunNormal": _sqrt32(f32(1.0) / f32(fan_in))}[self.name] / _TRUNC_COEF
            return ctx.random(shape, L.RANDOM_TRUNCATED_NORMAL, seed, float(std))
        if self.name == "Orthogonal":                         # :202-219; the QR of the small matrix stays on the host
            if len(shape) < 2:
                raise ValueError(f"requirement failed: at least rank 2 is required but was {len(shape)}")
            rows, cols = int(np.prod(shape[:-1])), shape[-1]
            a = ctx.random((max(rows, cols), min(rows, cols)), L.RANDOM_NORMAL, seed)
            q, rr = np.linalg.qr(a)
            q = q * np.sign(np.diag(rr))
            if rows < cols:
                q = q.T
            if self.args:
                q = q * np.float32(self.args[0])
            return np.ascontiguousarray(q.reshape(shape), np.float32)
        raise ValueError(self.name)


Zeros, Ones = Initializer("Zeros"), Initializer("Ones")


def Const(v: float) -> Initializer:
    return Initializer("Const", float(v))


def RandomUniform(min: float = -0.05, max: float = 0.05, seed: Optional[int] = None) -> Initializer:
    return Initializer("RandomUniform", seed=seed, args=(float(min), float(max)))


def RandomNormal(mean: float = 0.0, std: float = 0.05, seed: Optional[int] = None) -> Initializer:
    return Initializer("RandomNormal", seed=seed, args=(float(mean), float(std)))


def RandomNormalTruncated(mean: float = 0.0, std: float = 0.05, seed: Optional[int] = None) -> Initializer:
    return Initializer("RandomNormalTruncated", seed=seed, args=(float(mean), float(std)))


def GlorotUniform(seed: Optional[int] = None) -> Initializer:
    return Initializer("GlorotUniform", seed=seed)


def GlorotNormal(seed: Optional[int] = None) -> Initializer:
    return Initializer("GlorotNormal", seed=seed)


def HeUniform(seed: Optional[int] = None) -> Initializer:
    return Initializer("HeUniform", seed=seed)


def HeNormal(seed: Optional[int] = None) -> Initializer:
    return Initializer("HeNormal", seed=seed)


def LecunUniform(seed: Optional[int] = None) -> Initializer:
    return Initializer("LecunUniform", seed=seed)


def LecunNormal(seed: Optional[int] = None) -> Initializer:
    return Initializer("LecunNormal", seed=seed)


def Orthogonal(gain: Optional[float] = None, seed: Optional[int] = None) -> Initializer:
    return Initializer("Orthogonal", seed=seed, args=() if gain is None else (float(gain),))


# --------------------------------------------------------------------------- layers


@dataclass(frozen=True)
class Layer:
    """One primitive layer; `>>` composes (layer/Layer.scala:24-31)."""
    kind: int
    text: str
    units: int = 0
    activation: Activation = Identity
    kernel: Tuple[int, int] = (0, 0)
    strides: Tuple[int, int] = (1, 1)
    padding: int = Valid
    reg: Regularization = Zero
    use_bias: bool = True
    inits: Tuple[Initializer, ...] = ()
    explicit: Tuple[int, int, int, int] = (0, 0, 0, 0)   # Conv2D with explicit padding: top, bottom, left, right
    return_sequence: bool = False  # RNN layers only
    momentum: float = 0.99        # BatchNorm only
    epsilon: float = 1e-3
    fused: int = -1               # BatchNorm `fused`: -1 None, 0 Some(false), 1 Some(true)
    pool_reduce: int = 0          # Pool2D: L.POOL_MAX or L.POOL_AVG
    recurrent_reg: Regularization = Zero   # RNN layers: `recurrentReg`, `biasReg` (`reg` is their `kernelReg`)
    bias_reg: Regularization = Zero
    stateful: bool = False        # RNN layers: the state the last step leaves starts the next batch (layer/RNN.scala:27)

    def __rshift__(self, other):
        return Composed.of(self, other)

    @property
    def layers(self) -> List["Layer"]:
        return [self]

    def desc(self) -> L.LayerDesc:
        return L.LayerDesc(self.kind, self.units, self.activation.kind, self.activation.param, self.kernel[0], self.kernel[1],
                           self.strides[0], self.strides[1], self.padding, self.reg.kind, self.reg.lam, 1 if self.use_bias else 0,
                           1 if self.return_sequence else 0, self.momentum, self.epsilon,
                           self.explicit[0], self.explicit[1], self.explicit[2], self.explicit[3], self.fused,
                           self.recurrent_reg.kind, self.recurrent_reg.lam, self.bias_reg.kind, self.bias_reg.lam, self.pool_reduce,
                           1 if self.stateful else 0)

    def __repr__(self):
        return self.text


class Composed:
    """Flattened sequence of layers (layer/Composed.scala:14-103)."""

    def __init__(self, layers: Sequence[Layer]):
        if not layers:
            raise ValueError("requirement failed: at least 1 layer is required")
        self.layers = list(layers)

    @staticmethod
    def of(left, right):
        return Composed(list(left.layers) + list(right.layers))

    def __rshift__(self, other):
        return Composed.of(self, other)

    def __repr__(self):
        return " >> ".join(repr(l) for l in self.layers)


def _chain(first: Layer, *rest: Optional[Layer]):
    out = [first] + [l for l in rest if l is not None]
    return out[0] if len(out) == 1 else Composed(out)


def Bias(features: int, reg: Regularization = Zero, initializer: Initializer = Zeros) -> Layer:
    return Layer(L.LAYER_BIAS, f"Bias({features})", units=features, reg=reg, inits=(initializer,))


def Activate(activation: Activation) -> Layer:
    return Layer(L.LAYER_ACTIVATE, repr(activation), activation=activation)


def Dense(outputs: int, activation: Activation = Identity, reg: Regularization = Zero, bias: bool = True,
          kernelInitializer: Initializer = GlorotUniform(), biasInitializer: Initializer = Zeros):
    """layer/Dense.scala:30-40: Dense ?>> Bias ?>> Activate."""
    dense = Layer(L.LAYER_DENSE, f"Dense({outputs})", units=outputs, reg=reg, inits=(kernelInitializer,))
    return _chain(dense, Bias(outputs, reg, biasInitializer) if bias else None,
                  Activate(activation) if not activation.identity else None)


def Conv2D(filters: int, kernel: Tuple[int, int] = (3, 3), strides: Tuple[int, int] = (1, 1), padding: int = Valid,
           activation: Activation = Identity, bias: bool = False, kernelInitializer: Initializer = GlorotUniform(),
           biasInitializer: Initializer = Zeros):
    """layer/Conv2D.scala:54-68; `padding` is Valid, Same or an `Explicit(..)`."""
    explicit = (0, 0, 0, 0)
    pad_name = repr(padding) if isinstance(padding, Explicit) else _PAD_NAME[padding]
    if isinstance(padding, Explicit):
        explicit = (int(padding.height[0]), int(padding.height[1]), int(padding.width[0]), int(padding.width[1]))
        padding = L.PAD_EXPLICIT
    conv = Layer(L.LAYER_CONV2D, f"Conv2D({filters},{tuple(kernel)},{tuple(strides)},{pad_name},NHWC)".replace(" ", ""),
                 units=filters, kernel=tuple(kernel), strides=tuple(strides), padding=padding, explicit=explicit,
                 inits=(kernelInitializer,))
    return _chain(conv, Bias(filters, Zero, biasInitializer) if bias else None,
                  Activate(activation) if not activation.identity else None)


ReduceMax, ReduceAvg = "Max", "Avg"


def Pool2D(window: Tuple[int, int] = (2, 2), strides: Tuple[int, int] = (1, 1), padding: int = Valid, reduce: str = ReduceMax,
           as_reference_layer: bool = True) -> Layer:
    """layer/Pool2D.scala:28-42.  The reference's layer does not hand `reduce` to `pool2D` when it builds its graph
    (:36-42), so a model with `reduce = Avg` max-pools there; `as_reference_layer=True` (the default) does the same.
    With `as_reference_layer=False` the layer computes what the kernel function `pool2D(reduce = Avg)` computes
    (math/nn/AllKernels.scala:326-397)."""
    if reduce not in (ReduceMax, ReduceAvg):
        raise ValueError(f"reduce should be Max or Avg, got {reduce!r}")
    avg = reduce == ReduceAvg and not as_reference_layer
    return Layer(L.LAYER_POOL2D, f"Pool2D({tuple(window)},{tuple(strides)},{_PAD_NAME[padding]},NHWC,{reduce})".replace(" ", ""),
                 kernel=tuple(window), strides=tuple(strides), padding=padding, pool_reduce=L.POOL_AVG if avg else L.POOL_MAX)


Flatten = Layer(L.LAYER_FLATTEN, "Flatten")


def LSTM(units: int, bias: bool = True, kernelInitializer: Initializer = GlorotUniform(),
         recurrentInitializer: Initializer = Orthogonal(), biasInitializer: Initializer = Zeros,
         biasForgetInitializer: Initializer = Ones, returnSequence: bool = False, kernelReg: Regularization = Zero,
         recurrentReg: Regularization = Zero, biasReg: Regularization = Zero, stateful: bool = False) -> Layer:
    """layer/RNN.scala:208-258: tanh cell, sigmoid gates, forget bias one; the three regularizers apply to every gate."""
    return Layer(L.LAYER_LSTM, f"RNN(LSTMCell({units},Tanh,Sigmoid,{'true' if bias else 'false'}))", units=units,
                 activation=Tanh, use_bias=bias, return_sequence=returnSequence, reg=kernelReg, recurrent_reg=recurrentReg,
                 bias_reg=biasReg, stateful=stateful,
                 inits=(kernelInitializer, recurrentInitializer, biasInitializer, biasForgetInitializer))


def BatchNorm(axes: Sequence[int] = (-1,), momentum: float = 0.99, epsilon: float = 1e-3, betaInitializer: Initializer = Zeros,
              gammaInitializer: Initializer = Ones, movingMeanInitializer: Initializer = Zeros,
              movingVarianceInitializer: Initializer = Ones, fused: Optional[bool] = None,
              betaRegularizer: Regularization = Zero, gammaRegularizer: Regularization = Zero) -> Layer:
    """layer/BatchNorm.scala:64-76 over the last axis.  As in the reference, rank-4 input takes the FusedBatchNormV3
    branch unless `fused=False` (wired as the reference wires that op's outputs, which is not the generic form's
    gradient nor its moving variance); every other rank takes the generic form.  The reference's penalty is
    betaRegularizer(gamma) + betaRegularizer(gamma) (:158-160); `gammaRegularizer` is accepted and, as there, unused."""
    if tuple(axes) != (-1,):
        raise ValueError("only axes = Seq(-1) is built")
    return Layer(L.LAYER_BATCHNORM, f"BatchNorm({list(axes)})", momentum=momentum, epsilon=epsilon,
                 fused=-1 if fused is None else int(bool(fused)), reg=betaRegularizer,
                 inits=(betaInitializer, gammaInitializer, movingMeanInitializer, movingVarianceInitializer))


def SimpleRNN(units: int, activation: Activation = Tanh, bias: bool = True, kernelInitializer: Initializer = GlorotUniform(),
              recurrentInitializer: Initializer = Orthogonal(), biasInitializer: Initializer = Zeros,
              returnSequence: bool = False, kernelReg: Regularization = Zero, recurrentReg: Regularization = Zero,
              biasReg: Regularization = Zero, stateful: bool = False) -> Layer:
    """layer/RNN.scala:96-137: `RNN(SimpleRNNCell(..))`; the last step's output leaves the layer."""
    if activation.kind == L.ACT_SOFTMAX:
        raise ValueError("requirement failed: Softmax is not a cell activation")
    return Layer(L.LAYER_SIMPLE_RNN, f"RNN(SimpleRNNCell({units},{activation!r},{'true' if bias else 'false'}))", units=units,
                 activation=activation, use_bias=bias, return_sequence=returnSequence, reg=kernelReg, recurrent_reg=recurrentReg,
                 bias_reg=biasReg, stateful=stateful, inits=(kernelInitializer, recurrentInitializer, biasInitializer))


def LinearRegression(reg: Regularization = Zero, bias: bool = True):
    """models/LinearRegression.scala: Dense(1), zero-initialised."""
    return Dense(1, Identity, reg, bias, Zeros, Zeros)


def LogisticRegression(reg: Regularization = Zero, bias: bool = True):
    """models/LogisticRegression.scala: Dense(1, Sigmoid), zero-initialised."""
    return Dense(1, Sigmoid, reg, bias, Zeros, Zeros)


# --------------------------------------------------------------------------- algorithms


def _alg(kind, rate=0.0, beta1=0.0, beta2=0.0, epsilon=0.0, init_acc=0.0, nesterov=False) -> L.OptimizerDesc:
    return L.OptimizerDesc(kind, rate, beta1, beta2, epsilon, init_acc, 1 if nesterov else 0, 0)


def SGD(rate=0.01, momentum=0.0, nesterov=False):
    return _alg(L.OPT_SGD, rate, momentum, nesterov=nesterov)


def AdaGrad(rate=0.001, epsilon=1e-7):
    return _alg(L.OPT_ADAGRAD, rate, epsilon=epsilon)


def AdaDelta(rate=1.0, rho=0.9, epsilon=1e-7):
    return _alg(L.OPT_ADADELTA, rate, rho, epsilon=epsilon)


def RMSProp(rate=0.001, rho=0.9, epsilon=1e-7):
    return _alg(L.OPT_RMSPROP, rate, rho, epsilon=epsilon)


def Adam(rate=0.001, beta1=0.9, beta2=0.999, epsilon=1e-7):
    return _alg(L.OPT_ADAM, rate, beta1, beta2, epsilon)


def Nadam(beta1=0.9, beta2=0.999, epsilon=1e-7, initAcc=0.001):
    return _alg(L.OPT_NADAM, 0.0, beta1, beta2, epsilon, initAcc)


def Adamax(rate=0.001, beta1=0.9, beta2=0.999, epsilon=1e-7, initAcc=0.001):
    return _alg(L.OPT_ADAMAX, rate, beta1, beta2, epsilon, initAcc)


def AMSGrad(rate=0.001, beta1=0.9, beta2=0.999, epsilon=1e-7):
    return _alg(L.OPT_AMSGRAD, rate, beta1, beta2, epsilon)


STATE_NAMES = {
    L.OPT_SGD: ["velocity"], L.OPT_ADAGRAD: ["grad_acc"], L.OPT_ADADELTA: ["avg_grad", "avg_delta"],
    L.OPT_RMSPROP: ["avg_grad"], L.OPT_ADAM: ["momentum", "velocity"], L.OPT_NADAM: ["momentum", "velocity"],
    L.OPT_ADAMAX: ["momentum_1", "momentum_2"], L.OPT_AMSGRAD: ["momentum", "velocity", "corrected_velocity"],
}

# --------------------------------------------------------------------------- datasets / training


class Dataset:
    """Rows of (features, labels) with per-sample shapes, cut into `partitions` contiguous parts
    (the reference keeps shapes in Spark column metadata, optimizers/SparkExt.scala:16-33)."""

    def __init__(self, x, y, partitions: int = 1):
        self.x = np.ascontiguousarray(x, np.float32)
        self.y = np.ascontiguousarray(y, np.float32)
        if self.x.shape[0] != self.y.shape[0]:
            raise ValueError("features and labels differ in row count")
        self.partitions = int(partitions)

    @property
    def shapes(self):
        return self.x.shape[1:], self.y.shape[1:]

    def __len__(self):
        return self.x.shape[0]

    def coalesce(self, n: int) -> "Dataset":
        return Dataset(self.x, self.y, n)

    def split(self) -> List[Tuple[np.ndarray, np.ndarray]]:
        idx = np.array_split(np.arange(len(self)), self.partitions)
        return [(self.x[i[0]:i[-1] + 1], self.y[i[0]:i[-1] + 1]) for i in idx if len(i)]

    def train(self, model) -> "Builder":
        return Builder(model=model, dataset=self)


def minimize(model) -> "Builder":
    """`Optimizer.minimize(model)` (optimizers/Optimizer.scala:312-324)."""
    return Builder(model=model)


def maximize(model) -> "Builder":
    """`Optimizer.maximize(model)` (optimizers/Optimizer.scala:326-336): every update adds its delta."""
    return Builder(model=model, minimizing=False)


Skip, Partial, PadZeros = "Skip", "Partial", "PadZeros"


class TensorIterator:
    """optimizers/Iterators.scala:39-83: groups (features, labels) records into batches of `batch` rows.  What is left
    over at the end is dropped (`Skip`, what the optimizer uses, Optimizer.scala:115), handed out short (`Partial`, what
    the estimators use, estimators/package.scala:25) or filled up with zero rows (`PadZeros`)."""

    def __init__(self, rows, shapes, batch: int, remaining: str = Skip):
        if remaining not in (Skip, Partial, PadZeros):
            raise ValueError(f"remaining should be Skip, Partial or PadZeros, got {remaining!r}")
        self._rows = iter(rows)
        self.shape_x, self.shape_y = tuple(shapes[0]), tuple(shapes[1])
        self.batch = int(batch)
        self.remaining = remaining
        self._group = None

    def _fill(self):
        if self._group is None:
            group = []
            for record in self._rows:
                group.append(record)
                if len(group) == self.batch:
                    break
            if group and (len(group) == self.batch or self.remaining != Skip):
                self._group = group
        return self._group is not None

    def __iter__(self):
        return self

    def has_next(self) -> bool:
        return self._fill()

    def __next__(self):
        if not self._fill():
            raise StopIteration
        group, self._group = self._group, None
        rows = self.batch if self.remaining == PadZeros else len(group)
        x = np.zeros((rows,) + self.shape_x, np.float32)
        y = np.zeros((rows,) + self.shape_y, np.float32)
        for i, (fx, fy) in enumerate(group):
            x[i] = np.asarray(fx, np.float32).reshape(self.shape_x)
            y[i] = np.asarray(fy, np.float32).reshape(self.shape_y)
        return x, y


def _init_params(model, compiled: CompiledModel, seed: int) -> Dict[str, np.ndarray]:
    """ParamDef.initialize for every weight (optimizers/Optimizer.scala:124-128)."""
    rng = np.random.default_rng(seed)
    layers = model.layers
    single = len(layers) == 1
    out: Dict[str, np.ndarray] = {}
    shapes = {p: s for p, s, _ in compiled.params}
    for i, l in enumerate(layers):
        pre = "" if single else f"{i}/"
        if l.kind in (L.LAYER_DENSE, L.LAYER_BIAS, L.LAYER_CONV2D):
            out[pre + "weights"] = l.inits[0].build(shapes[pre + "weights"], compiled.ctx, rng)
        elif l.kind == L.LAYER_BATCHNORM:
            for name, init in zip(("beta", "gamma", "moving_mean", "moving_variance"), l.inits):
                out[pre + name] = init.build(shapes[pre + name], compiled.ctx, rng)
        elif l.kind == L.LAYER_SIMPLE_RNN:
            if l.stateful:
                out[pre + "0/state"] = np.zeros(shapes[pre + "0/state"], np.float32)          # RNN.scala:188
            k_init, r_init, b_init = l.inits
            out[pre + "0/kernel_weights"] = k_init.build(shapes[pre + "0/kernel_weights"], compiled.ctx, rng)
            out[pre + "0/recurrent_weights"] = r_init.build(shapes[pre + "0/recurrent_weights"], compiled.ctx, rng)
            if l.use_bias:
                out[pre + "1/weights"] = b_init.build(shapes[pre + "1/weights"], compiled.ctx, rng)
        elif l.kind == L.LAYER_LSTM:
            if l.stateful:
                for name in ("cell_state", "hidden_state"):                                      # RNN.scala:302-303
                    out[pre + name] = np.zeros(shapes[pre + name], np.float32)
            k_init, r_init, b_init, bf_init = l.inits
            for gate in ("forget", "input", "gate", "output"):
                out[f"{pre}{gate}/0/kernel_weights"] = k_init.build(shapes[f"{pre}{gate}/0/kernel_weights"], compiled.ctx, rng)
                out[f"{pre}{gate}/0/recurrent_weights"] = r_init.build(shapes[f"{pre}{gate}/0/recurrent_weights"], compiled.ctx, rng)
                if l.use_bias:
                    b = bf_init if gate == "forget" else b_init
                    out[f"{pre}{gate}/1/weights"] = b.build(shapes[f"{pre}{gate}/1/weights"], compiled.ctx, rng)
    return out


@dataclass
class TrainedModel:
    """`TrainedModel` (models/Model.scala:154-187): a model, its loss and the learned parameters."""
    model: object
    loss_fn: Loss
    params: Dict[str, np.ndarray]
    opt_state: Dict[str, List[np.ndarray]]
    history: List[float]
    iterations: int
    input_shape: Tuple[int, ...]
    flags: int = 0
    ctx: Optional[Context] = None

    def _run(self, x, batch, fn):
        x = np.ascontiguousarray(x, np.float32)
        ctx = self.ctx or Context()
        try:
            cm = CompiledModel(ctx, [l.desc() for l in self.model.layers], self.loss_fn.kind, self.input_shape, batch, self.flags)
            rep = cm.replica(None)
            rep.set_params(self.params)
            try:
                return fn(ctx, cm, rep)
            finally:
                rep.close()
                cm.close()
        finally:
            if self.ctx is None:
                ctx.close()

    def result(self, x) -> np.ndarray:
        x = np.ascontiguousarray(x, np.float32)

        def go(ctx, cm, rep):
            xb = ctx.to_device(x)
            try:
                return rep.forward(xb, x.shape[0])
            finally:
                xb.free()
        return self._run(x, x.shape[0], go)

    def loss(self, x, y) -> float:
        x = np.ascontiguousarray(x, np.float32)

        def go(ctx, cm, rep):
            xb, yb = ctx.to_device(x), ctx.to_device(y)
            try:
                return rep.loss(xb, yb, x.shape[0])
            finally:
                xb.free()
                yb.free()
        return self._run(x, x.shape[0], go)


def accuracy(trained: TrainedModel, ds: Dataset, batch: int = 1000) -> float:
    """estimators.accuracy (estimators/package.scala:18-47): batches of `batch` rows, the last one partial."""
    n = len(ds)
    batch = min(batch, n)

    def go(ctx, cm, rep):
        positives = 0
        for s in range(0, n, batch):
            xs, ys = ds.x[s:s + batch], ds.y[s:s + batch]
            xb, yb = ctx.to_device(xs), ctx.to_device(ys)
            try:
                positives += rep.count_correct(xb, yb, xs.shape[0])
            finally:
                xb.free()
                yb.free()
        return positives / n
    return trained._run(ds.x, batch, go)


def _mean_error(trained: TrainedModel, ds: Dataset, batch: int, kind: int) -> float:
    """estimators.meanError (estimators/package.scala:72-101): per-batch error sums (on the device), added in float
    on the host, divided by the number of rows."""
    n = len(ds)
    batch = min(batch, n)

    def go(ctx, cm, rep):
        total = np.float32(0.0)
        for s in range(0, n, batch):
            xs, ys = ds.x[s:s + batch], ds.y[s:s + batch]
            xb, yb = ctx.to_device(xs), ctx.to_device(ys)
            try:
                total = np.float32(total + np.float32(rep.error_sum(xb, yb, kind, xs.shape[0])))
            finally:
                xb.free()
                yb.free()
        return float(total / np.float32(n))
    return trained._run(ds.x, batch, go)


def MSE(trained: TrainedModel, ds: Dataset, batch: int = 1000) -> float:
    """estimators.MSE (estimators/package.scala:56-62)."""
    return _mean_error(trained, ds, batch, L.ERROR_SQUARED)


def RMSE(trained: TrainedModel, ds: Dataset, batch: int = 1000) -> float:
    """estimators.RMSE (estimators/package.scala:50-54)."""
    return float(np.float32(math.sqrt(MSE(trained, ds, batch))))


def MAE(trained: TrainedModel, ds: Dataset, batch: int = 1000) -> float:
    """estimators.MAE (estimators/package.scala:64-70)."""
    return _mean_error(trained, ds, batch, L.ERROR_ABSOLUTE)


def R2Score(trained: TrainedModel, ds: Dataset, batch: int = 1000) -> float:
    """estimators.R2Score (estimators/package.scala:103-138): predictions per batch from the device, the two sums in
    double on the host.  As in the reference the total sum of squares is taken around the mean PREDICTION
    (`mean = expectedVsPredicted.map(_._2)`, :126-131), not around the mean label."""
    if tuple(ds.y.shape[1:]) != (1,):
        raise ValueError("requirement failed: labels should have shape (1)")
    n = len(ds)
    batch = min(batch, n)

    def go(ctx, cm, rep):
        preds = []
        for s in range(0, n, batch):
            xs = ds.x[s:s + batch]
            xb = ctx.to_device(xs)
            try:
                preds.append(rep.forward(xb, xs.shape[0]).reshape(-1))
            finally:
                xb.free()
        predicted = np.concatenate(preds).astype(np.float64)
        expected = ds.y.reshape(-1).astype(np.float64)
        mean = predicted.mean()
        ssr = float(((predicted - expected) ** 2).sum())
        sst = float(((predicted - mean) ** 2).sum())
        return float(np.float32(1.0 - ssr / sst))
    return trained._run(ds.x, batch, go)


class RecordLoss:
    """Effect.RecordLoss (optimizers/Effect.scala:41-52): the epoch's loss to the console and, if asked, as the
    scalar "loss" at the current iteration to the builder's TensorBoard directory."""
    wants_context = True

    def __init__(self, console: bool = True, tensorboard: bool = False):
        self.console, self.tensorboard = console, tensorboard

    def __call__(self, epoch, iterations, loss, board=None, trained=None, batch=None):
        if self.tensorboard and board is not None:
            board.add_scalar("loss", loss, iterations)
        if self.console:
            print(f"{epoch}/{iterations} loss: {loss}")


class RecordAccuracy:
    """Effect.RecordAccuracy (optimizers/Effect.scala:54-66): accuracy of the model as trained so far on `ds`."""
    wants_context = True

    def __init__(self, ds: "Dataset", console: bool = True, tensorboard: bool = False):
        self.ds, self.console, self.tensorboard = ds, console, tensorboard

    def __call__(self, epoch, iterations, loss, board=None, trained=None, batch=None):
        a = accuracy(trained(), self.ds, batch or 1000)
        if self.tensorboard and board is not None:
            board.add_scalar("accuracy", a, iterations)
        if self.console:
            print(f"{epoch}/{iterations} accuracy: {a}")


@dataclass
class Builder:
    """The type-state builder of the reference without the types (optimizers/Optimizer.scala:267-310)."""
    model: object
    dataset: Optional[Dataset] = None
    loss_fn: Optional[Loss] = None
    alg: Optional[L.OptimizerDesc] = None
    batch_size: int = 10000                      # Optimizer.scala:321
    n_epochs: Optional[int] = None
    n_iterations: Optional[int] = None
    init: Optional[Callable[[], Dict[str, np.ndarray]]] = None
    effects: List[Callable] = field(default_factory=list)
    flags: int = 0
    seed: int = 0
    device: int = 0
    board_dir: str = "board"                     # Optimizer.scala:54
    minimizing: bool = True                      # Optimizer.scala:186: w - delta, or w + delta for `Optimizer.maximize`

    def board(self, directory: str):
        """Directory of the TensorBoard event files effects write (Optimizer.scala:297-298)."""
        return replace(self, board_dir=directory)

    def loss(self, loss: Loss):
        return replace(self, loss_fn=loss)

    def using(self, alg: L.OptimizerDesc):
        return replace(self, alg=alg)

    def initParams(self, params):
        return replace(self, init=(params if callable(params) else (lambda: params)))

    def on(self, dataset: Dataset):
        return replace(self, dataset=dataset)

    def batch(self, size: int):
        return replace(self, batch_size=int(size))

    def epochs(self, number: int):
        return replace(self, n_epochs=int(number))

    stopAfterEpochs = epochs

    def iterations(self, number: int):
        return replace(self, n_iterations=int(number))

    def each(self, effect: Callable):
        """effect(epoch, iterations, loss) after every epoch (optimizers/Effect.scala)."""
        return replace(self, effects=self.effects + [effect])

    def bf16(self, on: bool = True):
        return replace(self, flags=(self.flags | L.FLAG_GEMM_BF16) if on else (self.flags & ~L.FLAG_GEMM_BF16))

    def run(self) -> TrainedModel:
        for name, v in (("loss", self.loss_fn), ("using", self.alg), ("on/train", self.dataset)):
            if v is None:
                raise ValueError(f"builder is incomplete: call .{name}(..) first")
        if self.n_epochs is None and self.n_iterations is None:
            raise ValueError("builder is incomplete: call .epochs(..) or .iterations(..) first")
        ds = self.dataset
        in_shape, _ = ds.shapes
        parts = ds.split()
        ctx = Context(self.device)
        bufs: List[DeviceBuffer] = []
        reps: List[Replica] = []
        cm = None
        try:
            cm = CompiledModel(ctx, [l.desc() for l in self.model.layers], self.loss_fn.kind, in_shape, self.batch_size, self.flags)
            params = self.init() if self.init else _init_params(self.model, cm, self.seed)
            data = []
            for px, py in parts:
                xb, yb = ctx.to_device(px), ctx.to_device(py)
                bufs += [xb, yb]
                data.append((xb, yb, px.shape[0]))
                alg = L.OptimizerDesc.from_buffer_copy(self.alg)
                alg.maximize = 0 if self.minimizing else 1
                rep = cm.replica(alg)
                rep.set_params(params)
                reps.append(rep)
            global_iter, epoch, history = 0, 0, []
            board = None
            while True:
                iters, losses = 0, []
                for rep, (xb, yb, rows) in zip(reps, data):       # one partition after the other on the one GPU
                    it, lo = rep.train_epoch(xb, yb, rows, self.batch_size, global_iter)
                    iters += it
                    losses.append(lo)
                average_replicas(reps)                              # Optimizer.scala:86,196-230
                loss = float(np.mean(np.asarray(losses, np.float32)))   # `(l.loss + r.loss) / 2`, uniform over K here
                global_iter += iters                                # Optimizer.scala:88
                epoch += 1
                history.append(loss)
                for e in self.effects:
                    if getattr(e, "wants_context", False):
                        if board is None and getattr(e, "tensorboard", False):
                            board = TensorBoard(self.board_dir)
                        e(epoch, global_iter, loss, board=board, batch=self.batch_size,
                          trained=lambda: TrainedModel(self.model, self.loss_fn, reps[0].get_params(), {}, list(history), global_iter,
                                                       tuple(in_shape), self.flags))
                    else:
                        e(epoch, global_iter, loss)
                if (self.n_epochs is not None and epoch >= self.n_epochs) or \
                        (self.n_iterations is not None and global_iter >= self.n_iterations):
                    break
            final = reps[0].get_params()
            n_states = len(STATE_NAMES[self.alg.kind])
            slots = [reps[0].get_opt_state(s) for s in range(n_states)]
            opt_state = {p: [slots[s][p] for s in range(n_states)] for p in final if p not in cm.state_paths}   # weights only
            return TrainedModel(self.model, self.loss_fn, final, opt_state, history, global_iter, tuple(in_shape), self.flags)
        finally:
            for r in reps:
                r.close()
            if cm is not None:
                cm.close()
            for b in bufs:
                b.free()
            ctx.close()
