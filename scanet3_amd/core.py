"""Thin object layer over the C ABI: context, device buffers, compiled model, replica.

Mirrors the reference's compile/execute boundary (core/Session.scala, core/TF.scala):
a `Context` plays the part of a `Session`, a `CompiledModel` is the compiled
`LossModel`, a `Replica` is one partition's parameters plus optimizer state.
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import _lib as L
from ._lib import check, lib


def _f32c(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


class Context:
    """One device + one HIP stream (reference: `Session`, core/Session.scala:55-107)."""

    def __init__(self, device: int = 0, stream: Optional[int] = None):
        h = C.c_void_p()
        check(lib.sn_ctx_create(device, C.c_void_p(stream) if stream else None, C.byref(h)))
        self.handle = h
        self.device = device
        self._pinned = []

    def close(self):
        if self.handle:
            for p in self._pinned:
                check(lib.sn_host_free(self.handle, p))
            self._pinned = []
            check(lib.sn_ctx_destroy(self.handle))
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def sync(self):
        check(lib.sn_sync(self.handle))

    def device_info(self) -> Tuple[str, int, int]:
        name = C.create_string_buffer(256)
        hbm, cu = C.c_int64(), C.c_int32()
        check(lib.sn_device_info(self.handle, name, 256, C.byref(hbm), C.byref(cu)))
        return name.value.decode(), hbm.value, cu.value

    # ---- memory -------------------------------------------------------------
    def pinned_array(self, shape) -> np.ndarray:
        """float32 numpy array over page-locked host memory (`sn_host_alloc`); freed when the context closes."""
        n = int(np.prod(shape))
        p = C.c_void_p()
        check(lib.sn_host_alloc(self.handle, max(n, 1) * 4, C.byref(p)))
        self._pinned.append(p)
        buf = (C.c_float * max(n, 1)).from_address(p.value)
        return np.frombuffer(buf, dtype=np.float32, count=n).reshape(shape)

    def alloc(self, n_floats: int) -> "DeviceBuffer":
        return DeviceBuffer(self, int(n_floats))

    def to_device(self, array) -> "DeviceBuffer":
        a = _f32c(array)
        buf = DeviceBuffer(self, a.size, a.shape)
        buf.copy_from(a)
        return buf

    # ---- flat kernels ---------------------------------------------------------
    def optimizer_update(self, desc: L.OptimizerDesc, w: "DeviceBuffer", g: "DeviceBuffer",
                         states: Sequence["DeviceBuffer"], iteration: int, n: Optional[int] = None):
        s = [st.ptr for st in states] + [None] * (3 - len(states))
        check(lib.sn_optimizer_update(self.handle, C.byref(desc), w.ptr, g.ptr, s[0], s[1], s[2],
                                      w.size if n is None else n, iteration))

    def average(self, inputs: Sequence["DeviceBuffer"], out: "DeviceBuffer", n: Optional[int] = None):
        arr = (C.c_void_p * len(inputs))(*[b.ptr for b in inputs])
        check(lib.sn_average(self.handle, arr, len(inputs), out.size if n is None else n, out.ptr))

    def random_fill(self, out: "DeviceBuffer", dist: int, seed: int, scale: Optional[float] = None,
                    shift: Optional[float] = None, n: Optional[int] = None):
        """`rand(shape, dist, seed, scale, shift)` (math/rand/AllKernels.scala:68-81) with TensorFlow's seeded stream."""
        sc = None if scale is None else C.byref(C.c_float(scale))
        sh = None if shift is None else C.byref(C.c_float(shift))
        ptr = out.ptr if isinstance(out, DeviceBuffer) else out          # a raw device pointer needs `n`
        count = out.size if n is None else n
        check(lib.sn_random_fill(self.handle, ptr, count, dist, C.c_uint64(seed), sc, sh))

    def random(self, shape, dist: int, seed: int, scale: Optional[float] = None, shift: Optional[float] = None) -> np.ndarray:
        shape = tuple(int(d) for d in shape)
        buf = DeviceBuffer(self, int(np.prod(shape)) if shape else 1, shape)
        try:
            self.random_fill(buf, dist, seed, scale, shift)
            return buf.numpy()
        finally:
            buf.free()

    # ---- per-kernel timing ------------------------------------------------------
    def profile(self, on: bool):
        check(lib.sn_profile_enable(self.handle, 1 if on else 0))

    def profile_reset(self):
        check(lib.sn_profile_reset(self.handle))

    def profile_report(self) -> Dict[str, Tuple[float, int]]:
        """{kernel name: (total milliseconds, launches)} since the last reset."""
        n = C.c_int32()
        check(lib.sn_profile_count(self.handle, C.byref(n)))
        out = {}
        for i in range(n.value):
            name = C.create_string_buffer(128)
            ms, cnt = C.c_double(), C.c_int64()
            check(lib.sn_profile_get(self.handle, i, name, 128, C.byref(ms), C.byref(cnt)))
            out[name.value.decode()] = (ms.value, cnt.value)
        return out


class DeviceBuffer:
    """float32 device memory owned by a context (reference: a device-resident `Tensor`)."""

    def __init__(self, ctx: Context, size: int, shape: Optional[Tuple[int, ...]] = None):
        self.ctx = ctx
        self.size = int(size)
        self.shape = tuple(shape) if shape is not None else (self.size,)
        p = C.c_void_p()
        check(lib.sn_buffer_alloc(ctx.handle, self.size * 4, C.byref(p)))
        self.ptr = p

    def free(self):
        if self.ptr and self.ctx.handle:
            check(lib.sn_buffer_free(self.ctx.handle, self.ptr))
        self.ptr = None

    def offset(self, n_floats: int) -> C.c_void_p:
        return C.c_void_p(self.ptr.value + 4 * int(n_floats))

    def copy_from(self, array):
        a = _f32c(array)
        if a.size != self.size:
            raise ValueError(f"buffer holds {self.size} floats, array has {a.size}")
        check(lib.sn_copy_h2d(self.ctx.handle, self.ptr, a.ctypes.data_as(C.c_void_p), a.nbytes))
        self.ctx.sync()          # `a` may be a temporary

    def fill(self, value: float):
        check(lib.sn_fill(self.ctx.handle, self.ptr, float(value), self.size))

    def numpy(self) -> np.ndarray:
        out = np.empty(self.size, np.float32)
        check(lib.sn_copy_d2h(self.ctx.handle, out.ctypes.data_as(C.c_void_p), self.ptr, out.nbytes))
        return out.reshape(self.shape)


class CompiledModel:
    """`model.withLoss(loss)` compiled for one input shape and batch size."""

    def __init__(self, ctx: Context, layer_descs: Sequence[L.LayerDesc], loss: int, input_shape: Sequence[int], batch: int,
                 flags: int = 0):
        self.ctx = ctx
        self.batch = int(batch)
        self.input_shape = tuple(int(d) for d in input_shape)
        arr = (L.LayerDesc * len(layer_descs))(*layer_descs)
        dims = (C.c_int64 * len(self.input_shape))(*self.input_shape)
        h = C.c_void_p()
        check(lib.sn_model_create(ctx.handle, arr, len(layer_descs), loss, dims, len(self.input_shape), self.batch, flags,
                                  C.byref(h)))
        self.handle = h
        n, flat = C.c_int32(), C.c_int64()
        check(lib.sn_model_param_count(h, C.byref(n), C.byref(flat)))
        self.flat_elems = flat.value
        self.params: List[Tuple[str, Tuple[int, ...], int]] = []     # (path, shape, offset)
        self.state_paths = set()     # layer state (`trainable = false`): no gradient, no optimizer state
        for i in range(n.value):
            info = L.ParamInfo()
            check(lib.sn_model_param_info(h, i, C.byref(info)))
            self.params.append((info.path.decode(), tuple(info.dims[:info.rank]), info.offset))
            if not info.trainable:
                self.state_paths.add(info.path.decode())
        rank, odims = C.c_int32(), (C.c_int64 * L.SN_MAX_RANK)()
        check(lib.sn_model_output_shape(h, C.byref(rank), odims))
        self.output_shape = tuple(odims[:rank.value])
        self.index = {p: i for i, (p, _, _) in enumerate(self.params)}

    @property
    def in_elems(self) -> int:
        return int(np.prod(self.input_shape))

    @property
    def out_elems(self) -> int:
        return int(np.prod(self.output_shape))

    def close(self):
        if self.handle:
            check(lib.sn_model_destroy(self.handle))
            self.handle = None

    def replica(self, opt: Optional[L.OptimizerDesc] = None) -> "Replica":
        return Replica(self, opt)


class Replica:
    """Weights + gradients + optimizer state of one partition (optimizers/Optimizer.scala:117-131)."""

    def __init__(self, model: CompiledModel, opt: Optional[L.OptimizerDesc]):
        self.model = model
        self.ctx = model.ctx
        self.opt = opt
        h = C.c_void_p()
        check(lib.sn_replica_create(model.handle, C.byref(opt) if opt is not None else None, C.byref(h)))
        self.handle = h

    def close(self):
        if self.handle:
            check(lib.sn_replica_destroy(self.handle))
            self.handle = None

    # ---- parameters -----------------------------------------------------------
    def set_params(self, params: Dict[str, np.ndarray]):
        for path, value in params.items():
            if path not in self.model.index:
                raise KeyError(f"missing {path} param")
            a = _f32c(value)
            check(lib.sn_params_set(self.handle, self.model.index[path], a.ctypes.data_as(C.c_void_p), a.size))

    def _get(self, fn, *lead, weights_only: bool = False) -> Dict[str, np.ndarray]:
        out = {}
        for i, (path, shape, _) in enumerate(self.model.params):
            if weights_only and path in self.model.state_paths:
                continue
            a = np.empty(int(np.prod(shape)) if shape else 1, np.float32)
            check(fn(self.handle, i, *lead, a.ctypes.data_as(C.c_void_p), a.size))
            out[path] = a.reshape(shape)
        return out

    def get_params(self) -> Dict[str, np.ndarray]:
        return self._get(lib.sn_params_get)

    def get_grads(self) -> Dict[str, np.ndarray]:
        return self._get(lib.sn_grads_get, weights_only=True)

    def get_opt_state(self, slot: int) -> Dict[str, np.ndarray]:
        return self._get(lib.sn_optstate_get, slot, weights_only=True)

    def set_opt_state(self, slot: int, values: Dict[str, np.ndarray]):
        for path, value in values.items():
            a = _f32c(value)
            check(lib.sn_optstate_set(self.handle, self.model.index[path], slot, a.ctypes.data_as(C.c_void_p), a.size))

    def flat(self, slot: int = -2) -> Tuple[C.c_void_p, int]:
        p, n = C.c_void_p(), C.c_int64()
        check(lib.sn_replica_flat(self.handle, slot, C.byref(p), C.byref(n)))
        return p, n.value

    # ---- compiled functions ------------------------------------------------------
    @staticmethod
    def _ptr(b):
        return b.ptr if isinstance(b, DeviceBuffer) else b

    def step(self, x, y, iteration: int, rows: Optional[int] = None, want_loss: bool = False) -> Optional[float]:
        loss = C.c_float()
        check(lib.sn_step(self.handle, self._ptr(x), self._ptr(y), self.model.batch if rows is None else rows, iteration,
                          C.byref(loss) if want_loss else None))
        return loss.value if want_loss else None

    def grad(self, x, y, rows: Optional[int] = None) -> float:
        loss = C.c_float()
        check(lib.sn_grad(self.handle, self._ptr(x), self._ptr(y), self.model.batch if rows is None else rows, C.byref(loss)))
        return loss.value

    def forward(self, x, rows: Optional[int] = None, training: bool = False) -> np.ndarray:
        """training=False: the frozen model (`TrainedModel.result`); True: `model.resultStateful`'s output."""
        rows = self.model.batch if rows is None else rows
        out = DeviceBuffer(self.ctx, rows * self.model.out_elems, (rows,) + self.model.output_shape)
        try:
            check((lib.sn_forward_training if training else lib.sn_forward)(self.handle, self._ptr(x), rows, out.ptr))
            return out.numpy()
        finally:
            out.free()

    def forward_static(self, x, out: "DeviceBuffer", rows: Optional[int] = None) -> None:
        """`sn_forward_static`: the frozen forward pass into the caller's buffer, with no device allocation in the call."""
        check(lib.sn_forward_static(self.handle, self._ptr(x), self.model.batch if rows is None else rows, self._ptr(out)))

    def loss(self, x, y, rows: Optional[int] = None) -> float:
        loss = C.c_float()
        check(lib.sn_loss(self.handle, self._ptr(x), self._ptr(y), self.model.batch if rows is None else rows, C.byref(loss)))
        return loss.value

    def error_sum(self, x, y, kind: int, rows: Optional[int] = None) -> float:
        """Sum of squared (kind 0) or absolute (kind 1) errors of the frozen model over one batch."""
        out = C.c_float()
        check(lib.sn_error_sum(self.handle, self._ptr(x), self._ptr(y), self.model.batch if rows is None else rows, kind, C.byref(out)))
        return out.value

    def count_correct(self, x, y, rows: Optional[int] = None) -> int:
        n = C.c_int64()
        check(lib.sn_count_correct(self.handle, self._ptr(x), self._ptr(y), self.model.batch if rows is None else rows,
                                   C.byref(n)))
        return n.value

    def train_epoch(self, x, y, total_rows: int, batch: int, global_iter: int, want_loss: bool = True) -> Tuple[int, Optional[float]]:
        it, loss = C.c_int32(), C.c_float()
        check(lib.sn_train_epoch(self.handle, self._ptr(x), self._ptr(y), total_rows, batch, global_iter, C.byref(it),
                                 C.byref(loss) if want_loss else None))
        return it.value, (loss.value if want_loss else None)


    def train_epoch_host(self, x, y, batch: int, global_iter: int, want_loss: bool = True) -> Tuple[int, Optional[float]]:
        """One epoch over a partition held in host memory (numpy float32 arrays, rows first; pinned ones from
        `Context.pinned_array` make the batch copies overlap with training)."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        y = np.ascontiguousarray(y, dtype=np.float32)
        if x.shape[0] != y.shape[0]:
            raise ValueError("x and y hold different numbers of rows")
        it, loss = C.c_int32(), C.c_float()
        check(lib.sn_train_epoch_host(self.handle, x.ctypes.data_as(C.c_void_p), y.ctypes.data_as(C.c_void_p), x.shape[0], batch,
                                      global_iter, C.byref(it), C.byref(loss) if want_loss else None))
        return it.value, (loss.value if want_loss else None)


def average_replicas(replicas: Sequence[Replica]):
    """`aggregateParams` over K replicas (optimizers/Optimizer.scala:196-230), uniform mean."""
    arr = (C.c_void_p * len(replicas))(*[r.handle for r in replicas])
    check(lib.sn_replicas_average(arr, len(replicas)))
