"""ctypes binding of libscanet_hip.so (the C ABI declared in include/scanet_hip.h).

There is no CPU fallback: importing this module fails when the HIP library has
not been built, and every call raises `ScanetError` when the library reports a
failure.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libscanet_hip.so")

SN_MAX_RANK = 8
SN_MAX_OPT_STATES = 3
SN_MAX_AVG_INPUTS = 32

# enums of include/scanet_hip.h
LAYER_DENSE, LAYER_BIAS, LAYER_ACTIVATE, LAYER_FLATTEN, LAYER_CONV2D, LAYER_POOL2D, LAYER_LSTM, LAYER_SIMPLE_RNN, LAYER_BATCHNORM = range(9)
ACT_IDENTITY, ACT_SIGMOID, ACT_TANH, ACT_RELU, ACT_SOFTMAX = range(5)
RANDOM_UNIFORM, RANDOM_NORMAL, RANDOM_TRUNCATED_NORMAL = range(3)
ERROR_SQUARED, ERROR_ABSOLUTE = range(2)
LOSS_IDENTITY, LOSS_MSE, LOSS_BINARY_CROSSENTROPY, LOSS_CATEGORICAL_CROSSENTROPY = range(4)
PAD_VALID, PAD_SAME, PAD_EXPLICIT = 0, 1, 2
POOL_MAX, POOL_AVG = 0, 1
REG_NONE, REG_L1, REG_L2 = 0, 1, 2
OPT_SGD, OPT_ADAGRAD, OPT_ADADELTA, OPT_RMSPROP, OPT_ADAM, OPT_NADAM, OPT_ADAMAX, OPT_AMSGRAD = range(8)
FLAG_GEMM_BF16 = 1
FLAG_STABLE_SOFTMAX = 2


class ScanetError(RuntimeError):
    """A failing library call; carries the SN_E_* code and sn_last_error()'s text."""

    def __init__(self, code: int, message: str):
        super().__init__(f"[{code}] {message}")
        self.code = code
        self.message = message


class LayerDesc(C.Structure):
    _fields_ = [("kind", C.c_int32), ("units", C.c_int32), ("activation", C.c_int32), ("act_param", C.c_float),
                ("kernel_h", C.c_int32), ("kernel_w", C.c_int32), ("stride_h", C.c_int32), ("stride_w", C.c_int32),
                ("padding", C.c_int32), ("reg_kind", C.c_int32), ("reg_lambda", C.c_float), ("use_bias", C.c_int32),
                ("return_sequence", C.c_int32), ("bn_momentum", C.c_float), ("bn_epsilon", C.c_float),
                ("pad_top", C.c_int32), ("pad_bottom", C.c_int32), ("pad_left", C.c_int32), ("pad_right", C.c_int32),
                ("bn_fused", C.c_int32), ("recurrent_reg_kind", C.c_int32), ("recurrent_reg_lambda", C.c_float),
                ("bias_reg_kind", C.c_int32), ("bias_reg_lambda", C.c_float), ("pool_reduce", C.c_int32), ("stateful", C.c_int32)]


class OptimizerDesc(C.Structure):
    _fields_ = [("kind", C.c_int32), ("rate", C.c_float), ("beta1", C.c_float), ("beta2", C.c_float),
                ("epsilon", C.c_float), ("init_acc", C.c_float), ("nesterov", C.c_int32), ("maximize", C.c_int32)]


class ParamInfo(C.Structure):
    _fields_ = [("path", C.c_char * 96), ("offset", C.c_int64), ("size", C.c_int64), ("rank", C.c_int32),
                ("dims", C.c_int64 * SN_MAX_RANK), ("trainable", C.c_int32), ("aggregated", C.c_int32)]


_P = C.c_void_p
_F = C.POINTER(C.c_float)

# name -> (restype, argtypes); every name here must be declared in include/scanet_hip.h
SIGNATURES = {
    "sn_ctx_create": (C.c_int, [C.c_int, _P, C.POINTER(_P)]),
    "sn_ctx_destroy": (C.c_int, [_P]),
    "sn_last_error": (C.c_char_p, []),
    "sn_sync": (C.c_int, [_P]),
    "sn_device_info": (C.c_int, [_P, C.c_char_p, C.c_int, C.POINTER(C.c_int64), C.POINTER(C.c_int32)]),
    "sn_buffer_alloc": (C.c_int, [_P, C.c_size_t, C.POINTER(_P)]),
    "sn_buffer_free": (C.c_int, [_P, _P]),
    "sn_host_alloc": (C.c_int, [_P, C.c_size_t, C.POINTER(_P)]),
    "sn_host_free": (C.c_int, [_P, _P]),
    "sn_copy_h2d": (C.c_int, [_P, _P, _P, C.c_size_t]),
    "sn_copy_d2h": (C.c_int, [_P, _P, _P, C.c_size_t]),
    "sn_fill": (C.c_int, [_P, _P, C.c_float, C.c_int64]),
    "sn_model_create": (C.c_int, [_P, C.POINTER(LayerDesc), C.c_int32, C.c_int32, C.POINTER(C.c_int64), C.c_int32,
                                  C.c_int32, C.c_uint32, C.POINTER(_P)]),
    "sn_model_destroy": (C.c_int, [_P]),
    "sn_model_param_count": (C.c_int, [_P, C.POINTER(C.c_int32), C.POINTER(C.c_int64)]),
    "sn_model_param_info": (C.c_int, [_P, C.c_int32, C.POINTER(ParamInfo)]),
    "sn_model_output_shape": (C.c_int, [_P, C.POINTER(C.c_int32), C.POINTER(C.c_int64)]),
    "sn_replica_create": (C.c_int, [_P, C.POINTER(OptimizerDesc), C.POINTER(_P)]),
    "sn_replica_destroy": (C.c_int, [_P]),
    "sn_params_set": (C.c_int, [_P, C.c_int32, _P, C.c_int64]),
    "sn_params_get": (C.c_int, [_P, C.c_int32, _P, C.c_int64]),
    "sn_optstate_set": (C.c_int, [_P, C.c_int32, C.c_int32, _P, C.c_int64]),
    "sn_optstate_get": (C.c_int, [_P, C.c_int32, C.c_int32, _P, C.c_int64]),
    "sn_grads_get": (C.c_int, [_P, C.c_int32, _P, C.c_int64]),
    "sn_replica_flat": (C.c_int, [_P, C.c_int32, C.POINTER(_P), C.POINTER(C.c_int64)]),
    "sn_step": (C.c_int, [_P, _P, _P, C.c_int32, C.c_int32, _F]),
    "sn_grad": (C.c_int, [_P, _P, _P, C.c_int32, _F]),
    "sn_forward": (C.c_int, [_P, _P, C.c_int32, _P]),
    "sn_forward_training": (C.c_int, [_P, _P, C.c_int32, _P]),
    "sn_forward_static": (C.c_int, [_P, _P, C.c_int32, _P]),
    "sn_error_sum": (C.c_int, [_P, _P, _P, C.c_int32, C.c_int32, _F]),
    "sn_loss": (C.c_int, [_P, _P, _P, C.c_int32, _F]),
    "sn_count_correct": (C.c_int, [_P, _P, _P, C.c_int32, C.POINTER(C.c_int64)]),
    "sn_train_epoch": (C.c_int, [_P, _P, _P, C.c_int64, C.c_int32, C.c_int32, C.POINTER(C.c_int32), _F]),
    "sn_train_epoch_host": (C.c_int, [_P, _P, _P, C.c_int64, C.c_int32, C.c_int32, C.POINTER(C.c_int32), _F]),
    "sn_replicas_average": (C.c_int, [C.POINTER(_P), C.c_int32]),
    "sn_optimizer_update": (C.c_int, [_P, C.POINTER(OptimizerDesc), _P, _P, _P, _P, _P, C.c_int64, C.c_int32]),
    "sn_average": (C.c_int, [_P, C.POINTER(_P), C.c_int32, C.c_int64, _P]),
    "sn_random_fill": (C.c_int, [_P, _P, C.c_int64, C.c_int32, C.c_uint64, _F, _F]),
    "sn_profile_enable": (C.c_int, [_P, C.c_int32]),
    "sn_profile_reset": (C.c_int, [_P]),
    "sn_profile_count": (C.c_int, [_P, C.POINTER(C.c_int32)]),
    "sn_profile_get": (C.c_int, [_P, C.c_int32, C.c_char_p, C.c_int32, C.POINTER(C.c_double), C.POINTER(C.c_int64)]),
}


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build the HIP library first with `python scanet3_amd/build.py` "
            "(there is no CPU fallback)")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError when a declared symbol is not exported
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def check(rc: int) -> None:
    if rc != 0:
        raise ScanetError(rc, lib.sn_last_error().decode("utf-8", "replace"))
