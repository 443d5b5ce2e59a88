"""scanet3_amd: MI355X (gfx950) execution backend for scanet's training / inference step.

`scanet3_amd.dsl` mirrors the reference's user-facing DSL, `scanet3_amd.core` wraps the C ABI
of libscanet_hip.so (include/scanet_hip.h).  Importing the package loads the HIP library and
fails when it has not been built (`python scanet3_amd/build.py`).
"""
from . import _lib
from ._lib import ScanetError
from .core import CompiledModel, Context, DeviceBuffer, Replica, average_replicas
from .dsl import *  # noqa: F401,F403
