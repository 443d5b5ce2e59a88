"""The C ABI library loads without a GPU and exports every function include/scanet_hip.h declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "scanet_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(?:int|const char\s*\*)\s+(sn_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for must in ("sn_ctx_create", "sn_model_create", "sn_replica_create", "sn_step", "sn_forward", "sn_loss",
                 "sn_train_epoch", "sn_replicas_average", "sn_optimizer_update", "sn_average", "sn_count_correct"):
        assert must in names
    assert len(names) >= 35


def test_library_exports_every_declared_symbol():
    path = os.path.join(ROOT, "scanet3_amd", "libscanet_hip.so")
    assert os.path.exists(path), "build the library first: python scanet3_amd/build.py"
    lib = ctypes.CDLL(path)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in include/scanet_hip.h but not exported"


def test_binding_table_covers_the_header():
    from scanet3_amd import _lib
    assert sorted(_lib.SIGNATURES) == declared_functions()
    assert _lib.lib.sn_last_error() is not None


def test_no_cpu_fallback_in_the_product_path():
    """The package never imports the oracle, and has no torch/numpy compute path to fall back to."""
    pkg = os.path.join(ROOT, "scanet3_amd")
    for fn in os.listdir(pkg):
        if fn.endswith(".py"):
            src = open(os.path.join(pkg, fn)).read()
            assert "oracle" not in src, fn
            assert "import torch" not in src, fn
