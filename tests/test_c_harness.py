"""The C ABI from a caller that is not Python: include/scanet_hip.h compiled as strict C99, and (on a GPU) a C program
that drives three training steps, compared with the CPU oracle on the same numbers."""
import importlib.util
import os
import subprocess

import numpy as np
import pytest

from oracle import scanet_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HARNESS_DIR = os.path.join(ROOT, "tests", "c_harness")
f32 = np.float32


def _build_script():
    spec = importlib.util.spec_from_file_location("c_harness_build", os.path.join(HARNESS_DIR, "build.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_header_is_clean_c99():
    _build_script().syntax_check_header()


class Lcg:
    """step_harness.c's generator: 16 bits of a 32-bit linear congruential state as a float in [0, 1)."""

    def __init__(self, seed=20251125):
        self.state = seed

    def unit(self):
        self.state = (self.state * 1664525 + 1013904223) & 0xFFFFFFFF
        return f32(((self.state >> 8) & 0xFFFF) / 65536.0)


@pytest.mark.gpu
def test_c_program_trains_three_steps_like_the_oracle():
    binary = os.path.join(HARNESS_DIR, "step_harness")
    assert os.path.exists(binary), "build the harness first: python tests/c_harness/build.py (build() of __graft_entry__ does)"
    rows, features, hidden, classes, steps = 16, 5, 8, 3, 3
    out = subprocess.run([binary], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    losses, params_c = {}, {}
    for line in out.stdout.splitlines():
        parts = line.split()
        if parts[0] == "loss":
            losses[int(parts[1])] = float(parts[2])
        elif parts[0] == "param":
            params_c[parts[1]] = np.asarray([float(v) for v in parts[2:]], f32)
    om = O.Model([O.Dense(hidden, O.ACT_SIGMOID), O.Dense(classes, O.ACT_SOFTMAX)], O.LOSS_CCE)
    gen = Lcg()
    params = {}
    for path, shape in om.param_defs((rows, features)):
        n = int(np.prod(shape))
        params[path] = np.asarray([(gen.unit() - f32(0.5)) * f32(0.5) for _ in range(n)], f32).reshape(shape)
    x = np.asarray([gen.unit() for _ in range(rows * features)], f32).reshape(rows, features)
    y = np.zeros((rows, classes), f32)
    for r in range(rows):
        y[r, int(gen.unit() * f32(classes))] = 1.0
    assert list(params_c) == list(params)            # the parameter table in the reference's path naming and order
    alg = O.Adam(0.05)
    state = O.init_opt_state(alg, params)
    for t in range(1, steps + 1):
        params, state, loss, _ = O.train_step(om, alg, x, y, params, state, t)
        assert abs(losses[t] - float(loss)) <= 1e-5 * max(1.0, abs(float(loss))), t
    for path in params:
        np.testing.assert_allclose(params_c[path].reshape(params[path].shape), params[path], rtol=1e-4, atol=1e-6, err_msg=path)
