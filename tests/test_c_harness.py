"""The C ABI from a caller that is not Python: include/scanet_hip.h compiled as strict C99, and (on a GPU) two C
programs, one that drives three training steps and one that runs an epoch the way a JVM binding would (host partitions,
two replicas, their average, predictions, accuracy count, optimizer state), compared with the CPU oracle on the same
numbers."""
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


@pytest.mark.gpu
def test_c_program_runs_an_epoch_on_two_replicas_like_the_oracle():
    """epoch_harness.c: sn_host_alloc -> sn_train_epoch_host on two replicas -> sn_replicas_average -> sn_params_get /
    sn_optstate_get / sn_forward / sn_count_correct, against `O.optimize_on_partition`, `O.average_uniform`,
    `Model.forward` and `O.count_correct`."""
    binary = os.path.join(HARNESS_DIR, "epoch_harness")
    assert os.path.exists(binary), "build the harness first: python tests/c_harness/build.py (build() of __graft_entry__ does)"
    batch, batches, tail, features, hidden, classes, replicas = 16, 4, 5, 6, 8, 3, 2
    part_rows = batch * batches + tail
    out = subprocess.run([binary], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    epochs, vectors, correct = {}, {}, None
    for line in out.stdout.splitlines():
        parts = line.split()
        if parts[0] == "epoch":
            epochs[int(parts[1])] = (int(parts[2]), float(parts[3]))
        elif parts[0] == "correct":
            correct = int(parts[1])
        else:
            vectors[(parts[0], parts[1])] = np.asarray([float(v) for v in parts[2:]], f32)
    om = O.Model([O.Dense(hidden, O.ACT_TANH), O.Dense(classes, O.ACT_SOFTMAX)], O.LOSS_CCE)
    gen = Lcg()
    params = {}
    for path, shape in om.param_defs((batch, features)):
        n = int(np.prod(shape))
        params[path] = np.asarray([(gen.unit() - f32(0.5)) * f32(0.5) for _ in range(n)], f32).reshape(shape)
    partitions = []
    for _ in range(replicas):
        x = np.asarray([gen.unit() for _ in range(part_rows * features)], f32).reshape(part_rows, features)
        y = np.zeros((part_rows, classes), f32)
        for r in range(part_rows):
            y[r, int(gen.unit() * f32(classes))] = 1.0
        partitions.append((x, y))
    alg = O.Adam(0.05)
    results = []
    for r, (x, y) in enumerate(partitions):
        iters, p, st, loss = O.optimize_on_partition(om, alg, x, y, batch, 0, params, O.init_opt_state(alg, params))
        assert epochs[r][0] == iters == batches                       # the 5-row tail is skipped
        assert abs(epochs[r][1] - float(loss)) <= 1e-5 * max(1.0, abs(float(loss))), r
        results.append((p, st))
    mean = {p: O.average_uniform([res[0][p] for res in results]) for p in params}
    first = next(iter(params))
    slots = [O.average_uniform([res[1][first][s] for res in results]) for s in range(2)]
    for r in range(replicas):                                          # both replicas hold the average afterwards
        for path in params:
            np.testing.assert_allclose(vectors[(f"param{r}", path)].reshape(mean[path].shape), mean[path], rtol=1e-4, atol=1e-6, err_msg=path)
        for s in range(2):
            np.testing.assert_allclose(vectors[(f"slot{s}_{r}", first)].reshape(slots[s].shape), slots[s], rtol=1e-4, atol=1e-7)
    x0, y0 = partitions[0][0][:batch], partitions[0][1][:batch]
    np.testing.assert_allclose(vectors[("pred", "batch0")].reshape(batch, classes), om.forward(x0, mean), rtol=1e-4, atol=1e-6)
    assert correct == O.count_correct(om, x0, y0, mean)
