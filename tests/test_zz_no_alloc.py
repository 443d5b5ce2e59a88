"""`sn_forward_static` (the forward pass that allocates no device memory) against `sn_forward`.

Both run the same kernels on the same weights, one with its intermediates in the replica's own buffers, the other
with them in the library's static device array, so the outputs must be bit-identical.  Two calls in a row, the second
with fewer rows: the static array still holds the first call's contents.  Needs an MI355X: run with `-m gpu`.
"""
import ctypes

import numpy as np
import pytest

from tests.helpers import build_pair, f32, glorot_params

pytestmark = pytest.mark.gpu

CNN = [("conv", 8, (3, 3), (1, 1), "same", "relu", True), ("pool", (2, 2), (2, 2), "valid"), ("batchnorm", 0.9, 1e-3),
       ("conv", 16, (3, 3), (1, 1), "valid", "relu", False), ("pool", (2, 2), (1, 1), "valid"), ("flatten",),
       ("dense", 32, "sigmoid"), ("dense", 10, "softmax")]


def test_static_forward_matches_forward_on_two_calls_in_a_row():
    import scanet3_amd as S
    from scanet3_amd._lib import ScanetError
    rng = np.random.default_rng(20251125)
    in_shape, batch = (16, 16, 3), 96
    omodel, layers, sloss = build_pair(CNN, "cce")
    with S.Context(0) as ctx:
        cm = S.CompiledModel(ctx, [l.desc() for l in layers.layers], sloss.kind, in_shape, batch)
        rep = cm.replica(None)
        params = glorot_params(omodel, (batch,) + in_shape, rng)
        for p in params:                     # moving statistics that are not the identity transform
            if p.endswith("moving_mean"):
                params[p] = rng.normal(0.1, 0.05, params[p].shape).astype(f32)
            if p.endswith("moving_variance"):
                params[p] = rng.uniform(0.5, 1.5, params[p].shape).astype(f32)
        rep.set_params(params)
        x = rng.random((batch,) + in_shape, f32)
        xb = ctx.to_device(x)
        out = ctx.alloc(batch * cm.out_elems)
        # the HIP runtime instance the library itself is linked to (a second copy of the runtime would know no device)
        with open("/proc/self/maps") as maps:
            hip_path = next(line.split()[-1] for line in maps if "libamdhip64" in line and "/torch/" not in line)
        hip = ctypes.CDLL(hip_path)

        def free_device_bytes():
            free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
            assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
            return free.value

        for rows in (96, 40):                # the second call is smaller and finds the first one's data in the array
            want = rep.forward(xb, rows)
            out.fill(-1.0)
            ctx.sync()
            before = free_device_bytes()
            rep.forward_static(xb, out, rows)
            ctx.sync()
            assert free_device_bytes() == before, "the call allocated or freed device memory"
            got = out.numpy()[: rows * cm.out_elems].reshape(want.shape)
            assert np.array_equal(got, want), rows
            assert np.all(out.numpy()[rows * cm.out_elems:] == -1.0)      # nothing written past `rows`
            assert np.all(np.abs(want.sum(axis=1) - 1.0) < 1e-5)           # a real softmax came out
        # beyond the array's size: a clear refusal, nothing launched
        big = S.CompiledModel(ctx, [l.desc() for l in layers.layers], sloss.kind, (256, 256, 3), 64)
        big_rep = big.replica(None)
        xbig = ctx.alloc(64 * 256 * 256 * 3)
        obig = ctx.alloc(64 * big.out_elems)
        with pytest.raises(ScanetError, match="static scratch array holds"):
            big_rep.forward_static(xbig, obig, 64)
        for b in (xb, out, xbig, obig):
            b.free()
        big_rep.close()
        big.close()
        rep.close()
        cm.close()


def test_static_forward_refuses_recurrent_models():
    import scanet3_amd as S
    from scanet3_amd._lib import ScanetError
    _, layers, sloss = build_pair([("lstm", 8), ("dense", 1, "tanh")], "mse")
    with S.Context(0) as ctx:
        cm = S.CompiledModel(ctx, [l.desc() for l in layers.layers], sloss.kind, (5, 4), 8)
        rep = cm.replica(None)
        xb, out = ctx.alloc(8 * 5 * 4), ctx.alloc(8)
        with pytest.raises(ScanetError, match="recurrent"):
            rep.forward_static(xb, out, 8)
        xb.free()
        out.free()
        rep.close()
        cm.close()
