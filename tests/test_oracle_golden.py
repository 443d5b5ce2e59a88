"""Pins the CPU oracle: reference known-answer vectors, brute force, an independent
library (torch CPU) and float64 numerical gradients.  Nothing here touches a GPU."""
import itertools

import numpy as np
import pytest
import torch
import torch.nn.functional as TF

from oracle import scanet_oracle as O

f32 = np.float32


def A(v, dt=f32):
    return np.asarray(v, dtype=dt)


def round_at(x, p):
    """`roundAt(p)` of the reference: Rint(x * 10^p) / 10^p (AllKernels.scala:528-531)."""
    s = x.dtype.type(10.0 ** p)
    return np.rint(x * s) / s


# ----------------------------------------------------------------- conv / pool goldens
@pytest.mark.parametrize("key,strides,padding,explicit", [
    ("same_s1", (1, 1), O.PAD_SAME, (0, 0, 0, 0)),
    ("same_s2", (2, 2), O.PAD_SAME, (0, 0, 0, 0)),
    ("valid_s1", (1, 1), O.PAD_VALID, (0, 0, 0, 0)),
    ("valid_s2", (2, 2), O.PAD_VALID, (0, 0, 0, 0)),
    ("explicit_1010_s2", (2, 2), O.PAD_EXPLICIT, (1, 0, 1, 0)),
])
def test_conv2d_golden(golden, key, strides, padding, explicit):
    x = A(golden["image_5x5"], np.float64).reshape(1, 5, 5, 1)
    w = A(golden["filter_2x2"], np.float64).reshape(2, 2, 1, 1)
    out = O.conv2d(x, w, strides, padding, explicit)
    exp = A(golden["conv2d"][key], np.float64)
    assert out.shape == (1,) + exp.shape + (1,)
    np.testing.assert_array_equal(round_at(out, 2).reshape(exp.shape), exp)


def test_conv2d_grads_golden(golden):
    x = A(golden["image_5x5"], np.float64).reshape(1, 5, 5, 1)
    w = A(golden["filter_2x2"], np.float64).reshape(2, 2, 1, 1)
    dy = np.ones((1, 4, 4, 1))
    gf = O.conv2d_grad_filter(x, w.shape, dy)
    gi = O.conv2d_grad_input(x.shape, w, dy)
    np.testing.assert_array_equal(gf.reshape(2, 2), A(golden["conv2d"]["valid_s1_grad_filter_of_sum"], np.float64))
    np.testing.assert_array_equal(gi.reshape(5, 5), A(golden["conv2d"]["valid_s1_grad_input_of_sum"], np.float64))


@pytest.mark.parametrize("key,strides,padding", [
    ("same_s1", (1, 1), O.PAD_SAME), ("same_s2", (2, 2), O.PAD_SAME),
    ("valid_s1", (1, 1), O.PAD_VALID), ("valid_s2", (2, 2), O.PAD_VALID),
])
def test_max_pool_golden(golden, key, strides, padding):
    x = A(golden["image_5x5"], np.float64).reshape(1, 5, 5, 1)
    out = O.max_pool(x, (2, 2), strides, padding)
    exp = A(golden["max_pool_2x2"][key], np.float64)
    np.testing.assert_array_equal(out.reshape(exp.shape), exp)


def test_max_pool_grad_ties_golden(golden):
    x = A(golden["image_5x5"], np.float64).reshape(1, 5, 5, 1)
    g = O.max_pool_grad(x, np.ones((1, 5, 5, 1)), (2, 2), (1, 1), O.PAD_SAME)
    np.testing.assert_array_equal(g.reshape(5, 5), A(golden["max_pool_2x2"]["same_s1_grad_input_of_sum"], np.float64))


def test_avg_pool_golden(golden):
    """Kernel-level `pool2D(reduce = Avg)` with Same padding: windows at the bottom / right edge average fewer cells."""
    x = A(golden["image_5x5"], np.float64).reshape(1, 5, 5, 1)
    out = O.avg_pool(x, (2, 2), (1, 1), O.PAD_SAME)
    np.testing.assert_array_equal(out.reshape(5, 5), A(golden["avg_pool_2x2"]["same_s1"], np.float64))
    g = O.avg_pool_grad(x.shape, np.ones((1, 5, 5, 1)), (2, 2), (1, 1), O.PAD_SAME)
    np.testing.assert_array_equal(g.reshape(5, 5), A(golden["avg_pool_2x2"]["same_s1_grad_input_of_sum"], np.float64))


# ----------------------------------------------------------------- brute force + torch
def _brute_conv(x, w, strides, padding):
    n, h, wd, c = x.shape
    kh, kw, _, f = w.shape
    ho = O.out_size(padding, h, kh, strides[0])
    wo = O.out_size(padding, wd, kw, strides[1])
    pt, _ = O.pads_for(padding, h, kh, strides[0])
    pl, _ = O.pads_for(padding, wd, kw, strides[1])
    out = np.zeros((n, ho, wo, f))
    for b, i, j, o in itertools.product(range(n), range(ho), range(wo), range(f)):
        s = 0.0
        for r, q, ci in itertools.product(range(kh), range(kw), range(c)):
            y, xx = i * strides[0] + r - pt, j * strides[1] + q - pl
            if 0 <= y < h and 0 <= xx < wd:
                s += x[b, y, xx, ci] * w[r, q, ci, o]
        out[b, i, j, o] = s
    return out


@pytest.mark.parametrize("strides", [(1, 1), (2, 2), (2, 1)])
@pytest.mark.parametrize("padding", [O.PAD_VALID, O.PAD_SAME])
def test_conv2d_brute_and_torch(strides, padding):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 7, 6, 3))
    w = rng.standard_normal((3, 2, 3, 4))
    out = O.conv2d(x, w, strides, padding)
    np.testing.assert_allclose(out, _brute_conv(x, w, strides, padding), rtol=1e-12, atol=1e-12)
    # gradients against torch autograd (independent library), explicit padding reproduced by F.pad
    pt, pb = O.pads_for(padding, 7, 3, strides[0])
    pl, pr = O.pads_for(padding, 6, 2, strides[1])
    xt = torch.tensor(x.transpose(0, 3, 1, 2), requires_grad=True)
    wt = torch.tensor(w.transpose(3, 2, 0, 1), requires_grad=True)
    yt = TF.conv2d(TF.pad(xt, (pl, pr, pt, pb)), wt, stride=strides)
    np.testing.assert_allclose(out, yt.detach().numpy().transpose(0, 2, 3, 1), rtol=1e-12, atol=1e-12)
    dy = rng.standard_normal(out.shape)
    yt.backward(torch.tensor(dy.transpose(0, 3, 1, 2)))
    np.testing.assert_allclose(O.conv2d_grad_input(x.shape, w, dy, strides, padding),
                               xt.grad.numpy().transpose(0, 2, 3, 1), rtol=1e-11, atol=1e-11)
    np.testing.assert_allclose(O.conv2d_grad_filter(x, w.shape, dy, strides, padding),
                               wt.grad.numpy().transpose(2, 3, 1, 0), rtol=1e-11, atol=1e-11)


@pytest.mark.parametrize("strides", [(1, 1), (2, 2)])
@pytest.mark.parametrize("padding", [O.PAD_VALID, O.PAD_SAME])
def test_max_pool_brute_first_max(strides, padding):
    rng = np.random.default_rng(5)
    x = rng.integers(0, 3, size=(2, 6, 5, 3)).astype(np.float64)      # many ties
    kh = kw = 2
    n, h, wd, c = x.shape
    ho, wo = O.out_size(padding, h, kh, strides[0]), O.out_size(padding, wd, kw, strides[1])
    pt, _ = O.pads_for(padding, h, kh, strides[0])
    pl, _ = O.pads_for(padding, wd, kw, strides[1])
    dy = rng.standard_normal((n, ho, wo, c))
    out = np.zeros((n, ho, wo, c))
    dx = np.zeros_like(x)
    for b, i, j, ch in itertools.product(range(n), range(ho), range(wo), range(c)):
        best, at = -np.inf, None
        for r, q in itertools.product(range(kh), range(kw)):
            y, xx = i * strides[0] + r - pt, j * strides[1] + q - pl
            if 0 <= y < h and 0 <= xx < wd and x[b, y, xx, ch] > best:     # strict: first max wins
                best, at = x[b, y, xx, ch], (y, xx)
        out[b, i, j, ch] = best
        dx[b, at[0], at[1], ch] += dy[b, i, j, ch]
    np.testing.assert_array_equal(O.max_pool(x, (2, 2), strides, padding), out)
    np.testing.assert_allclose(O.max_pool_grad(x, dy, (2, 2), strides, padding), dx, rtol=0, atol=1e-15)


@pytest.mark.parametrize("window,strides", [((2, 2), (1, 1)), ((2, 2), (2, 2)), ((3, 2), (2, 1))])
@pytest.mark.parametrize("padding", [O.PAD_VALID, O.PAD_SAME])
def test_avg_pool_brute_and_torch(window, strides, padding):
    """Cell-by-cell mean over the in-bounds part of each window, its transpose as the gradient, and (where torch's
    padding can express TF's) torch's avg_pool2d with count_include_pad=False."""
    rng = np.random.default_rng(6)
    x = rng.standard_normal((2, 6, 5, 3))
    kh, kw = window
    n, h, wd, c = x.shape
    ho, wo = O.out_size(padding, h, kh, strides[0]), O.out_size(padding, wd, kw, strides[1])
    pt, _ = O.pads_for(padding, h, kh, strides[0])
    pl, _ = O.pads_for(padding, wd, kw, strides[1])
    dy = rng.standard_normal((n, ho, wo, c))
    out = np.zeros((n, ho, wo, c))
    dx = np.zeros_like(x)
    for b, i, j, ch in itertools.product(range(n), range(ho), range(wo), range(c)):
        cells = [(i * strides[0] + r - pt, j * strides[1] + q - pl) for r, q in itertools.product(range(kh), range(kw))]
        cells = [(y, xx) for y, xx in cells if 0 <= y < h and 0 <= xx < wd]
        out[b, i, j, ch] = sum(x[b, y, xx, ch] for y, xx in cells) / len(cells)
        for y, xx in cells:
            dx[b, y, xx, ch] += dy[b, i, j, ch] / len(cells)
    np.testing.assert_allclose(O.avg_pool(x, window, strides, padding), out, rtol=1e-13, atol=1e-13)
    np.testing.assert_allclose(O.avg_pool_grad(x.shape, dy, window, strides, padding), dx, rtol=1e-13, atol=1e-13)
    if padding == O.PAD_VALID:
        xt = torch.tensor(x.transpose(0, 3, 1, 2), requires_grad=True)
        yt = torch.nn.functional.avg_pool2d(xt, window, strides, count_include_pad=False)
        np.testing.assert_allclose(yt.detach().numpy().transpose(0, 2, 3, 1), out, rtol=1e-12, atol=1e-12)
        yt.backward(torch.tensor(dy.transpose(0, 3, 1, 2)))
        np.testing.assert_allclose(xt.grad.numpy().transpose(0, 2, 3, 1), dx, rtol=1e-12, atol=1e-12)


# ----------------------------------------------------------------- layer goldens
def test_dense_sigmoid_forward_golden(golden):
    g = golden["dense_sigmoid"]
    m = O.Model([O.Dense(4, O.ACT_SIGMOID)])
    assert [p for p, _ in m.param_defs((4, 3))] == ["0/weights", "1/weights"]
    y = m.forward(A(g["x"]), {"0/weights": A(g["w"]), "1/weights": A(g["b"])})
    np.testing.assert_array_equal(round_at(y, 6), A(g["y_6dp"]))


def test_dense_bce_gradient_golden(golden):
    g = golden["dense_sigmoid"]
    m = O.Model([O.Dense(4, O.ACT_SIGMOID)], O.LOSS_BCE)
    p = {"0/weights": np.zeros((3, 4), f32), "1/weights": np.zeros(4, f32)}
    _, grads = m.grad(A(g["x"]), A(g["bce_y"]), p)
    # the reference asserts exact float equality against TF; the restatement agrees to the last ulp or two
    np.testing.assert_allclose(grads["0/weights"], A(g["bce_grad_w"]), rtol=3e-7, atol=0)
    np.testing.assert_allclose(grads["1/weights"], A(g["bce_grad_b"]), rtol=3e-7, atol=0)


def test_mlp_forward_and_loss_golden(golden):
    g = golden["mlp_4_1"]
    m = O.Model([O.Dense(4, O.ACT_SIGMOID), O.Dense(1, O.ACT_SIGMOID)])
    assert [p for p, _ in m.param_defs((4, 3))] == ["0/weights", "1/weights", "3/weights", "4/weights"]
    y = m.forward(A(g["x"]), {"0/weights": A(g["w1"]), "1/weights": A(g["b1"]),
                              "3/weights": A(g["w2"]), "4/weights": A(g["b2"])})
    # the last row is 0.80188651..: one float32 ulp decides which way the reference's 6-digit rounding falls,
    # so this vector is compared as "equal before rounding, to within one ulp"
    np.testing.assert_allclose(y, A(g["y_6dp"]), rtol=0, atol=0.5e-6 + 1.2e-7)
    g = golden["mlp_3_1_loss"]
    params = {"0/weights": A(g["w1"]), "1/weights": A(g["b1"]), "3/weights": A(g["w2"]), "4/weights": A(g["b2"])}
    m = O.Model([O.Dense(3, O.ACT_SIGMOID), O.Dense(1, O.ACT_SIGMOID)], O.LOSS_MSE)
    assert round_at(np.asarray(m.loss_of(A(g["x"]), A(g["y"]), params)), 6) == f32(g["mse_6dp"])
    m2 = O.Model([O.Dense(3, O.ACT_SIGMOID, reg=O.REG_L2, reg_lambda=1.0),
                  O.Dense(1, O.ACT_SIGMOID, reg=O.REG_L2, reg_lambda=1.0)], O.LOSS_MSE)
    np.testing.assert_allclose(m2.loss_of(A(g["x"]), A(g["y"]), params), f32(g["mse_plus_l2"]), rtol=2e-7)


def test_penalty_golden(golden):
    g = golden["penalty_l2"]
    m = O.Model([O.Dense(4, O.ACT_SIGMOID, reg=O.REG_L2, reg_lambda=1.0)])
    np.testing.assert_allclose(m.penalty({"0/weights": A(g["dense_w"]), "1/weights": np.zeros(2, f32)}),
                               f32(g["dense_penalty"]), rtol=2e-7)
    m = O.Model([O.Dense(4, O.ACT_SIGMOID, reg=O.REG_L2, reg_lambda=1.0),
                 O.Dense(1, O.ACT_SIGMOID, reg=O.REG_L2, reg_lambda=1.0)])
    p = {"0/weights": A(g["mlp_w1"]), "1/weights": np.zeros(4, f32), "3/weights": A(g["mlp_w2"]),
         "4/weights": np.zeros(1, f32)}
    np.testing.assert_allclose(m.penalty(p), f32(g["mlp_penalty"]), rtol=2e-7)


def test_regression_goldens(golden):
    g = golden["linear_regression"]
    m = O.Model([O.Dense(1)], O.LOSS_MSE)
    p = {"0/weights": A(g["w"]), "1/weights": A(g["b"])}
    assert m.loss_of(A(g["x"]), A(g["y"]), p) == f32(g["mse"])
    np.testing.assert_array_equal(m.forward(A(g["x"]), p), A(g["result"]))
    _, grads = m.grad(A(g["x"]), A(g["y"]), {"0/weights": np.zeros((2, 1), f32), "1/weights": np.zeros(1, f32)})
    np.testing.assert_array_equal(grads["0/weights"], A(g["grad_at_zero_w"]))
    np.testing.assert_array_equal(grads["1/weights"], A(g["grad_at_zero_b"]))
    g = golden["logistic_regression"]
    m = O.Model([O.Dense(1, O.ACT_SIGMOID)], O.LOSS_BCE)
    p = {"0/weights": A(g["w"]), "1/weights": A(g["b"])}
    assert abs(float(m.loss_of(A(g["x"]), A(g["y"]), p)) - g["bce"]) <= 1e-6
    np.testing.assert_array_equal(round_at(m.forward(A(g["x"]), p), 6), A(g["result_6dp"]))
    _, grads = m.grad(A(g["x"]), A(g["y"]), p)
    np.testing.assert_array_equal(round_at(grads["0/weights"], 6), A(g["grad_w_6dp"]))
    np.testing.assert_array_equal(round_at(grads["1/weights"], 6), A(g["grad_b_6dp"]))


def test_activation_goldens(golden):
    g = golden["activations"]
    np.testing.assert_allclose(np.tanh(f32(0.5)), f32(g["tanh_0.5"]), rtol=1.3e-7)     # one ulp
    np.testing.assert_allclose(O.tanh_grad(A([-0.5, 0.0, 0.5]), np.ones(3, f32)),
                               A([g["tanh_grad_at_pm0.5"], 1.0, g["tanh_grad_at_pm0.5"]]), rtol=1.2e-7)
    np.testing.assert_array_equal(round_at(O.softmax(A(g["softmax_in"])), 5), A(g["softmax_5dp"]))
    for k, v in g["relu"].items():
        assert O.relu(f32(k)) == f32(v)
    np.testing.assert_array_equal(round_at(O.sigmoid(A(g["sigmoid_in"])), 6), A(g["sigmoid_6dp"]))
    np.testing.assert_allclose(np.exp(A(g["exp_in"])), A(g["exp"]), rtol=1.2e-7)
    np.testing.assert_allclose(np.log(A(g["log_in"])), A(g["log"]), rtol=1.2e-7)
    np.testing.assert_array_equal(O.rint(A(g["round_in"])), A(g["round"]))
    assert O.relu_grad(f32(0.0), f32(1.0)) == 0.0       # strict comparison: no gradient at the threshold


def test_matmul_and_helpers_golden(golden):
    g = golden["matmul"]
    np.testing.assert_array_equal(A(g["a"]) @ A(g["b"]), A(g["c"]))
    ones = np.ones((2, 2), f32)
    np.testing.assert_array_equal(A(g["a"]).T @ ones, A(g["grad_right_of_sum"]))          # left^T . parent
    np.testing.assert_array_equal(ones @ A(g["x_right"]).T, A(g["grad_left_of_sum"]))     # parent . right^T
    h = golden["helpers"]
    d = h["decaying_avg"]
    assert O.decaying_avg(np.float64(d["avg"]), np.float64(d["next"]), d["decay"]) == pytest.approx(d["out"], abs=1e-12)
    s = h["sqrt_zero_safe"]
    assert O.sqrt_zero_safe(f32(s["x"]), s["eps"]) == f32(s["out"])
    for k in ("boost_t2", "boost_t1e6"):
        b = h[k]
        assert O.boost(f32(b["x"]), b["rate"], b["iter"]) == f32(b["out"])


def test_simple_rnn_golden(golden):
    g = golden["simple_rnn"]
    m = O.Model([O.SimpleRNN(2, activation=O.ACT_IDENTITY)])
    p = {"0/kernel_weights": A(g["wx"]), "0/recurrent_weights": A(g["wh"]), "1/weights": A(g["b"])}
    y = m.forward(A(g["x"]).reshape(1, 3, 1), p)
    np.testing.assert_array_equal(round_at(y, 6), A(g["y_6dp"]))


def _batch_norm_case(g, mode):
    t = g[mode]
    p = {"0/weights": A(g["dense_w"]), "1/weights": A(g["dense_b"])}
    p.update({f"2/{k}": A(t[k]) for k in O.BN_PARAMS})
    return t, p


def test_batch_norm_golden(golden):
    """BatchNormSpec.scala:30-65: training mode (output and the next moving statistics) and the frozen model."""
    g = golden["batch_norm"]
    m = O.Model([O.Dense(4), O.BatchNorm(momentum=0.5)])
    assert [p for p, _ in m.param_defs((4, 3))][2:] == ["2/beta", "2/gamma", "2/moving_mean", "2/moving_variance"]
    assert all(s == (1, 4) for _, s in m.param_defs((4, 3))[2:])
    t, p = _batch_norm_case(g, "training")
    nxt = {}
    y = m.forward(A(g["x"]), p, training=True, next_state=nxt)
    np.testing.assert_array_equal(round_at(y, 3), A(t["y_3dp"]))
    np.testing.assert_array_equal(round_at(nxt["2/moving_mean"], 3), A(t["next_moving_mean_3dp"]))
    np.testing.assert_array_equal(round_at(nxt["2/moving_variance"], 3), A(t["next_moving_variance_3dp"]))
    t, p = _batch_norm_case(g, "frozen")
    np.testing.assert_array_equal(round_at(m.forward(A(g["x"]), p), 3), A(t["y_3dp"]))


def test_batch_norm_state_bypasses_the_algorithm(golden):
    """`nextWeights ++ nextState` (Optimizer.scala:142-144): moving statistics are replaced by the layer's own
    update, every other tensor by the algorithm; a training-mode output has zero mean and unit variance."""
    g = golden["batch_norm"]
    m = O.Model([O.Dense(4), O.BatchNorm(momentum=0.5)], O.LOSS_MSE)
    _, p = _batch_norm_case(g, "training")
    x, y = A(g["x"]), np.zeros((4, 4), np.float32)
    alg = O.SGD(0.1)
    new_p, _, _, grads = O.train_step(m, alg, x, y, p, O.init_opt_state(alg, p), 1)
    assert set(grads) == {"0/weights", "1/weights", "2/beta", "2/gamma"}
    np.testing.assert_array_equal(round_at(new_p["2/moving_mean"], 3), A(g["training"]["next_moving_mean_3dp"]))
    np.testing.assert_array_equal(new_p["2/beta"], p["2/beta"] - np.float32(0.1) * grads["2/beta"])
    out = m.forward(x, p, training=True)
    np.testing.assert_allclose(out.mean(axis=0), 0.0, atol=1e-6)
    np.testing.assert_allclose(out.var(axis=0), 1.0, atol=1e-3)      # var / (var + epsilon)


def test_fused_batch_norm_op_definitions(golden):
    """`FusedBatchNormV3` / `GradV3` as TensorFlow defines them, before the reference's wiring: y is the generic form's y
    (so the reference's BatchNormSpec values hold for it, in training and in inference mode), output 2 is the unbiased
    variance, and the gradient op handed the true batch statistics returns the true gradient."""
    g = golden["batch_norm"]
    x = (A(g["x"]) @ A(g["dense_w"]) + A(g["dense_b"])).reshape(4, 1, 1, 4)     # the Dense output, as an NHWC image
    ones, zeros = np.ones(4, np.float32), np.zeros(4, np.float32)
    outs = O.fused_batch_norm(x, ones, zeros, zeros, ones, 1e-3, True)
    np.testing.assert_array_equal(round_at(outs[0].reshape(4, 4), 3), A(g["training"]["y_3dp"]))
    np.testing.assert_allclose(outs[1], x.reshape(4, 4).mean(axis=0), rtol=1e-6)
    np.testing.assert_allclose(outs[2], x.reshape(4, 4).astype(np.float64).var(axis=0, ddof=1), rtol=1e-5)
    np.testing.assert_allclose(outs[4], x.reshape(4, 4).astype(np.float64).var(axis=0), rtol=1e-5)
    np.testing.assert_array_equal(outs[3], outs[1])
    t = g["frozen"]
    frozen = O.fused_batch_norm(x, A(t["gamma"]), A(t["beta"]), A(t["moving_mean"]), A(t["moving_variance"]), 1e-3, False)
    np.testing.assert_array_equal(round_at(frozen[0].reshape(4, 4), 3), A(t["y_3dp"]))
    # a single row: n - 1 is taken as 1
    one = O.fused_batch_norm(x[:1], ones, zeros, zeros, ones, 1e-3, True)
    np.testing.assert_array_equal(one[2], np.zeros(4, np.float32))
    # the gradient op with the true statistics against central differences of sum(y * dy), float64
    rng = np.random.default_rng(12)
    x = rng.standard_normal((3, 2, 2, 5))
    scale, offset, dy = rng.uniform(0.5, 1.5, 5), rng.standard_normal(5), rng.standard_normal((3, 2, 2, 5))
    f = lambda xx, sc, of: float((O.fused_batch_norm(xx, sc, of, None, None, 1e-3, True)[0] * dy).sum())
    outs = O.fused_batch_norm(x, scale, offset, None, None, 1e-3, True)
    dx, dscale, doffset = O.fused_batch_norm_grad(dy, x, scale, outs[3], outs[4], 1e-3)
    h = 1e-6
    for idx in [(0, 0, 0, 0), (2, 1, 0, 3), (1, 1, 1, 4)]:
        e = np.zeros_like(x); e[idx] = h
        assert abs((f(x + e, scale, offset) - f(x - e, scale, offset)) / (2 * h) - dx[idx]) < 1e-7
    for ch in range(5):
        e = np.zeros(5); e[ch] = h
        assert abs((f(x, scale + e, offset) - f(x, scale - e, offset)) / (2 * h) - dscale[ch]) < 1e-7
        assert abs((f(x, scale, offset + e) - f(x, scale, offset - e)) / (2 * h) - doffset[ch]) < 1e-7


def test_fused_batch_norm_layer_wiring():
    """The layer's fused branch as the reference wires the op's outputs (math/nn/AllKernels.scala:437-448): the output
    is the op's; the moving variance moves towards the batch MEAN; the gradient op is handed the unbiased variance as
    its mean and the batch mean as its variance.  (Read off the reference's source: no reference test holds values.)"""
    rng = np.random.default_rng(13)
    x = rng.uniform(0.5, 2.0, (6, 3, 2, 4)).astype(np.float32)          # positive, so that `mean + epsilon` has a root
    m = O.Model([O.BatchNorm(momentum=0.9, epsilon=1e-3, fused=True)], O.LOSS_MSE)
    p = {"beta": rng.standard_normal((1, 1, 1, 4)).astype(np.float32), "gamma": rng.uniform(0.5, 1.5, (1, 1, 1, 4)).astype(np.float32),
         "moving_mean": np.zeros((1, 1, 1, 4), np.float32), "moving_variance": np.ones((1, 1, 1, 4), np.float32)}
    assert [s for _, s in m.param_defs((6, 3, 2, 4))] == [(1, 1, 1, 4)] * 4
    generic = O.Model([O.BatchNorm(momentum=0.9, epsilon=1e-3)], O.LOSS_MSE)
    nxt, nxt_g = {}, {}
    y = m.forward(x, p, training=True, next_state=nxt)
    np.testing.assert_allclose(y, generic.forward(x, p, training=True, next_state=nxt_g), rtol=1e-5, atol=1e-6)
    mean = x.reshape(-1, 4).mean(axis=0)
    var = x.reshape(-1, 4).var(axis=0)
    np.testing.assert_allclose(nxt["moving_mean"].ravel(), 0.1 * mean, rtol=1e-5)
    np.testing.assert_allclose(nxt["moving_variance"].ravel(), 0.9 + 0.1 * mean, rtol=1e-5)
    np.testing.assert_allclose(nxt_g["moving_variance"].ravel(), 0.9 + 0.1 * var, rtol=1e-5)
    target = rng.standard_normal(y.shape).astype(np.float32)
    grads = m.grad_stateful(x, target, p)[1]
    dy = (y - target) * np.float32(2.0 / y.size)
    n = 36
    _, dscale, doffset = O.fused_batch_norm_grad(dy, x, p["gamma"], var * n / (n - 1), mean, 1e-3)
    np.testing.assert_allclose(grads["gamma"].ravel(), dscale, rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(grads["beta"].ravel(), doffset, rtol=1e-5, atol=1e-7)
    true_grads = generic.grad_stateful(x, target, p)[1]
    assert not np.allclose(grads["gamma"], true_grads["gamma"], rtol=1e-2)     # the wiring is not the true gradient


def test_penalties_of_recurrent_and_batch_norm_layers():
    """Which weights a penalty lands on (RNN.scala:198-199,341-346; BatchNorm.scala:158-160; Bias.scala:35-36), checked
    against the closed forms, and the L2 part of the gradient against central differences in float64."""
    rng = np.random.default_rng(0)
    m = O.Model([O.LSTM(4, kernel_reg=(O.REG_L2, 0.05), recurrent_reg=(O.REG_L1, 0.02), bias_reg=(O.REG_L2, 0.3)),
                 O.BatchNorm(beta_reg=(O.REG_L2, 0.1)), O.Dense(2, reg=O.REG_L2, reg_lambda=0.01)], O.LOSS_MSE)
    x, y = rng.standard_normal((5, 3, 2)), rng.standard_normal((5, 2))
    params = {p: rng.standard_normal(s) * 0.5 for p, s in m.param_defs(x.shape)}
    params["1/moving_variance"] = np.abs(params["1/moving_variance"]) + 0.5
    sq = lambda p: float((params[p] ** 2).sum())
    ab = lambda p: float(np.abs(params[p]).sum())
    always = sum(0.05 * sq(f"0/{g}/0/kernel_weights") / 2 + 0.02 * ab(f"0/{g}/0/recurrent_weights") / 2 for g in O.GATES) \
        + 0.01 * sq("2/weights") / 2
    trainable_only = sum(0.3 * sq(f"0/{g}/1/weights") / 2 for g in O.GATES) + 2 * (0.1 * sq("1/gamma") / 2) + 0.01 * sq("3/weights") / 2
    np.testing.assert_allclose(m.penalty(params, training=True), always + trainable_only, rtol=1e-12)
    np.testing.assert_allclose(m.penalty(params, training=False), always, rtol=1e-12)        # the frozen model
    # gradient of loss + penalty for the L2-regularised tensors (the reference's L1 gradient is |parent| by construction)
    _, grads, _ = m.grad_stateful(x, y, params)
    for p in ("0/forget/0/kernel_weights", "0/gate/1/weights", "1/gamma", "2/weights", "3/weights"):
        w = params[p]
        idx = tuple(int(rng.integers(0, d)) for d in w.shape)
        e = np.zeros_like(w)
        e[idx] = 1e-6
        up, down = dict(params), dict(params)
        up[p], down[p] = w + e, w - e
        num = (m.loss_of(x, y, up, training=True) - m.loss_of(x, y, down, training=True)) / 2e-6
        assert abs(num - grads[p][idx]) < 1e-6 * max(1.0, abs(num)), p
    # beta itself carries no penalty, whatever regularizer the layer was given
    plain = O.Model([O.LSTM(4), O.BatchNorm(), O.Dense(2)], O.LOSS_MSE)
    np.testing.assert_allclose(grads["1/beta"], plain.grad_stateful(x, y, params)[1]["1/beta"], rtol=1e-12)


def test_seeded_initializers_golden(golden):
    """InitializerSpec.scala:23-66: TensorFlow's seeded streams, restated."""
    for case in golden["initializers"]["cases"]:
        out = O.initialize(case["name"], tuple(case["shape"]), case["seed"], **case["args"])
        assert out.dtype == np.float32 and out.shape == tuple(case["shape"])
        np.testing.assert_array_equal(round_at(out, case["digits"]), A(case["out"]), err_msg=case["name"])


def test_seeded_streams_structure():
    """What the goldens (3 values each) leave open, fixed by the construction: four outputs per counter whatever the
    length asked for, Philox's published known-answer vector, the truncation, the moments."""
    # Random123 known-answer test for philox4x32-10: zero counter and key; and the all-ones one
    kat = O.philox4x32_10(np.zeros((1, 4), np.uint32), (0, 0))[0]
    assert [hex(int(v)) for v in kat] == ["0x6627e8d5", "0xe169c58d", "0xbc57ac4c", "0x9b00dbd8"]
    kat = O.philox4x32_10(np.full((1, 4), 0xFFFFFFFF, np.uint32), (0xFFFFFFFF, 0xFFFFFFFF))[0]
    assert [hex(int(v)) for v in kat] == ["0x408f276d", "0x41c83b0e", "0xa20bc7c6", "0x6d5451fd"]
    for fn in (O.tf_random_uniform, O.tf_random_normal, O.tf_truncated_normal):
        np.testing.assert_array_equal(fn(1001, 5)[:37], fn(37, 5))          # a prefix does not depend on the length
        assert not np.array_equal(fn(16, 5), fn(16, 6))
    u = O.tf_random_uniform(200000, 3)
    assert 0.0 <= u.min() and u.max() < 1.0 and abs(u.mean() - 0.5) < 2e-3 and abs(u.var() - 1 / 12) < 1e-3
    z = O.tf_random_normal(200000, 3)
    assert abs(z.mean()) < 5e-3 and abs(z.std() - 1.0) < 5e-3
    t = O.tf_truncated_normal(8000, 3)
    assert np.abs(t).max() < 2.0 and abs(t.std() - 0.8796) < 2e-2
    # the first group of the truncated stream is the normal stream with rejections removed
    zn = O.tf_random_normal(64, 11)
    np.testing.assert_array_equal(O.tf_truncated_normal(4, 11), zn[np.abs(zn) < 2.0][:4])
    q = O.initialize("Orthogonal", (5, 3), 4)
    np.testing.assert_allclose(q.T @ q, np.eye(3), atol=1e-6)
    q = O.initialize("Orthogonal", (3, 5), 4, gain=2.0)
    np.testing.assert_allclose(q @ q.T, 4.0 * np.eye(3), atol=1e-5)
    assert O.initializer_fans((3, 3, 2, 8)) == (16 * 3, 16 * 3)              # `out :: in :: receptive` (Initializer.scala:20-23)


def forecast_case(sunspots):
    """RNNSpec.scala:22-33: SimpleRNN(3) >> Dense(1, Tanh), Adam(0.01), batch 10, 100 epochs on the sunspot series.
    The reference splits 80/20 at random through Spark; here every fifth sample is held out.  Initial weights come
    from seeded initializers so that both sides of a parity test start from the same point."""
    X, Y = sunspots
    held = np.arange(X.shape[0]) % 5 == 4
    m = O.Model([O.SimpleRNN(3), O.Dense(1, O.ACT_TANH)], O.LOSS_MSE)
    init = {"0/0/kernel_weights": O.initialize("GlorotUniform", (1, 3), 11),
            "0/0/recurrent_weights": O.initialize("Orthogonal", (3, 3), 12), "0/1/weights": np.zeros(3, f32),
            "1/weights": O.initialize("GlorotUniform", (3, 1), 13), "2/weights": np.zeros(1, f32)}
    return m, init, (X[~held], Y[~held]), (X[held], Y[held])


def test_rnn_forecast_reaches_the_reference_thresholds(sunspots):
    """RNNSpec.scala:46-47: RMSE < 0.2 and R2Score > 0.78 on the held-out part."""
    assert sunspots[0].shape == (234, 12, 1)
    m, init, (xtr, ytr), (xte, yte) = forecast_case(sunspots)
    params, _, hist = O.train(m, O.Adam(0.01), [(xtr, ytr)], 10, 100, init)
    assert hist[-1] < hist[0]
    mse = O.mean_error(m, xte, yte, params)
    assert np.sqrt(mse) < 0.2 and O.r2_score(m, xte, yte, params) > 0.78
    # the estimators against their definitions on one batch
    pred = m.forward(xte, params).astype(np.float64)
    assert mse == pytest.approx(float(((pred - yte) ** 2).sum() / len(xte)), rel=1e-5)
    assert O.mean_error(m, xte, yte, params, absolute=True) == pytest.approx(float(np.abs(pred - yte).sum() / len(xte)), rel=1e-5)
    assert O.mean_error(m, xte, yte, params, batch=7) == pytest.approx(mse, rel=1e-5)          # batch sums add up


def _lstm_params(g, pre=""):
    p = {}
    for gate in O.GATES:
        p[f"{pre}{gate}/0/kernel_weights"] = A(g[gate]["k"])
        p[f"{pre}{gate}/0/recurrent_weights"] = A(g[gate]["r"])
        p[f"{pre}{gate}/1/weights"] = A(g[gate]["b"])
    return p


def test_lstm_forward_golden(golden):
    g = golden["lstm"]
    m = O.Model([O.LSTM(2)])
    y = m.forward(A(g["x"]).reshape(1, 3, 1), _lstm_params(g))
    np.testing.assert_array_equal(round_at(y, 6), A(g["y_6dp"]))


def test_cnn_shape_table_golden(golden):
    g = golden["cnn_shapes"]
    m = O.Model([O.Conv2D(32, activation=O.ACT_RELU), O.Pool2D(), O.Conv2D(64, activation=O.ACT_RELU), O.Pool2D(),
                 O.Flatten(), O.Dense(10, O.ACT_SOFTMAX)])
    defs = dict(m.param_defs((1, 24, 24, 1)))
    assert {k: list(v) for k, v in defs.items()} == g["weights"]
    assert sum(int(np.prod(v)) for v in defs.values()) == g["total_params"]
    s, outs = (1, 24, 24, 1), []
    for l in m.layers:
        s = l.out_shape(s)
        outs.append(list(s[1:]))
    assert outs == g["outputs"]


# ----------------------------------------------------------------- gradients: float64 numerics + torch
def _numeric_grad(m, x, y, params, path, eps=1e-6, training=False):
    w = params[path]
    g = np.zeros_like(w)
    it = np.nditer(w, flags=["multi_index"])
    for _ in it:
        idx = it.multi_index
        old = w[idx]
        w[idx] = old + eps
        lp = float(m.loss_of(x, y, params, training=training))
        w[idx] = old - eps
        lm = float(m.loss_of(x, y, params, training=training))
        w[idx] = old
        g[idx] = (lp - lm) / (2 * eps)
    return g


def _rand_params(m, in_shape, rng, dt=np.float64, scale=0.4):
    return {p: (rng.standard_normal(s) * scale).astype(dt) for p, s in m.param_defs(in_shape)}


@pytest.mark.parametrize("name", ["mlp_cce", "cnn_cce", "lstm_mse", "rnn_mse", "lstm_stacked", "rnn_stacked", "mlp_batchnorm",
                                  "cnn_batchnorm", "mlp_bce_l2"])
def test_model_gradients_match_numeric_float64(name):
    rng = np.random.default_rng(11)
    if name == "mlp_cce":
        m = O.Model([O.Dense(5, O.ACT_SIGMOID), O.Dense(6, O.ACT_TANH), O.Dense(4, O.ACT_SOFTMAX)], O.LOSS_CCE)
        x = rng.random((3, 7))
        y = np.eye(4)[rng.integers(0, 4, 3)]
    elif name == "cnn_cce":
        m = O.Model([O.Conv2D(3, activation=O.ACT_RELU), O.Pool2D(), O.Conv2D(2, (2, 2), (2, 2), O.PAD_SAME, O.ACT_RELU, bias=True),
                     O.Pool2D(strides=(2, 2)), O.Flatten(), O.Dense(3, O.ACT_SOFTMAX)], O.LOSS_CCE)
        x = rng.random((2, 9, 8, 2))
        y = np.eye(3)[rng.integers(0, 3, 2)]
    elif name == "lstm_mse":
        m = O.Model([O.LSTM(4), O.Dense(1, O.ACT_TANH)], O.LOSS_MSE)
        x = rng.standard_normal((3, 5, 2))
        y = rng.uniform(-1, 1, (3, 1))
    elif name == "rnn_mse":
        m = O.Model([O.SimpleRNN(3), O.Dense(2)], O.LOSS_MSE)
        x = rng.standard_normal((2, 4, 3))
        y = rng.uniform(-1, 1, (2, 2))
    elif name == "lstm_stacked":      # `returnSequence = true` feeds every step's output to the next layer (RNN.scala:74-77)
        m = O.Model([O.LSTM(3, return_sequence=True), O.LSTM(2), O.Dense(1)], O.LOSS_MSE)
        x = rng.standard_normal((3, 4, 2))
        y = rng.uniform(-1, 1, (3, 1))
    elif name == "rnn_stacked":
        m = O.Model([O.SimpleRNN(3, O.ACT_SIGMOID, return_sequence=True), O.SimpleRNN(2), O.Dense(1)], O.LOSS_MSE)
        x = rng.standard_normal((3, 4, 2))
        y = rng.uniform(-1, 1, (3, 1))
    elif name == "mlp_batchnorm":     # batch statistics depend on the input: the gradient runs through mean and variance
        m = O.Model([O.Dense(5, O.ACT_TANH), O.BatchNorm(0.9, 1e-3), O.Dense(3, O.ACT_SOFTMAX)], O.LOSS_CCE)
        x = rng.standard_normal((6, 4))
        y = np.eye(3)[rng.integers(0, 3, 6)]
    elif name == "cnn_batchnorm":     # rank 4: statistics over batch, height and width
        m = O.Model([O.Conv2D(3, activation=O.ACT_RELU), O.BatchNorm(0.9, 1e-2), O.Pool2D(), O.Flatten(), O.Dense(2)], O.LOSS_MSE)
        x = rng.random((3, 6, 5, 2))
        y = rng.uniform(-1, 1, (3, 2))
    else:
        m = O.Model([O.Dense(3, O.ACT_SIGMOID, reg=O.REG_L2, reg_lambda=0.3), O.Dense(2, O.ACT_SIGMOID)], O.LOSS_BCE)
        x = rng.random((4, 3))
        y = rng.integers(0, 2, (4, 2)).astype(np.float64)
    params = _rand_params(m, x.shape, rng)
    for path in params:
        if O.is_state_path(path):
            params[path] = np.abs(params[path]) + 0.5
    _, grads = m.grad(x, y, params)
    assert set(grads) == {p for p in params if not O.is_state_path(p)}
    for path in grads:
        num = _numeric_grad(m, x, y, params, path, training=True)
        np.testing.assert_allclose(grads[path], num, rtol=2e-5, atol=2e-8, err_msg=path)


@pytest.mark.parametrize("kind", ["lstm", "simple_rnn"])
def test_stateful_rnn_carries_its_state_between_batches(kind):
    """`RNN(cell, stateful = true)` (RNN.scala:27,34,66-72).  No reference test runs it, so the restatement is pinned by
    what the definition fixes: (1) with a zero state it is the stateless layer; (2) a sequence of 6 steps fed as two
    batches of 3 steps, the second starting from the state the first one left, gives the output of the 6 steps in one
    go; (3) the state takes no gradient and bypasses the algorithm; (4) float64 numerical gradients from a non-zero
    state; (5) averaging re-initialises it (Optimizer.scala:207-210)."""
    rng = np.random.default_rng(5)
    make = (lambda **kw: O.LSTM(4, **kw)) if kind == "lstm" else (lambda **kw: O.SimpleRNN(4, O.ACT_TANH, **kw))
    m_state = O.Model([make(stateful=True), O.Dense(1)], O.LOSS_MSE)
    m_plain = O.Model([make(), O.Dense(1)], O.LOSS_MSE)
    b = 3
    x = rng.standard_normal((b, 6, 2))
    y = rng.uniform(-1, 1, (b, 1))
    plain = _rand_params(m_plain, x.shape, rng)
    state_paths = [p for p, _ in m_state.param_defs(x.shape) if O.is_state_path(p)]
    assert state_paths == (["0/cell_state", "0/hidden_state"] if kind == "lstm" else ["0/0/state"])
    assert all(O.is_unaggregated_path(p) for p in state_paths)
    with_state = dict(plain)
    for p in state_paths:
        with_state[p] = np.zeros((b, 4))
    # (1)
    np.testing.assert_array_equal(m_state.forward(x, with_state), m_plain.forward(x, plain))
    # (2)
    nxt = {}
    m_state.forward(x[:, :3], with_state, training=True, next_state=nxt)
    assert set(nxt) == set(state_paths)
    second = dict(with_state)
    second.update(nxt)
    np.testing.assert_allclose(m_state.forward(x[:, 3:], second), m_plain.forward(x, plain), rtol=1e-12)
    # (3)
    alg = O.SGD(0.1)
    new_params, _, _, grads = O.train_step(m_state, alg, x[:, :3], y, with_state, O.init_opt_state(alg, with_state), 1)
    assert set(grads) == set(plain)
    for p in state_paths:
        np.testing.assert_array_equal(new_params[p], nxt[p])
    # (4)
    loss, grads = m_state.grad(x[:, 3:], y, second)
    for path in grads:
        num = _numeric_grad(m_state, x[:, 3:], y, second, path, training=True)
        np.testing.assert_allclose(grads[path], num, rtol=2e-5, atol=2e-8, err_msg=path)
    # (5)
    parts = [(x[:, :3].astype(f32), y.astype(f32)), (x[:, 3:].astype(f32), y.astype(f32))]
    init = {p: v.astype(f32) for p, v in with_state.items()}
    trained, _, _ = O.train(m_state, O.Adam(0.01), parts, b, 2, init)
    for p in state_paths:
        assert not np.any(trained[p])


def test_maximizing_adds_the_delta():
    """`Optimizer.maximize` (Optimizer.scala:186,326-336): `if (minimizing) w - del else w + del`."""
    rng = np.random.default_rng(3)
    m = O.Model([O.Dense(2)], O.LOSS_MSE)
    x, y = rng.standard_normal((5, 3)).astype(f32), rng.standard_normal((5, 2)).astype(f32)
    params = {p: rng.standard_normal(s_).astype(f32) for p, s_ in m.param_defs(x.shape)}
    alg = O.Adam(0.1)
    down, st_down, _, grads = O.train_step(m, alg, x, y, params, O.init_opt_state(alg, params), 1)
    up, st_up, _, _ = O.train_step(m, alg, x, y, params, O.init_opt_state(alg, params), 1, minimizing=False)
    for p in params:
        np.testing.assert_allclose(up[p] - params[p], -(down[p] - params[p]), rtol=0, atol=1e-6)     # the same delta, other sign
        np.testing.assert_array_equal(st_up[p][0], st_down[p][0])
    assert float(m.loss_of(x, y, up)) > float(m.loss_of(x, y, params)) > float(m.loss_of(x, y, down))


def test_lstm_matches_torch_lstm_cell():
    """Independent library check: torch.nn.LSTM (gate order i,f,g,o) with the reference's weights mapped in."""
    rng = np.random.default_rng(2)
    b, t, f, h = 3, 6, 4, 5
    m = O.Model([O.LSTM(h)], O.LOSS_MSE)
    params = _rand_params(m, (b, t, f), rng)
    x = rng.standard_normal((b, t, f))
    y = rng.standard_normal((b, h))
    lstm = torch.nn.LSTM(f, h, batch_first=True).double()
    order = ["input", "forget", "gate", "output"]
    with torch.no_grad():
        lstm.weight_ih_l0.copy_(torch.tensor(np.concatenate([params[f"{g}/0/kernel_weights"].T for g in order])))
        lstm.weight_hh_l0.copy_(torch.tensor(np.concatenate([params[f"{g}/0/recurrent_weights"].T for g in order])))
        lstm.bias_ih_l0.copy_(torch.tensor(np.concatenate([params[f"{g}/1/weights"] for g in order])))
        lstm.bias_hh_l0.zero_()
    out, _ = lstm(torch.tensor(x))
    last = out[:, -1, :]
    np.testing.assert_allclose(m.forward(x, params), last.detach().numpy(), rtol=1e-10, atol=1e-12)
    loss = ((last - torch.tensor(y)) ** 2).mean()
    loss.backward()
    lo, grads = m.grad(x, y, params)
    assert float(lo) == pytest.approx(float(loss.detach()), rel=1e-12)
    gk = np.concatenate([grads[f"{g}/0/kernel_weights"].T for g in order])
    gr = np.concatenate([grads[f"{g}/0/recurrent_weights"].T for g in order])
    gb = np.concatenate([grads[f"{g}/1/weights"] for g in order])
    np.testing.assert_allclose(gk, lstm.weight_ih_l0.grad.numpy(), rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(gr, lstm.weight_hh_l0.grad.numpy(), rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(gb, lstm.bias_ih_l0.grad.numpy(), rtol=1e-9, atol=1e-12)


def test_softmax_cce_general_form_vs_textbook():
    """With one-hot rows and eps negligible the chain reduces to (p - y) / B."""
    rng = np.random.default_rng(4)
    z = rng.standard_normal((6, 5))
    y = np.eye(5)[rng.integers(0, 5, 6)]
    p = O.softmax(z)
    dz = O.softmax_grad(z, O.loss_grad(O.LOSS_CCE, p, y))
    np.testing.assert_allclose(dz, (p - y) / 6, rtol=1e-6, atol=1e-9)


# ----------------------------------------------------------------- optimizers
ALGS = {"SGD": O.SGD, "Adam": O.Adam, "AdaGrad": O.AdaGrad, "AdaDelta": O.AdaDelta, "RMSProp": O.RMSProp,
        "Nadam": O.Nadam, "Adamax": O.Adamax, "AMSGrad": O.AMSGrad}


def test_state_names_and_inits():
    assert O.SGD().state_names == ["velocity"]                                   # SGD.scala:29
    assert O.AdaGrad().state_names == ["grad_acc"]                               # AdaGrad.scala:36
    assert O.AdaDelta().state_names == ["avg_grad", "avg_delta"]                 # AdaDelta.scala:48-49
    assert O.RMSProp().state_names == ["avg_grad"]
    assert O.Adam().state_names == ["momentum", "velocity"]
    assert O.Adamax().state_names == ["momentum_1", "momentum_2"]
    assert O.AMSGrad().state_names == ["momentum", "velocity", "corrected_velocity"]
    assert float(O.Nadam().init_state((1,))[0][0]) == f32(0.001)                 # Nadam.scala:26-35
    assert float(O.Adamax().init_state((1,))[1][0]) == f32(0.001)                # Adamax.scala:30-39
    assert float(O.Adam().init_state((1,))[0][0]) == 0.0


def test_convergence_thresholds(golden, linear_function):
    X, Y = linear_function
    assert X.shape == (97, 1)
    m = O.Model([O.Dense(1)], O.LOSS_MSE)
    init = {"0/weights": np.zeros((1, 1), f32), "1/weights": np.zeros(1, f32)}
    for case in golden["convergence"]["cases"]:
        alg = ALGS[case["alg"]](**case["args"])
        params, _, _ = O.train(m, alg, [(X, Y)], 97, case["epochs"], init)
        final = float(m.loss_of(X, Y, params))
        assert final <= case["max_loss"], (case, final)
        assert final > 4.0            # the data's least-squares optimum is about 4.48; nothing can beat it


def test_logistic_adam_golden(golden, logistic_data):
    g = golden["convergence"]["logistic_adam"]
    X, Y = logistic_data
    m = O.Model([O.Dense(1, O.ACT_SIGMOID)], O.LOSS_BCE)
    init = {"0/weights": np.zeros((2, 1), f32), "1/weights": np.zeros(1, f32)}
    params, _, _ = O.train(m, O.Adam(g["rate"]), [(X, Y)], g["batch"], g["epochs"], init)
    assert float(m.loss_of(X, Y, params)) <= g["max_loss"]
    assert O.count_correct(m, X, Y, params) / X.shape[0] >= g["min_accuracy"]
    np.testing.assert_array_equal(O.rint(m.forward(A(g["predict_in"]), params)), A(g["predict_rounded"]))


def test_sgd_x2_closed_form(golden):
    g = golden["convergence"]["sgd_x2"]
    alg = O.SGD(g["rate"])
    w, st = np.array(g["w0"], np.float64), alg.init_state((), np.float64)
    for t in range(1, g["epochs"] + 1):
        delta, st = alg.build(2 * w, st, t)        # d/dw w^2
        w = w - delta
    assert float(w) == pytest.approx(g["w0"] * 0.8 ** g["epochs"], rel=1e-9)
    assert float(w * w) <= g["max_loss"]


def test_optimizer_closed_forms_constant_gradient():
    """With a constant gradient and zero state the bias-corrected moments equal g and g^2 at every step,
    so each rule collapses to a closed form that a dropped (1-beta), a wrong exponent or a misplaced
    epsilon would break."""
    g = np.array([0.3, -1.7, 2.5e-3], np.float64)
    w0 = np.array([1.0, -2.0, 0.5], np.float64)
    lr, eps = 0.01, 1e-7
    a = O.Adam(lr)
    st = a.init_state(g.shape, np.float64)
    for t in range(1, 8):
        d, st = a.build(g, st, t)
        np.testing.assert_allclose(d, lr * g / np.sqrt(g * g + eps), rtol=1e-10)
    a = O.AdaGrad(lr)
    st = a.init_state(g.shape, np.float64)
    for t in range(1, 6):
        d, st = a.build(g, st, t)
        np.testing.assert_allclose(d, lr * g / np.sqrt(t * g * g + eps), rtol=1e-12)
    a = O.RMSProp(lr)
    st = a.init_state(g.shape, np.float64)
    for t in range(1, 6):
        d, st = a.build(g, st, t)
        np.testing.assert_allclose(d, lr * g / np.sqrt((1 - 0.9 ** t) * g * g + eps), rtol=1e-10)
    a = O.AMSGrad(lr)
    st = a.init_state(g.shape, np.float64)
    for t in range(1, 6):
        d, st = a.build(g, st, t)
        np.testing.assert_allclose(d, lr * (1 - 0.9 ** t) * g / (np.sqrt((1 - 0.999 ** t) * g * g) + eps), rtol=1e-10)
    a = O.Adamax(lr, init_acc=0.0)
    st = a.init_state(g.shape, np.float64)
    for t in range(1, 6):
        d, st = a.build(g, st, t)      # m2 = max(beta2*m2, (1-beta2)|g|) stays (1-beta2)|g|
        np.testing.assert_allclose(d, lr * g / (0.001 * np.abs(g) + eps), rtol=1e-9)
    a = O.Nadam(init_acc=0.0)
    st = a.init_state(g.shape, np.float64)
    for t in range(1, 6):
        d, st = a.build(g, st, t)      # m_hat = g, g_hat = g/(1-b1^t)
        np.testing.assert_allclose(d, (0.9 * g + 0.1 * g / (1 - 0.9 ** t)) / (np.abs(g) + eps), rtol=1e-9)
    a = O.SGD(lr, momentum=0.5)
    st = a.init_state(g.shape, np.float64)
    v = np.zeros_like(g)
    for t in range(1, 6):
        d, st = a.build(g, st, t)      # v_t = lr g - mu v_{t-1} = lr g (1 - (-mu)^t) / (1 + mu)
        np.testing.assert_allclose(d, lr * g * (1 - (-0.5) ** t) / 1.5, rtol=1e-12)
    a = O.AdaDelta()
    st = a.init_state(g.shape, np.float64)
    d, st = a.build(g, st, 1)
    np.testing.assert_allclose(d, np.sqrt(eps) / np.sqrt(0.1 * g * g + eps) * g, rtol=1e-12)
    np.testing.assert_allclose(st[1], 0.1 * d * d, rtol=1e-12)


def test_average_uniform_and_pairwise():
    rng = np.random.default_rng(0)
    reps = [rng.standard_normal(1000).astype(f32) for _ in range(8)]
    ref = np.mean(np.stack(reps).astype(np.float64), axis=0)
    np.testing.assert_allclose(O.average_uniform(reps), ref, rtol=1e-6, atol=1e-7)
    np.testing.assert_array_equal(O.avg2(reps[0], reps[1]), (reps[0] + reps[1]) / f32(2))
    # one replica: identity
    np.testing.assert_array_equal(O.average_uniform(reps[:1]), reps[0])


def test_partition_loop_semantics(linear_function):
    """1-based iteration numbers, partial batch dropped, final loss evaluated after the last update."""
    X, Y = linear_function
    m = O.Model([O.Dense(1)], O.LOSS_MSE)
    init = {"0/weights": np.zeros((1, 1), f32), "1/weights": np.zeros(1, f32)}
    alg = O.Adam(0.1)
    it, p, st, loss = O.optimize_on_partition(m, alg, X, Y, 40, 0, init, O.init_opt_state(alg, init))
    assert it == 2                                   # 97 rows, batch 40: 2 full batches, 17 rows skipped
    # replay by hand
    q, s = init, O.init_opt_state(alg, init)
    for i in range(2):
        q, s, _, _ = O.train_step(m, alg, X[i * 40:(i + 1) * 40], Y[i * 40:(i + 1) * 40], q, s, i + 1)
    np.testing.assert_array_equal(p["0/weights"], q["0/weights"])
    assert loss == m.loss_of(X[40:80], Y[40:80], q)
    with pytest.raises(StopIteration):
        O.optimize_on_partition(m, alg, X[:10], Y[:10], 40, 0, init, O.init_opt_state(alg, init))
