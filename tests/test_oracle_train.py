"""Pins the oracle's restatement of the batched training step (deltas, gradients, clipping,
optimizer updates) against what the mathematics fixes: central differences in float64, closed
forms of the first optimizer step, numpy norms.  CPU only."""
import numpy as np
import pytest

import oracle as O
from helpers import make_oracle_net

ACTS64 = {
    "sigmoid": lambda x: 1.0 / (1.0 + np.exp(-x)),
    "relu": lambda x: np.where(x > 0, x, 0.0),
    "tanh": np.tanh,
    "leaky_relu": lambda x: np.where(x > 0, x, 0.01 * x),
    "foo52": lambda x: np.where(x > 1, 1 + 0.01 * (x - 1), np.where(x < 0, 0.01 * x, x)),
    "none": lambda x: x,
}


def forward64(Ws, bs, acts, X):
    a = X.astype(np.float64)
    for W, b, act in zip(Ws, bs, acts):
        z = a @ W.T + b
        if act == "softmax":
            e = np.exp(z - z.max(axis=1, keepdims=True))
            a = e / e.sum(axis=1, keepdims=True)
        else:
            a = ACTS64[act](z)
    return a


def objective64(Ws, bs, acts, X, T, loss):
    """The function whose gradient each output-layer rule of the reference is: cross-entropy through a
    softmax or sigmoid output layer, half the squared error in every other combination."""
    a = forward64(Ws, bs, acts, X)
    if loss == 1 and acts[-1] == "softmax":
        return -np.sum(T * np.log(a)) / X.shape[0]
    if loss == 1 and acts[-1] == "sigmoid":
        return -np.sum(T * np.log(a) + (1 - T) * np.log(1 - a)) / X.shape[0]
    return 0.5 * np.sum((a - T) ** 2) / X.shape[0]


@pytest.mark.parametrize("act", ["sigmoid", "relu", "tanh", "leaky_relu", "foo52", "none"])
def test_derivative_is_the_slope_of_the_activation(act):
    x = np.array([-2.3, -0.7, -0.2, 0.3, 0.6, 0.9, 1.4, 2.5], dtype=np.float64)
    h = 1e-6
    slope = (ACTS64[act](x + h) - ACTS64[act](x - h)) / (2 * h)
    a = O.activate(x.astype(np.float32), O.ACT[act])
    np.testing.assert_allclose(O.derivative(a, O.ACT[act]), slope, rtol=2e-6, atol=2e-7)


def test_derivative_constants_at_the_kinks():
    assert O.derivative(np.float32([0.0]), O.ACT["relu"])[0] == 0.0
    assert O.derivative(np.float32([0.0]), O.ACT["leaky_relu"])[0] == np.float32(0.01)
    np.testing.assert_array_equal(O.derivative(np.float32([0.0, 1.0, -1e-30, 1.0000001]), O.ACT["foo52"]),
                                  np.float32([1.0, 1.0, 0.01, 0.01]))
    # softmax shares the sigmoid's form (only met on an output layer outside the two dedicated rules)
    assert O.derivative(np.float32([0.25]), O.ACT["softmax"])[0] == np.float32(0.1875)


CASES = [
    # (hidden activations, output activation, loss)
    (["sigmoid", "tanh"], "softmax", 0),
    (["relu", "leaky_relu"], "softmax", 1),
    (["foo52", "none"], "sigmoid", 1),
    (["tanh", "sigmoid"], "tanh", 0),
    (["leaky_relu", "relu"], "none", 0),
    (["none", "tanh"], "sigmoid", 0),
    (["sigmoid", "foo52"], "relu", 1),          # cross-entropy without softmax / sigmoid takes the general rule
]


@pytest.mark.parametrize("hidden,out_act,loss", CASES)
def test_gradients_match_central_differences(hidden, out_act, loss):
    topo = [5, 7, 4, 3]
    acts = hidden + [out_act]
    net = make_oracle_net(O, topo, acts, seed=11 + loss, bias_std=0.3, loss=loss)
    rng = np.random.default_rng(5)
    N = 6
    X = rng.standard_normal((N, topo[0])).astype(np.float32)
    if out_act in ("softmax", "sigmoid") and loss == 1:
        T = np.eye(topo[-1], dtype=np.float32)[rng.integers(0, topo[-1], N)]
    else:
        T = rng.uniform(0, 1, (N, topo[-1])).astype(np.float32)
    gW, gB, out = net.batch_gradients(X, T)
    Ws = [net.W(l).astype(np.float64) for l in range(3)]
    bs = [net.b(l).astype(np.float64) for l in range(3)]
    np.testing.assert_allclose(out, forward64(Ws, bs, acts, X), rtol=1e-5, atol=1e-6)

    h = 1e-6
    for l in range(3):
        fdW = np.zeros_like(Ws[l])
        for idx in np.ndindex(*Ws[l].shape):
            keep = Ws[l][idx]
            Ws[l][idx] = keep + h
            up = objective64(Ws, bs, acts, X, T, loss)
            Ws[l][idx] = keep - h
            dn = objective64(Ws, bs, acts, X, T, loss)
            Ws[l][idx] = keep
            fdW[idx] = (up - dn) / (2 * h)
        fdB = np.zeros_like(bs[l])
        for j in range(bs[l].size):
            keep = bs[l][j]
            bs[l][j] = keep + h
            up = objective64(Ws, bs, acts, X, T, loss)
            bs[l][j] = keep - h
            dn = objective64(Ws, bs, acts, X, T, loss)
            bs[l][j] = keep
            fdB[j] = (up - dn) / (2 * h)
        got_w = gW[net.woff[l]: net.woff[l] + fdW.size].reshape(fdW.shape)
        got_b = gB[net.boff[l]: net.boff[l] + fdB.size]
        scale = max(np.abs(fdW).max(), 1e-3)
        assert np.abs(got_w - fdW).max() <= 2e-5 * scale + 1e-7, (l, np.abs(got_w - fdW).max(), scale)
        assert np.abs(got_b - fdB).max() <= 2e-5 * max(np.abs(fdB).max(), 1e-3) + 1e-7, l


def test_grad_scale_is_a_plain_factor_and_bias_gradient_is_the_column_sum():
    net = make_oracle_net(O, [4, 6, 2], ["tanh", "none"], seed=3)
    rng = np.random.default_rng(0)
    X = rng.standard_normal((9, 4)).astype(np.float32)
    T = rng.standard_normal((9, 2)).astype(np.float32)
    gW1, gB1, _ = net.batch_gradients(X, T, grad_scale=1.0)
    gW2, gB2, _ = net.batch_gradients(X, T, grad_scale=0.25)
    np.testing.assert_allclose(gW2, 0.25 * gW1, rtol=1e-6)
    np.testing.assert_allclose(gB2, 0.25 * gB1, rtol=1e-6)
    # a constant-one input column turns its weight gradient into the bias gradient
    Xone = X.copy()
    Xone[:, 0] = 1.0
    gW, gB, _ = net.batch_gradients(Xone, T, grad_scale=1.0)
    np.testing.assert_allclose(gW[: 6 * 4].reshape(6, 4)[:, 0], gB[:6], rtol=1e-6, atol=1e-7)


def test_clip_grad_norm():
    net = make_oracle_net(O, [3, 5, 2], ["relu", "none"])
    rng = np.random.default_rng(1)
    gW = rng.standard_normal(net.weights.size).astype(np.float32)
    gB = rng.standard_normal(net.biases.size).astype(np.float32)
    norm = float(np.sqrt(np.sum(gW.astype(np.float64) ** 2) + np.sum(gB.astype(np.float64) ** 2)))
    w0, b0 = gW.copy(), gB.copy()
    assert net.clip_grad_norm(gW, gB, 2 * norm) == pytest.approx(norm, rel=1e-6)
    np.testing.assert_array_equal(gW, w0)
    np.testing.assert_array_equal(gB, b0)
    assert net.clip_grad_norm(gW, gB, 0.5) == pytest.approx(norm, rel=1e-6)
    after = float(np.sqrt(np.sum(gW.astype(np.float64) ** 2) + np.sum(gB.astype(np.float64) ** 2)))
    assert after == pytest.approx(0.5, rel=1e-5)
    np.testing.assert_allclose(gW, w0 * (0.5 / norm), rtol=1e-5)
    # max_norm <= 0 switches clipping off and reports 0
    assert net.clip_grad_norm(gW, gB, 0.0) == 0.0


def _fresh(seed=2):
    net = make_oracle_net(O, [3, 4, 2], ["tanh", "none"], seed=seed)
    rng = np.random.default_rng(seed)
    gW = rng.standard_normal(net.weights.size).astype(np.float32)
    gB = rng.standard_normal(net.biases.size).astype(np.float32)
    return net, O.TrainState(net), gW, gB


def test_sgd_first_step_and_decay():
    net, st, gW, gB = _fresh()
    w0, b0 = net.weights.copy(), net.biases.copy()
    net.apply_gradients(st, gW.copy(), gB.copy(), O.OPT_SGD, lr=0.1)
    np.testing.assert_allclose(net.weights, w0 - 0.1 * gW, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(net.biases, b0 - 0.1 * gB, rtol=1e-6, atol=1e-7)
    net, st, gW, gB = _fresh()
    net.apply_gradients(st, gW.copy(), gB.copy(), O.OPT_SGD, lr=0.1, weight_decay=0.5)
    np.testing.assert_allclose(net.weights, w0 - 0.1 * (gW + 0.5 * w0), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(net.biases, b0 - 0.1 * gB, rtol=1e-6, atol=1e-7)       # never decayed


def test_momentum_geometric_sum():
    net, st, gW, gB = _fresh()
    w0 = net.weights.copy()
    steps, mom, lr = 5, 0.8, 0.05
    for _ in range(steps):
        net.apply_gradients(st, gW.copy(), gB.copy(), O.OPT_MOMENTUM, lr=lr, momentum=mom)
    # velocity after t steps of a constant gradient: g (1 - mom^t) / (1 - mom)
    total = sum((1 - mom ** t) / (1 - mom) for t in range(1, steps + 1))
    np.testing.assert_allclose(net.weights, w0 - lr * total * gW, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(st.mW, gW * (1 - mom ** steps) / (1 - mom), rtol=1e-5)


@pytest.mark.parametrize("opt", [O.OPT_ADAM, O.OPT_ADAMW])
@pytest.mark.parametrize("b1,b2", [(0.9, 0.999), (0.5, 0.7)])
def test_adam_first_step_is_lr_times_sign(opt, b1, b2):
    net, st, gW, gB = _fresh()
    w0, b0 = net.weights.copy(), net.biases.copy()
    eps = 1e-8
    net.apply_gradients(st, gW.copy(), gB.copy(), opt, lr=0.01, beta1=b1, beta2=b2, epsilon=eps)
    # bias-corrected first moments are g and g^2 whatever the betas
    np.testing.assert_allclose(net.weights, w0 - 0.01 * gW / np.sqrt(gW.astype(np.float64) ** 2 + eps), rtol=2e-5, atol=1e-7)
    np.testing.assert_allclose(net.biases, b0 - 0.01 * gB / np.sqrt(gB.astype(np.float64) ** 2 + eps), rtol=2e-5, atol=1e-7)
    # the reference forms 1 - beta in FP32 (Training.c:447-448)
    np.testing.assert_allclose(st.mW, (np.float32(1) - np.float32(b1)) * gW, rtol=1e-6)
    np.testing.assert_allclose(st.vW, (np.float32(1) - np.float32(b2)) * gW * gW, rtol=1e-6)
    assert float(st.beta1_pow) == pytest.approx(b1) and float(st.beta2_pow) == pytest.approx(b2)


def test_adam_folds_decay_into_the_gradient_and_adamw_shrinks_the_weight():
    lr, wd, eps = 0.01, 0.3, 1e-8
    net, st, gW, gB = _fresh()
    w0 = net.weights.copy()
    net.apply_gradients(st, gW.copy(), gB.copy(), O.OPT_ADAM, lr=lr, weight_decay=wd, epsilon=eps)
    g = gW + wd * w0
    np.testing.assert_allclose(net.weights, w0 - lr * g / np.sqrt(g.astype(np.float64) ** 2 + eps), rtol=2e-5, atol=1e-7)
    net, st, gW, gB = _fresh()
    net.apply_gradients(st, gW.copy(), gB.copy(), O.OPT_ADAMW, lr=lr, weight_decay=wd, epsilon=eps)
    np.testing.assert_allclose(net.weights, w0 * (1 - lr * wd) - lr * gW / np.sqrt(gW.astype(np.float64) ** 2 + eps),
                               rtol=2e-5, atol=1e-7)


def test_rmsprop_first_step():
    lr, b2, eps, wd = 0.02, 0.9, 1e-6, 0.1
    net, st, gW, gB = _fresh()
    w0, b0 = net.weights.copy(), net.biases.copy()
    net.apply_gradients(st, gW.copy(), gB.copy(), O.OPT_RMSPROP, lr=lr, beta2=b2, epsilon=eps, weight_decay=wd)
    g64 = gW.astype(np.float64)
    omb2 = float(np.float32(1) - np.float32(b2))
    np.testing.assert_allclose(net.weights, w0 - lr * (wd * w0 + g64 / np.sqrt(omb2 * g64 ** 2 + eps)), rtol=2e-5, atol=1e-7)
    gb = gB.astype(np.float64)
    np.testing.assert_allclose(net.biases, b0 - lr * gb / np.sqrt(omb2 * gb ** 2 + eps), rtol=2e-5, atol=1e-7)
    assert not st.mW.any()                                    # no first moment


def test_rmsprop_per_sample_rule_folds_decay_into_the_gradient():
    """backpropagation() (Training.c:196-211): decay * W joins the gradient before the second moment."""
    lr, b2, eps, wd = 0.02, 0.9, 1e-6, 0.4
    net, st, gW, gB = _fresh()
    w0, b0 = net.weights.copy(), net.biases.copy()
    net.apply_gradients(st, gW.copy(), gB.copy(), O.OPT_RMSPROP, lr=lr, beta2=b2, epsilon=eps, weight_decay=wd,
                        decay_in_grad=True)
    omb2 = float(np.float32(1) - np.float32(b2))
    g = gW.astype(np.float64) + wd * w0
    np.testing.assert_allclose(net.weights, w0 - lr * g / np.sqrt(omb2 * g ** 2 + eps), rtol=2e-5, atol=1e-7)
    np.testing.assert_allclose(st.vW, omb2 * g ** 2, rtol=1e-5)
    gb = gB.astype(np.float64)                                # biases carry no decay in either rule
    np.testing.assert_allclose(net.biases, b0 - lr * gb / np.sqrt(omb2 * gb ** 2 + eps), rtol=2e-5, atol=1e-7)
    # without decay the two rules coincide up to the rounding of lr * g / sqrt(.) against lr * (g / sqrt(.))
    n1, s1, g1, h1 = _fresh()
    n2, s2, g2, h2 = _fresh()
    n1.apply_gradients(s1, g1, h1, O.OPT_RMSPROP, lr=lr, beta2=b2, epsilon=eps)
    n2.apply_gradients(s2, g2, h2, O.OPT_RMSPROP, lr=lr, beta2=b2, epsilon=eps, decay_in_grad=True)
    np.testing.assert_allclose(n1.weights, n2.weights, rtol=1e-6)


@pytest.mark.parametrize("opt", [O.OPT_ADAM, O.OPT_ADAMW])
@pytest.mark.parametrize("b1,b2", [(0.9, 0.999), (0.5, 0.7)])
def test_adam_moment_recurrences_under_a_constant_gradient(opt, b1, b2):
    """Steps 1..5 with the same gradient (SIMD.c:279-382): m_t = (1 - b1^t) g and v_t = (1 - b2^t) g^2, so the
    bias-corrected moments stay g and g^2 and every step moves a weight by lr g / sqrt(g^2 + eps); AdamW
    shrinks the weight by (1 - lr wd) before each of them.  A wrong coefficient on the beta m / beta v terms,
    which a first step from zero moments cannot see, breaks the moments from step 2 on."""
    lr, eps, wd = 0.01, 1e-8, (0.3 if opt == O.OPT_ADAMW else 0.0)
    net, st, gW, gB = _fresh()
    w = net.weights.astype(np.float64)
    b = net.biases.astype(np.float64)
    g64, gb64 = gW.astype(np.float64), gB.astype(np.float64)
    omb1, omb2 = float(np.float32(1) - np.float32(b1)), float(np.float32(1) - np.float32(b2))
    for t in range(1, 6):
        net.apply_gradients(st, gW.copy(), gB.copy(), opt, lr=lr, beta1=b1, beta2=b2, epsilon=eps, weight_decay=wd)
        w = w * (1 - lr * wd) - lr * g64 / np.sqrt(g64 ** 2 + eps)
        b = b - lr * gb64 / np.sqrt(gb64 ** 2 + eps)                        # biases are never decayed
        np.testing.assert_allclose(net.weights, w, rtol=5e-5, atol=2e-7, err_msg=f"step {t}")
        np.testing.assert_allclose(net.biases, b, rtol=5e-5, atol=2e-7, err_msg=f"step {t}")
        # geometric sums of the recurrences, with 1 - beta as the reference forms it in FP32
        np.testing.assert_allclose(st.mW, omb1 * g64 * sum(b1 ** k for k in range(t)), rtol=2e-5, err_msg=f"m, step {t}")
        np.testing.assert_allclose(st.vW, omb2 * g64 ** 2 * sum(b2 ** k for k in range(t)), rtol=2e-5, err_msg=f"v, step {t}")
        assert float(st.beta1_pow) == pytest.approx(b1 ** t, rel=1e-5) and float(st.beta2_pow) == pytest.approx(b2 ** t, rel=1e-5)


def test_adam_second_step_with_a_doubled_gradient():
    """g then 2 g: m_2 = (1 - b1)(b1 + 2) g and v_2 = (1 - b2)(b2 + 4) g^2, corrected by 1 - b^2: the two betas
    enter with different weights, so exchanging them (or their moments) shows."""
    lr, eps, b1, b2 = 0.01, 1e-8, 0.6, 0.9
    net, st, gW, gB = _fresh()
    w0 = net.weights.astype(np.float64)
    g = gW.astype(np.float64)
    net.apply_gradients(st, gW.copy(), gB.copy(), O.OPT_ADAM, lr=lr, beta1=b1, beta2=b2, epsilon=eps)
    net.apply_gradients(st, 2 * gW, 2 * gB, O.OPT_ADAM, lr=lr, beta1=b1, beta2=b2, epsilon=eps)
    m2 = (1 - b1) * (b1 + 2) * g / (1 - b1 ** 2)
    v2 = (1 - b2) * (b2 + 4) * g ** 2 / (1 - b2 ** 2)
    want = w0 - lr * g / np.sqrt(g ** 2 + eps) - lr * m2 / np.sqrt(v2 + eps)
    np.testing.assert_allclose(net.weights, want, rtol=5e-5, atol=2e-7)


def test_rmsprop_second_moment_recurrence_under_a_constant_gradient():
    """SIMD.c:455-494: v_t = (1 - b2^t) g^2 (no bias correction), so step t moves a weight by
    lr g / sqrt((1 - b2^t) g^2 + eps)."""
    lr, b2, eps = 0.02, 0.8, 1e-6
    net, st, gW, gB = _fresh()
    w = net.weights.astype(np.float64)
    g = gW.astype(np.float64)
    omb2 = float(np.float32(1) - np.float32(b2))
    for t in range(1, 6):
        net.apply_gradients(st, gW.copy(), gB.copy(), O.OPT_RMSPROP, lr=lr, beta2=b2, epsilon=eps)
        vt = omb2 * g ** 2 * sum(b2 ** k for k in range(t))
        w = w - lr * g / np.sqrt(vt + eps)
        np.testing.assert_allclose(st.vW, vt, rtol=2e-5, err_msg=f"v, step {t}")
        np.testing.assert_allclose(net.weights, w, rtol=5e-5, atol=2e-7, err_msg=f"step {t}")


def test_clipping_precedes_the_update():
    net, st, gW, gB = _fresh()
    w0 = net.weights.copy()
    norm = float(np.sqrt(np.sum(gW.astype(np.float64) ** 2) + np.sum(gB.astype(np.float64) ** 2)))
    net.apply_gradients(st, gW.copy(), gB.copy(), O.OPT_SGD, lr=0.1, max_grad_norm=0.25)
    np.testing.assert_allclose(net.weights, w0 - 0.1 * gW * (0.25 / norm), rtol=1e-5, atol=1e-7)


def test_training_lowers_the_objective_on_xor():
    """End to end on the reference's own sanity problem (Examples/XOR.c:20-64): full-batch steps on the
    four XOR samples drive the outputs to the right side of 0.5."""
    net = make_oracle_net(O, [2, 8, 1], ["tanh", "sigmoid"], seed=4, init="xavier", bias_std=0.0, loss=0)
    X = np.float32([[0, 0], [0, 1], [1, 0], [1, 1]])
    T = np.float32([[0], [1], [1], [0]])
    st = O.TrainState(net)
    first = None
    for _ in range(400):
        gW, gB, out = net.batch_gradients(X, T)
        if first is None:
            first = float(np.sum((out - T) ** 2))
        net.apply_gradients(st, gW, gB, O.OPT_ADAM, lr=0.05)
    out = net.forward_batch(X)
    assert float(np.sum((out - T) ** 2)) < 0.05 * first
    np.testing.assert_array_equal(out[:, 0] > 0.5, T[:, 0] > 0.5)
