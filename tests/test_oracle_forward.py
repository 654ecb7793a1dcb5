"""Pins the oracle's forward (GEMV/GEMM + bias + activation) against float64
brute force, closed forms and invariants — none of which restate its loops."""
import os

import numpy as np
import pytest
from scipy import special

from helpers import ALL_ACTS, make_oracle_net

GOLD = os.path.join(os.path.dirname(__file__), "golden")
E = np.load(os.path.join(GOLD, "expected.npz"))
F32 = np.float32


def test_piecewise_linear_activations_closed_form(O):
    x = np.array([-3.0, -1.0, -0.0, 0.0, 0.25, 1.0, 1.5, 10.0], dtype=F32)
    a = F32(0.01)
    assert np.array_equal(O.activate(x, O.ACT["relu"]), np.maximum(x, 0))
    assert np.array_equal(O.activate(x, O.ACT["leaky_relu"]), np.where(x > 0, x, a * x))
    assert np.array_equal(O.activate(x, O.ACT["foo52"]),
                          np.where(x > 1, F32(1) + a * (x - F32(1)), np.where(x < 0, a * x, x)).astype(F32))
    assert np.array_equal(O.activate(x, O.ACT["none"]), x)


def test_transcendental_activations_against_library(O):
    x = np.linspace(-12, 12, 4001).astype(F32)
    assert np.allclose(O.activate(x, O.ACT["sigmoid"]), special.expit(x.astype(np.float64)), rtol=3e-7, atol=1e-9)
    assert np.allclose(O.activate(x, O.ACT["tanh"]), np.tanh(x.astype(np.float64)), rtol=3e-7, atol=1e-9)
    s = O.activate(x, O.ACT["sigmoid"])
    assert np.allclose(s + s[::-1], 1.0, atol=2e-7)                 # sigmoid(-x) = 1 - sigmoid(x)


def test_softmax_invariants(O):
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((6, 1000)) * 4).astype(F32)
    y = O.activate(x, O.ACT["softmax"])
    assert np.allclose(y.sum(axis=1), 1.0, atol=1e-5)
    assert np.array_equal(y.argmax(axis=1), x.argmax(axis=1))
    assert np.allclose(y, special.softmax(x.astype(np.float64), axis=1), rtol=2e-5, atol=1e-9)
    shifted = O.activate(x + F32(3.0), O.ACT["softmax"])
    assert np.allclose(shifted, y, rtol=1e-4, atol=1e-9)
    # rows are independent: a huge value in one row must not leak into another
    x2 = x.copy(); x2[0, 0] = 80.0
    y2 = O.activate(x2, O.ACT["softmax"])
    assert np.array_equal(y2[1:], y[1:]) and y2[0, 0] > 0.999999


@pytest.mark.parametrize("fmt", ["f32", "f16", "bf16", "i8", "i4", "i2"])
def test_golden_forward_outputs(O, fmt):
    with open(os.path.join(GOLD, f"tiny_{fmt}.nn"), "rb") as f:
        net = O.Net.parse(f.read())
    X = E["tiny_X"]
    want = E[f"tiny_{fmt}_Y"]                                  # numpy float64, independent of the oracle
    assert np.allclose(net.forward_batch(X), want, rtol=2e-6, atol=2e-7)
    assert np.allclose(net.forward_batch_f64(X), want, rtol=1e-12, atol=1e-14)
    for i in range(X.shape[0]):
        assert np.allclose(net.forward_single(X[i]), want[i], rtol=2e-6, atol=2e-7)


@pytest.mark.parametrize("fmt", ["bf16", "i4"])
def test_golden_softmax_net(O, fmt):
    with open(os.path.join(GOLD, f"soft_{fmt}.nn"), "rb") as f:
        net = O.Net.parse(f.read())
    want = E[f"soft_{fmt}_Y"]
    assert np.allclose(net.forward_batch(E["soft_X"]), want, rtol=5e-6, atol=1e-7)


@pytest.mark.parametrize("act", ALL_ACTS)
def test_each_activation_in_a_net_against_numpy(O, act):
    net = make_oracle_net(O, [19, 33, 11], [act, "none"], seed=5)
    rng = np.random.default_rng(1)
    X = rng.standard_normal((7, 19)).astype(F32)
    h = X.astype(np.float64) @ net.W(0).astype(np.float64).T + net.b(0)
    f = {"sigmoid": special.expit, "relu": lambda v: np.maximum(v, 0), "tanh": np.tanh,
         "leaky_relu": lambda v: np.where(v > 0, v, np.float64(F32(0.01)) * v),
         "foo52": lambda v: np.where(v > 1, 1 + np.float64(F32(0.01)) * (v - 1), np.where(v < 0, np.float64(F32(0.01)) * v, v)),
         "softmax": lambda v: special.softmax(v, axis=1), "none": lambda v: v}[act]
    want = f(h) @ net.W(1).astype(np.float64).T + net.b(1)
    assert np.allclose(net.forward_batch(X), want, rtol=1e-5, atol=1e-6)


def test_layout_is_row_major_out_by_in(O):
    # a transposed-operand mistake fails: W[j][k] multiplies x[k] and lands in y[j]
    net = O.Net.new([3, 2], [O.ACT["none"]])
    net.W(0)[:] = np.array([[1, 2, 3], [10, 20, 30]], dtype=F32)
    net.b(0)[:] = np.array([0.5, -0.5], dtype=F32)
    y = net.forward_single(np.array([1, 0, -1], dtype=F32))
    assert np.array_equal(y, np.array([1 - 3 + 0.5, 10 - 30 - 0.5], dtype=F32))
    assert np.array_equal(net.weights[:6], np.array([1, 2, 3, 10, 20, 30], dtype=F32))


def test_mid_size_against_numpy_matmul(O):
    net = make_oracle_net(O, [784, 512, 1000, 10], ["relu", "relu", "softmax"], seed=2)
    rng = np.random.default_rng(3)
    X = rng.random((16, 784), dtype=F32)
    a = X.astype(np.float64)
    for l, act in enumerate(["relu", "relu", "softmax"]):
        a = a @ net.W(l).astype(np.float64).T + net.b(l)
        a = special.softmax(a, axis=1) if act == "softmax" else np.maximum(a, 0)
    got = net.forward_batch(X)
    assert np.max(np.abs(got - a)) / np.max(np.abs(a)) < 1e-5
    assert np.array_equal(got.argmax(1), a.argmax(1))
    sec, out = net.time_forward_batch(X, 1, None, 2)            # built-in threaded GEMM leg
    assert np.max(np.abs(out - a)) / np.max(np.abs(a)) < 1e-5 and sec > 0
    fn, desc, setter = O.find_sgemm()
    if fn is not None:                                          # BLAS leg, when a BLAS is present
        sec, out = net.time_forward_batch(X, 1, fn, 2)
        assert np.max(np.abs(out - a)) / np.max(np.abs(a)) < 1e-5


# ---------------------------------------------------------------------------
# evaluation step (compute_sample_loss SIMD.c:522-552, batch_compute_loss Training.c:421-435)
# ---------------------------------------------------------------------------
def test_sample_loss_closed_forms(O):
    """Pins: squared error of known vectors; cross-entropy of a one-hot target is -log of that
    output; the 1e-9 clamp at zero; the binary form under a sigmoid output layer (symmetric in
    (o, t) -> (1 - o, 1 - t)) with its clamp at one."""
    SIG, SOFT, NONE = O.ACT["sigmoid"], O.ACT["softmax"], O.ACT["none"]
    assert O.sample_loss([1.0, 2.0, -1.0], [0.5, 0.0, 1.0], 0, NONE) == pytest.approx(0.25 + 4.0 + 4.0, rel=1e-7)
    o = np.array([0.2, 0.7, 0.1], np.float32)
    assert O.sample_loss(o, [0, 1, 0], 1, SOFT) == pytest.approx(-np.log(0.7), rel=1e-6)
    assert O.sample_loss(o, [0.5, 0.25, 0.25], 1, SOFT) == pytest.approx(
        -(0.5 * np.log(0.2) + 0.25 * np.log(0.7) + 0.25 * np.log(0.1)), rel=1e-6)
    # an output of exactly zero is clamped to 1e-9, not -inf
    assert O.sample_loss([0.0, 1.0], [1, 0], 1, SOFT) == pytest.approx(-np.log(np.float32(1e-9)), rel=1e-6)
    # sigmoid output layer: binary cross-entropy per output
    a = O.sample_loss([0.3, 0.9], [1.0, 0.0], 1, SIG)
    assert a == pytest.approx(-(np.log(0.3) + np.log(1 - 0.9)), rel=1e-5)
    assert O.sample_loss([0.7, 0.1], [0.0, 1.0], 1, SIG) == pytest.approx(a, rel=1e-5)
    # the upper clamp 1 - 1e-9 rounds to 1 in FP32, so an output of exactly 1 still reaches log(0):
    # +inf against a target of 0, and 0 * -inf = NaN against a target of 1 (the arithmetic of
    # SIMD.c:538-541 as written)
    assert O.sample_loss([1.0], [0.0], 1, SIG) == float("inf")
    assert np.isnan(O.sample_loss([1.0], [1.0], 1, SIG))
    # a loss value outside the enum contributes nothing (neither branch runs)
    assert O.sample_loss(o, [0, 1, 0], 2, SOFT) == 0.0


def test_batch_loss_and_argmax(O):
    rng = np.random.default_rng(3)
    Y = rng.random((37, 11)).astype(np.float32)
    Y /= Y.sum(1, keepdims=True)
    T = np.eye(11, dtype=np.float32)[rng.integers(0, 11, 37)]
    want = sum(-np.log(Y[i, T[i].argmax()].astype(np.float64)) for i in range(37))
    assert O.batch_loss(Y, T, 1, O.ACT["softmax"]) == pytest.approx(want, rel=1e-5)
    assert O.batch_loss(Y, T, 0, O.ACT["softmax"]) == pytest.approx(((Y.astype(np.float64) - T) ** 2).sum(), rel=1e-5)
    assert np.array_equal(O.argmax_rows(Y), Y.argmax(1))
    tie = np.array([[1.0, 3.0, 3.0, 2.0], [5.0, 5.0, 5.0, 5.0]], np.float32)
    assert list(O.argmax_rows(tie)) == [1, 0]                      # first maximum


def test_single_sample_baseline_leg_computes_the_forward(O):
    """The CPU-baseline leg of the public forward (bias copy, sgemv or OpenMP rows of 4 x 8-lane dot products,
    activation: Network.c:218-247, SIMD.c:190-240) is only ever timed; what it computes must still be the forward:
    both variants against numpy float64 on a ragged net whose widths exercise the 32-, 8- and 1-element steps."""
    rng = np.random.default_rng(11)
    topo, acts = [301, 77, 45, 9], ["relu", "tanh", "softmax"]
    net = O.Net.new(topo, [O.ACT[a] for a in acts], 1)
    for l in range(3):
        net.W(l)[:] = (rng.standard_normal(net.W(l).shape) * 0.2).astype(np.float32)
        net.b(l)[:] = (rng.standard_normal(net.b(l).shape) * 0.1).astype(np.float32)
    x = rng.standard_normal(topo[0]).astype(np.float32)
    a = x.astype(np.float64)
    for l, act in enumerate(acts):
        z = net.W(l).astype(np.float64) @ a + net.b(l)
        a = {"relu": lambda z: np.maximum(z, 0), "tanh": np.tanh,
             "softmax": lambda z: np.exp(z - z.max()) / np.exp(z - z.max()).sum()}[act](z)
    legs = [None]
    if O.find_sgemv() is not None:
        legs.append(O.find_sgemv())
    for fn in legs:
        sec, out = net.time_forward_single(x, 2, fn, 2)
        assert sec > 0
        assert np.abs(out - a).max() <= 1e-5
