"""The batched training step on the device against the oracle's restatement of the reference's
(Training.c:313-419, 439-507): gradients, every optimizer, clipping, and train() end to end.
FP32 throughout; tolerance 1e-4 relative to the largest magnitude of the compared array."""
import os

import numpy as np
import pytest

import oracle as O
import spingalett_amd as S
from helpers import make_oracle_net, rel_max_abs

pytestmark = pytest.mark.gpu

TOL = 1e-4


def device_net(onet):
    d = S.DeviceNet(onet.topology, onet.act, S.PRECISION_FLOAT32)
    for l in range(onet.layers - 1):
        d.upload(l, 0, onet.W(l).ravel())
        d.upload(l, 1, onet.b(l))
    return d


def targets_for(rng, n, width, one_hot):
    if one_hot:
        return np.eye(width, dtype=np.float32)[rng.integers(0, width, n)]
    return rng.uniform(0, 1, (n, width)).astype(np.float32)


def step_args(optimizer, loss, **kw):
    a = S.SphipTrainArgs()
    a.optimizer = optimizer
    a.loss_func = loss
    a.learning_rate = kw.get("lr", 0.01)
    a.weight_decay = kw.get("weight_decay", 0.0)
    a.momentum = kw.get("momentum", 0.9)
    a.beta1 = kw.get("beta1", 0.9)
    a.beta2 = kw.get("beta2", 0.999)
    a.epsilon = kw.get("epsilon", 1e-8)
    a.max_grad_norm = kw.get("max_grad_norm", 0.0)
    a.beta1_pow_t = 1.0
    a.beta2_pow_t = 1.0
    return a


GRAD_CASES = [
    # topology, hidden activations, output activation, loss, batch
    ([20, 33, 17, 5], ["sigmoid", "tanh"], "softmax", 0, 50),            # vector-path forward, ragged sizes
    ([20, 33, 17, 5], ["relu", "leaky_relu"], "softmax", 1, 7),
    ([9, 64, 3], ["foo52"], "sigmoid", 1, 64),
    ([70, 130, 90, 10], ["tanh", "relu"], "softmax", 1, 300),            # matrix-core forward, K splits everywhere
    ([70, 130, 90, 10], ["leaky_relu", "sigmoid"], "none", 0, 257),
    ([64, 128, 64], ["none"], "tanh", 0, 1024),
    ([390, 520, 300, 10], ["tanh", "relu"], "softmax", 1, 700),          # ragged edges in every product
    ([5, 3], [], "relu", 1, 33),                                         # single layer, general output rule
    ([128, 256, 10], ["relu"], "softmax", 1, 1),                         # one sample
]


@pytest.mark.parametrize("topo,hidden,out_act,loss,n", GRAD_CASES)
def test_gradients_match_oracle(topo, hidden, out_act, loss, n):
    acts = hidden + [out_act]
    onet = make_oracle_net(O, topo, acts, seed=len(topo) * 7 + n, bias_std=0.2, loss=loss)
    rng = np.random.default_rng(n)
    X = rng.standard_normal((n, topo[0])).astype(np.float32)
    T = targets_for(rng, n, topo[-1], loss == 1 and out_act in ("softmax", "sigmoid"))
    gW, gB, out = onet.batch_gradients(X, T)
    want_loss = O.batch_loss(out, T, loss, O.ACT[out_act])

    d = device_net(onet)
    d.train_begin()
    got_loss = d.train_step(X, T, step_args(-1, loss), want_loss=True)
    assert got_loss == pytest.approx(want_loss, rel=1e-4, abs=1e-5)
    for l in range(len(topo) - 1):
        w = gW[onet.woff[l]: onet.woff[l] + topo[l] * topo[l + 1]]
        b = gB[onet.boff[l]: onet.boff[l] + topo[l + 1]]
        assert rel_max_abs(d.train_get(S.SPHIP_TRAIN_GW, l), w) <= TOL, l
        assert rel_max_abs(d.train_get(S.SPHIP_TRAIN_GB, l), b) <= TOL, l
        # gradients only: nothing moved
        np.testing.assert_array_equal(d.train_get(S.SPHIP_TRAIN_W, l), onet.W(l).ravel())
    d.destroy()


OPT_CASES = [
    (S.OPTIMIZER_SGD, {}),
    (S.OPTIMIZER_SGD, {"weight_decay": 0.3}),
    (S.OPTIMIZER_MOMENTUM, {"momentum": 0.8, "weight_decay": 0.1}),
    (S.OPTIMIZER_RMSPROP, {"beta2": 0.9, "epsilon": 1e-6, "weight_decay": 0.05}),
    (S.OPTIMIZER_ADAM, {}),
    (S.OPTIMIZER_ADAM, {"weight_decay": 0.2, "beta1": 0.8, "beta2": 0.95}),
    (S.OPTIMIZER_ADAMW, {"weight_decay": 0.2}),
    (S.OPTIMIZER_ADAM, {"max_grad_norm": 0.05}),
    (S.OPTIMIZER_SGD, {"max_grad_norm": 1e6}),                           # norm below the limit: untouched
]


@pytest.mark.parametrize("opt,kw", OPT_CASES)
def test_four_steps_of_each_optimizer_match_oracle(opt, kw):
    topo, acts, loss, n = [30, 70, 40, 6], ["tanh", "leaky_relu", "softmax"], 1, 96
    onet = make_oracle_net(O, topo, acts, seed=opt + 3, bias_std=0.1, loss=loss)
    rng = np.random.default_rng(opt)
    X = rng.standard_normal((n, topo[0])).astype(np.float32)
    T = targets_for(rng, n, topo[-1], True)
    d = device_net(onet)
    d.train_begin()
    st = O.TrainState(onet)
    a = step_args(opt, loss, lr=0.02, **kw)
    okw = {"lr": 0.02, **kw}
    for step in range(4):
        gW, gB, _ = onet.batch_gradients(X, T)
        onet.apply_gradients(st, gW, gB, opt, **okw)
        a.beta1_pow_t = float(st.beta1_pow)
        a.beta2_pow_t = float(st.beta2_pow)
        d.train_step(X, T, a)
        for l in range(len(topo) - 1):
            assert rel_max_abs(d.train_get(S.SPHIP_TRAIN_W, l), onet.W(l).ravel()) <= TOL, (step, l)
            assert rel_max_abs(d.train_get(S.SPHIP_TRAIN_B, l), onet.b(l)) <= TOL, (step, l)
    for l in range(len(topo) - 1):
        wo, wc = onet.woff[l], topo[l] * topo[l + 1]
        if opt in (S.OPTIMIZER_MOMENTUM, S.OPTIMIZER_ADAM, S.OPTIMIZER_ADAMW):
            assert rel_max_abs(d.train_get(S.SPHIP_TRAIN_MW, l), st.mW[wo: wo + wc]) <= TOL
        if opt in (S.OPTIMIZER_RMSPROP, S.OPTIMIZER_ADAM, S.OPTIMIZER_ADAMW):
            assert rel_max_abs(d.train_get(S.SPHIP_TRAIN_VW, l), st.vW[wo: wo + wc]) <= 2 * TOL
    d.destroy()


def test_moments_can_be_seeded_and_read_back():
    onet = make_oracle_net(O, [6, 9, 4], ["relu", "none"])
    d = device_net(onet)
    d.train_begin()
    rng = np.random.default_rng(0)
    for which in (S.SPHIP_TRAIN_MW, S.SPHIP_TRAIN_VW, S.SPHIP_TRAIN_MB, S.SPHIP_TRAIN_VB):
        for l in range(2):
            v = rng.standard_normal(54 if which in (S.SPHIP_TRAIN_MW, S.SPHIP_TRAIN_VW) and l == 0 else
                                    36 if which in (S.SPHIP_TRAIN_MW, S.SPHIP_TRAIN_VW) else (9, 4)[l]).astype(np.float32)
            d.train_set(which, l, v)
            np.testing.assert_array_equal(d.train_get(which, l), v)
    d.destroy()


def test_step_argument_checks():
    onet = make_oracle_net(O, [6, 9, 4], ["relu", "none"])
    d = device_net(onet)
    X, T = np.zeros((2, 6), np.float32), np.zeros((2, 4), np.float32)
    with pytest.raises(S.SpingalettError, match="sphip_train_begin"):
        d.train_step(X, T, step_args(0, 0))
    d.train_begin()
    with pytest.raises(S.SpingalettError, match="optimizer"):
        d.train_step(X, T, step_args(9, 0))
    d.destroy()
    # packed formats cannot be trained in place, hidden softmax is rejected as in the reference
    q = S.DeviceNet([4, 4], [S.ACT_NONE], S.PRECISION_INT8)
    q.upload(0, 0, np.zeros(16, np.uint8), 1.0)
    q.upload(0, 1, np.zeros(4, np.uint8), 1.0)
    with pytest.raises(S.SpingalettError, match="FP32"):
        q.train_begin()
    q.destroy()
    sm = device_net(make_oracle_net(O, [4, 5, 3], ["softmax", "none"]))
    with pytest.raises(S.SpingalettError, match="softmax"):
        sm.train_begin()
    sm.destroy()


# ------------------------------------------------------------------ train() through the public interface
def public_net(topo, acts, loss, seed=0):
    onet = make_oracle_net(O, topo, acts, seed=seed, bias_std=0.1, loss=loss)
    net = S.new_spingalett(loss)
    S.layer(net, topo[0], 0, S.WEIGHT_INITIALIZATION_NONE)
    for l in range(1, len(topo)):
        S.layer(net, topo[l], O.ACT[acts[l - 1]], S.WEIGHT_INITIALIZATION_NONE)
    for l in range(len(topo) - 1):
        S.weights_view(net, l)[:] = onet.W(l)
        S.biases_view(net, l)[:] = onet.b(l)
    return net, onet


def test_full_batch_train_matches_oracle_epochs():
    topo, acts, loss, n, epochs = [12, 40, 8, 3], ["tanh", "relu", "softmax"], 1, 150, 6
    net, onet = public_net(topo, acts, loss, seed=5)
    rng = np.random.default_rng(1)
    X = rng.standard_normal((n, topo[0])).astype(np.float32)
    T = targets_for(rng, n, topo[-1], True)
    seen = []
    S.clear_error()
    S.train(net, X, T, epochs, S.STRATEGY_FULL_BATCH, S.OPTIMIZER_ADAM, learning_rate=0.01,
            callback=lambda p, epoch, err: seen.append((epoch, err)) or False, callback_interval=2)
    assert S.last_error()[0] == S.SPINGALETT_OK, S.last_error()
    st = O.TrainState(onet)
    want_err = {}
    for epoch in range(1, epochs + 1):
        gW, gB, out = onet.batch_gradients(X, T)
        want_err[epoch] = O.batch_loss(out, T, loss, O.ACT["softmax"]) / n
        onet.apply_gradients(st, gW, gB, O.OPT_ADAM, lr=0.01)
    for l in range(len(topo) - 1):
        assert rel_max_abs(S.weights_view(net, l), onet.W(l)) <= TOL
        assert rel_max_abs(S.biases_view(net, l), onet.b(l)) <= TOL
    assert [e for e, _ in seen] == [2, 4, 6]
    for e, err in seen:
        assert err == pytest.approx(want_err[e], rel=1e-4)
    assert net.contents.time_step == epochs
    # moments came back too (they are what a later save with the optimizer block writes)
    mw = np.ctypeslib.as_array(net.contents.opt_m_weights, shape=(int(net.contents.total_weights),))
    assert rel_max_abs(mw, st.mW) <= TOL
    # and forward() now runs the trained weights
    y = S.forward_batch(net, X[:5])
    assert rel_max_abs(y, onet.forward_batch(X[:5])) <= TOL
    S.free_network(net)


def test_repeated_train_calls_pick_up_host_side_edits_and_keep_their_state():
    """The device net and its training buffers survive a train() call; the next call uploads the host arrays
    again (they are the caller's to edit), continues the optimizer state, and may bring a different batch size."""
    topo, acts, loss = [10, 24, 4], ["relu", "softmax"], 1
    net, onet = public_net(topo, acts, loss, seed=11)
    rng = np.random.default_rng(3)
    X = rng.standard_normal((90, topo[0])).astype(np.float32)
    T = targets_for(rng, 90, topo[-1], True)
    st = O.TrainState(onet)

    def oracle_epochs(x, t, k):
        st.beta1_pow = st.beta2_pow = np.float32(1.0)      # the running powers restart with every call (Training.c:684-685)
        for _ in range(k):
            gW, gB, _ = onet.batch_gradients(x, t)
            onet.apply_gradients(st, gW, gB, O.OPT_ADAM, lr=0.01)

    S.clear_error()
    S.train(net, X, T, 3, S.STRATEGY_FULL_BATCH, S.OPTIMIZER_ADAM, learning_rate=0.01)
    oracle_epochs(X, T, 3)
    # second call: same net, moments continue (time step 4, 5)
    S.train(net, X, T, 2, S.STRATEGY_FULL_BATCH, S.OPTIMIZER_ADAM, learning_rate=0.01)
    oracle_epochs(X, T, 2)
    assert net.contents.time_step == 5
    for l in range(2):
        assert rel_max_abs(S.weights_view(net, l), onet.W(l)) <= TOL
    # the caller edits the host arrays between calls; a larger batch follows
    S.weights_view(net, 0)[:] *= 0.5
    S.biases_view(net, 1)[:] += 0.25
    onet.W(0)[:] *= 0.5
    onet.b(1)[:] += 0.25
    X2 = rng.standard_normal((200, topo[0])).astype(np.float32)
    T2 = targets_for(rng, 200, topo[-1], True)
    S.train(net, X2, T2, 2, S.STRATEGY_FULL_BATCH, S.OPTIMIZER_ADAM, learning_rate=0.01)
    oracle_epochs(X2, T2, 2)
    assert S.last_error()[0] == S.SPINGALETT_OK, S.last_error()
    for l in range(2):
        assert rel_max_abs(S.weights_view(net, l), onet.W(l)) <= TOL
        assert rel_max_abs(S.biases_view(net, l), onet.b(l)) <= TOL
    assert rel_max_abs(S.forward_batch(net, X2[:7]), onet.forward_batch(X2[:7])) <= TOL
    S.free_network(net)


def test_small_batch_train_learns_xor_and_counts_steps():
    """The reference's sanity problem (Examples/XOR.c:20-64)."""
    net, _ = public_net([2, 8, 1], ["tanh", "sigmoid"], 0, seed=4)
    X = np.float32([[0, 0], [0, 1], [1, 0], [1, 1]] * 8)
    T = np.float32([[0], [1], [1], [0]] * 8)
    errs = []
    S.clear_error()
    S.train(net, X, T, 150, S.STRATEGY_SMALL_BATCH, S.OPTIMIZER_ADAM, batch_size=12, learning_rate=0.05,
            callback=lambda p, epoch, err: errs.append(err) or False, callback_interval=1)
    assert S.last_error()[0] == S.SPINGALETT_OK, S.last_error()
    assert net.contents.time_step == 150 * 3                   # 32 samples in batches of 12: 3 steps per epoch
    assert errs[-1] < 0.05 * errs[0]
    y = S.forward_batch(net, X[:4])
    np.testing.assert_array_equal(y[:, 0] > 0.5, T[:4, 0] > 0.5)
    S.free_network(net)


def test_layer_after_train_keeps_gradients_and_moments():
    """layer() copies all six gradient / moment arrays into the regrown net (Network.c:130-146): adding a head after
    train() (fine-tuning) must not zero what train() left in the host arrays."""
    net, _ = public_net([2, 8, 3], ["tanh", "sigmoid"], 0, seed=5)
    X = np.float32([[0, 0], [0, 1], [1, 0], [1, 1]] * 4)
    T = np.float32([[0, 1, 0], [1, 0, 1], [1, 1, 0], [0, 0, 1]] * 4)
    S.clear_error()
    S.train(net, X, T, 5, S.STRATEGY_FULL_BATCH, S.OPTIMIZER_ADAM, learning_rate=0.05)
    assert S.last_error()[0] == S.SPINGALETT_OK, S.last_error()
    nc = net.contents
    tw, tb = int(nc.total_weights), int(nc.total_biases)
    view = lambda name, cnt: np.ctypeslib.as_array(getattr(net.contents, name), shape=(cnt,)).copy()
    names_w = ["weights", "grad_weights", "opt_m_weights", "opt_v_weights"]
    names_b = ["biases", "grad_biases", "opt_m_biases", "opt_v_biases"]
    before = {k: view(k, tw) for k in names_w} | {k: view(k, tb) for k in names_b}
    assert all(np.any(before[k] != 0) for k in before)              # train() really left something in every one
    steps = nc.time_step
    S.layer(net, 4, S.ACT_NONE, S.WEIGHT_INITIALIZATION_XAVIER)
    assert net.contents.time_step == steps
    for k in names_w:
        assert np.array_equal(view(k, tw), before[k]), k            # old prefix unchanged
    for k in names_b:
        assert np.array_equal(view(k, tb), before[k]), k
    assert not view("opt_m_weights", tw + 12)[tw:].any() and not view("grad_biases", tb + 4)[tb:].any()   # new part zero
    S.free_network(net)


def test_callback_stops_training_and_autosave_writes_files(tmp_path):
    net, _ = public_net([4, 6, 2], ["relu", "none"], 0)
    rng = np.random.default_rng(0)
    X = rng.standard_normal((10, 4)).astype(np.float32)
    T = rng.standard_normal((10, 2)).astype(np.float32)
    path = str(tmp_path / "auto.nn")
    S.clear_error()
    S.train(net, X, T, 10, S.STRATEGY_FULL_BATCH, S.OPTIMIZER_SGD, callback=lambda p, epoch, err: epoch == 4,
            autosave_mode=S.AUTOSAVE_NEW_FILES, autosave_interval=2, autosave_path=path,
            autosave_precision=S.PRECISION_FLOAT32)
    assert S.last_error()[0] == S.SPINGALETT_OK, S.last_error()
    assert net.contents.time_step == 4
    assert sorted(os.listdir(tmp_path)) == ["auto_epoch_2.nn", "auto_epoch_4.nn"]
    # the file holds the weights of that epoch: reloading the last one gives the net as it stands
    again = S.load_spingalett(str(tmp_path / "auto_epoch_4.nn"))
    np.testing.assert_array_equal(S.weights_view(again, 0), S.weights_view(net, 0))
    S.free_network(again)
    S.free_network(net)


@pytest.mark.parametrize("opt,kw", [(S.OPTIMIZER_SGD, {"weight_decay": 0.1}), (S.OPTIMIZER_MOMENTUM, {}),
                                    (S.OPTIMIZER_RMSPROP, {"weight_decay": 0.2}), (S.OPTIMIZER_ADAM, {}),
                                    (S.OPTIMIZER_ADAMW, {"weight_decay": 0.1})])
def test_per_sample_strategy_matches_oracle(opt, kw):
    """STRATEGY_SAMPLE: one update per sample in order with the rules of backpropagation() (Training.c:78-213);
    max_grad_norm is not applied there."""
    topo, acts, loss, n, epochs = [6, 12, 4], ["tanh", "softmax"], 1, 9, 2
    net, onet = public_net(topo, acts, loss, seed=13)
    rng = np.random.default_rng(4)
    X = rng.standard_normal((n, topo[0])).astype(np.float32)
    T = targets_for(rng, n, topo[-1], True)
    errs = []
    S.clear_error()
    S.train(net, X, T, epochs, S.STRATEGY_SAMPLE, opt, learning_rate=0.02, max_grad_norm=1e-3,
            callback=lambda p, epoch, err: errs.append(err) or False, **kw)
    assert S.last_error()[0] == S.SPINGALETT_OK, S.last_error()
    st = O.TrainState(onet)
    want = []
    for _ in range(epochs):
        total = 0.0
        for s_ in range(n):
            gW, gB, out = onet.batch_gradients(X[s_:s_ + 1], T[s_:s_ + 1], grad_scale=1.0)
            total += O.batch_loss(out, T[s_:s_ + 1], loss, O.ACT["softmax"])
            onet.apply_gradients(st, gW, gB, opt, lr=0.02, decay_in_grad=True, **kw)
        want.append(total / n)
    for l in range(len(topo) - 1):
        assert rel_max_abs(S.weights_view(net, l), onet.W(l)) <= TOL, l
        assert rel_max_abs(S.biases_view(net, l), onet.b(l)) <= TOL, l
    assert errs == pytest.approx(want, rel=1e-4)
    assert net.contents.time_step == epochs * n
    S.free_network(net)


def test_xor_with_the_example_settings_converges():
    """The reference's end-to-end sanity check (Examples/XOR.c:27-64): 2-8-1, FOO52 / sigmoid, He / Xavier start, squared
    error, full batch, AdamW 0.01 with decay 1e-4, 10,000 epochs; every output within 0.1 of its target."""
    X = np.float32([[0, 0], [0, 1], [1, 0], [1, 1]])
    T = np.float32([[0], [1], [1], [0]])
    passed = 0
    for attempt in range(3):                                   # the start is random, as in the example
        net = S.new_spingalett(S.LOSS_MSE)
        S.layer(net, 2)
        S.layer(net, 8, S.ACT_FOO52, S.WEIGHT_INITIALIZATION_HE)
        S.layer(net, 1, S.ACT_SIGMOID, S.WEIGHT_INITIALIZATION_XAVIER)
        reports = []
        S.clear_error()
        S.train(net, X, T, 10000, S.STRATEGY_FULL_BATCH, S.OPTIMIZER_ADAMW, learning_rate=0.01, weight_decay=1e-4,
                callback=lambda p, epoch, err: reports.append(epoch) or False, callback_interval=5000)
        assert S.last_error()[0] == S.SPINGALETT_OK, S.last_error()
        assert reports == [5000, 10000]
        passed = sum(abs(float(S.forward(net, X[i])[0]) - float(T[i, 0])) < 0.1 for i in range(4))
        S.free_network(net)
        if passed == 4:
            break
    assert passed == 4


def test_train_rejects_what_the_reference_rejects():
    net, _ = public_net([4, 6, 2], ["softmax", "none"], 0)
    X, T = np.zeros((3, 4), np.float32), np.zeros((3, 2), np.float32)
    S.clear_error()
    S.train(net, X, T, 1)
    assert S.last_error() == (S.SPINGALETT_ERR_INVALID, "Softmax is not supported in hidden layers")
    S.free_network(net)
    net, _ = public_net([4, 6, 2], ["relu", "none"], 0)
    w0 = S.weights_view(net, 0).copy()
    for kw, msg in (({"training_mode": S.MODE_GENERATOR_FUNCTION}, "Generator function"),
                    ({"sample_count": 0}, "Invalid training arguments"),
                    ({"strategy": 7}, "unknown optimizer, strategy or loss")):
        S.clear_error()
        S.train(net, X, T, 1, **kw)
        code, text = S.last_error()
        assert code == S.SPINGALETT_ERR_INVALID and msg in text, (kw, text)
    S.clear_error()
    S.train(net, X, T, 0)
    assert S.last_error()[0] == S.SPINGALETT_ERR_INVALID
    np.testing.assert_array_equal(S.weights_view(net, 0), w0)
    S.free_network(net)


def test_training_a_quantized_net_continues_from_its_fp32_arrays():
    onet = make_oracle_net(O, [16, 32, 4], ["relu", "softmax"], seed=9, loss=1)
    blob = onet.serialize(O.PREC["i8"])
    ref = O.Net.parse(blob)                                    # what the loader's FP32 arrays hold
    ref.c.loss = 1
    net = S.load_spingalett_memory(blob)
    rng = np.random.default_rng(2)
    X = rng.standard_normal((80, 16)).astype(np.float32)
    T = targets_for(rng, 80, 4, True)
    S.forward_batch(net, X)                                    # device copy holds the INT8 arrays now
    assert S.lib().spingalett_hip_precision(net) == S.PRECISION_INT8
    S.clear_error()
    S.train(net, X, T, 2, S.STRATEGY_FULL_BATCH, S.OPTIMIZER_SGD, learning_rate=0.1)
    assert S.last_error()[0] == S.SPINGALETT_OK, S.last_error()
    st = O.TrainState(ref)
    for _ in range(2):
        gW, gB, _ = ref.batch_gradients(X, T)
        ref.apply_gradients(st, gW, gB, O.OPT_SGD, lr=0.1)
    assert rel_max_abs(S.weights_view(net, 0), ref.W(0)) <= TOL
    assert S.lib().spingalett_hip_precision(net) == S.PRECISION_FLOAT32
    assert rel_max_abs(S.forward_batch(net, X), ref.forward_batch(X)) <= TOL
    S.free_network(net)


def test_full_size_benchmark_step_properties():
    """The reference's benchmark net at its full batch (Examples/Benchmark.c: 784-512-1000-10, 20,000 samples), through
    properties that do not need the oracle at that size: the gradient of the whole batch is the mean of the gradients
    of its two halves, the reported loss is the sum of the halves' losses, and Adam steps lower the loss of one-hot targets."""
    topo, n = [784, 512, 1000, 10], 20000
    rng = np.random.default_rng(3)
    d = S.DeviceNet(topo, [S.ACT_RELU, S.ACT_RELU, S.ACT_SOFTMAX], S.PRECISION_FLOAT32)
    for l in range(3):
        std = np.sqrt((2.0 if l < 2 else 1.0) / topo[l])
        d.upload(l, 0, (rng.standard_normal(topo[l] * topo[l + 1]) * std).astype(np.float32))
        d.upload(l, 1, np.zeros(topo[l + 1], np.float32))
    X = rng.random((n, topo[0]), dtype=np.float32)
    T = rng.random((n, topo[-1]), dtype=np.float32)
    d.train_begin()
    grads = {}
    losses = {}
    for name, sl in (("all", slice(0, n)), ("a", slice(0, n // 2)), ("b", slice(n // 2, n))):
        losses[name] = d.train_step(X[sl], T[sl], step_args(-1, 1), want_loss=True)
        grads[name] = [d.train_get(S.SPHIP_TRAIN_GW, l) for l in range(3)] + [d.train_get(S.SPHIP_TRAIN_GB, l) for l in range(3)]
    assert losses["all"] == pytest.approx(losses["a"] + losses["b"], rel=1e-5)
    for g_all, g_a, g_b in zip(grads["all"], grads["a"], grads["b"]):
        assert np.isfinite(g_all).all()
        assert rel_max_abs(g_all, 0.5 * (g_a.astype(np.float64) + g_b)) <= TOL
    # descent needs targets the output rule is the gradient for (rows that sum to 1; the benchmark's uniform targets do not)
    hot = np.eye(topo[-1], dtype=np.float32)[rng.integers(0, topo[-1], n)]
    a = step_args(S.OPTIMIZER_ADAM, 1, lr=0.001)
    seen = []
    for step in range(1, 7):
        a.beta1_pow_t, a.beta2_pow_t = 0.9 ** step, 0.999 ** step
        seen.append(d.train_step(X, hot, a, want_loss=True))
    assert seen[-1] < seen[0]
    d.destroy()
