"""Shared builders for the tests (not collected by pytest)."""
import numpy as np

ALL_ACTS = ["sigmoid", "relu", "tanh", "leaky_relu", "foo52", "softmax", "none"]
FORMATS = ["f32", "f16", "bf16", "i8", "i4", "i2"]


def make_oracle_net(O, topology, acts, seed=0, init="he", bias_std=0.1, loss=0):
    """A seeded FP32 net in the oracle's container. acts: names."""
    rng = np.random.default_rng(seed)
    net = O.Net.new(topology, [O.ACT[a] for a in acts], loss)
    for l in range(len(topology) - 1):
        fan_in = topology[l]
        std = np.sqrt((2.0 if init == "he" else 1.0) / fan_in)
        net.W(l)[:] = (rng.standard_normal((topology[l + 1], fan_in)) * std).astype(np.float32)
        net.b(l)[:] = (rng.standard_normal(topology[l + 1]) * bias_std).astype(np.float32)
    return net


def quantized_pair(O, S, net, fmt, mode=0, with_optimizer=False):
    """Serialize `net` in `fmt` with the oracle writer; return (file bytes,
    oracle net decoded from them, library net loaded from them)."""
    blob = net.serialize(O.PREC[fmt], with_optimizer)
    ref = O.Net.parse(blob, mode)
    S.clear_error()
    lib_net = S.load_spingalett_memory(blob)
    assert lib_net is not None, S.last_error()
    return blob, ref, lib_net


def rel_max_abs(got, ref):
    ref = np.asarray(ref, dtype=np.float64)
    got = np.asarray(got, dtype=np.float64)
    den = np.max(np.abs(ref))
    return float(np.max(np.abs(got - ref)) / (den if den > 0 else 1.0))


def argmax_agreement(got, want):
    """(raw, decided): raw = fraction of rows with the same argmax; decided = the
    same fraction over rows whose reference top-2 gap exceeds twice the largest
    absolute deviation of this run.  A flip outside that band cannot be rounding."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    same = got.argmax(1) == want.argmax(1)
    err = np.max(np.abs(got - want))
    top2 = np.sort(want, axis=1)[:, -2:]
    decided = (top2[:, 1] - top2[:, 0]) > 2.0 * err
    return float(same.mean()), float(same[decided].mean()) if decided.any() else 1.0
