"""Seeded random nets through the public batched forward: every weight format, ragged and aligned widths, one to
four layers, every activation, batch sizes on both sides of every routing threshold, plain and split mode, against the
oracle's float64 forward on the decoded weights.  The fixed cases elsewhere pin each kernel family; this sweep is what
catches a routing rule that sends a shape to a kernel that does not fit it."""
import numpy as np
import pytest

from helpers import make_oracle_net, quantized_pair, rel_max_abs

pytestmark = pytest.mark.gpu

ACTS = ["sigmoid", "relu", "tanh", "leaky_relu", "foo52", "none"]
FMTS = ["f32", "f16", "bf16", "i8", "i4", "i2"]
BATCHES = [1, 2, 3, 4, 5, 7, 8, 9, 16, 31, 64, 65, 100, 129, 256, 257, 300, 777, 2000]


def _case(i):
    rng = np.random.default_rng(20260 + i)
    depth = int(rng.integers(1, 5))
    kind = int(rng.integers(0, 3))
    if kind == 0:
        topo = [int(rng.integers(1, 700)) for _ in range(depth + 1)]              # any width
    elif kind == 1:
        topo = [int(rng.integers(1, 40)) * 8 for _ in range(depth + 1)]           # whole 16-byte units of 16-bit values
    else:
        topo = [int(rng.choice([64, 128, 256, 512, 1024, 2048])) for _ in range(depth + 1)]
    acts = [str(rng.choice(ACTS)) for _ in range(depth)]
    if rng.random() < 0.4:
        acts[-1] = "softmax"
    return rng, topo, acts, str(rng.choice(FMTS)), int(rng.choice(BATCHES)), bool(rng.random() < 0.3)


@pytest.mark.parametrize("block", range(8))
def test_random_nets_against_the_float64_forward(S, O, block):
    for i in range(block * 12, block * 12 + 12):
        rng, topo, acts, fmt, n, split = _case(i)
        src = make_oracle_net(O, topo, acts, seed=i, bias_std=0.1)
        _, ref, net = quantized_pair(O, S, src, fmt)
        X = rng.standard_normal((n, topo[0])).astype(np.float32)
        want = ref.forward_batch_f64(X)
        if split:
            assert S.lib().spingalett_set_net_activations(net, S.NET_ACTIVATIONS_SPLIT) == 0
        got = S.forward_batch(net, X)
        S.free_network(net)
        assert got is not None, (i, S.last_error())
        # FP32 weights, up to four samples, and split mode are FP32-grade; the 16-bit matrix-core paths 2e-2
        tol = 1e-4 if (fmt == "f32" or n <= 4 or split) else 2e-2
        assert np.isfinite(got).all(), (i, fmt, topo, n)
        assert rel_max_abs(got, want) <= tol, (i, fmt, topo, acts, n, split, rel_max_abs(got, want))
