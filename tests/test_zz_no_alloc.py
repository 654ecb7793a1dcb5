"""sphip_forward_noalloc (the entry point that allocates nothing) against sphip_forward through the C-ABI.

Same kernels, same routing, a workspace laid out in the library's fixed scratch array instead of the net's own
buffers: the outputs must be bit-identical.  Every case makes two calls in a row, the second with fewer samples,
so that anything a kernel would read from the previous call's leftovers in the shared array shows up."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

F32 = np.float32


def _net(S, fmt, topo, acts, seed):
    prec = {"f32": S.PRECISION_FLOAT32, "f16": S.PRECISION_FP16, "bf16": S.PRECISION_BFLOAT16, "i8": S.PRECISION_INT8,
            "i4": S.PRECISION_INT4, "i2": S.PRECISION_INT2}[fmt]
    bits = {"f32": 32, "f16": 16, "bf16": 16, "i8": 8, "i4": 4, "i2": 2}[fmt]
    rng = np.random.default_rng(seed)
    net = S.DeviceNet(topo, acts, prec)
    for l in range(len(topo) - 1):
        K, N = topo[l], topo[l + 1]
        if bits >= 16:
            w = (rng.standard_normal(N * K) * np.sqrt(2.0 / K)).astype(F32)
            b = (rng.standard_normal(N) * 0.1).astype(F32)
            enc = {32: lambda a: a, 16: (lambda a: (a.view(np.uint32) >> 16).astype(np.uint16)) if fmt == "bf16"
                   else (lambda a: a.astype(np.float16).view(np.uint16))}[bits]
            net.upload(l, 0, enc(w))
            net.upload(l, 1, enc(b))
        else:
            net.upload(l, 0, rng.integers(0, 256, size=(N * K * bits + 7) // 8, dtype=np.uint8), 0.4 / np.sqrt(K))
            net.upload(l, 1, rng.integers(0, 256, size=(N * bits + 7) // 8, dtype=np.uint8), 0.1)
    return net


CASES = [
    # fmt, topology, activations, (first n, second smaller n), flags
    ("i8", [784, 512, 1000, 10], ["relu", "relu", "softmax"], (4096, 300), 0),     # tiled GEMMs, classifier head; at 300 the one-launch small-layer kernel
    ("i8", [784, 512, 1000, 10], ["relu", "relu", "softmax"], (4, 1), 0),          # vector kernels
    ("i4", [1024, 4096, 4096, 512], ["relu", "tanh", "none"], (64, 8), 0),         # streaming kernels, K splits + reduce
    ("i4", [1024, 4096, 4096, 512], ["relu", "tanh", "none"], (3, 2), 0),          # self-quantising integer GEMV
    ("i2", [2048, 2048, 96, 10], ["sigmoid", "relu", "softmax"], (33, 5), 16),     # forced two-launch integer GEMV (planes)
    ("i2", [512, 2048, 40, 10], ["sigmoid", "relu", "softmax"], (700, 64), 0),     # FP16 copies of small integer layers
    ("bf16", [1024, 1024, 1024, 1000], ["leaky_relu", "foo52", "softmax"], (1024, 100), 0),
    ("f16", [512, 768, 300], ["tanh", "none"], (300, 5), 0),
    ("f32", [784, 512, 1000, 10], ["relu", "relu", "softmax"], (256, 70), 0),      # FP32 matrix-core GEMM, split K
    ("f32", [96, 160, 10], ["foo52", "softmax"], (64, 1), 0),
    ("i4", [256, 512, 384, 40], ["relu", "tanh", "softmax"], (300, 9), 128),       # split activations: partial sums of both matrices
    ("bf16", [512, 1024, 1000], ["leaky_relu", "softmax"], (2048, 70), 128),
    ("i8", [777, 1030, 515, 33], ["relu", "tanh", "none"], (64, 5), 0),            # ragged rows: K split of the single-stage kernel
    ("i2", [256, 256, 256, 64, 10], ["relu", "relu", "tanh", "softmax"], (3, 1), 0),   # word-per-lane vector kernel
]


@pytest.mark.parametrize("fmt,topo,acts,ns,flags", CASES)
def test_noalloc_forward_equals_forward(S, fmt, topo, acts, ns, flags):
    act = {"sigmoid": S.ACT_SIGMOID, "relu": S.ACT_RELU, "tanh": S.ACT_TANH, "leaky_relu": S.ACT_LEAKY_RELU,
           "foo52": S.ACT_FOO52, "softmax": S.ACT_SOFTMAX, "none": S.ACT_NONE}
    net = _net(S, fmt, topo, [act[a] for a in acts], seed=sum(topo))
    fresh = _net(S, fmt, topo, [act[a] for a in acts], seed=sum(topo))   # never sees sphip_forward: no buffers of its own
    rng = np.random.default_rng(ns[0])
    for n in ns:                                          # two calls in a row, the second smaller
        X = rng.standard_normal((n, topo[0])).astype(F32)
        d_x = S.DeviceBuffer.from_numpy(X)
        d_y = S.DeviceBuffer(n * topo[-1] * 4)
        rc = fresh.forward_noalloc(d_x, n, d_y, flags)
        assert rc == 0, S.lib().sphip_last_error_string()
        S.synchronize()
        got = d_y.to_numpy(F32, (n, topo[-1]))
        want = net.forward(X, flags)
        assert np.isfinite(want).all()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (fmt, n)
        # What the entry point exists for: a warmed call takes no device memory.  `fresh` has no buffers of its own,
        # so an allocation on any route of this case would lower the free figure.
        free_before, _ = S.device_memory()
        assert fresh.forward_noalloc(d_x, n, d_y, flags) == 0
        S.synchronize()
        free_after, _ = S.device_memory()
        assert free_after == free_before, (fmt, n, free_before - free_after)
        assert np.array_equal(d_y.to_numpy(F32, (n, topo[-1])).view(np.uint32), want.view(np.uint32)), (fmt, n)
    net.destroy()
    fresh.destroy()


def test_noalloc_forward_in_the_split_mode_of_an_fp32_net(S):
    """That mode reads FP16 parts of the weights, which are made (allocated) by the first sphip_forward in the mode:
    before it the entry point refuses, after it the call works out of the scratch array like every other route."""
    topo, n = [1024, 2048, 10], 768                       # first layer 3.2 GFLOP: three FP16 products; the head: FP32 kernel
    net = _net(S, "f32", topo, [S.ACT_RELU, S.ACT_SOFTMAX], seed=3)
    X = np.random.default_rng(4).random((n, topo[0]), dtype=F32)
    d_x = S.DeviceBuffer.from_numpy(X)
    d_y = S.DeviceBuffer(n * topo[-1] * 4)
    assert net.forward_noalloc(d_x, n, d_y, S.SPHIP_SPLIT_ACTIVATIONS) == 1
    assert "FP16 parts" in S.lib().sphip_last_error_string().decode()
    want = net.forward(X, S.SPHIP_SPLIT_ACTIVATIONS)
    for m in (n, 740):
        assert net.forward_noalloc(d_x, m, d_y, S.SPHIP_SPLIT_ACTIVATIONS) == 0, S.lib().sphip_last_error_string()
        S.synchronize()
        free_before, _ = S.device_memory()
        assert net.forward_noalloc(d_x, m, d_y, S.SPHIP_SPLIT_ACTIVATIONS) == 0
        S.synchronize()
        free_after, _ = S.device_memory()
        assert free_after == free_before
        ref = want[:m] if m == n else net.forward(X[:m], S.SPHIP_SPLIT_ACTIVATIONS)
        assert np.array_equal(d_y.to_numpy(F32, (n, topo[-1]))[:m].view(np.uint32), ref.view(np.uint32)), m
    net.destroy()


def test_noalloc_forward_refuses_what_does_not_fit(S):
    """64 MiB of scratch: 8192 samples of a 4096-wide net need two 128 MiB activation buffers."""
    net = _net(S, "bf16", [256, 4096, 16], [S.ACT_RELU, S.ACT_NONE], seed=5)
    n = 8192
    d_x = S.DeviceBuffer(n * 256 * 4)
    d_y = S.DeviceBuffer(n * 16 * 4)
    assert net.forward_noalloc(d_x, n, d_y) == 1
    msg = S.lib().sphip_last_error_string().decode()
    assert "scratch" in msg and str(64 << 20) in msg, msg
    # a size that fits still works afterwards
    X = np.random.default_rng(1).standard_normal((100, 256)).astype(F32)
    d_x2 = S.DeviceBuffer.from_numpy(X)
    d_y2 = S.DeviceBuffer(100 * 16 * 4)
    assert net.forward_noalloc(d_x2, 100, d_y2) == 0
    S.synchronize()
    assert np.array_equal(d_y2.to_numpy(F32, (100, 16)), net.forward(X))
    assert S.lib().sphip_forward_noalloc(net.h, None, 100, d_y2.ptr, 0) == 1          # argument check
    net.destroy()
