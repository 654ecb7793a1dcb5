"""Device dequantisation must equal the reference decode bit for bit
(Serialize.c:45-85, 195-297).  Every case goes through the C-ABI:
load_spingalett_memory -> spingalett_hip_decode (which launches the decode
kernel over the packed array held on the device)."""
import os
import struct

import numpy as np
import pytest

from helpers import FORMATS, make_oracle_net

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(__file__), "golden")
E = np.load(os.path.join(GOLD, "expected.npz"))
F32 = np.float32


def bits(a):
    return np.asarray(a, dtype=F32).view(np.uint32)


def nn_file(topo, acts, prec, arrays):
    """Hand-assembled file: arrays = [W0 payload, b0 payload, W1 payload, ...] as bytes."""
    h = struct.pack("<HIBBB", 1, len(topo), 0, 0, prec) + struct.pack(f"<{len(topo)}I", *topo) + bytes(acts)
    return h + b"".join(arrays)


def load(S, blob):
    S.clear_error()
    net = S.load_spingalett_memory(blob)
    assert net is not None, S.last_error()
    return net


@pytest.mark.parametrize("fmt,prec", [("f16", 1), ("bf16", 2)])
def test_all_65536_codes(S, O, fmt, prec):
    codes = np.arange(65536, dtype=np.uint16)
    blob = nn_file([256, 256], [6], prec, [codes.tobytes(), codes[:256].tobytes()])
    net = load(S, blob)
    got = S.hip_decode(net, 0, 0)
    want = O.decode_array(codes.tobytes(), 65536, prec)
    assert np.array_equal(bits(got), bits(want))
    if fmt == "bf16":
        assert np.array_equal(bits(got), codes.astype(np.uint32) << 16)
    else:
        ieee = codes.view(np.float16).astype(F32)
        ok = ~np.isnan(ieee)
        assert np.array_equal(bits(got)[ok], bits(ieee)[ok])
        assert set(bits(got)[~ok]) == {0x7FC00000, 0xFFC00000}
    assert np.array_equal(bits(S.hip_decode(net, 0, 1)), bits(want[:256]))
    S.free_network(net)


@pytest.mark.parametrize("mx", [1.0, 0.37, 3.3e-5, 1e20, 2.0 ** -130, 0.0, -1.0, float("nan")])
@pytest.mark.parametrize("mode", [0, 1])
def test_all_integer_codes(S, O, mx, mode):
    L = S.lib()
    L.spingalett_set_dequant_mode(mode)
    try:
        head = struct.pack("<f", mx)
        # INT8: 16x16 holds all 256 codes; INT4: 4x4 all 16; INT2: 2x2 all 4
        cases = [
            (3, [16, 16], np.arange(256, dtype=np.uint8).tobytes(), np.arange(16, dtype=np.uint8).tobytes()),
            (4, [4, 4], bytes((2 * i) | ((2 * i + 1) << 4) for i in range(8)), bytes([0x98, 0x7F])),
            (5, [2, 2], bytes([0b11100100]), bytes([0b00001110])),
        ]
        for prec, topo, wcodes, bcodes in cases:
            blob = nn_file(topo, [6], prec, [head + wcodes, head + bcodes])
            net = load(S, blob)
            n = topo[0] * topo[1]
            got = S.hip_decode(net, 0, 0)
            want = O.decode_array(head + wcodes, n, prec, mode)
            assert np.array_equal(bits(got), bits(want)), (prec, mx, mode)
            gb = S.hip_decode(net, 0, 1)
            assert np.array_equal(bits(gb), bits(O.decode_array(head + bcodes, topo[1], prec, mode)))
            # the host arrays of the loader are the same numbers
            assert np.array_equal(bits(S.weights_view(net, 0).ravel()), bits(want))
            S.free_network(net)
    finally:
        L.spingalett_set_dequant_mode(0)


@pytest.mark.parametrize("fmt", FORMATS)
def test_golden_files(S, fmt):
    net = S.load_spingalett(os.path.join(GOLD, f"tiny_{fmt}.nn"))
    assert net is not None
    W = np.concatenate([S.hip_decode(net, l, 0) for l in range(3)])
    b = np.concatenate([S.hip_decode(net, l, 1) for l in range(3)])
    assert np.array_equal(bits(W), bits(E[f"tiny_{fmt}_W"]))      # odd dims: INT4/INT2 rows straddle bytes
    assert np.array_equal(bits(b), bits(E[f"tiny_{fmt}_b"]))
    S.lib().spingalett_set_dequant_mode(1)
    try:
        Wr = np.concatenate([S.hip_decode(net, l, 0) for l in range(3)])
        assert np.array_equal(bits(Wr), bits(E[f"tiny_{fmt}_W_release"]))
    finally:
        S.lib().spingalett_set_dequant_mode(0)
    S.free_network(net)


@pytest.mark.parametrize("fmt", ["i8", "i4", "i2", "f16"])
def test_mid_size_random_net(S, O, fmt):
    src = make_oracle_net(O, [784, 512, 1000, 10], ["relu", "relu", "softmax"], seed=1)
    blob = src.serialize(O.PREC[fmt])
    ref = O.Net.parse(blob)
    net = load(S, blob)
    for l in range(3):
        assert np.array_equal(bits(S.hip_decode(net, l, 0)), bits(ref.W(l).ravel()))
        assert np.array_equal(bits(S.hip_decode(net, l, 1)), bits(ref.b(l)))
    S.free_network(net)


def test_invalidate_switches_the_device_to_the_fp32_arrays(S):
    net = S.load_spingalett(os.path.join(GOLD, "tiny_i4.nn"))
    assert S.lib().spingalett_hip_precision(net) == S.PRECISION_INT4
    S.hip_decode(net, 0, 0)
    S.weights_view(net, 0)[0, 0] = 123.0
    S.lib().spingalett_hip_invalidate(net)
    assert S.lib().spingalett_hip_precision(net) == S.PRECISION_FLOAT32
    assert S.hip_decode(net, 0, 0)[0] == 123.0
    S.free_network(net)


def test_decode_argument_checks(S):
    net = S.load_spingalett(os.path.join(GOLD, "tiny_i4.nn"))
    out = np.empty(4, F32)
    assert S.lib().spingalett_hip_decode(net, 3, 0, out.ctypes.data) == 1      # layer out of range
    assert S.last_error()[0] == S.SPINGALETT_ERR_INVALID
    S.clear_error()
    assert S.lib().spingalett_hip_decode(net, 0, 2, out.ctypes.data) == 1
    S.clear_error()
    assert S.lib().spingalett_hip_decode(net, 0, 0, None) == 1
    S.free_network(net)
