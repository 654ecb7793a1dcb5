"""Pins the oracle's file parser/writer against hand-assembled .nn files made by
tests/golden/make_golden.py (numpy + struct only) and against byte counts."""
import os
import struct

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(__file__), "golden")
E = np.load(os.path.join(GOLD, "expected.npz"))
FMTS = ["f32", "f16", "bf16", "i8", "i4", "i2"]


def bits(a):
    return np.asarray(a, dtype=np.float32).view(np.uint32)


def read(name):
    with open(os.path.join(GOLD, name), "rb") as f:
        return f.read()


@pytest.mark.parametrize("fmt", FMTS)
def test_parse_golden_file(O, fmt):
    net = O.Net.parse(read(f"tiny_{fmt}.nn"), O.STRICT)
    assert net.topology == [37, 53, 29, 10]
    assert net.act == [O.ACT["foo52"], O.ACT["leaky_relu"], O.ACT["sigmoid"]]
    assert net.c.precision == O.PREC[fmt] and net.c.has_optimizer == 0 and not net.c.truncated
    assert np.array_equal(bits(net.weights), bits(E[f"tiny_{fmt}_W"]))
    assert np.array_equal(bits(net.biases), bits(E[f"tiny_{fmt}_b"]))
    rel = O.Net.parse(read(f"tiny_{fmt}.nn"), O.RELEASE)
    assert np.array_equal(bits(rel.weights), bits(E[f"tiny_{fmt}_W_release"]))
    assert np.array_equal(bits(rel.biases), bits(E[f"tiny_{fmt}_b_release"]))


def test_optimizer_block_is_skipped_array_by_array(O):
    blob = read("tiny_i8_opt.nn")
    assert len(blob) == 16 + 5 * 4 + 3 * (3932 - 28)          # header 16+5L, every array three times
    net = O.Net.parse(blob)
    assert net.c.has_optimizer == 1 and net.c.time_step == 77 and not net.c.truncated
    assert np.array_equal(bits(net.weights), bits(E["tiny_i8_W"]))
    assert np.array_equal(bits(net.biases), bits(E["tiny_i8_b"]))


@pytest.mark.parametrize("fmt", FMTS)
def test_file_sizes(O, fmt):
    # header 8 + 5L without optimizer block; payload sizes per format
    per = {"f32": lambda n: 4 * n, "f16": lambda n: 2 * n, "bf16": lambda n: 2 * n,
           "i8": lambda n: 4 + n, "i4": lambda n: 4 + (n + 1) // 2, "i2": lambda n: 4 + (n + 3) // 4}[fmt]
    topo = [37, 53, 29, 10]
    want = 8 + 5 * 4 + sum(per(topo[l] * topo[l + 1]) + per(topo[l + 1]) for l in range(3))
    assert len(read(f"tiny_{fmt}.nn")) == want


@pytest.mark.parametrize("fmt", FMTS)
def test_writer_reproduces_golden_bytes(O, fmt):
    # FP32 source -> oracle writer must give the file make_golden.py assembled from the same source
    src = O.Net.parse(read("tiny_f32.nn"))
    src.c.loss = 1
    assert src.serialize(O.PREC[fmt]) == read(f"tiny_{fmt}.nn")


def test_config2_file_size(O):
    # the INT8 file of the 784-512-1000-10 net is 924,982 bytes
    net = O.Net.new([784, 512, 1000, 10], [1, 1, 5])
    assert len(net.serialize(O.PREC["i8"])) == 924982
    assert len(net.serialize(O.PREC["f32"])) == 3699748


@pytest.mark.parametrize("cut", [1, 5, 9, 27, 28, 29, 500, 1990])
def test_truncated_files(O, cut):
    blob = read("tiny_i4.nn")[:cut]
    if cut < 28:                      # inside the header: no net
        with pytest.raises(ValueError):
            O.Net.parse(blob)
    else:                             # inside the payload: net comes back flagged (Serialize.c:596-608)
        net = O.Net.parse(blob)
        assert net.c.truncated == 1


def test_header_validation(O):
    good = bytearray(read("tiny_i8.nn"))
    def err(mut):
        b = bytearray(good); mut(b)
        with pytest.raises(ValueError) as e:
            O.Net.parse(bytes(b))
        return str(e.value)
    assert "err=2" in err(lambda b: b.__setitem__(0, 2))                       # version
    assert "err=3" in err(lambda b: b.__setitem__(slice(2, 6), struct.pack("<I", 1)))   # layers < 2
    assert "err=4" in err(lambda b: b.__setitem__(6, 2))                       # loss
    assert "err=5" in err(lambda b: b.__setitem__(8, 6))                       # precision
    assert "err=6" in err(lambda b: b.__setitem__(9 + 16, 7))                  # activation


def test_soft_files(O):
    for fmt in ("bf16", "i4"):
        net = O.Net.parse(read(f"soft_{fmt}.nn"))
        assert net.topology == [24, 40, 7] and net.act == [O.ACT["tanh"], O.ACT["softmax"]]
        assert np.array_equal(bits(net.weights), bits(E[f"soft_{fmt}_W"]))
