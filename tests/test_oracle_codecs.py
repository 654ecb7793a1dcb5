"""Pins the oracle's codecs (oracle/sp_oracle.c) against what the mathematics
fixes: IEEE float32 arithmetic done by numpy on every integer code, numpy's
half->single conversion on all 65,536 FP16 codes, the closed form code<<16 for
BF16, and hand-derived payloads (tests/golden/kat.json)."""
import json
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(__file__), "golden")
F32 = np.float32
MAXES = [1.0, 0.37, 3.3e-5, 1e20, 2.0 ** -130, 127.0, 7.0]


def bits(a):
    return np.asarray(a, dtype=F32).view(np.uint32)


def test_fp16_all_codes_match_ieee_with_nan_rule(O):
    codes = np.arange(65536, dtype=np.uint16)
    got = O.decode_array(codes.tobytes(), 65536, O.PREC["f16"])
    want = codes.view(np.float16).astype(F32)
    wb = bits(want).copy()
    nan = np.isnan(want)
    assert nan.sum() == 2046
    wb[nan] = ((codes[nan].astype(np.uint32) >> 15) << 31) | 0x7FC00000     # Serialize.c:64
    assert np.array_equal(bits(got), wb)


def test_bf16_all_codes_closed_form(O):
    codes = np.arange(65536, dtype=np.uint16)
    got = O.decode_array(codes.tobytes(), 65536, O.PREC["bf16"])
    assert np.array_equal(bits(got), codes.astype(np.uint32) << 16)


@pytest.mark.parametrize("mx", MAXES)
def test_int8_all_codes_both_evaluations(O, mx):
    q = np.arange(-128, 128).astype(np.int8)
    pay = F32(mx).tobytes() + q.tobytes()
    strict = (q.astype(F32) / F32(127)) * F32(mx)                 # Serialize.c:233 as written
    release = q.astype(F32) * (F32(mx) * (F32(1) / F32(127)))     # -freciprocal-math form
    assert np.array_equal(bits(O.decode_array(pay, 256, O.PREC["i8"], O.STRICT)), bits(strict))
    assert np.array_equal(bits(O.decode_array(pay, 256, O.PREC["i8"], O.RELEASE)), bits(release))


@pytest.mark.parametrize("mx", MAXES)
def test_int4_all_codes_and_nibble_order(O, mx):
    # element 2i in the low nibble of byte i, element 2i+1 in the high nibble (Serialize.c:148-152)
    q = np.array([0, 1, 2, 3, 4, 5, 6, 7, -8, -7, -6, -5, -4, -3, -2, -1, 7])
    u = (q & 15).astype(np.uint8)
    u2 = np.concatenate([u, [0]]).astype(np.uint8)
    pay = F32(mx).tobytes() + (u2[0::2] | (u2[1::2] << 4)).astype(np.uint8).tobytes()
    strict = (q.astype(F32) / F32(7)) * F32(mx)
    release = q.astype(F32) * (F32(mx) * (F32(1) / F32(7)))
    assert np.array_equal(bits(O.decode_array(pay, 17, O.PREC["i4"], O.STRICT)), bits(strict))
    assert np.array_equal(bits(O.decode_array(pay, 17, O.PREC["i4"], O.RELEASE)), bits(release))


@pytest.mark.parametrize("mx", MAXES)
def test_int2_all_codes_and_field_order(O, mx):
    q = np.array([0, 1, -2, -1, 1, 0, -1])
    u = np.concatenate([(q & 3), [0]]).astype(np.uint8)
    pay = F32(mx).tobytes() + (u[0::4] | (u[1::4] << 2) | (u[2::4] << 4) | (u[3::4] << 6)).astype(np.uint8).tobytes()
    want = q.astype(F32) * F32(mx)                                 # Serialize.c:285
    for mode in (O.STRICT, O.RELEASE):
        assert np.array_equal(bits(O.decode_array(pay, 7, O.PREC["i2"], mode)), bits(want))


def test_strict_and_release_differ_somewhere(O):
    # a plausible mistake (one evaluation used for both modes) fails here
    q = np.arange(-128, 128).astype(np.int8)
    pay = F32(0.37).tobytes() + q.tobytes()
    a = O.decode_array(pay, 256, O.PREC["i8"], O.STRICT)
    b = O.decode_array(pay, 256, O.PREC["i8"], O.RELEASE)
    assert (bits(a) != bits(b)).sum() > 10


def test_known_answer_payloads(O):
    for k in json.load(open(os.path.join(GOLD, "kat.json"))):
        pay = bytes.fromhex(k["payload"])
        for mode, key in ((O.STRICT, "strict_bits"), (O.RELEASE, "release_bits")):
            got = O.decode_array(pay, k["n"], O.PREC[k["fmt"]], mode)
            assert [int(v) for v in bits(got)] == k[key], (k["fmt"], mode)


def test_short_payload_is_refused(O):
    with pytest.raises(ValueError):
        O.decode_array(b"\x00" * 7, 4, O.PREC["i8"])              # needs 4 + 4 bytes


# ---- writer ---------------------------------------------------------------
def test_int8_encode_rounds_half_away_and_keeps_sign(O):
    # x/max*127 hits exact halves for max = 127: 0.5 -> 1, -0.5 -> -1, 1.5 -> 2, 2.5 -> 3
    x = np.array([127.0, 0.5, -0.5, 1.5, 2.5, -2.5, 0.49, -127.0], dtype=F32)
    pay = O.encode_array(x, O.PREC["i8"])
    assert pay[:4].view(F32)[0] == F32(127.0)
    assert list(pay[4:].view(np.int8)) == [127, 1, -1, 2, 3, -3, 0, -127]


def test_int4_encode_clamps_and_packs(O):
    x = np.array([7.0, -7.0, 3.5, -3.5, 0.4, -0.6, 1.0], dtype=F32)     # max 7 -> scaled = x
    pay = O.encode_array(x, O.PREC["i4"])
    q = [7, -7, 4, -4, 0, -1, 1]
    u = [(v & 15) for v in q] + [0]
    want = bytes(u[i] | (u[i + 1] << 4) for i in range(0, 8, 2))
    assert pay[4:].tobytes() == want


def test_int2_encode_thresholds(O):
    x = np.array([1.0, 0.5, 0.50001, -0.5, -0.50001, 0.0, -1.0], dtype=F32)   # max 1
    pay = O.encode_array(x, O.PREC["i2"])
    q = [1, 0, 1, 0, -1, 0, -1]                                     # strictly beyond +-0.5 (Serialize.c:177-179)
    u = [(v & 3) for v in q] + [0]
    want = bytes(u[i] | (u[i + 1] << 2) | (u[i + 2] << 4) | (u[i + 3] << 6) for i in range(0, 8, 4))
    assert pay[4:].tobytes() == want


def test_zero_array_encodes_zero_scale_and_codes(O):
    for fmt in ("i8", "i4", "i2"):
        pay = O.encode_array(np.zeros(9, F32), O.PREC[fmt])
        assert not pay.any()


def test_fp16_encode_truncates(O):
    # 1 + 2^-11 lies exactly between two halves: truncation keeps 1.0; RNE would too, so also test 1 + 3*2^-12
    x = np.array([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -12, 65520.0, 1e-8, 6e-8, -2.5, 70000.0], dtype=F32)
    got = O.encode_array(x, O.PREC["f16"]).view(np.uint16)
    assert list(got) == [0x3C00, 0x3C00, 0x7BFF, 0x0000, 0x0001, 0xC100, 0x7C00]


def test_bf16_encode_truncates(O):
    x = np.array([1.0 + 2.0 ** -8 + 2.0 ** -9, -3.0], dtype=F32)       # RNE would round the first one up
    got = O.encode_array(x, O.PREC["bf16"]).view(np.uint16)
    assert list(got) == [0x3F80, 0xC040]


@pytest.mark.parametrize("fmt", ["f32", "f16", "bf16", "i8", "i4", "i2"])
def test_encode_decode_is_idempotent(O, fmt):
    rng = np.random.default_rng(3)
    x = rng.standard_normal(1001).astype(F32)
    p = O.PREC[fmt]
    once = O.decode_array(O.encode_array(x, p), x.size, p)
    twice = O.decode_array(O.encode_array(once, p), x.size, p)
    if fmt == "i2":
        # ternary: decoded values are {-max,0,max}; re-encoding keeps codes, scale becomes max again
        assert np.array_equal(once, twice)
    else:
        assert np.allclose(once, twice, rtol=0, atol=np.abs(x).max() * 2.0 ** -20)
    assert O.array_bytes(x.size, p) == {"f32": 4004, "f16": 2002, "bf16": 2002, "i8": 1005, "i4": 505, "i2": 255}[fmt]
