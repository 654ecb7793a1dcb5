#!/usr/bin/env python3
"""Writes the golden fixtures in this directory.

The reference ships no test vectors and cannot be built here, so the fixtures
are made by a third, independent statement of the file format: numpy and
struct only — neither the oracle nor the library is imported.  Every number
follows from the reference's source expressions evaluated in IEEE float32
(numpy's float32 is IEEE): Serialize.c:87-193 for the writer, :195-297 for the
reader, :348-372 for the header, Activation.c:5-38 for the activations.

Outputs (all small):
  tiny_<fmt>.nn        37->53->29->10 net, one file per precision
  tiny_i8_opt.nn       same net, INT8, with optimizer block (time_step 77)
  soft_<fmt>.nn        24->40->7 net ending in softmax (bf16, i4)
  expected.npz         decoded FP32 arrays (strict and release evaluation),
                       inputs, float64 outputs
  kat.json             hand-assembled array payloads with expected bit patterns
Run:  python tests/golden/make_golden.py
"""
import json
import os
import struct

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
F32 = np.float32
ACT = dict(sigmoid=0, relu=1, tanh=2, leaky_relu=3, foo52=4, softmax=5, none=6)
PREC = dict(f32=0, f16=1, bf16=2, i8=3, i4=4, i2=5)


# ---- writer side (Serialize.c:12-43,74-78,110-190) -------------------------
def f32_to_f16_trunc(x):
    u = x.astype(F32).view(np.uint32).astype(np.uint64)
    sign = ((u >> 16) & 0x8000).astype(np.uint32)
    e = ((u >> 23) & 0xFF).astype(np.int64)
    m = (u & 0x7FFFFF).astype(np.int64)
    ue = e - 127
    out = np.zeros(x.shape, dtype=np.uint32)
    normal = (e != 0) & (e != 255) & (ue >= -14) & (ue <= 15)
    out[normal] = (((ue[normal] + 15) << 10) | (m[normal] >> 13)).astype(np.uint32)
    sub = (e != 0) & (ue < -14) & (ue >= -24)
    sh = (-1 - ue[sub]).astype(np.int64)
    out[sub] = ((m[sub] | 0x800000) >> sh).astype(np.uint32)
    out[(e != 255) & (ue > 15)] = 0x7C00
    out[(e == 255) & (m == 0)] = 0x7C00
    out[(e == 255) & (m != 0)] = 0x7E00
    return (out | sign).astype(np.uint16)


def round_half_away(s):
    s = s.astype(np.float64)            # exact for the +0.5
    return np.sign(s) * np.floor(np.abs(s) + 0.5)


def encode(x, fmt):
    x = np.ascontiguousarray(x, dtype=F32).ravel()
    if fmt == "f32":
        return x.tobytes()
    if fmt == "f16":
        return f32_to_f16_trunc(x).tobytes()
    if fmt == "bf16":
        return (x.view(np.uint32) >> 16).astype(np.uint16).tobytes()
    mx = F32(np.max(np.abs(x))) if x.size else F32(0)
    head = struct.pack("<f", float(mx))
    n = x.size
    if fmt == "i8":
        q = np.zeros(n, np.int8)
        if mx > 0:
            q = round_half_away((x / mx) * F32(127)).astype(np.int8)
        return head + q.tobytes()
    if fmt == "i4":
        q = np.zeros(n, np.int64)
        if mx > 0:
            q = np.clip(round_half_away((x / mx) * F32(7)), -8, 7).astype(np.int64)
        u = (q & 15).astype(np.uint8)
        if n & 1:
            u = np.concatenate([u, np.zeros(1, np.uint8)])
        return head + (u[0::2] | (u[1::2] << 4)).astype(np.uint8).tobytes()
    q = np.zeros(n, np.int64)
    if mx > 0:
        r = x / mx
        q = np.where(r > F32(0.5), 1, np.where(r < F32(-0.5), -1, 0))
    u = (q & 3).astype(np.uint8)
    u = np.concatenate([u, np.zeros((-n) % 4, np.uint8)])
    return head + (u[0::4] | (u[1::4] << 2) | (u[2::4] << 4) | (u[3::4] << 6)).astype(np.uint8).tobytes()


# ---- reader side (Serialize.c:45-85,195-297) --------------------------------
def decode(payload, n, fmt, release=False):
    b = np.frombuffer(payload, dtype=np.uint8)
    if fmt == "f32":
        return b[:4 * n].view(F32).copy()
    if fmt == "bf16":
        return (b[:2 * n].view(np.uint16).astype(np.uint32) << 16).view(F32)
    if fmt == "f16":
        h = b[:2 * n].view(np.uint16)
        v = h.view(np.float16).astype(F32)
        bits = v.view(np.uint32).copy()
        nan = np.isnan(v)
        bits[nan] = ((h[nan].astype(np.uint32) >> 15) << 31) | 0x7FC00000
        return bits.view(F32)
    mx = b[:4].view(F32)[0]
    c = b[4:]
    idx = np.arange(n)
    if fmt == "i8":
        q = c[:n].view(np.int8).astype(np.int32); d = F32(127)
    elif fmt == "i4":
        nib = (c[idx // 2] >> ((idx & 1) * 4)) & 15
        q = nib.astype(np.int32) - np.where(nib & 8, 16, 0); d = F32(7)
    else:
        cr = (c[idx // 4] >> ((idx & 3) * 2)) & 3
        q = cr.astype(np.int32) - np.where(cr & 2, 4, 0); d = F32(1)
    if not (mx > 0):
        return np.zeros(n, F32)
    qf = q.astype(F32)
    if fmt == "i2":
        return qf * mx
    if release:
        return qf * (mx * (F32(1) / d))
    return (qf / d) * mx


def header(topo, acts, fmt, loss=1, time_step=None):
    h = struct.pack("<HIBB", 1, len(topo), loss, 0 if time_step is None else 1)
    if time_step is not None:
        h += struct.pack("<Q", time_step)
    h += struct.pack("<B", PREC[fmt]) + struct.pack(f"<{len(topo)}I", *topo)
    return h + bytes(ACT[a] for a in acts)


def make_file(topo, acts, Ws, bs, fmt, time_step=None, rng=None):
    out = header(topo, acts, fmt, time_step=time_step)
    for W, b in zip(Ws, bs):
        out += encode(W, fmt)
        if time_step is not None:           # mW, vW in the same precision, each with its own scale
            out += encode(rng.standard_normal(W.size).astype(F32) * F32(1e-3), fmt)
            out += encode(np.abs(rng.standard_normal(W.size)).astype(F32) * F32(1e-5), fmt)
        out += encode(b, fmt)
        if time_step is not None:
            out += encode(rng.standard_normal(b.size).astype(F32) * F32(1e-3), fmt)
            out += encode(np.abs(rng.standard_normal(b.size)).astype(F32) * F32(1e-5), fmt)
    return out


def act64(x, a):
    if a == "sigmoid":
        return 1.0 / (1.0 + np.exp(-x))
    if a == "relu":
        return np.where(x > 0, x, 0.0)
    if a == "tanh":
        return np.tanh(x)
    if a == "leaky_relu":
        return np.where(x > 0, x, np.float64(F32(0.01)) * x)
    if a == "foo52":
        al = np.float64(F32(0.01))
        return np.where(x > 1, 1 + al * (x - 1), np.where(x < 0, al * x, x))
    if a == "softmax":
        e = np.exp(x - x.max(axis=1, keepdims=True))
        return e / e.sum(axis=1, keepdims=True)
    return x


def forward64(Ws, bs, acts, X):
    a = X.astype(np.float64)
    for W, b, act in zip(Ws, bs, acts):
        a = act64(a @ W.astype(np.float64).T + b.astype(np.float64), act)
    return a


def main():
    rng = np.random.default_rng(20260101)
    exp = {}
    nets = {
        "tiny": ([37, 53, 29, 10], ["foo52", "leaky_relu", "sigmoid"]),
        "soft": ([24, 40, 7], ["tanh", "softmax"]),
    }
    for name, (topo, acts) in nets.items():
        Ws = [(rng.standard_normal((topo[l + 1], topo[l])) * np.sqrt(2.0 / topo[l])).astype(F32) for l in range(len(topo) - 1)]
        bs = [(rng.standard_normal(topo[l + 1]) * 0.1).astype(F32) for l in range(len(topo) - 1)]
        X = rng.standard_normal((5, topo[0])).astype(F32)
        exp[f"{name}_X"] = X
        fmts = list(PREC) if name == "tiny" else ["bf16", "i4"]
        for fmt in fmts:
            variants = [(f"{name}_{fmt}", None)]
            if name == "tiny" and fmt == "i8":
                variants.append((f"{name}_{fmt}_opt", 77))
            for stem, ts in variants:
                blob = make_file(topo, acts, Ws, bs, fmt, time_step=ts, rng=rng)
                with open(os.path.join(HERE, stem + ".nn"), "wb") as f:
                    f.write(blob)
            # decoded arrays as the reader must produce them
            dW, dB, dWr, dBr = [], [], [], []
            for W, b in zip(Ws, bs):
                pw, pb = encode(W, fmt), encode(b, fmt)
                dW.append(decode(pw, W.size, fmt)); dB.append(decode(pb, b.size, fmt))
                dWr.append(decode(pw, W.size, fmt, True)); dBr.append(decode(pb, b.size, fmt, True))
            exp[f"{name}_{fmt}_W"] = np.concatenate(dW)
            exp[f"{name}_{fmt}_b"] = np.concatenate(dB)
            exp[f"{name}_{fmt}_W_release"] = np.concatenate(dWr)
            exp[f"{name}_{fmt}_b_release"] = np.concatenate(dBr)
            shaped = [w.reshape(topo[l + 1], topo[l]) for l, w in enumerate(dW)]
            exp[f"{name}_{fmt}_Y"] = forward64(shaped, dB, acts, X)
    np.savez_compressed(os.path.join(HERE, "expected.npz"), **exp)

    # hand-assembled payloads: expected values written out, derived by reading the decoder
    kat = [
        # INT4: byte 0x81 -> element0 = low nibble 1, element1 = high nibble 8 = -8; 0x7F -> -1, 7; 0x08 -> -8
        dict(fmt="i4", n=5, payload=(struct.pack("<f", 7.0) + bytes([0x81, 0x7F, 0x08])).hex(),
             q=[1, -8, -1, 7, -8]),
        # INT2: byte 0b11_10_01_00 -> 0, 1, -2, -1 ; byte 0b00_00_00_01 -> 1
        dict(fmt="i2", n=5, payload=(struct.pack("<f", 0.5) + bytes([0b11100100, 0b00000001])).hex(),
             q=[0, 1, -2, -1, 1]),
        # INT8: -128 is decoded, not clamped
        dict(fmt="i8", n=4, payload=(struct.pack("<f", 127.0) + bytes([0x80, 0xFF, 0x00, 0x7F])).hex(),
             q=[-128, -1, 0, 127]),
        # scale <= 0 or NaN: zeros whatever the codes say
        dict(fmt="i8", n=3, payload=(struct.pack("<f", 0.0) + bytes([1, 2, 3])).hex(), q=None),
        dict(fmt="i4", n=3, payload=(struct.pack("<f", -1.0) + bytes([0x21, 0x03])).hex(), q=None),
        dict(fmt="i2", n=3, payload=(struct.pack("<f", float("nan")) + bytes([0x1B])).hex(), q=None),
    ]
    d = dict(i8=F32(127), i4=F32(7), i2=F32(1))
    for k in kat:
        mx = F32(struct.unpack("<f", bytes.fromhex(k["payload"])[:4])[0])
        if k["q"] is None:
            vals = np.zeros(k["n"], F32)
            vr = vals
        else:
            q = np.array(k["q"], F32)
            vals = (q / d[k["fmt"]]) * mx if k["fmt"] != "i2" else q * mx
            vr = q * (mx * (F32(1) / d[k["fmt"]])) if k["fmt"] != "i2" else q * mx
        k["strict_bits"] = [int(v) for v in vals.astype(F32).view(np.uint32)]
        k["release_bits"] = [int(v) for v in vr.astype(F32).view(np.uint32)]
    # FP16 / BF16 spot values (IEEE tables): 1.0, -2.0, smallest subnormal, largest subnormal, max, inf, NaN
    kat.append(dict(fmt="f16", n=7, payload=np.array([0x3C00, 0xC000, 0x0001, 0x03FF, 0x7BFF, 0xFC00, 0xFE01], np.uint16).tobytes().hex(),
                    strict_bits=[0x3F800000, 0xC0000000, 0x33800000, 0x387FC000, 0x477FE000, 0xFF800000, 0xFFC00000]))
    kat[-1]["release_bits"] = kat[-1]["strict_bits"]
    kat.append(dict(fmt="bf16", n=4, payload=np.array([0x3F80, 0xC000, 0x7FC1, 0x0001], np.uint16).tobytes().hex(),
                    strict_bits=[0x3F800000, 0xC0000000, 0x7FC10000, 0x00010000]))
    kat[-1]["release_bits"] = kat[-1]["strict_bits"]
    with open(os.path.join(HERE, "kat.json"), "w") as f:
        json.dump(kat, f, indent=1)
    print("wrote", sorted(os.listdir(HERE)))


if __name__ == "__main__":
    main()
