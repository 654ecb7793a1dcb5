#!/usr/bin/env python3
"""Benchmark of the MI355X inference forward pass.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-extra] [--no-cpu]

A step is one forward of one batch of seeded synthetic inputs through a net
whose weights were written by the library's own serializer and loaded back
(load_spingalett keeps the packed arrays; the device computes on them).
Inputs and outputs are device-resident during the timed region.  One JSON line
is printed: the headline workload plus, under "workloads", the other
benchmark configurations (C1, C2, C3, C5) with their own roofline figures and, under "training",
the reference's published training benchmark (--workload T1 makes that the
headline instead).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import spingalett_amd as S  # noqa: E402

HBM_PEAK = 8.0e12          # B/s
MFMA16_PEAK = 2.5e15       # FLOP/s, dense bf16/fp16
FP32_PEAK = 157.3e12

PREC_NAMES = {S.PRECISION_FLOAT32: "fp32", S.PRECISION_FP16: "fp16", S.PRECISION_BFLOAT16: "bf16",
              S.PRECISION_INT8: "int8", S.PRECISION_INT4: "int4", S.PRECISION_INT2: "int2"}
BITS = {S.PRECISION_FLOAT32: 32, S.PRECISION_FP16: 16, S.PRECISION_BFLOAT16: 16,
        S.PRECISION_INT8: 8, S.PRECISION_INT4: 4, S.PRECISION_INT2: 2}

A = dict(sigmoid=S.ACT_SIGMOID, relu=S.ACT_RELU, tanh=S.ACT_TANH, leaky=S.ACT_LEAKY_RELU,
         foo52=S.ACT_FOO52, softmax=S.ACT_SOFTMAX, none=S.ACT_NONE)

# name -> (topology, activations, init per layer, precision, input distribution, batches, headline batch)
WORKLOADS = {
    "C1": dict(topo=[784, 512, 1000, 10], acts=["relu", "relu", "softmax"], init=["he", "he", "xavier"],
               prec=S.PRECISION_FLOAT32, inputs="u01", batches=[256]),
    "C2": dict(topo=[784, 512, 1000, 10], acts=["relu", "relu", "softmax"], init=["he", "he", "xavier"],
               prec=S.PRECISION_INT8, inputs="u01", batches=[1, 256, 4096]),
    "C3": dict(topo=[4096, 16384, 16384, 4096], acts=["relu", "tanh", "none"], init=["xavier"] * 3,
               prec=S.PRECISION_INT4, inputs="n01", batches=[1, 8, 64]),
    "C4": dict(topo=[8192] * 9 + [1000], acts=["leaky", "foo52"] * 4 + ["softmax"], init=["he"] * 9,
               prec=S.PRECISION_BFLOAT16, inputs="n01", batches=[8192]),
    "C5": dict(topo=[2048, 8192, 8192, 8192, 8192, 1000], acts=["sigmoid", "relu", "relu", "tanh", "softmax"],
               init=["he"] * 5, prec=S.PRECISION_INT2, inputs="u11", batches=[1 << i for i in range(17)],
               # the batches whose dominant layer is also timed on its own (a roofline entry per row)
               roofline_batches=[1, 8, 64, 512, 4096, 65536]),
    # not one of the reference's configurations: FP32 weights at a batch where the matrix cores decide, to show the
    # FP32 matrix-core kernels next to the split mode (three FP16 products per layer)
    "F1": dict(topo=[4096] * 4 + [1000], acts=["relu", "tanh", "relu", "softmax"], init=["he"] * 4,
               prec=S.PRECISION_FLOAT32, inputs="n01", batches=[8192]),
}


def compute_dtype(prec: int, n: int) -> str:
    """Arithmetic type of the path taken (not a precision claim about the weights)."""
    if prec == S.PRECISION_FLOAT32:
        return "f32"
    if n <= 4:
        return "i8 (exact integer digits, f32 accumulate)" if prec >= S.PRECISION_INT8 else "f32"
    return "f16"         # FP16 matrix cores, f32 accumulate (BF16 weights: against their FP16 copy)


def array_payload(n: int, prec: int) -> int:
    """Serialized size of an n-element array including its 4-byte scale (Serialize.c:87-193)."""
    if prec == S.PRECISION_FLOAT32:
        return 4 * n
    if prec in (S.PRECISION_FP16, S.PRECISION_BFLOAT16):
        return 2 * n
    return 4 + (n * BITS[prec] + 7) // 8


def algorithmic_bytes(topo, prec, batch) -> int:
    w = sum(array_payload(topo[l] * topo[l + 1], prec) + array_payload(topo[l + 1], prec) for l in range(len(topo) - 1))
    return w + 4 * batch * (topo[0] + topo[-1])


def flops_per_sample(topo) -> int:
    return 2 * sum(topo[l] * topo[l + 1] for l in range(len(topo) - 1))


def build_net(name: str, seed: int = 42):
    """Seeded FP32 net -> library writer -> file -> load_spingalett.  Returns (net, file path)."""
    cfg = WORKLOADS[name]
    topo, acts = cfg["topo"], cfg["acts"]
    rng = np.random.default_rng(seed)
    net = S.new_spingalett(S.LOSS_CROSS_ENTROPY)
    S.layer(net, topo[0])
    for l in range(1, len(topo)):
        S.layer(net, topo[l], A[acts[l - 1]], S.WEIGHT_INITIALIZATION_NONE)
    for l in range(len(topo) - 1):
        std = np.float32(np.sqrt((2.0 if cfg["init"][l] == "he" else 1.0) / topo[l]))
        W = S.weights_view(net, l)
        # generated row block by row block to bound temporary memory
        step = max(1, (1 << 26) // topo[l])
        for r0 in range(0, topo[l + 1], step):
            r1 = min(topo[l + 1], r0 + step)
            W[r0:r1] = rng.standard_normal((r1 - r0, topo[l]), dtype=np.float32) * std
        S.biases_view(net, l)[:] = rng.standard_normal(topo[l + 1], dtype=np.float32) * np.float32(0.05)
    tmpdir = tempfile.mkdtemp(prefix="spbench_")
    path = os.path.join(tmpdir, name + ".nn")
    S.clear_error()
    S.save_spingalett(net, path, cfg["prec"], do_not_save_optimizer=True)
    code, msg = S.last_error()
    if code:
        raise RuntimeError("save_spingalett: " + msg)
    S.free_network(net)
    loaded = S.load_spingalett(path)
    if loaded is None:
        raise RuntimeError("load_spingalett: " + S.last_error()[1])
    return loaded, path


def make_inputs(kind: str, n: int, width: int, seed: int = 7) -> np.ndarray:
    rng = np.random.default_rng(seed)
    if kind == "u01":
        return rng.random((n, width), dtype=np.float32)
    if kind == "u11":
        return rng.random((n, width), dtype=np.float32) * np.float32(2) - np.float32(1)
    return rng.standard_normal((n, width), dtype=np.float32)


class DevNetRef:
    """Borrowed kernel-TU handle of a loaded net (so timing helpers can take it)."""
    def __init__(self, handle):
        self.h = C.c_void_p(handle)


def device_copies(net, topo, prec, min_total_bytes: int):
    """The net's own device copy plus clones until the rotation exceeds the last-level cache."""
    h = S.lib().spingalett_hip_handle(net)
    if not h:
        raise RuntimeError("hip handle: " + S.last_error()[1])
    base = DevNetRef(h)
    nbytes = algorithmic_bytes(topo, prec, 0)
    copies = [base]
    clones = []
    while nbytes * len(copies) < min_total_bytes:
        hc = C.c_void_p()
        if S.lib().sphip_clone(base.h, C.byref(hc)):
            raise RuntimeError("sphip_clone: " + S.lib().sphip_last_error_string().decode())
        clones.append(hc)
        copies.append(DevNetRef(hc.value))
    return copies, clones


def time_workload(copies, topo, n, x_host, steps, warmup, flags=0):
    d_x = S.DeviceBuffer.from_numpy(x_host)
    d_y = S.DeviceBuffer(4 * n * topo[-1])
    if warmup > 0:
        S.time_forward(copies, d_x, n, d_y, warmup, flags)
    S.synchronize()
    t0 = time.perf_counter()
    ev_ms = S.time_forward(copies, d_x, n, d_y, steps, flags)      # records events, waits for the last one
    S.synchronize()
    wall = time.perf_counter() - t0
    y = d_y.to_numpy(np.float32, (n, topo[-1]))
    d_x.free()
    d_y.free()
    return wall * 1e3 / steps, ev_ms / steps, y


# HBM-side bytes per launch of the dominant kernels: profiles/traffic.json, written by bench_traffic.py from
# rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script (each entry carries its counter readings, the
# calibration factors from a plain copy of known size in the same run, and the commands).  Keyed by kernel and
# [n, N, K]; a dominant kernel without an entry reports traffic null and a warning on stderr.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def load_traffic():
    try:
        with open(TRAFFIC_FILE) as f:
            entries = json.load(f)["entries"]
    except (OSError, ValueError, KeyError):
        return {}
    return {(e["kernel"], tuple(e["shape"])): e["bytes"] for e in entries}


PROFILED_TRAFFIC = load_traffic()


def dominant_layer(topo):
    return 1 + int(np.argmax([topo[l] * topo[l + 1] for l in range(len(topo) - 1)]))


def timed_layer(copies, l, n, iters, flags=0):
    """Average milliseconds of layer l's launches, back to back, after enough of them to bring the part to the clocks
    it holds under this load (about 50 ms: the first launches after a pause on the host run 5-10 % slower)."""
    first = S.time_layer(copies, l, n, len(copies) + 2, flags) / (len(copies) + 2)
    S.time_layer(copies, l, n, int(min(2000, max(3, 50.0 / max(first, 1e-3)))), flags)
    return S.time_layer(copies, l, n, iters, flags) / iters


def roofline_for(copies, topo, prec, n, iters):
    """Times the main kernel of the largest layer alone (HIP events on its stream).  A net with several layers of that
    shape (the same kernel, the same launch) reports their average, as a profiler's per-kernel average does: the
    duration depends on the operand values (the part's clock under this load follows how many bits toggle), and the
    first such layer sees the raw inputs, the others activations."""
    l = dominant_layer(topo)
    K, N = topo[l - 1], topo[l]
    same = [i for i in range(1, len(topo)) if (topo[i - 1], topo[i]) == (K, N)]
    ms = float(np.mean([timed_layer(copies, i, n, iters) for i in same]))
    kernel = S.lib().sphip_layer_kernel_name(copies[0].h, l, n, 0).decode()
    # a batch that runs in blocks of rows launches the layer's kernel once per block: ms (and traffic) are those of
    # all of them together, the layer's share of one forward
    rows = S.lib().sphip_batch_block_rows(copies[0].h, n, 0)
    launches = -(-n // rows) if rows else 1
    traffic = PROFILED_TRAFFIC.get((kernel, (n, N, K)))
    if traffic is None:
        print(f"bench.py: no profiled traffic for {kernel} at [n, N, K] = {[n, N, K]} in profiles/traffic.json "
              "(bench_traffic.py adds it)", file=sys.stderr)
    if n <= 64:
        # memory regime: serialized weights + bias of the layer, FP32 inputs and outputs of the layer
        nbytes = array_payload(K * N, prec) + array_payload(N, prec) + 4 * n * (K + N)
        ach = nbytes / (ms * 1e-3)
        return dict(bound="hbm", achieved=ach / 1e9, peak=HBM_PEAK / 1e9, unit="GB/s", frac=ach / HBM_PEAK,
                    traffic=traffic, kernel=kernel, layer=l, shape=[n, N, K], avg_ms=ms, launches=launches)
    fl = 2.0 * n * K * N
    ach = fl / (ms * 1e-3)
    peak = FP32_PEAK if prec == S.PRECISION_FLOAT32 else MFMA16_PEAK
    return dict(bound="mfma", achieved=ach / 1e12, peak=peak / 1e12, unit="TFLOP/s", frac=ach / peak,
                traffic=traffic, kernel=kernel, layer=l, shape=[n, N, K], avg_ms=ms, launches=launches)


def cpu_baseline(path, cfg, n_sample, budget_s=12.0):
    """The reference's batched call sequence (sgemm NT + bias + activation,
    Training.c:327-343) restated on the host, threaded BLAS, on a sample of the batch."""
    import oracle as O
    with open(path, "rb") as f:
        blob = f.read()
    net = O.Net.parse(blob)
    del blob
    sgemm, desc, set_threads = O.find_sgemm()
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    if set_threads is not None:
        set_threads(cores)
    X = make_inputs(cfg["inputs"], n_sample, cfg["topo"][0], seed=11)
    sec, _ = net.time_forward_batch(X, 1, sgemm, cores)
    iters = int(max(1, min(200, budget_s / max(sec, 1e-6))))
    sec, _ = net.time_forward_batch(X, iters, sgemm, cores)
    return dict(value=n_sample / sec, unit="samples/s", cores=cores, kind="port",
                sample=f"{n_sample} samples x {iters} iterations of the same net, sgemm NT + bias + activation, {blas_short(desc)}")


def blas_short(desc: str) -> str:
    """'libscipy_openblas-....so (OpenBLAS 0.3.28 DYNAMIC_ARCH ...)' -> 'OpenBLAS 0.3.28 (libscipy_openblas)'"""
    import re
    m = re.search(r"OpenBLAS ([0-9.]+)", desc)
    lib = desc.split("-")[0].split(".so")[0].split(" ")[0]
    return f"OpenBLAS {m.group(1)} ({lib})" if m else desc[:60]


def cpu_baseline_single(path, cfg, budget_s=2.0):
    """The public single-sample forward's call sequence on the host (Network.c:218-247: bias copy, cblas_sgemv or an
    OpenMP loop over rows of AVX-style dot products, activation), timed on one seeded input."""
    import oracle as O
    with open(path, "rb") as f:
        blob = f.read()
    net = O.Net.parse(blob)
    del blob
    _, desc, set_threads = O.find_sgemm()
    sgemv = O.find_sgemv()
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    if set_threads is not None:
        set_threads(cores)
    x = make_inputs(cfg["inputs"], 1, cfg["topo"][0], seed=11)[0]
    out = {}
    for leg, fn in (("sgemv", sgemv), ("openmp_dot", None)):
        if leg == "sgemv" and fn is None:
            continue
        sec, _ = net.time_forward_single(x, 1, fn, cores)
        iters = int(max(1, min(500, budget_s / 2 / max(sec, 1e-6))))
        sec, _ = net.time_forward_single(x, iters, fn, cores)
        out[leg + "_us"] = sec * 1e6
    best = min(out.values())
    return dict(value=1e6 / best, unit="samples/s", cores=cores, kind="port", **out,
                sample=f"one sample, the public forward's call sequence, {blas_short(desc)} sgemv and OpenMP dot rows")


def run_workload(name, batches, steps, warmup, want_output=False, cpu_budget_s=0.0, alternatives=True):
    cfg = WORKLOADS[name]
    topo, prec = cfg["topo"], cfg["prec"]
    t0 = time.perf_counter()
    net, path = build_net(name)
    build_s = time.perf_counter() - t0
    # Rotation over device copies: at least 600 MB of arrays in all, and at least two copies, so that neither a whole
    # forward nor back-to-back launches of one layer find their weights in the 256 MB memory-side cache (a layer of
    # the 8192-wide BF16 net alone is 128 MiB: launched back to back from one copy it runs 1.3 % faster than in the net)
    wbytes = algorithmic_bytes(topo, prec, 0)
    copies, clones = device_copies(net, topo, prec, max(600 << 20, 2 * wbytes) if wbytes > (8 << 20) else 0)
    rows = []
    for n in batches:
        x = make_inputs(cfg["inputs"], n, topo[0])
        k = steps if n * flops_per_sample(topo) < 2e12 else max(3, min(steps, 20))
        ms_wall, ms_ev, y = time_workload(copies, topo, n, x, k, warmup)
        fl = flops_per_sample(topo) * n
        row = dict(workload=name, format=PREC_NAMES[prec], batch=n, steps=k, ms_per_step=ms_wall, ms_per_step_events=ms_ev,
                   samples_per_s=n / (ms_wall * 1e-3),
                   hbm_frac=algorithmic_bytes(topo, prec, n) / (ms_ev * 1e-3) / HBM_PEAK,
                   mfma_frac=fl / (ms_ev * 1e-3) / (FP32_PEAK if prec == S.PRECISION_FLOAT32 else MFMA16_PEAK),
                   copies=len(copies), finite=bool(np.isfinite(y).all()))
        if n in cfg.get("roofline_batches", batches):
            row["roofline"] = roofline_for(copies, topo, prec, n, 20 if n >= 1024 else 200)
        if alternatives and prec == S.PRECISION_BFLOAT16 and n >= 5:
            # the same workload with BF16 activations on the BF16 matrix cores (SPHIP_BF16_ACTIVATIONS /
            # spingalett_set_bf16_activations): the faster, less accurate setting; the figures above are the default's
            # (FP16 activations against the FP16 copy of the BF16 weights)
            alt = S.SPHIP_BF16_ACTIVATIONS
            w_wall, w_ev, _ = time_workload(copies, topo, n, x, k, warmup, alt)
            l = dominant_layer(topo)
            w_layer = timed_layer(copies, l, n, 20, alt)
            row["bf16_activations"] = dict(ms_per_step=w_wall, samples_per_s=n / (w_wall * 1e-3),
                                           mfma_frac=fl / (w_ev * 1e-3) / MFMA16_PEAK, dominant_layer_ms=w_layer,
                                           dominant_layer_frac=2.0 * n * topo[l - 1] * topo[l] / (w_layer * 1e-3) / MFMA16_PEAK)
        if prec == S.PRECISION_FLOAT32 and n > 64 and (alternatives or name == "F1") and \
                any(topo[l + 1] >= 128 and 2.0 * n * topo[l] * topo[l + 1] >= 3e9 for l in range(len(topo) - 1)):
            # FP32 weights in split mode: every layer as three FP16 products into one FP32 accumulator (FP32-grade
            # outputs); fractions are of the algorithmic flops against the FP32 matrix peak, which this mode may exceed
            alt = S.SPHIP_SPLIT_ACTIVATIONS
            w_wall, w_ev, y3 = time_workload(copies, topo, n, x, k, warmup, alt)
            row["split_mode"] = dict(ms_per_step=w_wall, samples_per_s=n / (w_wall * 1e-3),
                                     fp32_mfma_frac=fl / (w_ev * 1e-3) / FP32_PEAK,
                                     max_abs_diff_to_fp32_kernels=float(np.max(np.abs(y3.astype(np.float64) - y))))
        if alternatives and want_output and prec != S.PRECISION_FLOAT32 and n >= 5:
            # the same workload with split activations (SPHIP_SPLIT_ACTIVATIONS / spingalett_set_net_activations): two
            # FP16 numbers per activation, twice the matrix-core work, FP32-grade outputs; the opt-in setting that
            # meets 99.9 % argmax agreement on 1000-class heads.  Fractions are of the algorithmic flops, not of the
            # doubled work.
            alt = S.SPHIP_SPLIT_ACTIVATIONS
            w_wall, w_ev, _ = time_workload(copies, topo, n, x, max(3, k // 2), warmup, alt)
            row["split_activations"] = dict(ms_per_step=w_wall, samples_per_s=n / (w_wall * 1e-3),
                                            mfma_frac=fl / (w_ev * 1e-3) / MFMA16_PEAK)
        if n == 1:
            # the public forward(): host pointer in, all activations mirrored into net->neurons (PCIe both ways)
            x1 = np.ascontiguousarray(x[0])
            for _ in range(20):
                S.forward(net, x1)
            t1 = time.perf_counter()
            for _ in range(200):
                S.forward(net, x1)
            row["public_forward_us"] = (time.perf_counter() - t1) / 200 * 1e6
        rows.append(row)
    if cpu_budget_s > 0:
        # one CPU leg per configuration (a bounded sample of its largest batch), attached to every row of it
        sample = min(max(batches), 64 if flops_per_sample(topo) > 1e8 else 4096)
        try:
            cpu = cpu_baseline(path, cfg, sample, cpu_budget_s)
        except Exception as e:
            cpu = dict(error=str(e))
        for row in rows:
            row["cpu_baseline"] = cpu
            if row["batch"] == 1:
                try:
                    row["cpu_baseline_b1"] = cpu_baseline_single(path, cfg, cpu_budget_s)
                except Exception as e:
                    row["cpu_baseline_b1"] = dict(error=str(e))
    return dict(net=net, path=path, copies=copies, clones=clones, rows=rows, build_s=build_s)


def monotone_below(rows, limit=4096):
    """True when samples/s never drops as the batch doubles, up to `limit` samples (rows of one workload)."""
    rs = sorted((r for r in rows if r["batch"] <= limit), key=lambda r: r["batch"])
    return all(b["samples_per_s"] >= a["samples_per_s"] for a, b in zip(rs, rs[1:]))


def sig(x, digits=4):
    """Floats rounded to `digits` significant digits, recursively (the line must stay short enough to be kept whole)."""
    if isinstance(x, float):
        return float(f"{x:.{digits}g}") if np.isfinite(x) else None
    if isinstance(x, dict):
        return {k: sig(v, digits) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [sig(v, digits) for v in x]
    return x


def compact_row(row):
    """One workload row with short keys: w workload, b batch, ms per step (wall), sps samples/s, hbm / mfma whole-net
    fractions of the peaks, dom the dominant layer's kernel on its own (k kernel, l layer, frac of its bound's peak,
    ms average launch, traffic HBM-side bytes per launch), fwd_us the public forward() host to host."""
    if "error" in row:
        return row
    out = dict(w=row["workload"], b=row["batch"], ms=row["ms_per_step"], sps=row["samples_per_s"],
               hbm=row["hbm_frac"], mfma=row["mfma_frac"])
    if not row["finite"]:
        out["finite"] = False
    rl = row.get("roofline")
    if rl:
        out["dom"] = dict(k=rl["kernel"], l=rl["layer"], bound=rl["bound"], frac=rl["frac"], ms=rl["avg_ms"],
                          traffic=rl["traffic"])
        if rl["launches"] > 1:
            out["dom"]["launches"] = rl["launches"]
    if "public_forward_us" in row:
        out["fwd_us"] = row["public_forward_us"]
    if "cpu_baseline_b1" in row:
        out["cpu_b1"] = row["cpu_baseline_b1"]
    if "split_mode" in row:
        out["split_mode"] = row["split_mode"]
    return out


# The reference's own published benchmark (Examples/Benchmark.c:14-98, README.md:48-59): train() on
# 784 -> 512 ReLU -> 1000 ReLU -> 10 softmax, 20,000 samples, full batch, Adam 0.001, cross-entropy,
# inputs and targets uniform in [0, 1).
TRAIN_TOPO = [784, 512, 1000, 10]
TRAIN_SAMPLES = 20000
TRAIN_PUBLISHED = dict(value=88921.0, unit="samples/s", hardware="Intel i7-12650H, OpenBLAS, 12 threads", source="README.md:57")


def train_flops(n):
    """2 n (in out) per layer for the forward and for the weight gradients, and for the hidden deltas of layers 2.."""
    t = TRAIN_TOPO
    fwd = sum(t[l] * t[l + 1] for l in range(len(t) - 1))
    return 2 * n * (2 * fwd + sum(t[l] * t[l + 1] for l in range(1, len(t) - 1)))


def run_training(steps, warmup, cpu=True):
    rng = np.random.default_rng(42)
    t = TRAIN_TOPO
    acts = [S.ACT_RELU, S.ACT_RELU, S.ACT_SOFTMAX]
    W = [(rng.standard_normal((t[l + 1], t[l])) * np.sqrt((2.0 if l < 2 else 1.0) / t[l])).astype(np.float32) for l in range(3)]
    X = rng.random((TRAIN_SAMPLES, t[0]), dtype=np.float32)
    T = rng.random((TRAIN_SAMPLES, t[-1]), dtype=np.float32)
    d = S.DeviceNet(t, acts, S.PRECISION_FLOAT32)
    for l in range(3):
        d.upload(l, 0, W[l].ravel())
        d.upload(l, 1, np.zeros(t[l + 1], np.float32))
    d.train_begin()
    a = S.SphipTrainArgs(S.OPTIMIZER_ADAM, S.LOSS_CROSS_ENTROPY, 0.001, 0.0, 0.9, 0.9, 0.999, 1e-8, 0.0, 0.9, 0.999)
    dx, dt = S.DeviceBuffer.from_numpy(X), S.DeviceBuffer.from_numpy(T)
    d.time_train_step(dx, dt, TRAIN_SAMPLES, a, max(1, warmup))
    ms = d.time_train_step(dx, dt, TRAIN_SAMPLES, a, steps) / steps
    finite = bool(np.isfinite(d.train_get(S.SPHIP_TRAIN_W, 0)).all())
    d.destroy(); dx.free(); dt.free()
    # the public call as the reference's example times it: host arrays in, trained host arrays out, 5 epochs
    net = S.new_spingalett(S.LOSS_CROSS_ENTROPY)
    S.layer(net, t[0], 0, S.WEIGHT_INITIALIZATION_NONE)
    for l in range(3):
        S.layer(net, t[l + 1], acts[l], S.WEIGHT_INITIALIZATION_NONE)
        S.weights_view(net, l)[:] = W[l]
    S.train(net, X, T, 1, S.STRATEGY_FULL_BATCH, S.OPTIMIZER_ADAM, learning_rate=0.001)      # warm-up
    t0 = time.perf_counter()
    S.train(net, X, T, 5, S.STRATEGY_FULL_BATCH, S.OPTIMIZER_ADAM, learning_rate=0.001)
    call_s = time.perf_counter() - t0
    S.free_network(net)
    out = dict(workload=f"T1: {'->'.join(map(str, t))} FP32, full batch of {TRAIN_SAMPLES}, Adam, cross-entropy "
                        "(Examples/Benchmark.c)", samples_per_s=TRAIN_SAMPLES / (ms * 1e-3), ms_per_step=ms, steps=steps,
               fp32_mfma_frac=train_flops(TRAIN_SAMPLES) / (ms * 1e-3) / FP32_PEAK, finite=finite,
               train_call_samples_per_s=5 * TRAIN_SAMPLES / call_s,
               published=TRAIN_PUBLISHED, vs_published=TRAIN_SAMPLES / (ms * 1e-3) / TRAIN_PUBLISHED["value"])
    if cpu:
        import oracle as O
        n = 256
        onet = O.Net.new(t, acts, 1)
        for l in range(3):
            onet.W(l)[:] = W[l]
        st = O.TrainState(onet)
        t1 = time.perf_counter()
        gW, gB, _ = onet.batch_gradients(X[:n], T[:n])
        onet.apply_gradients(st, gW, gB, O.OPT_ADAM, lr=0.001)
        sec = time.perf_counter() - t1
        out["cpu_baseline"] = dict(value=n / sec, unit="samples/s", cores=1, kind="port",
                                   sample=f"one step on {n} samples, scalar restatement (no BLAS)")
    return out


def vendor_gemm(m, steps, warmup):
    """Speed-of-light comparison, not part of the product: the vendor library's 16-bit GEMM (torch.matmul ->
    hipBLASLt) on an m x m x m product of BF16 operands with this benchmark's value distribution (N(0,1) activations,
    N(0, 2/m) weights), timed with events after the same 50 ms of warm-up launches as the library's own layers."""
    import torch
    g = torch.Generator(device="cuda").manual_seed(42)
    a = torch.randn((m, m), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    w = (torch.randn((m, m), generator=g, device="cuda", dtype=torch.float32) * (2.0 / m) ** 0.5).to(torch.bfloat16)
    c = torch.empty((m, m), device="cuda", dtype=torch.bfloat16)
    for _ in range(max(warmup, 60)):
        torch.matmul(a, w.t(), out=c)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        torch.matmul(a, w.t(), out=c)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    fl = 2.0 * m * m * m
    return dict(kernel="torch.matmul (hipBLASLt), BF16", shape=[m, m, m], avg_ms=ms, frac=fl / (ms * 1e-3) / MFMA16_PEAK,
                achieved_tflops=fl / (ms * 1e-3) / 1e12)


def release(w):
    for hc in w["clones"]:
        S.lib().sphip_destroy(hc)
    S.free_network(w["net"])
    try:
        os.remove(w["path"])
        os.rmdir(os.path.dirname(w["path"]))
    except OSError:
        pass


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="C4", choices=sorted(WORKLOADS) + ["T1"],
                    help="C1..C5: forward configurations; T1: the reference's published training benchmark")
    ap.add_argument("--batch", type=int, default=0, help="headline batch (default: the workload's largest)")
    ap.add_argument("--no-extra", action="store_true", help="skip the other benchmark configurations and the training benchmark")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-alt", action="store_true",
                    help="skip the headline workload's alternative activation settings (BF16 activations, split "
                         "activations), so that a profile holds the default setting's launches only")
    ap.add_argument("--vendor-gemm", type=int, default=0, metavar="M",
                    help="instead of a workload, time the vendor library's BF16 GEMM on an M x M x M product (needs torch; "
                         "a comparison for the profiles, not part of the product)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also make one device-to-device copy of the net's arrays (a plain copy kernel of known "
                         "size, to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.vendor_gemm:
        # before anything of this library touches the GPU: torch brings its own copy of the HIP runtime
        print(json.dumps(sig(vendor_gemm(args.vendor_gemm, args.steps, args.warmup))))
        return 0
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 (no multi-GPU path exists)", file=sys.stderr)
        return 2
    S.set_verbose(False)
    if S.device_count() < 1:
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1

    if args.workload == "T1":
        tr = run_training(args.steps, args.warmup, cpu=not args.no_cpu)
        print(json.dumps({
            "metric": "training samples/sec (forward + backward + Adam), the reference's published benchmark",
            "value": tr["samples_per_s"], "unit": "samples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": tr["ms_per_step"], "higher_is_better": True, "scaling": "weak",
            "vs_baseline": tr["vs_published"], "dtype": "fp32", "data": "synthetic (seeded, as Examples/Benchmark.c draws them)",
            "config": {"workload": tr["workload"]},
            "roofline": {"bound": "mfma", "achieved": train_flops(TRAIN_SAMPLES) / (tr["ms_per_step"] * 1e-3) / 1e12,
                         "peak": FP32_PEAK / 1e12, "unit": "TFLOP/s", "frac": tr["fp32_mfma_frac"], "traffic": None},
            "cpu_baseline": tr.get("cpu_baseline"), "training": tr}))
        return 0
    cfg = WORKLOADS[args.workload]
    n = args.batch or max(cfg["batches"])
    head = run_workload(args.workload, [n], args.steps, args.warmup, want_output=True, alternatives=not args.no_alt)
    row = head["rows"][0]
    if args.calibrate_copy:
        hc = C.c_void_p()
        if S.lib().sphip_clone(head["copies"][0].h, C.byref(hc)) == 0:
            S.synchronize()
            S.lib().sphip_destroy(hc)
        print(f"calibration copy: {algorithmic_bytes(cfg['topo'], cfg['prec'], 0)} bytes of arrays "
              f"(largest single copy {max(array_payload(cfg['topo'][l] * cfg['topo'][l + 1], cfg['prec']) - (4 if cfg['prec'] >= S.PRECISION_INT8 else 0) for l in range(len(cfg['topo']) - 1))} bytes)",
              file=sys.stderr)
    cpu = None
    if not args.no_cpu:
        sample = min(n, 512 if flops_per_sample(cfg["topo"]) > 5e8 else 4096)
        cpu = cpu_baseline(head["path"], cfg, sample)
    release(head)

    extra, cpu_extra, monotone = [], {}, {}
    if not args.no_extra:
        for name in ("C2", "C3", "C5", "C1", "F1"):
            if name == args.workload:
                continue
            try:
                w = run_workload(name, WORKLOADS[name]["batches"], 50, 3, cpu_budget_s=0.0 if args.no_cpu else 2.0)
                extra += [compact_row(r) for r in w["rows"]]
                if w["rows"] and "cpu_baseline" in w["rows"][0]:
                    cpu_extra[name] = w["rows"][0]["cpu_baseline"]
                if len(w["rows"]) > 3:
                    monotone[name] = monotone_below(w["rows"])
                release(w)
            except Exception as e:  # keep the headline even if an extra configuration fails
                extra.append(dict(workload=name, error=str(e)))

    training = None
    if not args.no_extra:
        try:
            training = run_training(20, 3, cpu=not args.no_cpu)
        except Exception as e:
            training = dict(workload="T1", error=str(e))

    rl = dict(row["roofline"])
    out = {
        "metric": "forward samples/sec per weight format; % peak HBM BW (b=1), % MFMA peak (b>=4K)",
        "value": row["samples_per_s"], "unit": "samples/s", "n_gpus": 1, "steps": row["steps"], "warmup": args.warmup,
        "ms_per_step": row["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": compute_dtype(cfg["prec"], n),
        "data": "synthetic (seeded normal weights through the library's serializer, seeded inputs)",
        "config": {"workload": f"{args.workload}: {'->'.join(map(str, cfg['topo']))} {row['format']} weights, batch {n}",
                   "format": row["format"], "batch": n},
        "roofline": {k: rl[k] for k in ("bound", "achieved", "peak", "unit", "frac", "traffic")},
        "roofline_kernel": {k: rl[k] for k in ("kernel", "layer", "shape", "avg_ms", "launches")},
        "whole_net_mfma_frac": row["mfma_frac"], "whole_net_hbm_frac": row["hbm_frac"],
        "bf16_activations": row.get("bf16_activations"),
        "split_activations": row.get("split_activations"),
        "split_mode": row.get("split_mode"),
        "cpu_baseline": cpu,
        # the other configurations, one short row per batch (keys: compact_row), their CPU legs once per configuration,
        # and whether samples/s is monotone in the batch up to 4096 samples (the GEMV -> GEMM crossover)
        "workloads": extra,
        "cpu_baselines": cpu_extra,
        "monotone_to_4096": monotone,
        "training": training,
    }
    print(json.dumps(sig(out), separators=(",", ":")))
    return 0


if __name__ == "__main__":
    sys.exit(main())
