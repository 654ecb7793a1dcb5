"""ctypes binding of the CPU oracle (``oracle/sp_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``; never by the shipped package.
"""
from __future__ import annotations

import ctypes as C
import glob
import os
import subprocess
import sys

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libsp_oracle.so")

ACT = {"sigmoid": 0, "relu": 1, "tanh": 2, "leaky_relu": 3, "foo52": 4, "softmax": 5, "none": 6}
PREC = {"f32": 0, "f16": 1, "bf16": 2, "i8": 3, "i4": 4, "i2": 5}
STRICT, RELEASE = 0, 1


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile next to it; returns the library path."""
    src = os.path.join(_HERE, "sp_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-C", _HERE, "-B" if force else "-s", "all"])
    return _LIB_PATH


class _Net(C.Structure):
    _fields_ = [
        ("layers", C.c_uint32), ("topology", C.POINTER(C.c_uint32)), ("act", C.POINTER(C.c_uint8)),
        ("loss", C.c_uint8), ("has_optimizer", C.c_uint8), ("precision", C.c_uint8),
        ("time_step", C.c_uint64), ("woff", C.POINTER(C.c_uint64)), ("boff", C.POINTER(C.c_uint64)),
        ("total_weights", C.c_uint64), ("total_biases", C.c_uint64),
        ("weights", C.POINTER(C.c_float)), ("biases", C.POINTER(C.c_float)), ("truncated", C.c_int),
    ]


_lib = None


class _OptArgs(C.Structure):
    _fields_ = [("optimizer", C.c_int), ("learning_rate", C.c_float), ("weight_decay", C.c_float),
                ("momentum", C.c_float), ("beta1", C.c_float), ("beta2", C.c_float), ("epsilon", C.c_float),
                ("max_grad_norm", C.c_float), ("decay_in_grad", C.c_int)]


OPT_SGD, OPT_MOMENTUM, OPT_RMSPROP, OPT_ADAM, OPT_ADAMW = range(5)


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    L = C.CDLL(_LIB_PATH)
    P = C.POINTER
    L.orc_fp16_to_f32.restype = C.c_float; L.orc_fp16_to_f32.argtypes = [C.c_uint16]
    L.orc_bf16_to_f32.restype = C.c_float; L.orc_bf16_to_f32.argtypes = [C.c_uint16]
    L.orc_f32_to_fp16.restype = C.c_uint16; L.orc_f32_to_fp16.argtypes = [C.c_float]
    L.orc_f32_to_bf16.restype = C.c_uint16; L.orc_f32_to_bf16.argtypes = [C.c_float]
    L.orc_array_bytes.restype = C.c_size_t; L.orc_array_bytes.argtypes = [C.c_uint32, C.c_int]
    L.orc_decode_array.restype = C.c_size_t
    L.orc_decode_array.argtypes = [C.c_void_p, C.c_size_t, C.c_uint32, C.c_int, C.c_int, C.c_void_p]
    L.orc_encode_array.restype = C.c_size_t
    L.orc_encode_array.argtypes = [C.c_void_p, C.c_uint32, C.c_int, C.c_void_p]
    L.orc_new.restype = P(_Net); L.orc_new.argtypes = [C.c_uint32, C.c_void_p, C.c_void_p]
    L.orc_free.restype = None; L.orc_free.argtypes = [P(_Net)]
    L.orc_parse.restype = P(_Net); L.orc_parse.argtypes = [C.c_void_p, C.c_size_t, C.c_int, P(C.c_int)]
    L.orc_serialized_size.restype = C.c_size_t; L.orc_serialized_size.argtypes = [P(_Net), C.c_int, C.c_int]
    L.orc_serialize.restype = C.c_size_t; L.orc_serialize.argtypes = [P(_Net), C.c_int, C.c_int, C.c_void_p]
    L.orc_activate.restype = C.c_float; L.orc_activate.argtypes = [C.c_float, C.c_int]
    L.orc_softmax.restype = None; L.orc_softmax.argtypes = [C.c_void_p, C.c_uint32]
    L.orc_apply_activation.restype = None
    L.orc_apply_activation.argtypes = [C.c_void_p, C.c_uint64, C.c_uint32, C.c_int]
    L.orc_forward_single.restype = None; L.orc_forward_single.argtypes = [P(_Net), C.c_void_p, C.c_void_p]
    L.orc_forward_batch.restype = None
    L.orc_forward_batch.argtypes = [P(_Net), C.c_void_p, C.c_uint32, C.c_void_p]
    L.orc_forward_batch_f64.restype = None
    L.orc_forward_batch_f64.argtypes = [P(_Net), C.c_void_p, C.c_uint32, C.c_void_p]
    L.orc_time_forward_batch.restype = C.c_double
    L.orc_time_forward_batch.argtypes = [P(_Net), C.c_void_p, C.c_uint32, C.c_void_p, C.c_int, C.c_void_p, C.c_int]
    L.orc_time_forward_single.restype = C.c_double
    L.orc_time_forward_single.argtypes = [P(_Net), C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int]
    L.orc_sample_loss.restype = C.c_float
    L.orc_sample_loss.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_int, C.c_int]
    L.orc_batch_loss.restype = C.c_float
    L.orc_batch_loss.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_uint32, C.c_int, C.c_int]
    L.orc_argmax.restype = C.c_uint32; L.orc_argmax.argtypes = [C.c_void_p, C.c_uint32]
    L.orc_derivative.restype = C.c_float; L.orc_derivative.argtypes = [C.c_float, C.c_int]
    L.orc_batch_gradients.restype = None
    L.orc_batch_gradients.argtypes = [P(_Net), C.c_void_p, C.c_void_p, C.c_uint32, C.c_float,
                                      C.c_void_p, C.c_void_p, C.c_void_p]
    L.orc_clip_grad_norm.restype = C.c_float
    L.orc_clip_grad_norm.argtypes = [P(_Net), C.c_void_p, C.c_void_p, C.c_float]
    L.orc_apply_gradients.restype = None
    L.orc_apply_gradients.argtypes = [P(_Net), P(_OptArgs), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                      C.c_void_p, C.c_void_p, C.c_float, C.c_float]
    _lib = L
    return L


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


# --------------------------------------------------------------------------
# array codecs
# --------------------------------------------------------------------------
def array_bytes(n: int, prec: int) -> int:
    return lib().orc_array_bytes(n, prec)


def decode_array(payload: bytes | np.ndarray, n: int, prec: int, mode: int = STRICT) -> np.ndarray:
    buf = np.frombuffer(bytes(payload), dtype=np.uint8) if not isinstance(payload, np.ndarray) else payload
    out = np.empty(n, dtype=np.float32)
    got = lib().orc_decode_array(_ptr(buf), buf.size, n, prec, mode, _ptr(out))
    if got == 0 and n:
        raise ValueError("payload too short")
    return out


def encode_array(x: np.ndarray, prec: int) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    out = np.zeros(array_bytes(x.size, prec), dtype=np.uint8)
    got = lib().orc_encode_array(_ptr(x), x.size, prec, _ptr(out))
    assert got == out.size
    return out


def fp16_to_f32(codes: np.ndarray) -> np.ndarray:
    L = lib()
    return np.array([L.orc_fp16_to_f32(int(c)) for c in codes], dtype=np.float32)


# --------------------------------------------------------------------------
# network
# --------------------------------------------------------------------------
class Net:
    """Owning wrapper of an ``orc_net``; weights/biases are numpy views."""

    def __init__(self, handle):
        if not handle:
            raise ValueError("null oracle net")
        self._h = handle
        n = handle.contents
        self.layers = n.layers
        self.topology = [n.topology[i] for i in range(n.layers)]
        self.act = [n.act[i] for i in range(n.layers - 1)]
        self.weights = np.ctypeslib.as_array(n.weights, shape=(max(int(n.total_weights), 1),))
        self.biases = np.ctypeslib.as_array(n.biases, shape=(max(int(n.total_biases), 1),))
        self.woff = [n.woff[i] for i in range(n.layers - 1)]
        self.boff = [n.boff[i] for i in range(n.layers - 1)]

    @classmethod
    def new(cls, topology, acts, loss: int = 0) -> "Net":
        t = np.asarray(topology, dtype=np.uint32)
        a = np.asarray(acts, dtype=np.uint8)
        assert a.size == t.size - 1
        h = lib().orc_new(t.size, _ptr(t), _ptr(a))
        net = cls(h)
        h.contents.loss = loss
        return net

    @classmethod
    def parse(cls, data: bytes, mode: int = STRICT) -> "Net":
        buf = np.frombuffer(data, dtype=np.uint8)
        err = C.c_int(0)
        h = lib().orc_parse(_ptr(buf), buf.size, mode, C.byref(err))
        if not h:
            raise ValueError(f"orc_parse failed: err={err.value}")
        return cls(h)

    @property
    def c(self):
        return self._h.contents

    def W(self, l: int) -> np.ndarray:
        i, o = self.topology[l], self.topology[l + 1]
        return self.weights[self.woff[l]: self.woff[l] + i * o].reshape(o, i)

    def b(self, l: int) -> np.ndarray:
        o = self.topology[l + 1]
        return self.biases[self.boff[l]: self.boff[l] + o]

    def serialize(self, prec: int, with_optimizer: bool = False) -> bytes:
        L = lib()
        n = L.orc_serialized_size(self._h, prec, int(with_optimizer))
        out = np.zeros(n, dtype=np.uint8)
        got = L.orc_serialize(self._h, prec, int(with_optimizer), _ptr(out))
        assert got == n, (got, n)
        return out.tobytes()

    def forward_single(self, x: np.ndarray) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty(self.topology[-1], dtype=np.float32)
        lib().orc_forward_single(self._h, _ptr(x), _ptr(out))
        return out

    def forward_batch(self, X: np.ndarray) -> np.ndarray:
        X = np.ascontiguousarray(X, dtype=np.float32).reshape(-1, self.topology[0])
        out = np.empty((X.shape[0], self.topology[-1]), dtype=np.float32)
        lib().orc_forward_batch(self._h, _ptr(X), X.shape[0], _ptr(out))
        return out

    def forward_batch_f64(self, X: np.ndarray) -> np.ndarray:
        X = np.ascontiguousarray(X, dtype=np.float32).reshape(-1, self.topology[0])
        out = np.empty((X.shape[0], self.topology[-1]), dtype=np.float64)
        lib().orc_forward_batch_f64(self._h, _ptr(X), X.shape[0], _ptr(out))
        return out

    def time_forward_batch(self, X: np.ndarray, iters: int, sgemm=None, threads: int = 0):
        X = np.ascontiguousarray(X, dtype=np.float32).reshape(-1, self.topology[0])
        out = np.empty((X.shape[0], self.topology[-1]), dtype=np.float32)
        fn = C.cast(sgemm, C.c_void_p) if sgemm is not None else None
        sec = lib().orc_time_forward_batch(self._h, _ptr(X), X.shape[0], _ptr(out), iters, fn, threads)
        return sec, out

    def time_forward_single(self, x: np.ndarray, iters: int, sgemv=None, threads: int = 0):
        """(seconds per call, outputs) of the public single-sample forward's call sequence (Network.c:218-247) with a
        cblas_sgemv found at run time, or with sgemv=None its OpenMP loop over rows of dot products."""
        x = np.ascontiguousarray(x, dtype=np.float32).reshape(self.topology[0])
        out = np.empty(self.topology[-1], dtype=np.float32)
        fn = C.cast(sgemv, C.c_void_p) if sgemv is not None else None
        sec = lib().orc_time_forward_single(self._h, _ptr(x), _ptr(out), iters, fn, threads)
        return sec, out

    def batch_gradients(self, X: np.ndarray, T: np.ndarray, grad_scale: float | None = None):
        """(gW, gB, outputs) of one batch: flat arrays laid out like weights / biases."""
        X = np.ascontiguousarray(X, dtype=np.float32).reshape(-1, self.topology[0])
        T = np.ascontiguousarray(T, dtype=np.float32).reshape(X.shape[0], self.topology[-1])
        gW = np.zeros(self.weights.size, dtype=np.float32)
        gB = np.zeros(self.biases.size, dtype=np.float32)
        out = np.empty((X.shape[0], self.topology[-1]), dtype=np.float32)
        scale = 1.0 / X.shape[0] if grad_scale is None else grad_scale
        lib().orc_batch_gradients(self._h, _ptr(X), _ptr(T), X.shape[0], scale, _ptr(gW), _ptr(gB), _ptr(out))
        return gW, gB, out

    def clip_grad_norm(self, gW: np.ndarray, gB: np.ndarray, max_norm: float) -> float:
        return float(lib().orc_clip_grad_norm(self._h, _ptr(gW), _ptr(gB), max_norm))

    def apply_gradients(self, state: "TrainState", gW: np.ndarray, gB: np.ndarray, optimizer: int,
                        lr: float = 0.01, weight_decay: float = 0.0, momentum: float = 0.9, beta1: float = 0.9,
                        beta2: float = 0.999, epsilon: float = 1e-8, max_grad_norm: float = 0.0,
                        decay_in_grad: bool = False) -> None:
        """One optimizer step in place (weights, biases, state; gW / gB are modified like the reference's)."""
        state.beta1_pow *= np.float32(beta1)
        state.beta2_pow *= np.float32(beta2)
        a = _OptArgs(optimizer, lr, weight_decay, momentum, beta1, beta2, epsilon, max_grad_norm, int(decay_in_grad))
        lib().orc_apply_gradients(self._h, C.byref(a), _ptr(gW), _ptr(gB), _ptr(state.mW), _ptr(state.vW),
                                  _ptr(state.mB), _ptr(state.vB), float(state.beta1_pow), float(state.beta2_pow))

    def __del__(self):
        try:
            if self._h:
                lib().orc_free(self._h)
                self._h = None
        except Exception:
            pass


class TrainState:
    """Optimizer moments of a net plus the running powers beta^t of one train() call (Training.c:684-685)."""

    def __init__(self, net: Net):
        self.mW = np.zeros(net.weights.size, dtype=np.float32)
        self.vW = np.zeros(net.weights.size, dtype=np.float32)
        self.mB = np.zeros(net.biases.size, dtype=np.float32)
        self.vB = np.zeros(net.biases.size, dtype=np.float32)
        self.beta1_pow = np.float32(1.0)
        self.beta2_pow = np.float32(1.0)


def derivative(a: np.ndarray, act: int) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    L = lib()
    return np.array([L.orc_derivative(float(v), act) for v in a.ravel()], dtype=np.float32).reshape(a.shape)


def activate(x: np.ndarray, act: int) -> np.ndarray:
    """Row-wise activation of a 2-D (rows, width) array; returns a new array."""
    y = np.array(x, dtype=np.float32, copy=True)
    if y.ndim == 1:
        y = y.reshape(1, -1)
    y = np.ascontiguousarray(y)
    lib().orc_apply_activation(_ptr(y), y.shape[0], y.shape[1], act)
    return y.reshape(np.shape(x))


def sample_loss(output: np.ndarray, target: np.ndarray, loss: int, output_act: int) -> float:
    o = np.ascontiguousarray(output, dtype=np.float32)
    t = np.ascontiguousarray(target, dtype=np.float32)
    return float(lib().orc_sample_loss(_ptr(o), _ptr(t), o.size, loss, output_act))


def batch_loss(outputs: np.ndarray, targets: np.ndarray, loss: int, output_act: int) -> float:
    o = np.ascontiguousarray(outputs, dtype=np.float32)
    t = np.ascontiguousarray(targets, dtype=np.float32)
    return float(lib().orc_batch_loss(_ptr(o), _ptr(t), o.shape[0], o.shape[1], loss, output_act))


def argmax_rows(outputs: np.ndarray) -> np.ndarray:
    o = np.ascontiguousarray(outputs, dtype=np.float32)
    return np.array([lib().orc_argmax(_ptr(o[i]), o.shape[1]) for i in range(o.shape[0])], dtype=np.uint32)


# --------------------------------------------------------------------------
# BLAS discovery for the CPU-baseline leg
# --------------------------------------------------------------------------
def find_sgemv():
    """cblas_sgemv of the same library find_sgemm() uses (None if there is none)."""
    fn, _, _ = find_sgemm()
    return _sgemv_of.get(id(fn)) if fn is not None else None


_sgemv_of = {}


def find_sgemm():
    """Locate a cblas_sgemm at run time.

    Returns (function pointer or None, description, set_threads callable or None).
    Search order: a system libopenblas, then the LP64 OpenBLAS bundled in the
    SciPy wheel (symbols carry a ``scipy_`` prefix).
    """
    cands = []
    for pat in ("/usr/lib/x86_64-linux-gnu/libopenblas.so*", "/usr/lib64/libopenblas.so*",
                "/usr/local/lib/libopenblas.so*", "/opt/OpenBLAS/lib/libopenblas.so*"):
        cands += [(p, "") for p in sorted(glob.glob(pat))]
    for sp in sys.path:
        for p in sorted(glob.glob(os.path.join(sp, "scipy.libs", "libscipy_openblas*.so"))):
            cands.append((p, "scipy_"))
    for path, prefix in cands:
        try:
            h = C.CDLL(path, mode=C.RTLD_GLOBAL)
            fn = getattr(h, prefix + "cblas_sgemm")
        except (OSError, AttributeError):
            continue
        if hasattr(h, prefix + "cblas_sgemv"):
            _sgemv_of[id(fn)] = getattr(h, prefix + "cblas_sgemv")
        setter = None
        for name in (prefix + "openblas_set_num_threads", "openblas_set_num_threads"):
            if hasattr(h, name):
                f = getattr(h, name); f.argtypes = [C.c_int]; f.restype = None
                setter = f
                break
        desc = os.path.basename(path)
        for name in (prefix + "openblas_get_config", "openblas_get_config"):
            if hasattr(h, name):
                g = getattr(h, name); g.restype = C.c_char_p
                desc += " (" + g().decode(errors="replace").strip() + ")"
                break
        return fn, desc, setter
    return None, "built-in OpenMP sgemm (no OpenBLAS found)", None
