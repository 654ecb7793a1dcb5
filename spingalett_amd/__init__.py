"""spingalett_amd — Python mirror of the Spingalett C interface, bound with
ctypes to the in-tree ``libspingalett.so`` (HIP back-end for MI355X).

The names, argument meaning and error behaviour follow the reference's public
header (Include/Spingalett/Spingalett.h:202-238); the batched entry is the
public form of the reference's static ``batch_forward`` (Training.c:313-345).
There is no host compute path: without the built library the import fails, and
without a GPU every forward fails with the library's error set.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libspingalett.so")
CSRC = os.path.join(_HERE, "csrc")

# enum values: Spingalett.h:38-47, :49-53, :55-61, :85-91, :93-101
ACT_SIGMOID, ACT_RELU, ACT_TANH, ACT_LEAKY_RELU, ACT_FOO52, ACT_SOFTMAX, ACT_NONE, ACT_COUNT = range(8)
LOSS_MSE, LOSS_CROSS_ENTROPY = 0, 1
(WEIGHT_INITIALIZATION_RANDOM, WEIGHT_INITIALIZATION_XAVIER,
 WEIGHT_INITIALIZATION_HE, WEIGHT_INITIALIZATION_NONE) = range(4)
COMPUTE_SINGLE_THREADED, COMPUTE_OPENMP, COMPUTE_OPENBLAS, COMPUTE_CUDA, COMPUTE_HIP, COMPUTE_COUNT = range(6)
(PRECISION_FLOAT32, PRECISION_FP16, PRECISION_BFLOAT16,
 PRECISION_INT8, PRECISION_INT4, PRECISION_INT2, PRECISION_COUNT) = range(7)
SPINGALETT_OK, SPINGALETT_ERR_ALLOC, SPINGALETT_ERR_INVALID = 0, 1, 2
DEQUANT_STRICT, DEQUANT_RELEASE = 0, 1
LOG_DEBUG, LOG_INFO, LOG_WARNING, LOG_ERROR, LOG_NONE = range(5)

# Spingalett.h:63-83, 103-107
MODE_ARRAY, MODE_GENERATOR_FUNCTION = 0, 1
STRATEGY_SAMPLE, STRATEGY_FULL_BATCH, STRATEGY_SMALL_BATCH = 0, 1, 2
OPTIMIZER_SGD, OPTIMIZER_MOMENTUM, OPTIMIZER_RMSPROP, OPTIMIZER_ADAM, OPTIMIZER_ADAMW = range(5)
AUTOSAVE_OFF, AUTOSAVE_OVERWRITE, AUTOSAVE_NEW_FILES = 0, 1, 2

SPHIP_X_ON_DEVICE, SPHIP_Y_ON_DEVICE, SPHIP_FORCE_GEMM, SPHIP_FORCE_GEMV = 1, 2, 8, 16
SPHIP_BF16_ACTIVATIONS = 32
SPHIP_WHOLE_BATCH, SPHIP_SPLIT_ACTIVATIONS = 64, 128
NET_ACTIVATIONS_DEFAULT, NET_ACTIVATIONS_BF16, NET_ACTIVATIONS_SPLIT = 0, 1, 2
(SPHIP_TRAIN_W, SPHIP_TRAIN_B, SPHIP_TRAIN_MW, SPHIP_TRAIN_VW, SPHIP_TRAIN_MB, SPHIP_TRAIN_VB,
 SPHIP_TRAIN_GW, SPHIP_TRAIN_GB) = range(8)


class NeuralNetwork(C.Structure):
    """Spingalett.h:109-136, field for field."""
    _fields_ = [
        ("layers", C.c_uint32),
        ("topology", C.POINTER(C.c_uint32)),
        ("act_func", C.POINTER(C.c_int)),
        ("weights", C.POINTER(C.c_float)),
        ("biases", C.POINTER(C.c_float)),
        ("neurons", C.POINTER(C.c_float)),
        ("grad_weights", C.POINTER(C.c_float)),
        ("grad_biases", C.POINTER(C.c_float)),
        ("opt_m_weights", C.POINTER(C.c_float)),
        ("opt_m_biases", C.POINTER(C.c_float)),
        ("opt_v_weights", C.POINTER(C.c_float)),
        ("opt_v_biases", C.POINTER(C.c_float)),
        ("neuron_offsets", C.POINTER(C.c_uint64)),
        ("weight_offsets", C.POINTER(C.c_uint64)),
        ("bias_offsets", C.POINTER(C.c_uint64)),
        ("total_neurons", C.c_uint64),
        ("total_weights", C.c_uint64),
        ("total_biases", C.c_uint64),
        ("time_step", C.c_uint64),
        ("loss_func", C.c_int),
    ]


class NeuralNetworkArgs(C.Structure):
    _fields_ = [("loss_func", C.c_int)]


class LayerArgs(C.Structure):
    _fields_ = [("net", C.POINTER(NeuralNetwork)), ("neurons_amount", C.c_uint32),
                ("act_func", C.c_int), ("weight_initialization", C.c_int)]


class ForwardArgs(C.Structure):
    _fields_ = [("net", C.POINTER(NeuralNetwork)), ("input", C.POINTER(C.c_float))]


class SaveArgs(C.Structure):
    _fields_ = [("net", C.POINTER(NeuralNetwork)), ("filename", C.c_char_p),
                ("do_not_save_optimizer", C.c_bool), ("precision", C.c_int)]


TrainCallback = C.CFUNCTYPE(C.c_bool, C.POINTER(NeuralNetwork), C.c_size_t, C.c_float)


class TrainArgs(C.Structure):
    """Spingalett.h:156-189, field for field."""
    _fields_ = [
        ("net", C.POINTER(NeuralNetwork)), ("training_mode", C.c_int), ("training_strategy", C.c_int),
        ("optimizer_type", C.c_int),
        ("inputs", C.POINTER(C.c_float)), ("targets", C.POINTER(C.c_float)),
        ("sample_count", C.c_uint32), ("batch_size", C.c_uint32), ("epochs", C.c_size_t),
        ("learning_rate", C.c_float), ("weight_decay", C.c_float), ("momentum", C.c_float),
        ("beta1", C.c_float), ("beta2", C.c_float), ("epsilon", C.c_float), ("max_grad_norm", C.c_float),
        ("reset_optimizer", C.c_bool), ("nan_check_interval", C.c_size_t),
        ("report_interval", C.c_size_t),
        ("autosave_mode", C.c_int), ("autosave_interval", C.c_size_t), ("autosave_path", C.c_char_p),
        ("autosave_do_not_save_optimizer", C.c_bool), ("autosave_precision", C.c_int),
        ("callback", TrainCallback), ("callback_interval", C.c_size_t),
    ]


class SphipTrainArgs(C.Structure):
    _fields_ = [("optimizer", C.c_int32), ("loss_func", C.c_int32), ("learning_rate", C.c_float),
                ("weight_decay", C.c_float), ("momentum", C.c_float), ("beta1", C.c_float), ("beta2", C.c_float),
                ("epsilon", C.c_float), ("max_grad_norm", C.c_float), ("beta1_pow_t", C.c_float),
                ("beta2_pow_t", C.c_float), ("decay_in_grad", C.c_int32)]


class SphipDesc(C.Structure):
    _fields_ = [("layers", C.c_uint32), ("topology", C.POINTER(C.c_uint32)),
                ("act", C.POINTER(C.c_uint8)), ("precision", C.c_uint8)]


NetPtr = C.POINTER(NeuralNetwork)

# every symbol the two headers under include/ declare
PUBLIC_SYMBOLS = [
    "spingalett_last_error_code", "spingalett_last_error_message", "spingalett_clear_error",
    "spingalett_get_compute_mode", "spingalett_set_compute_mode", "spingalett_get_num_threads",
    "spingalett_set_num_threads", "spingalett_set_log_callback", "spingalett_set_log_level",
    "spingalett_set_verbose", "spingalett_get_verbose",
    "new_spingalett_struct_arguments", "layer_struct_arguments", "activate", "forward_struct_arguments",
    "save_spingalett_struct_arguments", "load_spingalett", "free_network",
    "spingalett_set_dequant_mode", "spingalett_get_dequant_mode", "spingalett_forward_batch",
    "spingalett_set_bf16_activations", "spingalett_get_bf16_activations", "spingalett_set_net_activations",
    "spingalett_forward_batch_device", "spingalett_hip_synchronize", "spingalett_hip_invalidate",
    "spingalett_hip_precision", "spingalett_hip_decode", "spingalett_hip_handle", "load_spingalett_memory",
    "spingalett_evaluate_batch", "train_struct_arguments", "derivative", "print_parameters",
]
SPHIP_SYMBOLS = [
    "sphip_device_count", "sphip_last_error_string", "sphip_create", "sphip_destroy", "sphip_upload_array",
    "sphip_forward", "sphip_forward_noalloc", "sphip_forward_layers", "sphip_decode", "sphip_synchronize", "sphip_malloc", "sphip_free",
    "sphip_device_memory",
    "sphip_memcpy_h2d", "sphip_memcpy_d2h", "sphip_clone", "sphip_time_forward", "sphip_time_layer",
    "sphip_layer_kernel_name", "sphip_batch_block_rows", "sphip_evaluate",
    "sphip_train_begin", "sphip_train_end", "sphip_train_set", "sphip_train_get", "sphip_train_step",
    "sphip_time_train_step",
]


def build(verbose: bool = False) -> str:
    """Compile libspingalett.so for gfx950 with the Makefile in csrc/ (always rebuilds)."""
    cmd = ["make", "-C", CSRC, "-B", "-j8", "all"]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode:
        print(res.stdout)
    if res.returncode:
        raise RuntimeError("building libspingalett.so failed")
    return LIB_PATH


_lib = None


def lib():
    """The loaded library; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is missing: build it with spingalett_amd.build() "
                          "or `make -C spingalett_amd/csrc`")
    L = C.CDLL(LIB_PATH)
    L.spingalett_last_error_code.restype = C.c_int
    L.spingalett_last_error_message.restype = C.c_char_p
    L.spingalett_clear_error.restype = None
    L.spingalett_get_compute_mode.restype = C.c_int
    L.spingalett_set_compute_mode.argtypes = [C.c_int]; L.spingalett_set_compute_mode.restype = None
    L.spingalett_get_num_threads.restype = C.c_uint
    L.spingalett_set_num_threads.argtypes = [C.c_uint]; L.spingalett_set_num_threads.restype = None
    L.spingalett_set_log_level.argtypes = [C.c_int]; L.spingalett_set_log_level.restype = None
    L.spingalett_set_verbose.argtypes = [C.c_bool]; L.spingalett_set_verbose.restype = None
    L.spingalett_get_verbose.restype = C.c_bool
    L.new_spingalett_struct_arguments.argtypes = [NeuralNetworkArgs]
    L.new_spingalett_struct_arguments.restype = NetPtr
    L.layer_struct_arguments.argtypes = [LayerArgs]; L.layer_struct_arguments.restype = None
    L.activate.argtypes = [C.c_float, C.c_int]; L.activate.restype = C.c_float
    L.forward_struct_arguments.argtypes = [ForwardArgs]
    L.forward_struct_arguments.restype = C.POINTER(C.c_float)
    L.save_spingalett_struct_arguments.argtypes = [SaveArgs]; L.save_spingalett_struct_arguments.restype = None
    L.load_spingalett.argtypes = [C.c_char_p]; L.load_spingalett.restype = NetPtr
    L.load_spingalett_memory.argtypes = [C.c_void_p, C.c_size_t]; L.load_spingalett_memory.restype = NetPtr
    L.free_network.argtypes = [NetPtr]; L.free_network.restype = None
    L.spingalett_set_dequant_mode.argtypes = [C.c_int]; L.spingalett_set_dequant_mode.restype = None
    L.spingalett_get_dequant_mode.restype = C.c_int
    L.spingalett_set_bf16_activations.argtypes = [C.c_int]; L.spingalett_set_bf16_activations.restype = None
    L.spingalett_set_net_activations.argtypes = [NetPtr, C.c_int]; L.spingalett_set_net_activations.restype = C.c_int
    L.spingalett_get_bf16_activations.restype = C.c_int
    L.spingalett_forward_batch.argtypes = [NetPtr, C.c_void_p, C.c_uint32, C.c_void_p]
    L.spingalett_forward_batch.restype = C.c_void_p
    L.spingalett_forward_batch_device.argtypes = [NetPtr, C.c_void_p, C.c_uint32, C.c_void_p]
    L.spingalett_forward_batch_device.restype = C.c_int
    L.spingalett_evaluate_batch.argtypes = [NetPtr, C.c_void_p, C.c_void_p, C.c_uint32, C.POINTER(C.c_float),
                                            C.c_void_p, C.POINTER(C.c_uint32)]
    L.spingalett_evaluate_batch.restype = C.c_int
    L.train_struct_arguments.argtypes = [TrainArgs]; L.train_struct_arguments.restype = None
    L.derivative.argtypes = [C.c_float, C.c_int]; L.derivative.restype = C.c_float
    L.print_parameters.argtypes = [NetPtr]; L.print_parameters.restype = None
    L.spingalett_hip_synchronize.restype = C.c_int
    L.spingalett_hip_invalidate.argtypes = [NetPtr]; L.spingalett_hip_invalidate.restype = None
    L.spingalett_hip_precision.argtypes = [NetPtr]; L.spingalett_hip_precision.restype = C.c_int
    L.spingalett_hip_decode.argtypes = [NetPtr, C.c_uint32, C.c_int, C.c_void_p]
    L.spingalett_hip_decode.restype = C.c_int
    L.spingalett_hip_handle.argtypes = [NetPtr]; L.spingalett_hip_handle.restype = C.c_void_p
    # kernel-TU ABI
    L.sphip_device_count.restype = C.c_int
    L.sphip_last_error_string.restype = C.c_char_p
    L.sphip_create.argtypes = [C.POINTER(SphipDesc), C.POINTER(C.c_void_p)]; L.sphip_create.restype = C.c_int
    L.sphip_destroy.argtypes = [C.c_void_p]; L.sphip_destroy.restype = None
    L.sphip_upload_array.argtypes = [C.c_void_p, C.c_uint32, C.c_int, C.c_void_p, C.c_size_t, C.c_float]
    L.sphip_upload_array.restype = C.c_int
    L.sphip_forward.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_void_p, C.c_uint32]
    L.sphip_forward.restype = C.c_int
    L.sphip_forward_noalloc.argtypes = [C.c_void_p, C.c_void_p, C.c_uint32, C.c_void_p, C.c_uint32]
    L.sphip_forward_noalloc.restype = C.c_int
    L.sphip_forward_layers.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]; L.sphip_forward_layers.restype = C.c_int
    L.sphip_decode.argtypes = [C.c_void_p, C.c_uint32, C.c_int, C.c_int, C.c_void_p]; L.sphip_decode.restype = C.c_int
    L.sphip_synchronize.restype = C.c_int
    L.sphip_malloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]; L.sphip_malloc.restype = C.c_int
    L.sphip_free.argtypes = [C.c_void_p]; L.sphip_free.restype = C.c_int
    L.sphip_device_memory.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]; L.sphip_device_memory.restype = C.c_int
    L.sphip_memcpy_h2d.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]; L.sphip_memcpy_h2d.restype = C.c_int
    L.sphip_memcpy_d2h.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]; L.sphip_memcpy_d2h.restype = C.c_int
    L.sphip_clone.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]; L.sphip_clone.restype = C.c_int
    L.sphip_time_forward.argtypes = [C.POINTER(C.c_void_p), C.c_int, C.c_void_p, C.c_uint32, C.c_void_p,
                                     C.c_uint32, C.c_int, C.POINTER(C.c_float)]
    L.sphip_time_forward.restype = C.c_int
    L.sphip_time_layer.argtypes = [C.POINTER(C.c_void_p), C.c_int, C.c_uint32, C.c_uint32, C.c_uint32, C.c_int,
                                   C.POINTER(C.c_float)]
    L.sphip_time_layer.restype = C.c_int
    L.sphip_batch_block_rows.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32]; L.sphip_batch_block_rows.restype = C.c_uint32
    L.sphip_layer_kernel_name.argtypes = [C.c_void_p, C.c_uint32, C.c_uint32, C.c_uint32]
    L.sphip_layer_kernel_name.restype = C.c_char_p
    L.sphip_train_begin.argtypes = [C.c_void_p]; L.sphip_train_begin.restype = C.c_int
    L.sphip_train_end.argtypes = [C.c_void_p]; L.sphip_train_end.restype = None
    L.sphip_train_set.argtypes = [C.c_void_p, C.c_int, C.c_uint32, C.c_void_p]; L.sphip_train_set.restype = C.c_int
    L.sphip_train_get.argtypes = [C.c_void_p, C.c_int, C.c_uint32, C.c_void_p]; L.sphip_train_get.restype = C.c_int
    L.sphip_train_step.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.POINTER(SphipTrainArgs),
                                   C.c_uint32, C.POINTER(C.c_float)]
    L.sphip_train_step.restype = C.c_int
    L.sphip_time_train_step.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint32, C.POINTER(SphipTrainArgs),
                                        C.c_int, C.POINTER(C.c_float)]
    L.sphip_time_train_step.restype = C.c_int
    _lib = L
    return L


class SpingalettError(RuntimeError):
    pass


# ---------------------------------------------------------------------------
# the reference's call surface
# ---------------------------------------------------------------------------
def last_error():
    L = lib()
    return L.spingalett_last_error_code(), (L.spingalett_last_error_message() or b"").decode()


def clear_error():
    lib().spingalett_clear_error()


def set_verbose(flag: bool):
    lib().spingalett_set_verbose(bool(flag))


def new_spingalett(loss_func: int = LOSS_MSE):
    """new_spingalett(.loss_func=...) — Network.c:34-45; NULL (None) on an invalid loss."""
    p = lib().new_spingalett_struct_arguments(NeuralNetworkArgs(loss_func))
    return p if p else None


def layer(net, neurons_amount: int, act_func: int = 0, weight_initialization: int = 0):
    """layer(net, n, act, init) — Network.c:47-200."""
    lib().layer_struct_arguments(LayerArgs(net, neurons_amount, act_func, weight_initialization))


def forward(net, x):
    """forward(net, input) — Network.c:202-251.  Returns a numpy view into
    net->neurons (valid until the next call on the net) or None."""
    L = lib()
    xp = None
    if x is not None:
        x = np.ascontiguousarray(x, dtype=np.float32)
        xp = x.ctypes.data_as(C.POINTER(C.c_float))
    out = L.forward_struct_arguments(ForwardArgs(net, xp))
    if not out:
        return None
    n = net.contents.topology[net.contents.layers - 1]
    return np.ctypeslib.as_array(out, shape=(n,))


def forward_batch(net, X):
    """spingalett_forward_batch — the batched form (Training.c:313-345)."""
    L = lib()
    nc = net.contents
    X = np.ascontiguousarray(X, dtype=np.float32).reshape(-1, nc.topology[0])
    out = np.empty((X.shape[0], nc.topology[nc.layers - 1]), dtype=np.float32)
    r = L.spingalett_forward_batch(net, X.ctypes.data, X.shape[0], out.ctypes.data)
    if not r:
        code, msg = last_error()
        raise SpingalettError(f"spingalett_forward_batch failed ({code}): {msg}")
    return out


def evaluate_batch(net, X, T):
    """spingalett_evaluate_batch: (total loss, predictions, number correct) of a labelled batch
    (SIMD.c:522-552, Training.c:421-435)."""
    nc = net.contents
    X = np.ascontiguousarray(X, dtype=np.float32).reshape(-1, nc.topology[0])
    T = np.ascontiguousarray(T, dtype=np.float32).reshape(X.shape[0], nc.topology[nc.layers - 1])
    loss, correct = C.c_float(0), C.c_uint32(0)
    pred = np.empty(X.shape[0], dtype=np.uint32)
    rc = lib().spingalett_evaluate_batch(net, X.ctypes.data, T.ctypes.data, X.shape[0], C.byref(loss),
                                         pred.ctypes.data, C.byref(correct))
    if rc:
        code, msg = last_error()
        raise SpingalettError(f"spingalett_evaluate_batch failed ({code}): {msg}")
    return loss.value, pred, correct.value


def train(net, inputs, targets, epochs: int, strategy: int = STRATEGY_FULL_BATCH, optimizer: int = OPTIMIZER_SGD,
          batch_size: int = 0, callback=None, **kw):
    """train(...) of the reference (Spingalett.h:229-230); kw: any other TrainArgs field.  Errors are left in
    the error slot, as there."""
    X = np.ascontiguousarray(inputs, dtype=np.float32)
    T = np.ascontiguousarray(targets, dtype=np.float32)
    n = X.size // net.contents.topology[0]
    a = TrainArgs()
    a.net = net
    a.training_mode = kw.pop("training_mode", MODE_ARRAY)
    a.training_strategy = strategy
    a.optimizer_type = optimizer
    a.inputs = X.ctypes.data_as(C.POINTER(C.c_float))
    a.targets = T.ctypes.data_as(C.POINTER(C.c_float))
    a.sample_count = kw.pop("sample_count", n)
    a.batch_size = batch_size
    a.epochs = epochs
    cb = TrainCallback(callback) if callback is not None else TrainCallback()
    a.callback = cb
    for k, v in kw.items():
        if k == "autosave_path" and isinstance(v, str):
            v = v.encode()
        setattr(a, k, v)
    lib().train_struct_arguments(a)


def save_spingalett(net, filename: str, precision: int = PRECISION_FLOAT32, do_not_save_optimizer: bool = False):
    fn = None if filename is None else os.fsencode(filename)
    lib().save_spingalett_struct_arguments(SaveArgs(net, fn, do_not_save_optimizer, precision))


def load_spingalett(filename):
    p = lib().load_spingalett(None if filename is None else os.fsencode(filename))
    return p if p else None


def load_spingalett_memory(data: bytes):
    buf = np.frombuffer(data, dtype=np.uint8)
    p = lib().load_spingalett_memory(buf.ctypes.data, buf.size)
    return p if p else None


def free_network(net):
    lib().free_network(net)


def derivative(x: float, act: int) -> float:
    return float(lib().derivative(x, act))


def print_parameters(net):
    lib().print_parameters(net)


def activate(x: float, act: int) -> float:
    return lib().activate(x, act)


# ---------------------------------------------------------------------------
# numpy views of the public struct
# ---------------------------------------------------------------------------
def topology(net):
    nc = net.contents
    return [nc.topology[i] for i in range(nc.layers)]


def weights_view(net, l: int) -> np.ndarray:
    nc = net.contents
    i, o = nc.topology[l], nc.topology[l + 1]
    base = C.cast(nc.weights, C.c_void_p).value + 4 * nc.weight_offsets[l]
    return np.ctypeslib.as_array(C.cast(base, C.POINTER(C.c_float)), shape=(o, i))


def biases_view(net, l: int) -> np.ndarray:
    nc = net.contents
    o = nc.topology[l + 1]
    base = C.cast(nc.biases, C.c_void_p).value + 4 * nc.bias_offsets[l]
    return np.ctypeslib.as_array(C.cast(base, C.POINTER(C.c_float)), shape=(o,))


def neurons_view(net) -> np.ndarray:
    nc = net.contents
    return np.ctypeslib.as_array(nc.neurons, shape=(int(nc.total_neurons),))


def hip_decode(net, l: int, which: int) -> np.ndarray:
    nc = net.contents
    n = nc.topology[l] * nc.topology[l + 1] if which == 0 else nc.topology[l + 1]
    out = np.empty(n, dtype=np.float32)
    if lib().spingalett_hip_decode(net, l, which, out.ctypes.data):
        code, msg = last_error()
        raise SpingalettError(f"spingalett_hip_decode failed ({code}): {msg}")
    return out


# ---------------------------------------------------------------------------
# kernel-TU level helpers (benchmarks, device-resident runs)
# ---------------------------------------------------------------------------
def _check(rc: int, what: str):
    if rc:
        raise SpingalettError(f"{what}: {lib().sphip_last_error_string().decode()}")


def device_memory():
    """(free, total) bytes of the device's memory."""
    f, t = C.c_size_t(), C.c_size_t()
    _check(lib().sphip_device_memory(C.byref(f), C.byref(t)), "sphip_device_memory")
    return f.value, t.value


class DeviceBuffer:
    def __init__(self, nbytes: int):
        self.ptr = C.c_void_p()
        self.nbytes = nbytes
        _check(lib().sphip_malloc(C.byref(self.ptr), nbytes), "sphip_malloc")

    @classmethod
    def from_numpy(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        _check(lib().sphip_memcpy_h2d(b.ptr, a.ctypes.data, a.nbytes), "sphip_memcpy_h2d")
        return b

    def to_numpy(self, dtype, shape) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        _check(lib().sphip_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes), "sphip_memcpy_d2h")
        return out

    def free(self):
        if self.ptr:
            lib().sphip_free(self.ptr)
            self.ptr = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class DeviceNet:
    """A net at the kernel-TU level (spingalett_hip.h), fed with serialized arrays."""

    def __init__(self, topology, acts, precision: int, handle=None):
        self.topology = list(topology)
        self.acts = list(acts)
        self.precision = precision
        if handle is not None:
            self.h = C.c_void_p(handle)
            self.owned = True
            return
        t = (C.c_uint32 * len(topology))(*topology)
        a = (C.c_uint8 * len(acts))(*acts)
        d = SphipDesc(len(topology), t, a, precision)
        self.h = C.c_void_p()
        self.owned = True
        _check(lib().sphip_create(C.byref(d), C.byref(self.h)), "sphip_create")

    def upload(self, l: int, which: int, codes: np.ndarray, max_val: float = 0.0):
        codes = np.ascontiguousarray(codes)
        _check(lib().sphip_upload_array(self.h, l, which, codes.ctypes.data, codes.nbytes, max_val),
               "sphip_upload_array")

    def upload_serialized_array(self, l: int, which: int, payload: np.ndarray):
        """payload = one array as it sits in a .nn file (scale prefix included for INT formats)."""
        payload = np.ascontiguousarray(payload, dtype=np.uint8)
        if self.precision >= PRECISION_INT8:
            mx = float(payload[:4].view(np.float32)[0])
            self.upload(l, which, payload[4:], mx)
        else:
            self.upload(l, which, payload, 0.0)

    def clone(self) -> "DeviceNet":
        h = C.c_void_p()
        _check(lib().sphip_clone(self.h, C.byref(h)), "sphip_clone")
        return DeviceNet(self.topology, self.acts, self.precision, handle=h.value)

    def forward(self, X: np.ndarray, flags: int = 0) -> np.ndarray:
        X = np.ascontiguousarray(X, dtype=np.float32).reshape(-1, self.topology[0])
        out = np.empty((X.shape[0], self.topology[-1]), dtype=np.float32)
        _check(lib().sphip_forward(self.h, X.ctypes.data, X.shape[0], out.ctypes.data, flags), "sphip_forward")
        return out

    def forward_device(self, d_x: DeviceBuffer, n: int, d_y: DeviceBuffer, flags: int = 0):
        _check(lib().sphip_forward(self.h, d_x.ptr, n, d_y.ptr, flags | SPHIP_X_ON_DEVICE | SPHIP_Y_ON_DEVICE),
               "sphip_forward")

    def forward_noalloc(self, d_x: DeviceBuffer, n: int, d_y: DeviceBuffer, flags: int = 0) -> int:
        """sphip_forward_noalloc; returns its status (the caller reads sphip_last_error_string on failure)."""
        return lib().sphip_forward_noalloc(self.h, d_x.ptr, n, d_y.ptr, flags)

    def decode(self, l: int, which: int, mode: int = DEQUANT_STRICT) -> np.ndarray:
        n = self.topology[l] * self.topology[l + 1] if which == 0 else self.topology[l + 1]
        out = np.empty(n, dtype=np.float32)
        _check(lib().sphip_decode(self.h, l, which, mode, out.ctypes.data), "sphip_decode")
        return out

    # ---- batched training step (FP32 nets) ----
    def train_begin(self):
        _check(lib().sphip_train_begin(self.h), "sphip_train_begin")

    def train_end(self):
        lib().sphip_train_end(self.h)

    def _train_count(self, which: int, l: int) -> int:
        weights = which in (SPHIP_TRAIN_W, SPHIP_TRAIN_MW, SPHIP_TRAIN_VW, SPHIP_TRAIN_GW)
        return self.topology[l] * self.topology[l + 1] if weights else self.topology[l + 1]

    def train_get(self, which: int, l: int) -> np.ndarray:
        out = np.empty(self._train_count(which, l), dtype=np.float32)
        _check(lib().sphip_train_get(self.h, which, l, out.ctypes.data), "sphip_train_get")
        return out

    def train_set(self, which: int, l: int, values: np.ndarray):
        v = np.ascontiguousarray(values, dtype=np.float32).ravel()
        assert v.size == self._train_count(which, l)
        _check(lib().sphip_train_set(self.h, which, l, v.ctypes.data), "sphip_train_set")

    def train_step(self, X: np.ndarray, T: np.ndarray, args: "SphipTrainArgs", want_loss: bool = False):
        X = np.ascontiguousarray(X, dtype=np.float32).reshape(-1, self.topology[0])
        T = np.ascontiguousarray(T, dtype=np.float32).reshape(X.shape[0], self.topology[-1])
        loss = C.c_float(0)
        _check(lib().sphip_train_step(self.h, X.ctypes.data, T.ctypes.data, X.shape[0], C.byref(args), 0,
                                      C.byref(loss) if want_loss else None), "sphip_train_step")
        return loss.value if want_loss else None

    def time_train_step(self, d_x: "DeviceBuffer", d_t: "DeviceBuffer", n: int, args: "SphipTrainArgs", iters: int) -> float:
        ms = C.c_float(0)
        _check(lib().sphip_time_train_step(self.h, d_x.ptr, d_t.ptr, n, C.byref(args), iters, C.byref(ms)),
               "sphip_time_train_step")
        return ms.value

    def destroy(self):
        if self.h and self.owned:
            lib().sphip_destroy(self.h)
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def synchronize():
    _check(lib().sphip_synchronize(), "sphip_synchronize")


def time_forward(nets, d_x: DeviceBuffer, n: int, d_y: DeviceBuffer, iters: int, flags: int = 0) -> float:
    """Milliseconds for `iters` forwards rotating over `nets` (HIP events on the library's stream)."""
    arr = (C.c_void_p * len(nets))(*[x.h for x in nets])
    ms = C.c_float(0)
    _check(lib().sphip_time_forward(arr, len(nets), d_x.ptr, n, d_y.ptr, flags, iters, C.byref(ms)),
           "sphip_time_forward")
    return ms.value


def time_layer(nets, layer_idx: int, n: int, iters: int, flags: int = 0) -> float:
    arr = (C.c_void_p * len(nets))(*[x.h for x in nets])
    ms = C.c_float(0)
    _check(lib().sphip_time_layer(arr, len(nets), layer_idx, n, flags, iters, C.byref(ms)), "sphip_time_layer")
    return ms.value


def device_count() -> int:
    return lib().sphip_device_count()
