"""Host side of the shipped library, no GPU needed: the C-ABI loads and exports
every declared symbol, the loader/writer agree with the oracle and the golden
files bit for bit, and the API contract of the reference holds
(Network.c:34-251, Serialize.c:307-609, Error.c, Settings.c)."""
import ctypes as C
import os
import re
import struct

import numpy as np
import pytest

from helpers import FORMATS, make_oracle_net

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = os.path.join(os.path.dirname(__file__), "golden")
E = np.load(os.path.join(GOLD, "expected.npz"))
PREC = {"f32": 0, "f16": 1, "bf16": 2, "i8": 3, "i4": 4, "i2": 5}


def bits(a):
    return np.asarray(a, dtype=np.float32).view(np.uint32)


def read(name):
    with open(os.path.join(GOLD, name), "rb") as f:
        return f.read()


def declared_symbols(header):
    text = "\n".join(ln for ln in open(os.path.join(ROOT, "include", header)).read().splitlines()
                     if not ln.lstrip().startswith("#"))
    return set(re.findall(r"(?:SPINGALETT_API|SPHIP_API)[^;(]*?\b(\w+)\s*\(", text))


def test_library_exports_every_declared_symbol(S):
    L = S.lib()
    pub = declared_symbols("spingalett.h")
    dev = declared_symbols("spingalett_hip.h")
    assert pub == set(S.PUBLIC_SYMBOLS), pub ^ set(S.PUBLIC_SYMBOLS)
    assert dev == set(S.SPHIP_SYMBOLS), dev ^ set(S.SPHIP_SYMBOLS)
    for name in pub | dev:
        assert hasattr(L, name), name


def test_internal_symbols_are_hidden(S):
    L = S.lib()
    for name in ("sp_set_error", "sp_decode_array", "sp_net_build", "sp_hip_release"):
        assert not hasattr(L, name), name


def test_struct_layout_matches_reference_abi(S):
    # LP64 layout of Spingalett.h:109-136: 4+pad, 14 pointers, 4 u64, int
    assert C.sizeof(S.NeuralNetwork) == 8 + 14 * 8 + 4 * 8 + 8
    assert S.NeuralNetwork.weights.offset == 24 and S.NeuralNetwork.total_neurons.offset == 120
    assert S.NeuralNetwork.loss_func.offset == 152
    assert C.sizeof(S.LayerArgs) == 24 and C.sizeof(S.ForwardArgs) == 16 and C.sizeof(S.SaveArgs) == 24


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("mode", [0, 1])
def test_load_matches_golden_and_oracle(S, O, fmt, mode):
    L = S.lib()
    L.spingalett_set_dequant_mode(mode)
    try:
        net = S.load_spingalett(os.path.join(GOLD, f"tiny_{fmt}.nn"))
        assert net is not None, S.last_error()
        assert S.topology(net) == [37, 53, 29, 10]
        sfx = "_release" if mode else ""
        W = np.concatenate([S.weights_view(net, l).ravel() for l in range(3)])
        b = np.concatenate([S.biases_view(net, l) for l in range(3)])
        assert np.array_equal(bits(W), bits(E[f"tiny_{fmt}_W{sfx}"]))
        assert np.array_equal(bits(b), bits(E[f"tiny_{fmt}_b{sfx}"]))
        ref = O.Net.parse(read(f"tiny_{fmt}.nn"), mode)
        assert np.array_equal(bits(W), bits(ref.weights))
        assert L.spingalett_hip_precision(net) == PREC[fmt]
        assert net.contents.loss_func == 1 and net.contents.time_step == 0
        S.free_network(net)
    finally:
        L.spingalett_set_dequant_mode(0)


def test_load_with_optimizer_block(S):
    net = S.load_spingalett(os.path.join(GOLD, "tiny_i8_opt.nn"))
    assert net is not None
    nc = net.contents
    assert nc.time_step == 77
    W = np.concatenate([S.weights_view(net, l).ravel() for l in range(3)])
    assert np.array_equal(bits(W), bits(E["tiny_i8_W"]))
    m = np.ctypeslib.as_array(nc.opt_m_weights, shape=(int(nc.total_weights),))
    v = np.ctypeslib.as_array(nc.opt_v_weights, shape=(int(nc.total_weights),))
    assert np.abs(m).max() > 0 and v.min() >= 0 and v.max() > 0      # the block was decoded, not skipped
    S.free_network(net)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("with_opt", [False, True])
def test_save_writes_the_bytes_the_oracle_writes(S, O, fmt, with_opt, tmp_path):
    src = make_oracle_net(O, [21, 34, 13], ["relu", "none"], seed=9)
    src.c.loss = 0
    net = S.new_spingalett(S.LOSS_MSE)
    S.layer(net, 21)
    S.layer(net, 34, S.ACT_RELU, S.WEIGHT_INITIALIZATION_NONE)
    S.layer(net, 13, S.ACT_NONE, S.WEIGHT_INITIALIZATION_NONE)
    for l in range(2):
        S.weights_view(net, l)[:] = src.W(l)
        S.biases_view(net, l)[:] = src.b(l)
    path = str(tmp_path / "model")                     # no extension: ".nn" is appended (Serialize.c:321-336)
    S.save_spingalett(net, path, PREC[fmt], do_not_save_optimizer=not with_opt)
    assert S.last_error()[0] == 0
    got = open(path + ".nn", "rb").read()
    assert got == src.serialize(O.PREC[fmt], with_opt)
    S.free_network(net)


def test_save_keeps_a_given_extension_and_reports_errors(S, tmp_path):
    net = S.new_spingalett()
    S.layer(net, 2); S.layer(net, 1, S.ACT_NONE, S.WEIGHT_INITIALIZATION_NONE)
    p = str(tmp_path / "dir.with.dot" )
    os.mkdir(p)
    S.save_spingalett(net, os.path.join(p, "m.bin"))
    assert os.path.exists(os.path.join(p, "m.bin"))
    S.save_spingalett(net, os.path.join(p, "plain"))    # dot only in the directory name -> still appended
    assert os.path.exists(os.path.join(p, "plain.nn"))
    S.clear_error()
    S.save_spingalett(net, os.path.join(p, "x"), precision=9)
    assert S.last_error() == (S.SPINGALETT_ERR_INVALID, "save: invalid precision mode")
    S.clear_error()
    S.save_spingalett(net, str(tmp_path / "nodir" / "x"))
    assert S.last_error()[0] == S.SPINGALETT_ERR_INVALID
    S.clear_error()
    S.save_spingalett(None, "x")
    assert S.last_error() == (S.SPINGALETT_ERR_INVALID, "save: net or filename is NULL")
    S.free_network(net)


def test_load_error_paths(S, tmp_path):
    assert S.load_spingalett(None) is None and S.last_error()[1] == "load: filename is NULL"
    S.clear_error()
    assert S.load_spingalett(str(tmp_path / "missing.nn")) is None
    assert S.last_error() == (S.SPINGALETT_ERR_INVALID, "load: cannot open file for reading")
    good = bytearray(read("tiny_i8.nn"))
    cases = [
        (lambda b: b.__setitem__(0, 9), "load: unsupported format version"),
        (lambda b: b.__setitem__(slice(2, 6), struct.pack("<I", 1)), "load: network must have at least 2 layers"),
        (lambda b: b.__setitem__(6, 2), "load: invalid loss type"),
        (lambda b: b.__setitem__(8, 6), "load: invalid precision type"),
        (lambda b: b.__setitem__(9 + 16 + 1, 7), "load: invalid activation function or layer size"),
    ]
    for mut, msg in cases:
        S.clear_error()
        b = bytearray(good); mut(b)
        assert S.load_spingalett_memory(bytes(b)) is None
        assert S.last_error() == (S.SPINGALETT_ERR_INVALID, msg)
    S.clear_error()
    assert S.load_spingalett_memory(bytes(good[:1])) is None
    assert S.last_error()[1] == "load: failed to read format version"


def test_truncated_payload_returns_net_with_error_set(S):
    S.clear_error()
    blob = read("tiny_bf16.nn")[:4000]
    net = S.load_spingalett_memory(blob)
    assert net is not None                                # Serialize.c:596-608
    assert S.last_error() == (S.SPINGALETT_ERR_INVALID, "load: file appears truncated or corrupt")
    W0 = S.weights_view(net, 0).ravel()
    assert np.array_equal(bits(W0), bits(E["tiny_bf16_W"][:W0.size]))     # 37*53*2 = 3922 bytes were complete
    assert not S.weights_view(net, 1).any()
    assert S.lib().spingalett_hip_precision(net) == 0     # incomplete packed arrays are dropped
    S.free_network(net)


def test_stale_error_makes_load_fail_like_the_reference(S):
    # the loader tests the sticky slot without clearing it (Serialize.c:556)
    S.save_spingalett(None, "x")
    assert S.last_error()[0] != 0
    assert S.load_spingalett(os.path.join(GOLD, "tiny_i8.nn")) is None
    S.clear_error()
    net = S.load_spingalett(os.path.join(GOLD, "tiny_i8.nn"))
    assert net is not None
    S.free_network(net)


def test_lifecycle_contract(S):
    assert S.new_spingalett(7) is None and S.last_error() == (S.SPINGALETT_ERR_INVALID, "Invalid loss function")
    S.clear_error()
    net = S.new_spingalett(S.LOSS_CROSS_ENTROPY)
    S.layer(net, 0)
    assert S.last_error()[1] == "Net is NULL or neurons amount is 0"
    S.clear_error()
    S.layer(net, 4)
    S.layer(net, 3, 99, 0)
    assert S.last_error()[1] == "Invalid activation function"
    S.clear_error()
    S.layer(net, 3, S.ACT_RELU, 99)
    assert S.last_error()[1] == "Invalid weight initialization"
    S.clear_error()
    x = np.ones(4, np.float32)
    assert S.forward(net, x) is None                      # one layer only
    assert S.last_error() == (S.SPINGALETT_ERR_INVALID, "Network must have at least 2 layers for forward pass")
    S.clear_error()
    assert S.forward(None, x) is None and S.forward(net, None) is None
    assert S.last_error()[0] == 0                         # silent NULL (Network.c:207)
    S.layer(net, 3, S.ACT_RELU, S.WEIGHT_INITIALIZATION_HE)
    S.layer(net, 2, S.ACT_SOFTMAX, S.WEIGHT_INITIALIZATION_XAVIER)
    nc = net.contents
    assert nc.layers == 3 and nc.total_weights == 18 and nc.total_biases == 5 and nc.total_neurons == 9
    assert [nc.weight_offsets[i] for i in range(2)] == [0, 12] and [nc.bias_offsets[i] for i in range(2)] == [0, 3]
    assert [nc.neuron_offsets[i] for i in range(4)] == [0, 4, 7, 9]
    assert S.weights_view(net, 0).any() and not S.biases_view(net, 0).any()
    assert C.addressof(nc.weights.contents) % 64 == 0     # Memory.c: 64-byte aligned
    S.free_network(net)
    S.free_network(None)


def test_weight_initialisation_distributions(S):
    net = S.new_spingalett()
    S.layer(net, 400)
    S.layer(net, 300, S.ACT_RELU, S.WEIGHT_INITIALIZATION_HE)
    S.layer(net, 200, S.ACT_RELU, S.WEIGHT_INITIALIZATION_XAVIER)
    S.layer(net, 100, S.ACT_RELU, S.WEIGHT_INITIALIZATION_RANDOM)
    S.layer(net, 10, S.ACT_RELU, S.WEIGHT_INITIALIZATION_NONE)
    he, xa, un, no = (S.weights_view(net, l) for l in range(4))
    assert abs(he.std() - np.sqrt(2 / 400)) < 0.003 and abs(he.mean()) < 0.002
    assert abs(xa.std() - np.sqrt(1 / 300)) < 0.003
    assert un.min() >= -1 and un.max() <= 1 and abs(un.std() - 1 / np.sqrt(3)) < 0.02
    assert not no.any()
    S.free_network(net)


def test_activate_matches_oracle(S, O):
    xs = np.array([-3.0, -0.5, 0.0, 0.3, 1.0, 1.7, 9.0], np.float32)
    for a in range(7):
        got = np.array([S.activate(float(x), a) for x in xs], np.float32)
        want = xs.copy() if a == O.ACT["softmax"] else O.activate(xs, a)
        assert np.allclose(got, want, rtol=2e-7, atol=0), a


def test_derivative_matches_oracle(S, O):
    xs = np.array([-0.5, 0.0, 0.25, 1.0, 1.5], np.float32)
    for a in range(7):
        got = np.array([S.derivative(float(x), a) for x in xs], np.float32)
        assert np.array_equal(got, O.derivative(xs, a)), a


def test_print_parameters_lists_every_bias_and_weight(S):
    """print_parameters (Network.c:253-281) goes through the log: one line per bias and per weight, weights listed input
    neuron by input neuron."""
    lines = []
    cb = C.CFUNCTYPE(None, C.c_int, C.c_char_p)(lambda level, msg: lines.append((level, msg.decode())))
    net = S.new_spingalett(S.LOSS_CROSS_ENTROPY)
    S.layer(net, 2)
    S.layer(net, 3, S.ACT_TANH, S.WEIGHT_INITIALIZATION_NONE)
    S.weights_view(net, 0)[:] = np.arange(6, dtype=np.float32).reshape(3, 2) + 1       # W[j][k] = 1 + 2 j + k
    S.biases_view(net, 0)[:] = [0.5, -0.5, 0.25]
    S.lib().spingalett_set_log_callback(cb)
    S.lib().spingalett_set_log_level(S.LOG_INFO)
    S.set_verbose(True)
    try:
        S.print_parameters(net)
    finally:
        S.set_verbose(False)
        S.lib().spingalett_set_log_callback(C.CFUNCTYPE(None, C.c_int, C.c_char_p)())
    text = [m for lvl, m in lines if lvl == S.LOG_INFO]
    assert any("Cross-Entropy" in m for m in text)
    assert any("Layer 0 (2 neurons) -> Layer 1 (3 neurons)" in m and "Tanh" in m for m in text)
    assert sum("bias:" in m for m in text) == 3
    weights = [m for m in text if "->" in m and m.lstrip().startswith("L0 N")]
    assert len(weights) == 6
    assert weights[0].split(":")[0].strip() == "L0 N0 -> L1 N0" and float(weights[0].split(":")[1]) == 1.0
    assert weights[1].split(":")[0].strip() == "L0 N0 -> L1 N1" and float(weights[1].split(":")[1]) == 3.0
    assert weights[3].split(":")[0].strip() == "L0 N1 -> L1 N0" and float(weights[3].split(":")[1]) == 2.0
    S.free_network(net)


def test_settings_and_error_slot(S):
    L = S.lib()
    assert L.spingalett_get_compute_mode() == S.COMPUTE_HIP
    L.spingalett_set_compute_mode(S.COMPUTE_OPENBLAS)
    assert L.spingalett_get_compute_mode() == S.COMPUTE_OPENBLAS
    L.spingalett_set_compute_mode(99)                     # ignored (Settings.c:26-29)
    assert L.spingalett_get_compute_mode() == S.COMPUTE_OPENBLAS
    L.spingalett_set_compute_mode(S.COMPUTE_HIP)
    L.spingalett_set_num_threads(5)
    assert L.spingalett_get_num_threads() == 5
    assert L.spingalett_get_verbose() is False
    S.save_spingalett(None, None)
    assert S.last_error()[0] == S.SPINGALETT_ERR_INVALID
    # the slot is per thread
    import threading
    seen = []
    t = threading.Thread(target=lambda: seen.append(S.last_error()))
    t.start(); t.join()
    assert seen == [(0, "")]
    S.clear_error()
    assert S.last_error() == (0, "")


def test_a_record_the_library_did_not_allocate_is_recognised(S):
    """The private state lives behind the public record, so the library looks a caller's pointer up in its own
    table of live nets before reading past the public part: a NeuralNetwork made up by the caller (exactly as
    large as the public struct) is refused by forward() and reports FP32, a freed-and-recreated one is fine."""
    import ctypes as C
    fake = S.NeuralNetwork()
    fake.layers = 2
    x = np.zeros(4, np.float32)
    S.clear_error()
    out = S.lib().forward_struct_arguments(S.ForwardArgs(C.pointer(fake), x.ctypes.data_as(C.POINTER(C.c_float))))
    assert not out
    code, msg = S.last_error()
    assert code == S.SPINGALETT_ERR_INVALID and "not created by this library" in msg
    S.clear_error()
    assert S.lib().spingalett_hip_precision(C.pointer(fake)) == S.PRECISION_FLOAT32
    S.lib().spingalett_hip_invalidate(C.pointer(fake))
    assert S.last_error()[0] == S.SPINGALETT_ERR_INVALID
    S.clear_error()
    for _ in range(40):                                  # the table grows and shrinks
        nets = [S.new_spingalett() for _ in range(5)]
        for n in nets:
            S.layer(n, 3)
            S.free_network(n)
    assert S.last_error()[0] == S.SPINGALETT_OK


def test_forward_fails_loudly_without_a_gpu(S):
    if S.device_count() > 0:
        pytest.skip("a GPU is present")
    net = S.load_spingalett(os.path.join(GOLD, "tiny_i4.nn"))
    S.clear_error()
    assert S.forward(net, np.zeros(37, np.float32)) is None
    code, msg = S.last_error()
    assert code == S.SPINGALETT_ERR_INVALID and "no GPU" in msg
    with pytest.raises(S.SpingalettError):
        S.forward_batch(net, np.zeros((3, 37), np.float32))
    S.free_network(net)


def test_reference_header_compiles_against_this_library(S, tmp_path):
    """A C program written against the reference's own header links and runs
    (host-only calls) against libspingalett.so."""
    ref_inc = "/root/reference/Include"
    if not os.path.isdir(ref_inc):
        pytest.skip("reference tree not present")
    import shutil
    import subprocess
    cc = shutil.which("gcc")
    if cc is None:
        pytest.skip("no C compiler")
    (tmp_path / "Spingalett.Config.h").write_text("")     # compile-time switches only; empty = none set
    src = tmp_path / "t.c"
    src.write_text(r'''
#include <Spingalett/Spingalett.h>
#include <stddef.h>
#include <stdio.h>
int main(void) {
    spingalett_set_verbose(false);
    NeuralNetwork *nn = new_spingalett(.loss_func = LOSS_MSE);
    layer(nn, 2);
    layer(nn, 8, ACT_FOO52, WEIGHT_INITIALIZATION_HE);
    layer(nn, 1, ACT_SIGMOID, WEIGHT_INITIALIZATION_XAVIER);
    printf("%u %llu %llu %d\n", nn->layers, (unsigned long long)nn->total_weights,
           (unsigned long long)nn->total_biases, (int)sizeof(NeuralNetwork));
    save_spingalett(.net = nn, .filename = "abi_model", .precision = PRECISION_INT8, .do_not_save_optimizer = true);
    free_network(nn);
    NeuralNetwork *l = load_spingalett("abi_model.nn");
    printf("%d %u\n", l != NULL, l ? l->topology[1] : 0u);
    /* train() links and rejects an empty job the way the reference does (Training.c:609-613) */
    float x[2] = {0, 1}, t[1] = {1};
    train(.net = l, .inputs = x, .targets = t, .sample_count = 1, .epochs = 0, .training_strategy = STRATEGY_FULL_BATCH);
    printf("%d\n", spingalett_last_error_code());
    spingalett_clear_error();
    printf("%zu %zu %zu %zu %zu\n", sizeof(TrainArgs), offsetof(TrainArgs, epochs), offsetof(TrainArgs, max_grad_norm),
           offsetof(TrainArgs, autosave_path), offsetof(TrainArgs, callback_interval));
    free_network(l);
    return spingalett_last_error_code();
}
''')
    exe = tmp_path / "t"
    subprocess.check_call([cc, "-std=c2x", "-I", ref_inc, "-I", str(tmp_path), str(src), "-o", str(exe),
                           "-L", os.path.dirname(S.LIB_PATH), "-lspingalett",
                           "-Wl,-rpath," + os.path.dirname(S.LIB_PATH)])
    out = subprocess.run([str(exe)], cwd=tmp_path, capture_output=True, text=True)
    assert out.returncode == 0, out
    T = S.TrainArgs
    assert out.stdout.split() == ["3", "24", "9", "160", "1", "8", "2"] + [
        str(v) for v in (C.sizeof(T), T.epochs.offset, T.max_grad_norm.offset, T.autosave_path.offset,
                         T.callback_interval.offset)]


def test_bf16_activation_setting_round_trips(S):
    """spingalett_set_bf16_activations: FP16 activations (0) by default, BF16 (1) on request, anything else ignored."""
    L = S.lib()
    assert L.spingalett_get_bf16_activations() == 0
    try:
        L.spingalett_set_bf16_activations(1)
        assert L.spingalett_get_bf16_activations() == 1
        L.spingalett_set_bf16_activations(7)
        assert L.spingalett_get_bf16_activations() == 1
    finally:
        L.spingalett_set_bf16_activations(0)
    assert L.spingalett_get_bf16_activations() == 0
