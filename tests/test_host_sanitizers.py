"""The host side of the library under AddressSanitizer and UndefinedBehaviorSanitizer (CPU only).

`make asan` links the library's C sources (container parser, codecs, lifecycle, runtime) with tests/host_sanitize.c,
which stands in for the kernel translation unit and pushes well-formed files of every format, every prefix of them and
seeded damaged copies through load_spingalett_memory (the replacement of Serialize.c:426-609, which parses bytes it did
not write).  Any sanitizer report aborts the program."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "..", "spingalett_amd", "csrc")


def test_host_sources_under_address_and_ub_sanitizers():
    res = subprocess.run(["make", "-C", CSRC, "-B", "asan"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0:halt_on_error=1",
               UBSAN_OPTIONS="print_stacktrace=1:halt_on_error=1")
    env.pop("LD_PRELOAD", None)
    run = subprocess.run([os.path.join(CSRC, "build", "host_sanitize")], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                         text=True, env=env, timeout=600)
    assert run.returncode == 0, run.stdout[-4000:]
    assert "host_sanitize:" in run.stdout and "refused" in run.stdout, run.stdout[-2000:]
