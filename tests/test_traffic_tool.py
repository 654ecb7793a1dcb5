"""bench_traffic.py turns two rocprofv3 counter runs into the HBM bytes per launch that bench.py reports as
roofline.traffic.  Host-only checks of how it picks the dominant layer's launches out of the dispatch list."""
import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench_traffic  # noqa: E402


def test_dominant_layer_is_the_most_launched_group_not_the_largest_reading():
    # two layers run a kernel of the same name; bench.py times the dominant one with many launches of its own
    first = "void (anonymous namespace)::sp_gemm16_small<3, true, true, 1>((anonymous namespace)::GemmArgs)"
    second = "void (anonymous namespace)::sp_gemm16_small<3, true, false, 1>((anonymous namespace)::GemmArgs)"
    rows = [(first, 3410.0)] * 45 + [(second, 1321.5)] * 700 + [(second, 1322.0)] * 22 + [("sp_skinny16_kw<1>", 429.5)] * 45
    mean, count = bench_traffic.dominant(rows, "sp_gemm16_small")
    assert count == 722
    assert mean == pytest.approx(1321.5, rel=1e-3)


def test_one_instantiation_on_two_shapes_is_split_by_reading():
    name = "void (anonymous namespace)::sp_gemm16_big<2, true, 2, 4, 4, 2>((anonymous namespace)::GemmArgs)"
    rows = [(name, 788000.0 + i) for i in range(300)] + [(name, 96000.0)] * 40
    mean, count = bench_traffic.dominant(rows, "sp_gemm16_big")
    assert count == 300 and 788000.0 <= mean <= 788300.0


def test_a_kernel_that_never_ran_is_an_error():
    with pytest.raises(SystemExit):
        bench_traffic.dominant([("sp_gemv<1>", 10.0)], "sp_gemm16_big")


def test_committed_entries_name_their_commands_and_sizes():
    with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
        doc = json.load(f)
    assert doc["entries"]
    for e in doc["entries"]:
        assert e["bytes"] > 0 and e["dispatches_averaged"] >= 20, e["kernel"]
        assert len(e["shape"]) == 3 and e["shape"][0] == e["batch"]
        assert any("--pmc FETCH_SIZE" in c for c in e["commands"]) and any("--pmc WRITE_SIZE" in c for c in e["commands"])
