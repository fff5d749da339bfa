"""Host-side pieces of bench.py: no GPU needed."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one GPU" in r.stderr


def test_kernel_identity_ignores_the_function_number_only():
    a = bench.kernel_id("template<int N> __global__ void function_12() { function_3<N>(); }")
    b = bench.kernel_id("template<int N> __global__ void function_97() { function_41<N>(); }")
    c = bench.kernel_id("template<int N> __global__ void function_12() { function_3<N + 1>(); }")
    assert a == b and a != c and len(a) == 12


class _FakePipeline:
    source = "__global__ void function_5() {}"
    kernel_name = "function_5"


def test_traffic_is_used_only_for_the_kernel_it_was_measured_on(tmp_path, monkeypatch):
    kid = bench.kernel_id(_FakePipeline.source)
    table = tmp_path / "hbm_traffic.md"
    table.write_text("# title\n\n| workload | kernel id | fetch bytes | write bytes | note |\n|---|---|---|---|---|\n"
                     "| `same` | `%s` | 1000 | 500 | x |\n| `changed` | `0123456789ab` | 7 | 7 | y |\n| not a row |\n" % kid)
    monkeypatch.setattr(bench, "TRAFFIC_TABLE", str(table))
    rows = bench.traffic_table()
    assert rows == {"same": (kid, 1000, 500), "changed": ("0123456789ab", 7, 7)}
    timing = {"ms": 2.0, "ms_median": 1.0, "ms_min": 0.5}
    roof = bench.roofline("same", rows, "hbm", 8e9, timing, _FakePipeline())
    assert roof["traffic"] == 1500 and roof["traffic_fetch"] == 1000 and roof["bound"] == "hbm"
    assert abs(roof["achieved"] - 4000.0) < 1e-9 and abs(roof["frac"] - 0.5) < 1e-12 and abs(roof["frac_at_median"] - 1.0) < 1e-12
    roof = bench.roofline("changed", rows, "hbm", 8e9, timing, _FakePipeline())
    assert roof["traffic"] is None and "changed" in roof["traffic_note"]
    roof = bench.roofline("absent", rows, "mfma", 2.5e12, timing, _FakePipeline())
    assert roof["traffic"] is None and roof["unit"] == "TFLOP/s" and abs(roof["frac"] - 0.5) < 1e-12


def test_a_missing_traffic_table_means_no_traffic(tmp_path, monkeypatch):
    monkeypatch.setattr(bench, "TRAFFIC_TABLE", str(tmp_path / "absent.md"))
    assert bench.traffic_table() == {}


def test_kernel_identity_does_not_depend_on_what_was_generated_before():
    import gern_amd
    first = bench.kernel_id(gern_amd.Softmax(4096, flags=gern_amd.COMPILE_ONLY).source)
    gern_amd.BlurChain("xy", flags=gern_amd.COMPILE_ONLY)  # moves the code generator's counters
    again = gern_amd.Softmax(4096, flags=gern_amd.COMPILE_ONLY)
    assert bench.kernel_id(again.source) == first
    assert bench.kernel_id(gern_amd.Softmax(1000, flags=gern_amd.COMPILE_ONLY).source) != first
