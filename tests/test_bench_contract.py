"""bench.py's command-line contract and the provenance of its traffic figures
(no GPU: nothing here launches a kernel)."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode != 0
    assert "one GPU" in (proc.stdout + proc.stderr)


def test_traffic_table_names_sources_that_exist_and_carries_its_commands():
    with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
        table = json.load(f)
    assert all("rocprofv3 --pmc" in c and "bench.py" in c for c in table["commands"])
    assert "radix_sort_u32_uniform_2^28" in table["workloads"]
    for name, entry in table["workloads"].items():
        assert os.path.exists(os.path.join(bench.CSRC, entry["source"])), name
        assert entry["bytes_per_launch"] > 0 and len(entry["sha256"]) == 16, name


def test_source_digest_ignores_comments_and_layout_but_not_code(tmp_path, monkeypatch):
    monkeypatch.setattr(bench, "CSRC", str(tmp_path))
    (tmp_path / "a.hip").write_text("int f() {\n  return 1;  // one\n}\n")
    (tmp_path / "b.hip").write_text("// header\n\nint f() {\n      return 1;\n}\n")
    (tmp_path / "c.hip").write_text("int f() {\n  return 2;\n}\n")
    assert bench.source_digest("a.hip") == bench.source_digest("b.hip")
    assert bench.source_digest("a.hip") != bench.source_digest("c.hip")
    # the shared headers and the compiler flags count too
    before = bench.source_digest("a.hip")
    (tmp_path / "common.hpp").write_text("constexpr int kWaveSize = 64;\n")
    with_header = bench.source_digest("a.hip")
    assert with_header != before
    (tmp_path / "common.hpp").write_text("constexpr int kWaveSize = 64;  // a wave\n")
    assert bench.source_digest("a.hip") == with_header
    from ilgpu_amd import build
    monkeypatch.setattr(build, "FLAGS", build.FLAGS + ["-DX"])
    assert bench.source_digest("a.hip") != with_header


def test_stale_counters_are_not_reported_as_traffic(tmp_path, monkeypatch):
    # counters read on other code: no figure, and the provenance says why
    table = {"workloads": {"w": {"bytes_per_launch": 5.0, "source": "a.hip", "sha256": "0" * 16}}}
    path = tmp_path / "t.json"
    path.write_text(json.dumps(table))
    (tmp_path / "a.hip").write_text("int f() { return 1; }\n")
    monkeypatch.setattr(bench, "CSRC", str(tmp_path))
    monkeypatch.setattr(bench, "TRAFFIC_FILE", str(path))
    value, provenance = bench.measured_traffic("w", True)
    assert value is None and "stale" in provenance
    table["workloads"]["w"]["sha256"] = bench.source_digest("a.hip")
    path.write_text(json.dumps(table))
    value, provenance = bench.measured_traffic("w", True)
    assert value == 5.0 and "stale" not in provenance


def test_profile_summaries_name_commands_that_run_committed_files():
    # Every summary under profiles/ gives the command that made it, and every
    # file such a command runs is part of the repository (or is built from it
    # by `python -m ilgpu_amd.build`: the library, its variants, bench_bounds).
    import glob
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    summaries = sorted(glob.glob(os.path.join(root, "profiles", "*.txt")))
    assert summaries
    built = ("ilgpu_amd/lib/bench_bounds", "ilgpu_amd/lib/variants/")
    for path in summaries:
        text = open(path, encoding="utf-8").read()
        assert "command" in text.split("\n\n")[0] + text, path
        for name in re.findall(r"(?:python3?|--) +([\w/]+\.py)\b", text):
            assert os.path.exists(os.path.join(root, name)), (path, name)
        for name in re.findall(r"^\s+(ilgpu_amd/lib/[\w/]+)", text, flags=re.M):
            assert name.startswith(built), (path, name)
        assert "_work/" not in text, path


def test_bounds_benchmark_is_part_of_the_build():
    from ilgpu_amd import build
    assert os.path.exists(build.BOUNDS_SRC)
    if os.path.exists(build.LIB_PATH):
        assert os.path.exists(build.BOUNDS_BIN), "python -m ilgpu_amd.build builds both"
