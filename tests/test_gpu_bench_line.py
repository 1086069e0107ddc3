"""The one JSON line of ``bench.py``: a short run of the headline configuration in a child process, and the keys
and relations that the callers of the line rely on."""
import json
import pathlib
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = pathlib.Path(__file__).resolve().parents[1]


def test_headline_line_has_the_contract_keys_and_consistent_figures():
    run = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "1", "--steps", "4", "--warmup", "2",
                          "--headline-config-only", "--sustain-seconds", "0", "--settle-seconds", "0.1"],
                         capture_output=True, text=True, timeout=600, cwd=str(ROOT))
    assert run.returncode == 0, run.stderr[-2000:]
    lines = [ln for ln in run.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1, "exactly one line on stdout"
    line = json.loads(lines[0])

    assert line["metric"] and line["unit"] == "tokens/s" and line["higher_is_better"] is True
    assert line["n_gpus"] == 1 and line["steps"] == 4 and line["warmup"] == 2
    assert line["dtype"] == "bf16" and "synthetic" in line["data"] and line["vs_baseline"] is None
    assert "workload" in line["config"] and "model" not in line["config"]
    # value is the whole job: 4096 tokens per step
    assert line["value"] == pytest.approx(4096 / (line["ms_per_step"] * 1e-3), rel=1e-6)
    assert 0.5 < line["ms_per_step"] < 5.0

    roof = line["roofline"]
    assert roof["bound"] == "mfma" and roof["unit"] == "TFLOP/s" and roof["peak"] == 2500.0
    assert roof["frac"] == pytest.approx(roof["achieved"] / roof["peak"], rel=1e-9)
    assert 0.2 < roof["frac"] < 1.0
    # the dominant kernel cannot be slower than the step that contains it: 2 x 481 GFLOP per pair of launches
    pair_ms = 2 * 481.036 / roof["achieved"]
    assert pair_ms < line["ms_per_step"]

    cpu = line["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
    assert line["value"] > cpu["value"]

    parts = line["overlap_speedup_parts"]
    assert line["overlap_speedup"] == pytest.approx(
        parts["one_stream_same_kernels_graph_ms"] / parts["two_streams_graph_ms"], rel=1e-9)
    assert parts["outputs_bit_identical_to_the_one_stream_issue"] is True
    assert "north_star_pattern_gemm_beside_tail_of_previous_nano_batch" in line
    assert "power_limit_check" in line
