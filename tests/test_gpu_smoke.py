"""The driver's smoke entry and the loud failure when the native library is missing."""

import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_smoke_entry():
    sys.path.insert(0, ROOT)
    import __graft_entry__

    __graft_entry__.smoke()


def test_no_silent_fallback_when_the_kernel_library_cannot_be_loaded(tmp_path):
    """With an unloadable kernel library the engine raises; it never computes on another path."""
    code = (
        "import sys; sys.path.insert(0, %r)\n"
        "from mini_gpt_inference_amd.csrc import build\n"
        "build.ensure_kernels = lambda: %r\n"
        "from mini_gpt_inference_amd.ops import library\n"
        "try:\n"
        "    library.kernels()\n"
        "except library.NativeLibraryError as e:\n"
        "    print('LOUD', e)\n"
    ) % (ROOT, str(tmp_path / "missing.so"))
    proc = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert "LOUD" in proc.stdout and "cannot load native library" in proc.stdout


def test_bench_prints_one_record_with_the_agreed_fields():
    """A short run of bench.py with a step count that whole bursts do not divide and a warm-up shorter
    than a burst: one JSON line, the fields the measurement is read from, a flat `config`.  bench.py
    itself asserts that no HIP graph was recorded inside the timed steps and that every timed step
    came from a graph."""
    import json
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "20", "--warmup", "5",
                           "--layers", "2", "--no-extras", "--blocks", "13"], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [line for line in proc.stdout.splitlines() if line.startswith("{")]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 20 and rec["warmup"] == 5 and rec["value"] > 0
    # 256 generated tokens hold 12 blocks of 20 steps behind 5 of warm-up: the 13th block needs new requests
    assert rec["blocks"] == 24 and rec["iqr_ms"] >= 0 and rec["config"]["generated"] == 256
    assert 128 + 5 + 1 < rec["config"]["mean_context"] < 128 + 256
    assert rec["config"]["hip_graph"] is True and 0 < rec["kernels_per_step"] < 40
    assert rec["config"]["n_layer"] == 2 and rec["config"]["n_layer_full"] == 8      # fewer layers are named
    assert len(rec["config"]) <= 20 and not any(isinstance(v, (dict, list)) for v in rec["config"].values())
    assert abs(rec["roofline"]["frac"] - rec["roofline"]["achieved"] / rec["roofline"]["peak"]) < 1e-4
