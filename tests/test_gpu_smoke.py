"""The driver's smoke entry point runs as part of the GPU suite."""
import pytest


@pytest.mark.gpu
def test_smoke_entry_point():
    import __graft_entry__

    __graft_entry__.smoke()


@pytest.mark.gpu
def test_bench_line_has_the_contract_fields():
    """A short bench.py run prints ONE JSON line with the fields the driver reads."""
    import json
    import pathlib
    import subprocess
    import sys

    root = pathlib.Path(__file__).resolve().parent.parent
    out = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "1", "--steps", "20", "--warmup", "5",
                          "--cpu-seconds", "0", "--no-sequential", "--configs", "cfg2b,cfg4"], capture_output=True, text=True, timeout=240, cwd=root)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [ln for ln in out.stdout.splitlines() if ln.startswith("{")]
    assert len(lines) == 1
    line = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 20 and line["unit"] == "edges/s" and line["value"] > 0
    assert line["vs_baseline"] is None and line["dtype"] == "f32" and "workload" in line["config"]
    # --steps counts calls; the number of batches per call does not shrink with it
    cfg = line["config"]
    assert cfg["hogwild_workers"] == 64 and cfg["timed_calls"] == 20 and cfg["timed_batches"] == 20 * 64
    assert line["value"] == pytest.approx(cfg["timed_edges"] / cfg["timed_wall_seconds"], rel=1e-6)
    roof = line["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in roof, key
    assert roof["bound"] in ("hbm", "mfma") and 0 < roof["frac"] < 1
    assert roof["frac"] == pytest.approx(roof["achieved"] / roof["peak"], rel=1e-6)
    # the other configurations ride along under "configs", each with its own roofline entry
    assert set(line["configs"]) == {"cfg2b", "cfg4"}
    for name, entry in line["configs"].items():
        assert entry["value"] > 0 and entry["sequential_value"] > 0, name
        assert entry["roofline"]["bound"] in ("hbm", "mfma") and 0 < entry["roofline"]["frac"] < 1, name
        assert cfg[f"{name}_edges_per_s"] == entry["value"]
