"""What the benchmark script promises without a GPU: its configurations, the refusal of more than one GPU, and that
the traffic figures it reports come from profile summaries that are there."""

import json
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def _bench():
    sys.path.insert(0, str(ROOT))
    import bench
    return bench


def test_every_companion_of_the_default_line_has_a_traffic_entry_and_a_profile():
    bench = _bench()
    table = json.loads((ROOT / "profiles" / "traffic.json").read_text())
    for config in ["c2"] + bench.COMPANIONS:
        assert config in bench.CONFIGS
        entry = table[config]
        assert entry["fetch_kib"] > 0 and entry["write_kib"] > 0, config
        summary = ROOT / "profiles" / entry["profile"]
        text = summary.read_text()
        assert "rocprofv3" in text and f"--config {config}" in text, summary.name  # the command that made it
        assert bench.traffic_bytes(config) == int(
            (bench.FETCH_SCALE * entry["fetch_kib"] + bench.WRITE_SCALE * entry["write_kib"]) * 1024)
    assert bench.traffic_bytes("no such configuration") is None


def test_profile_summaries_name_committed_files_only():
    """Every summary quotes the command that made it, and that command runs bench.py, nothing else of this tree."""
    for summary in sorted((ROOT / "profiles").glob("*.txt")):
        commands = [line for line in summary.read_text().splitlines() if line.startswith("# cd /tmp")]
        assert commands, summary.name
        for line in commands:
            assert "/root/repo/bench.py" in line and "_work" not in line, (summary.name, line)


def test_more_than_one_gpu_is_refused_with_a_message():
    run = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert run.returncode != 0 and "one GPU" in (run.stderr + run.stdout)
