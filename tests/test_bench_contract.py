"""CPU: the parts of bench.py's contract that need no GPU -- more than one GPU is refused with a message, and
standard output carries exactly one JSON line even though the native library reports on standard output itself
(checked on the host-only tokenizer workload)."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, cwd=ROOT,
                          timeout=300)


def test_more_than_one_gpu_is_refused():
    r = run("--gpus", "2")
    assert r.returncode == 2 and r.stdout == ""
    assert "one GPU" in r.stderr


def test_one_json_line_with_the_contract_fields():
    r = run("--workload", "tokenizer", "--steps", "3", "--warmup", "1", "--no-cpu-baseline")
    assert r.returncode == 0, r.stderr[-2000:]
    lines = r.stdout.splitlines()
    assert len(lines) == 1, lines
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["value"] > 0 and "workload" in d["config"]
    assert "Tokenizer:" in r.stderr                         # the library's report went to standard error
