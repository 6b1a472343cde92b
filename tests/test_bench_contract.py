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


def test_traffic_figures_belong_to_the_committed_kernel_sources(tmp_path, monkeypatch):
    """roofline.traffic comes from profiles/measured_traffic.txt, keyed by the hash of the kernel's source file at the
    time of the counter runs: the committed lines must name the sources as they are (so the bench prints the figures,
    not null), and a line whose source has changed since must read as None."""
    sys.path.insert(0, ROOT)
    import bench
    for key in ("gemv_stack_b1", "gemm_gate_up_b256"):
        v = bench.measured_traffic(key)
        assert v is not None and 5e7 < v < 5e8, (key, v)
    assert bench.measured_traffic("no_such_kernel") is None
    # the same file with one source's hash changed
    fake = tmp_path / "repo"
    (fake / "profiles").mkdir(parents=True)
    (fake / "src").mkdir()
    (fake / "src" / "k.hip").write_text("kernel v2\n")
    (fake / "profiles" / "measured_traffic.txt").write_text("# comment\nk 1.0e8 src/k.hip 0123456789abcdef\n")
    monkeypatch.setattr(bench, "ROOT", str(fake))
    assert bench.measured_traffic("k") is None
    import hashlib
    h = hashlib.sha256(b"kernel v2\n").hexdigest()[:16]
    (fake / "profiles" / "measured_traffic.txt").write_text("k 1.0e8 src/k.hip %s\n" % h)
    assert bench.measured_traffic("k") == 1.0e8
