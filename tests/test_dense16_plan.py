"""CPU: the host-side planner of the small-batch GEMM launch with two workgroup sizes (csrc/dense16_plan.h), built with
-fsanitize=address,undefined and run over a few hundred thousand random launches: a wrong plan would send the kernel
outside its tensors, so every plan is checked for heads and tails inside their tensors, tails that start on a whole
workgroup of the head size, all tails within one round of the chip, and no more rounds than the plain launch."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_plan_is_a_launch_the_kernel_can_run(tmp_path):
    exe = str(tmp_path / "plan_check")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-static-libasan",
           "-I" + os.path.join(ROOT, "turbo-lossless_amd", "csrc"), os.path.join(ROOT, "tests", "plan_dense16_check.cpp"), "-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    r = subprocess.run([exe, "300000"], capture_output=True, text=True, timeout=300,
                       env=dict(os.environ, ASAN_OPTIONS="detect_leaks=0"))
    assert r.returncode == 0, (r.stdout[-1000:], r.stderr[-3000:])
    assert r.stdout.startswith("ok:")
