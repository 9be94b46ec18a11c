"""The kernels' scalar arithmetic (quartet_amd/csrc/qm_math.h) compiled for the host and checked against the host's
IEEE-754 arithmetic: exact division by fl32(4/3) in both forms, bf16 rounding, E2M1 rounding rules, the mapping of
random bytes to uniforms, Philox known answers."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_qm_math_on_the_host(tmp_path):
    exe = tmp_path / "host_math_check"
    subprocess.run(["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-I", os.path.join(ROOT, "quartet_amd", "csrc"),
                    os.path.join(ROOT, "tests", "host_math_check.cpp"), "-o", str(exe)], check=True)
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0 and run.stdout.strip().endswith("ok"), run.stdout[-2000:]
