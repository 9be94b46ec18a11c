"""The kernels' scalar arithmetic (quartet_amd/csrc/qm_math.h) compiled for the host and checked against the host's
IEEE-754 arithmetic: exact division by fl32(4/3) in both forms, bf16 rounding, E2M1 rounding rules, the mapping of
random bytes to uniforms, Philox known answers, the fixed-sequence exponential (accuracy against the C library, and bit
for bit against the oracle's own statement of the same sequence over every bf16 input)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_qm_math_on_the_host(tmp_path):
    exe = tmp_path / "host_math_check"
    subprocess.run(["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-I", os.path.join(ROOT, "quartet_amd", "csrc"),
                    os.path.join(ROOT, "tests", "host_math_check.cpp"), "-o", str(exe)], check=True)
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0 and run.stdout.strip().endswith("ok"), run.stdout[-2000:]

    import re

    import numpy as np

    from oracle import oracle as o
    hashes = {"exp": 1469598103934665603, "silu": 1469598103934665603}
    L = o.lib()
    for h in range(65536):
        z = float(o.bf16_bits_to_f32(np.array([h], dtype=np.uint16))[0])
        if z != z:
            continue
        for name, fn in (("exp", L.qo_exp), ("silu", L.qo_silu)):
            bits = int(np.array([fn(z)], dtype=np.float32).view(np.uint32)[0])
            hashes[name] = ((hashes[name] ^ bits) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    got = re.search(r"exp_hash=([0-9a-f]+) silu_hash=([0-9a-f]+)", run.stdout)
    assert got and int(got.group(1), 16) == hashes["exp"] and int(got.group(2), 16) == hashes["silu"]
