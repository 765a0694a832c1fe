"""The kernels' tick arithmetic (LUT form, motifcl_amd/csrc/counter_math.hpp), compiled for
the CPU with g++ and compared with the oracle's literal form on millions of random and
adversarial inputs (every code, every C, integral, near-integral, huge and tiny values)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_lut_tick_equals_literal_tick(tmp_path, oracle):
    exe = str(tmp_path / "check_tick_math")
    subprocess.run(
        ["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-fno-fast-math",
         os.path.join(ROOT, "tests", "cpp", "check_tick_math.cpp"),
         os.path.join(ROOT, "oracle", "libcounter_oracle.so"),
         "-Wl,-rpath," + os.path.join(ROOT, "oracle"), "-o", exe],
        check=True, capture_output=True, text=True)
    r = subprocess.run([exe, "1500000"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-2000:]
    assert "0 mismatches" in r.stdout
