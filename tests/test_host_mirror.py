"""The C++ host mirror of ML::HIP / QuantMatmul (cogni-ml_amd/host/*.hpp) through tests/cpp/test_host_mirror."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
EXE = os.path.join(HERE, "cpp", "test_host_mirror")


def build():
    from oracle import oracle
    oracle.build()
    subprocess.run(["make", "-s", "-C", os.path.join(HERE, "cpp")], check=True)


def test_host_only_runner_spec_and_argument_errors():
    build()
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "PASSED (0 failures)" in r.stdout


@pytest.mark.gpu
def test_probe_sequence_through_cpp_classes():
    if not os.path.exists(EXE):
        build()
    r = subprocess.run([EXE, "--gpu"], capture_output=True, text=True, timeout=100)
    print(r.stdout)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ok=true" in r.stdout and "summary_ok=true" in r.stdout
    for key in ("device=", "type=Q4_K", "shape=4096x1024", "raw_bytes=", "reps=", "warmup=", "hip_ms=", "cos=", "max_diff="):
        assert key in r.stdout
