"""The probe harness end to end (tests/probe_quant_gemv.py): printed keys, summary and exit code."""
import io
from contextlib import redirect_stdout

import pytest

import probe_quant_gemv

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("tokens", [1, 4])
def test_probe_cases_all_ok(tokens):
    buf = io.StringIO()
    with redirect_stdout(buf):
        rc = probe_quant_gemv.main(["--reps", "5", "--warmup", "1", "--tokens", str(tokens)])
    out = buf.getvalue()
    assert rc == 0, out
    assert out.count("\nok=true") == len(probe_quant_gemv.CASES) and "summary_ok=true" in out
    for key in ("device=", "compute_capability=9.5", "case=", "type=Q4_K", "shape=4096x12288", "raw_bytes=28311552",
                "reps=5", "warmup=1", "hip_ms=", "cpu_ms=", "cos=", "max_diff="):
        assert key in out, key


def test_probe_argument_checks():
    with pytest.raises(SystemExit, match="reps must be positive"):
        probe_quant_gemv.main(["--reps", "0"])
    with pytest.raises(SystemExit, match="tokens must be positive"):
        probe_quant_gemv.main(["--tokens", "0"])
