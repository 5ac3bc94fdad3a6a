"""Session set-up shared by the GPU parity tests (all of them call through libcogni_hip.so)."""
import numpy as np
import pytest

from cogni_ml_amd import hip, quant


@pytest.fixture(scope="session")
def gpu():
    ctx = hip.Context.create(0)
    assert ctx.arch.startswith("gfx950"), ctx.arch
    quant.init(0)
    yield ctx
    ctx.close()


class DevArray:
    """A numpy array mirrored into a DeviceBuffer."""

    def __init__(self, host=None, nbytes=None):
        if host is not None:
            host = np.ascontiguousarray(host)
            nbytes = host.nbytes
        self.buf = hip.DeviceBuffer(nbytes)
        self.ptr, self.nbytes = self.buf.ptr, nbytes
        if host is not None and nbytes:
            hip.copy_htod(self.ptr, host, nbytes, "test input")

    def read(self, dtype, count):
        out = np.empty(count, dtype=dtype)
        hip.synchronize()
        hip.copy_dtoh(out, self.ptr, out.nbytes, "test output")
        return out

    def close(self):
        self.buf.close()
