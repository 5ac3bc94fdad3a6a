"""rmsnorm_f32 / add_rmsnorm_f32 through the C ABI against the CPU form (src/ml/gguf/qwen35_cpu.cr:484-490, :1705-1708).
The device sums the squares in fp32 where the CPU form uses Float64, so the bar is relative: 1e-6 of the largest output."""
import numpy as np
import pytest

from cogni_ml_amd import quant
from gpu_common import DevArray, gpu  # noqa: F401

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dim,tokens", [(4096, 1), (4096, 5), (1024, 3), (130, 2), (7, 1), (12288, 2), (1, 1)])
def test_rmsnorm_and_add_rmsnorm(gpu, oracle, dim, tokens):
    rng = np.random.default_rng(dim * 31 + tokens)
    x = (rng.standard_normal(tokens * dim) * 2.5).astype(np.float32)
    add = rng.standard_normal(tokens * dim).astype(np.float32)
    w = (1.0 + 0.1 * rng.standard_normal(dim)).astype(np.float32)
    eps = 1.0e-6
    xd, ad, wd = DevArray(x), DevArray(add), DevArray(w)
    od, rd, nd = (DevArray(nbytes=x.nbytes) for _ in range(3))
    try:
        quant.rmsnorm_dev(xd.ptr, wd.ptr, od.ptr, dim, tokens, eps)
        got = od.read(np.float32, x.size).reshape(tokens, dim)
        quant.add_rmsnorm_dev(xd.ptr, ad.ptr, wd.ptr, rd.ptr, nd.ptr, dim, tokens, eps)
        res, normed = rd.read(np.float32, x.size).reshape(tokens, dim), nd.read(np.float32, x.size).reshape(tokens, dim)
        summed = (x + add).reshape(tokens, dim)                   # one fp32 addition per element, as the CPU form
        assert np.array_equal(res, summed)
        for t in range(tokens):
            want = oracle.rms_norm(x[t * dim:(t + 1) * dim], w, eps)
            assert np.max(np.abs(got[t] - want)) <= 1e-6 * np.max(np.abs(want)), "rmsnorm token %d" % t
            want = oracle.rms_norm(summed[t], w, eps)
            assert np.max(np.abs(normed[t] - want)) <= 1e-6 * np.max(np.abs(want)), "add_rmsnorm token %d" % t
        # residual stream updated in place: residual_out aliases x
        quant.add_rmsnorm_dev(xd.ptr, ad.ptr, wd.ptr, xd.ptr, od.ptr, dim, tokens, eps)
        assert np.array_equal(xd.read(np.float32, x.size).reshape(tokens, dim), summed)
        assert np.array_equal(od.read(np.float32, x.size).reshape(tokens, dim), normed)
    finally:
        for d in (xd, ad, wd, od, rd, nd):
            d.close()


def test_rmsnorm_argument_errors(gpu):
    with pytest.raises(quant.QuantError, match="zero dimension"):
        quant.rmsnorm_dev(1, 1, 1, 0, 1)
    with pytest.raises(quant.QuantError, match="null device pointer"):
        quant.add_rmsnorm_dev(1, 0, 1, 1, 1, 16, 1)
    quant.rmsnorm_dev(1, 1, 1, 16, 0)       # no tokens: nothing is launched
