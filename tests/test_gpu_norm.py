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
    # (real device memory behind every pointer, large enough for the shapes named: a call that were accepted by mistake
    # would stay inside it)
    buf = DevArray(nbytes=4 << 20)
    p = buf.ptr
    with pytest.raises(quant.QuantError, match="zero dimension"):
        quant.rmsnorm_dev(p, p, p, 0, 1)
    with pytest.raises(quant.QuantError, match="null device pointer"):
        quant.add_rmsnorm_dev(p, 0, p, p, p, 16, 1)
    quant.rmsnorm_dev(p, p, p, 16, 0)       # no tokens: nothing is launched
    buf.close()


@pytest.mark.parametrize("w_type", [12, 13, 14])
@pytest.mark.parametrize("dim,tokens", [(4096, 8), (4096, 3), (2048, 1), (2048, 6), (1024, 5), (2560, 8), (3584, 2), (256, 4)])
def test_norms_that_also_write_the_activation_image(gpu, w_type, dim, tokens):
    """rmsnorm_pack / add_rmsnorm_pack: the normalised rows and residual stream of the plain kernels, bit for bit, and the
    image cogni_gemv_pack_dev writes from those rows, byte for byte (absent tokens' slots zeroed; the image buffer starts as
    garbage; rows that are not a multiple of 2048 values: the zero super-blocks that fill the image up as well). With the
    fp32 output left out the image is the same."""
    rng = np.random.default_rng(dim + 17 * tokens + w_type)
    x = (rng.standard_normal(tokens * dim) * 2.5).astype(np.float32)
    x[:min(300, dim)] *= np.float32(1e-20)                                   # a super-block far below the binary16 range
    add = rng.standard_normal(tokens * dim).astype(np.float32)
    w = (1.0 + 0.1 * rng.standard_normal(dim)).astype(np.float32)
    eps = 1.0e-6
    nbytes = quant.gemv_image_bytes(w_type, dim, 8)
    assert nbytes > 0
    junk = rng.integers(0, 256, nbytes, dtype=np.uint8)
    xd, ad, wd = DevArray(x), DevArray(add), DevArray(w)
    od, rd, nd, od2, rd2 = (DevArray(nbytes=x.nbytes) for _ in range(5))
    img_ref, img = DevArray(junk), DevArray(junk)
    try:
        for with_add in (False, True):
            if with_add:
                quant.add_rmsnorm_dev(xd.ptr, ad.ptr, wd.ptr, rd.ptr, nd.ptr, dim, tokens, eps)
                quant.add_rmsnorm_pack_dev(xd.ptr, ad.ptr, wd.ptr, rd2.ptr, od2.ptr, w_type, img.ptr, dim, tokens, eps)
                assert np.array_equal(rd2.read(np.float32, x.size), rd.read(np.float32, x.size))
            else:
                quant.rmsnorm_dev(xd.ptr, wd.ptr, nd.ptr, dim, tokens, eps)
                quant.rmsnorm_pack_dev(xd.ptr, wd.ptr, od2.ptr, w_type, img.ptr, dim, tokens, eps)
            assert np.array_equal(od2.read(np.float32, x.size), nd.read(np.float32, x.size))
            if tokens >= 2:       # (the pack kernel itself starts at two tokens)
                quant.gemv_pack_dev(nd.ptr, w_type, dim, tokens, img_ref.ptr)
                assert np.array_equal(img.read(np.uint8, nbytes), img_ref.read(np.uint8, nbytes))
            first = img.read(np.uint8, nbytes).copy()
            # without the fp32 rows
            hip_junk = DevArray(junk)
            if with_add:
                quant.add_rmsnorm_pack_dev(xd.ptr, ad.ptr, wd.ptr, rd2.ptr, 0, w_type, hip_junk.ptr, dim, tokens, eps)
            else:
                quant.rmsnorm_pack_dev(xd.ptr, wd.ptr, 0, w_type, hip_junk.ptr, dim, tokens, eps)
            assert np.array_equal(hip_junk.read(np.uint8, nbytes), first)
            hip_junk.close()
    finally:
        for d in (xd, ad, wd, od, rd, nd, od2, rd2, img_ref, img):
            d.close()


def test_norm_pack_argument_errors(gpu):
    # (real device memory behind every pointer, large enough for the shapes named: a call that were accepted by mistake
    # would stay inside it)
    buf = DevArray(nbytes=4 << 20)
    p = buf.ptr
    with pytest.raises(quant.QuantError, match="one-pass GEMV takes"):
        quant.rmsnorm_pack_dev(p, p, p, 12, p, 1000, 4)            # no one-pass kernel for rows of 1000
    with pytest.raises(quant.QuantError, match="one-pass GEMV takes"):
        quant.rmsnorm_pack_dev(p, p, p, 12, p, 6144, 4)            # longer than a thread keeps
    with pytest.raises(quant.QuantError, match="one-pass GEMV takes"):
        quant.add_rmsnorm_pack_dev(p, p, p, p, p, 2, p, 4096, 4)   # Q4_0 has no image
    with pytest.raises(quant.QuantError, match="one-pass GEMV takes"):
        quant.rmsnorm_pack_dev(p, p, p, 14, p, 4096, 9)
    with pytest.raises(quant.QuantError, match="null device pointer"):
        quant.add_rmsnorm_pack_dev(p, p, p, 0, p, 12, p, 4096, 4)
    buf.close()


@pytest.mark.parametrize("w_type", [12, 13, 14])
@pytest.mark.parametrize("dim,tokens", [(4096, 512), (4096, 9), (2048, 130), (1024, 64), (2560, 200), (256, 129), (3584, 65)])
def test_norms_that_write_the_packed_gemm_activations(gpu, w_type, dim, tokens):
    """cogni_rmsnorm_gemm_pack_dev / cogni_add_rmsnorm_gemm_pack_dev: every byte of the block cogni_gemm_pack_dev writes from
    the plain norm's output (the layouts of the three GEMM weight types; last token tiles that are not full carry zeros for
    the absent tokens), the residual stream and, when asked for, the normalised rows bit for bit the plain kernels'."""
    rng = np.random.default_rng(dim + 13 * tokens + w_type)
    x = (rng.standard_normal(tokens * dim) * 2.5).astype(np.float32)
    add = rng.standard_normal(tokens * dim).astype(np.float32)
    w = (1.0 + 0.1 * rng.standard_normal(dim)).astype(np.float32)
    eps = 1.0e-6
    nbytes = quant.gemm_workspace_bytes(w_type, dim, tokens)
    ff = np.full(nbytes, 0xFF, dtype=np.uint8)     # every byte of the packed block has to be written by the norm
    xd, ad, wd = DevArray(x), DevArray(add), DevArray(w)
    od, rd, nd, od2, rd2, nd2 = (DevArray(nbytes=x.nbytes) for _ in range(6))
    p_ref, p_a, p_b, p_c = DevArray(nbytes=nbytes), DevArray(ff), DevArray(ff), DevArray(ff)
    try:
        quant.rmsnorm_dev(xd.ptr, wd.ptr, od.ptr, dim, tokens, eps)
        quant.gemm_pack_dev(od.ptr, w_type, dim, tokens, p_ref.ptr, nbytes)
        want = p_ref.read(np.uint8, nbytes)
        quant.rmsnorm_gemm_pack_dev(xd.ptr, wd.ptr, od2.ptr, w_type, p_a.ptr, nbytes, dim, tokens, eps)
        assert np.array_equal(p_a.read(np.uint8, nbytes), want)
        assert np.array_equal(od2.read(np.float32, x.size), od.read(np.float32, x.size))
        quant.rmsnorm_gemm_pack_dev(xd.ptr, wd.ptr, 0, w_type, p_b.ptr, nbytes, dim, tokens, eps)
        assert np.array_equal(p_b.read(np.uint8, nbytes), want)

        quant.add_rmsnorm_dev(xd.ptr, ad.ptr, wd.ptr, rd.ptr, nd.ptr, dim, tokens, eps)
        quant.gemm_pack_dev(nd.ptr, w_type, dim, tokens, p_ref.ptr, nbytes)
        want = p_ref.read(np.uint8, nbytes)
        quant.add_rmsnorm_gemm_pack_dev(xd.ptr, ad.ptr, wd.ptr, rd2.ptr, nd2.ptr, w_type, p_c.ptr, nbytes, dim, tokens, eps)
        assert np.array_equal(p_c.read(np.uint8, nbytes), want)
        assert np.array_equal(rd2.read(np.float32, x.size), rd.read(np.float32, x.size))
        assert np.array_equal(nd2.read(np.float32, x.size), nd.read(np.float32, x.size))
        # the residual stream written in place (residual_out = x), no normalised rows
        quant.add_rmsnorm_gemm_pack_dev(xd.ptr, ad.ptr, wd.ptr, xd.ptr, 0, w_type, p_a.ptr, nbytes, dim, tokens, eps)
        assert np.array_equal(p_a.read(np.uint8, nbytes), want)
        assert np.array_equal(xd.read(np.float32, x.size), rd.read(np.float32, x.size))
    finally:
        for d in (xd, ad, wd, od, rd, nd, od2, rd2, nd2, p_ref, p_a, p_b, p_c):
            d.close()


def test_norm_gemm_pack_argument_errors(gpu):
    # (real device memory behind every pointer, as above)
    buf = DevArray(nbytes=8 << 20)
    p, n = buf.ptr, 8 << 20
    with pytest.raises(quant.QuantError, match="dim must be a multiple of 256 up to 4096"):
        quant.rmsnorm_gemm_pack_dev(p, p, p, 12, p, n, 1000, 16)
    with pytest.raises(quant.QuantError, match="dim must be a multiple of 256 up to 4096"):
        quant.add_rmsnorm_gemm_pack_dev(p, p, p, p, p, 14, p, n, 6144, 16)
    with pytest.raises(quant.QuantError, match="Unsupported quant type for the prefill GEMM: Q8_0"):
        quant.rmsnorm_gemm_pack_dev(p, p, p, 8, p, n, 1024, 16)
    with pytest.raises(quant.QuantError, match="workspace has 1000 bytes"):
        quant.rmsnorm_gemm_pack_dev(p, p, p, 12, p, 1000, 1024, 16)
    with pytest.raises(quant.QuantError, match="null device pointer"):
        quant.add_rmsnorm_gemm_pack_dev(p, p, p, 0, p, 12, p, n, 1024, 16)
    buf.close()


@pytest.mark.parametrize("w_type", [12, 13, 14])
@pytest.mark.parametrize("dim,tokens", [(4096, 16), (4096, 9), (2048, 12), (1024, 1), (2560, 13), (256, 16)])
def test_norms_that_write_the_sixteen_token_image(gpu, w_type, dim, tokens):
    """cogni_rmsnorm_pack16_dev / cogni_add_rmsnorm_pack16_dev: every byte of the image cogni_gemv_pack16_dev makes of the plain
    norm's output (zeros for the absent tokens and the super-blocks past the row's end), the residual stream and, when asked
    for, the normalised rows bit for bit the plain kernels'."""
    rng = np.random.default_rng(dim + 17 * tokens + w_type)
    x = (rng.standard_normal(tokens * dim) * 2.5).astype(np.float32)
    add = rng.standard_normal(tokens * dim).astype(np.float32)
    w = (1.0 + 0.1 * rng.standard_normal(dim)).astype(np.float32)
    eps = 1.0e-6
    nbytes = quant.gemv_image_bytes(w_type, dim, 8)
    ff = np.full(nbytes, 0xFF, dtype=np.uint8)
    xd, ad, wd = DevArray(x), DevArray(add), DevArray(w)
    od, rd, nd, od2, rd2 = (DevArray(nbytes=x.nbytes) for _ in range(5))
    i_ref, i_a, i_b = DevArray(ff), DevArray(ff), DevArray(ff)
    try:
        quant.rmsnorm_dev(xd.ptr, wd.ptr, od.ptr, dim, tokens, eps)
        quant.gemv_pack16_dev(od.ptr, w_type, dim, tokens, i_ref.ptr)
        quant.rmsnorm_pack16_dev(xd.ptr, wd.ptr, od2.ptr, w_type, i_a.ptr, dim, tokens, eps)
        assert np.array_equal(i_a.read(np.uint8, nbytes), i_ref.read(np.uint8, nbytes))
        assert np.array_equal(od2.read(np.float32, x.size), od.read(np.float32, x.size))
        quant.add_rmsnorm_dev(xd.ptr, ad.ptr, wd.ptr, rd.ptr, nd.ptr, dim, tokens, eps)
        quant.gemv_pack16_dev(nd.ptr, w_type, dim, tokens, i_ref.ptr)
        quant.add_rmsnorm_pack16_dev(xd.ptr, ad.ptr, wd.ptr, rd2.ptr, 0, w_type, i_b.ptr, dim, tokens, eps)
        assert np.array_equal(i_b.read(np.uint8, nbytes), i_ref.read(np.uint8, nbytes))
        assert np.array_equal(rd2.read(np.float32, x.size), rd.read(np.float32, x.size))
        with pytest.raises(quant.QuantError, match="1..16 tokens"):
            quant.rmsnorm_pack16_dev(xd.ptr, wd.ptr, od2.ptr, w_type, i_a.ptr, dim, 17, eps)
        with pytest.raises(quant.QuantError, match="1..16 tokens"):
            quant.rmsnorm_pack16_dev(xd.ptr, wd.ptr, od2.ptr, 8, i_a.ptr, dim, tokens, eps)
    finally:
        for d in (xd, ad, wd, od, rd, nd, od2, rd2, i_ref, i_a, i_b):
            d.close()
