"""Decode GEMV for 2..8 tokens in one pass over a Q4_K, Q5_K or Q6_K matrix (activations packed once, q4_k_gemv_mt_f32 /
q5_k_gemv_mt_f32 / q6_k_gemv_mt_f32) vs the CPU oracle.

Bars, both asserted: the north-star bound max|err| <= 1e-4 * ||x||_2 * max|w_row| per token and row, and the reference's own
probe gate (cos >= 0.99999, max_diff <= 1e-3 * max(1, max|ref| / 64): the probe's absolute 1e-3 is meant for outputs of order
10..100). The kernel feeds the activations as two binary16 terms (22 bits), so it is also held to 2e-5 of each token's
output scale."""
import numpy as np
import pytest

from cogni_ml_amd import hip, quant, synth
from gpu_common import DevArray, gpu  # noqa: F401
from helpers import Q4_K, Q5_K, Q6_K, Q8_0, cosine, gemv_tolerance

pytestmark = pytest.mark.gpu


def oracle_rows(oracle, raw, x, in_dim, out_dim, tokens, type_id=Q4_K):
    want = oracle.matmul_add(x, tokens, in_dim, raw, type_id, out_dim, np.zeros(out_dim, dtype=np.float32), threads=8).astype(np.float64)
    dense = np.abs(oracle.dequantize(raw, type_id, out_dim * in_dim)).reshape(out_dim, in_dim)
    return want, gemv_tolerance(x, dense, tokens, in_dim).reshape(-1)


def assert_bars(got, want, tol, tokens, out_dim, what):
    err = np.abs(got.astype(np.float64) - want)
    worst = int(np.argmax(err / np.maximum(tol, 1e-30)))
    assert np.all(err <= tol), "%s: err %.3e > tol %.3e at %d" % (what, err[worst], tol[worst], worst)
    g, w_ = got.reshape(tokens, out_dim).astype(np.float64), want.reshape(tokens, out_dim)
    for m in range(tokens):
        scale = float(np.max(np.abs(w_[m])))
        if scale == 0.0:
            assert not g[m].any()
            continue
        assert cosine(g[m], w_[m]) >= 0.99999, (what, m)
        assert np.max(np.abs(g[m] - w_[m])) <= 1e-3 * max(1.0, scale / 64.0), (what, m)
        assert np.max(np.abs(g[m] - w_[m])) <= 2e-5 * scale, (what, m)


ONE_PASS_SHAPES = [(4096, 12288), (4096, 4096), (2048, 1024), (4096, 37), (2048, 50), (4096, 1040), (2048, 16 * 3 * 256 * 2 + 40),
                   (4096, 16 * 300 + 7), (2048, 16 * 600)]


@pytest.mark.parametrize("in_dim,out_dim", ONE_PASS_SHAPES)
@pytest.mark.parametrize("tokens", [5, 6, 7, 8])
def test_five_to_eight_tokens_in_one_pass(gpu, oracle, in_dim, out_dim, tokens):
    """cogni_gemv_dev with 5..8 tokens: one pack and one launch. Shapes: one, two and three tiles per wavefront, a single
    partial tile, row counts that are not multiples of 16, more row groups than workgroups (24616 rows: the workgroups walk
    two groups each, refilling their slots), both super-block counts per k-slice; with and without residual."""
    print("case in_dim=%d out_dim=%d tokens=%d" % (in_dim, out_dim, tokens), flush=True)
    assert quant.gemv_image_bytes(Q4_K, in_dim, tokens) == (in_dim // 256) * (8192 + 1024)
    rng = np.random.default_rng(in_dim * 13 + out_dim * 7 + tokens)
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    res = rng.standard_normal(tokens * out_dim).astype(np.float32)
    want, tol = oracle_rows(oracle, raw, x, in_dim, out_dim, tokens)
    w, xd, od, rd = DevArray(raw), DevArray(x), DevArray(nbytes=4 * tokens * out_dim), DevArray(res)
    quant.gemv_dev(w.ptr, Q4_K, xd.ptr, od.ptr, in_dim, out_dim, tokens)
    plain = od.read(np.float32, tokens * out_dim)
    assert_bars(plain, want, tol, tokens, out_dim, "%dx%d M=%d" % (in_dim, out_dim, tokens))
    quant.gemv_dev(w.ptr, Q4_K, xd.ptr, od.ptr, in_dim, out_dim, tokens, rd.ptr)
    added = od.read(np.float32, tokens * out_dim)
    assert np.array_equal(added, plain + res)          # the residual is one fp32 add on the finished sum
    for a in (w, xd, od, rd):
        a.close()


@pytest.mark.parametrize("tokens", [2, 3, 4, 8])
def test_explicit_image_and_matrix_lists(gpu, oracle, tokens):
    """The caller-owned image: pack once, then a list of matrices (q | k | v | odd one) against it in one call. A matrix
    whose row count is not a multiple of 16 ends its launch; the values are those of the same kernel on each matrix alone,
    bit for bit (a row's arithmetic does not depend on its neighbours)."""
    in_dim, dims = 4096, (4096, 1024, 1040, 24, 16, 160)
    rng = np.random.default_rng(tokens)
    raws = [synth.make_weights(rng, Q4_K, d, in_dim) for d in dims]
    x = synth.make_activations(rng, tokens, in_dim)
    ws, xd = [DevArray(r) for r in raws], DevArray(x)
    image = DevArray(nbytes=quant.gemv_image_bytes(Q4_K, in_dim, tokens))
    outs = [DevArray(nbytes=4 * tokens * d) for d in dims]
    quant.gemv_pack_dev(xd.ptr, Q4_K, in_dim, tokens, image.ptr)
    quant.gemv_packed_dev([w.ptr for w in ws], Q4_K, image.ptr, [o.ptr for o in outs], list(dims), in_dim, tokens)
    single = DevArray(nbytes=4 * tokens * max(dims))
    for raw, w, o, d in zip(raws, ws, outs, dims):
        got = o.read(np.float32, tokens * d)
        want, tol = oracle_rows(oracle, raw, x, in_dim, d, tokens)
        assert_bars(got, want, tol, tokens, d, "list member %d rows M=%d" % (d, tokens))
        quant.gemv_packed_dev([w.ptr], Q4_K, image.ptr, [single.ptr], [d], in_dim, tokens)
        assert np.array_equal(got, single.read(np.float32, tokens * d))
    for a in ws + outs + [xd, image, single]:
        a.close()


def test_one_pass_activation_ranges(gpu, oracle):
    """Activations far outside the binary16 range, zeros and mixed magnitudes must come out as from fp32 arithmetic: the
    image scales every (token, super-block) by its own power of two."""
    rng = np.random.default_rng(78)
    in_dim, out_dim, tokens = 4096, 528, 8
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim).reshape(tokens, in_dim)
    x[0] *= np.float32(1e-30)                       # far below the smallest binary16 subnormal
    x[1] *= np.float32(1e30)                        # far above the largest binary16 number
    x[2, :256] = 0.0                                # an all-zero super-block
    x[2, 256:512] *= np.float32(1e-12)
    x[2, 700] = np.float32(3e7)                     # one huge value among small ones
    x[3] = np.where(rng.random(in_dim) < 0.5, x[3] * np.float32(1e-6), x[3] * np.float32(1e4)).astype(np.float32)
    x[4] = 0.0                                      # a whole token of zeros
    x[5] = np.float32(1.0)                          # constants: the min term alone decides the sign of many rows
    x[6] = -x[7]                                    # a token and its negative
    x = np.ascontiguousarray(x.reshape(-1))
    want, tol = oracle_rows(oracle, raw, x, in_dim, out_dim, tokens)
    w, xd, od = DevArray(raw), DevArray(x), DevArray(nbytes=4 * tokens * out_dim)
    quant.gemv_dev(w.ptr, Q4_K, xd.ptr, od.ptr, in_dim, out_dim, tokens)
    got = od.read(np.float32, tokens * out_dim)
    assert_bars(got, want, tol, tokens, out_dim, "activation ranges")
    g = got.reshape(tokens, out_dim)
    assert not g[4].any()
    # (not bit for bit: the matrix cores' internal sums are not symmetric under a change of sign)
    assert np.max(np.abs(g[6] + g[7])) <= 2e-5 * float(np.abs(g[7]).max())
    for a in (w, xd, od):
        a.close()


@pytest.mark.parametrize("type_id", [Q4_K, Q5_K, Q6_K])
def test_one_pass_activations_near_the_top_of_the_fp32_range(gpu, oracle, type_id):
    """|x| of 1e35 .. 1e36, beyond 2^116: the image's power of two brings any finite activation into the binary16 range (no
    clamp on the large side) and the sub-block sums are formed after the scaling, so nothing overflows before the result
    does. The outputs (up to about 1e38) are finite in the reference's f64 sums and must be here, to the usual bars."""
    rng = np.random.default_rng(338)
    in_dim, out_dim, tokens = 2048, 96, 8
    raw = synth.make_weights(rng, type_id, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim).reshape(tokens, in_dim)
    x[0] *= np.float32(1e35)
    x[1] *= np.float32(2e35)
    x[2, :256] = np.float32(2.0 ** 117) * np.where(np.arange(256) % 2 == 0, 1.0, -1.0).astype(np.float32)   # one magnitude, alternating signs
    x[3] *= np.float32(1e-37)                        # and the smallest normal numbers
    x = np.ascontiguousarray(x.reshape(-1)).astype(np.float32)
    want, tol = oracle_rows(oracle, raw, x, in_dim, out_dim, tokens, type_id)
    assert np.isfinite(want).all()
    w, xd, od = DevArray(raw), DevArray(x), DevArray(nbytes=4 * tokens * out_dim)
    quant.gemv_dev(w.ptr, type_id, xd.ptr, od.ptr, in_dim, out_dim, tokens)
    got = od.read(np.float32, tokens * out_dim)
    assert quant.gemv_passes(type_id, tokens, in_dim, out_dim) == 1
    assert np.isfinite(got).all()
    g, w_ = got.reshape(tokens, out_dim).astype(np.float64), want.reshape(tokens, out_dim)
    for m in range(tokens):
        assert np.max(np.abs(g[m] - w_[m])) <= 2e-5 * float(np.max(np.abs(w_[m]))), m
    for a in (w, xd, od):
        a.close()


def test_one_pass_element_order_and_scale_positions(gpu, oracle):
    """A matrix whose codes, scales and mins each appear in exactly one place at a time: a swapped sub-block, nibble half,
    k-group or scale byte puts the unit activation's weight in the wrong output."""
    in_dim, out_dim, tokens = 2048, 16, 8
    rng = np.random.default_rng(5)
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    w = DevArray(raw)
    od = DevArray(nbytes=4 * tokens * out_dim)
    dense = oracle.dequantize(raw, Q4_K, out_dim * in_dim).reshape(out_dim, in_dim)
    for base in (0, 31, 32, 255, 256 + 64 + 9, 1024 + 200, 2047):
        x = np.zeros((tokens, in_dim), dtype=np.float32)
        for m in range(tokens):                     # token m picks out column base + 37 m (mod in_dim)
            x[m, (base + 37 * m) % in_dim] = 1.0
        xd = DevArray(np.ascontiguousarray(x.reshape(-1)))
        quant.gemv_dev(w.ptr, Q4_K, xd.ptr, od.ptr, in_dim, out_dim, tokens)
        got = od.read(np.float32, tokens * out_dim).reshape(tokens, out_dim)
        for m in range(tokens):
            col = dense[:, (base + 37 * m) % in_dim]
            assert np.allclose(got[m], col, rtol=0, atol=2e-6 * float(np.abs(dense).max())), (base, m)
        xd.close()
    for a in (w, od):
        a.close()


def test_token_counts_above_eight_and_other_shapes_fall_back(gpu, oracle):
    """9 and 13 tokens: a group of eight in one pass, the rest as the token count decides (one token on the vector ALU,
    five in one pass); in_dim above 12288 has no one-pass kernel and keeps its older path (four tokens per pass)."""
    rng = np.random.default_rng(11)
    for in_dim, out_dim, tokens in ((4096, 272, 9), (2048, 100, 13), (14336, 64, 8)):
        raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
        x = synth.make_activations(rng, tokens, in_dim)
        want, tol = oracle_rows(oracle, raw, x, in_dim, out_dim, tokens)
        w, xd, od = DevArray(raw), DevArray(x), DevArray(nbytes=4 * tokens * out_dim)
        quant.gemv_dev(w.ptr, Q4_K, xd.ptr, od.ptr, in_dim, out_dim, tokens)
        assert_bars(od.read(np.float32, tokens * out_dim), want, tol, tokens, out_dim, "%dx%d M=%d" % (in_dim, out_dim, tokens))
        for a in (w, xd, od):
            a.close()
    assert quant.gemv_image_bytes(Q4_K, 1000, 8) == 0 and quant.gemv_image_bytes(Q5_K, 4096, 8) == 16 * (8192 + 1024)
    assert quant.gemv_image_bytes(Q4_K, 14336, 8) == 0 and quant.gemv_image_bytes(Q6_K, 4096, 8) == 16 * (8192 + 1024)
    assert quant.gemv_image_bytes(Q4_K, 4096, 1) == 0 and quant.gemv_image_bytes(Q4_K, 4096, 9) == 0
    big = DevArray(nbytes=4 << 20)
    with pytest.raises(quant.QuantError, match="no one-pass kernel"):
        quant.gemv_pack_dev(big.ptr, Q4_K, 14336, 8, big.ptr)   # (real memory of sufficient size behind the pointers)
    big.close()


RAGGED_ROWS = [(Q4_K, 1024, 4096), (Q4_K, 256, 48), (Q4_K, 2560, 16 * 3 * 256 + 24), (Q4_K, 3584, 1040), (Q4_K, 5120, 5120),
               (Q4_K, 6912, 530), (Q4_K, 11008, 4096), (Q4_K, 1792, 37),
               (Q5_K, 1024, 1040), (Q5_K, 2560, 4096), (Q5_K, 5120, 530), (Q5_K, 11776, 50),
               (Q6_K, 1024, 4096), (Q6_K, 768, 37), (Q6_K, 2560, 16 * 2 * 256 + 24), (Q6_K, 3584, 3584), (Q6_K, 5120, 1040),
               (Q6_K, 9472, 530), (Q6_K, 11008, 16 * 257),
               (Q8_0, 1024, 3584), (Q8_0, 3584, 1024), (Q8_0, 256, 37), (Q8_0, 2048, 16 * 2 * 256 + 24), (Q8_0, 4096, 1040),
               (Q8_0, 5120, 530), (Q8_0, 12288, 50), (Q8_0, 7936, 16 * 257), (Q8_0, 2560, 16 * 600)]


@pytest.mark.parametrize("type_id,in_dim,out_dim", RAGGED_ROWS)
@pytest.mark.parametrize("tokens", [5, 8])
def test_rows_that_do_not_fill_their_k_slices(gpu, oracle, type_id, in_dim, out_dim, tokens):
    """(Q8_0 as well, at full and at ragged row lengths: eight of its 34-byte blocks stand for a super-block, the codes of
    every second block sit 2 bytes off a dword in LDS.) in_dim any multiple of 256: the eight k-slices take ceil(super-blocks / 8) each, the image is filled up with zero
    super-blocks and a k-slice without a super-block of its own re-reads the row's last block against those zeros. Rows of
    1 (only one wavefront has real work), 3, 4, 7, 10, 14, 20, 27, 37, 43 and 46 super-blocks: resident and streamed
    operands, one to three tiles per wavefront, partial tiles; with and without residual; the explicit image as well."""
    print("case type=%d in_dim=%d out_dim=%d tokens=%d" % (type_id, in_dim, out_dim, tokens), flush=True)
    nsbp = -(-(in_dim // 256) // 8) * 8
    assert quant.gemv_image_bytes(type_id, in_dim, tokens) == nsbp * (8192 + 1024)
    assert quant.gemv_passes(type_id, tokens, in_dim, out_dim) == 1
    rng = np.random.default_rng(type_id * 1000003 + in_dim * 13 + out_dim * 7 + tokens)
    raw = synth.make_weights(rng, type_id, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    res = rng.standard_normal(tokens * out_dim).astype(np.float32)
    want, tol = oracle_rows(oracle, raw, x, in_dim, out_dim, tokens, type_id)
    w, xd, od, rd = DevArray(raw), DevArray(x), DevArray(nbytes=4 * tokens * out_dim), DevArray(res)
    quant.gemv_dev(w.ptr, type_id, xd.ptr, od.ptr, in_dim, out_dim, tokens)
    plain = od.read(np.float32, tokens * out_dim)
    assert_bars(plain, want, tol, tokens, out_dim, "type %d %dx%d M=%d" % (type_id, in_dim, out_dim, tokens))
    quant.gemv_dev(w.ptr, type_id, xd.ptr, od.ptr, in_dim, out_dim, tokens, rd.ptr)
    assert np.array_equal(od.read(np.float32, tokens * out_dim), plain + res)
    # the same through a caller-owned image that held other data before (the zero super-blocks are written by the pack)
    image = DevArray(np.full(quant.gemv_image_bytes(type_id, in_dim, tokens), 0x7B, dtype=np.uint8))
    quant.gemv_pack_dev(xd.ptr, type_id, in_dim, tokens, image.ptr)
    quant.gemv_packed_dev([w.ptr], type_id, image.ptr, [od.ptr], [out_dim], in_dim, tokens)
    assert np.array_equal(od.read(np.float32, tokens * out_dim), plain)
    for a in (w, xd, od, rd, image):
        a.close()


LONG_AND_Q6K = [(Q4_K, 12288, 4096), (Q4_K, 6144, 530), (Q4_K, 8192, 16 * 300 + 5), (Q4_K, 10240, 33),
                (Q5_K, 4096, 8192), (Q5_K, 2048, 1040), (Q5_K, 4096, 16 * 3 * 256 * 2 + 24), (Q5_K, 2048, 37), (Q5_K, 4096, 16 * 600),
                (Q5_K, 12288, 530), (Q5_K, 6144, 16 * 257), (Q5_K, 10240, 50),
                (Q6_K, 12288, 4096), (Q6_K, 4096, 4096), (Q6_K, 2048, 1040), (Q6_K, 4096, 16 * 2 * 256 * 2 + 24), (Q6_K, 6144, 50),
                (Q6_K, 8192, 16 * 257), (Q6_K, 2048, 37),
                (Q8_0, 4096, 4096), (Q8_0, 2048, 1040), (Q8_0, 4096, 16 * 2 * 256 * 2 + 24), (Q8_0, 6144, 50), (Q8_0, 8192, 16 * 257),
                (Q8_0, 10240, 530), (Q8_0, 12288, 4096)]


@pytest.mark.parametrize("type_id,in_dim,out_dim", LONG_AND_Q6K)
@pytest.mark.parametrize("tokens", [5, 8])
def test_long_rows_and_q6_k_in_one_pass(gpu, oracle, type_id, in_dim, out_dim, tokens):
    """Rows of 6144..12288 values (three to six super-blocks per k-slice: the activation operands are streamed through two
    register sets, Q6_K with four LDS slots for six units) and Q5_K and Q6_K at every row length: one, two and three tiles per
    wavefront, partial tiles, more row groups than workgroups, odd Q6_K super-blocks (blocks that start 2 bytes off a 4-byte
    boundary)."""
    print("case type=%d in_dim=%d out_dim=%d tokens=%d" % (type_id, in_dim, out_dim, tokens), flush=True)
    assert quant.gemv_image_bytes(type_id, in_dim, tokens) == (in_dim // 256) * (8192 + 1024)
    rng = np.random.default_rng(type_id * 1000003 + in_dim * 13 + out_dim * 7 + tokens)
    raw = synth.make_weights(rng, type_id, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    res = rng.standard_normal(tokens * out_dim).astype(np.float32)
    want, tol = oracle_rows(oracle, raw, x, in_dim, out_dim, tokens, type_id)
    w, xd, od, rd = DevArray(raw), DevArray(x), DevArray(nbytes=4 * tokens * out_dim), DevArray(res)
    quant.gemv_dev(w.ptr, type_id, xd.ptr, od.ptr, in_dim, out_dim, tokens)
    plain = od.read(np.float32, tokens * out_dim)
    assert_bars(plain, want, tol, tokens, out_dim, "type %d %dx%d M=%d" % (type_id, in_dim, out_dim, tokens))
    quant.gemv_dev(w.ptr, type_id, xd.ptr, od.ptr, in_dim, out_dim, tokens, rd.ptr)
    assert np.array_equal(od.read(np.float32, tokens * out_dim), plain + res)
    for a in (w, xd, od, rd):
        a.close()


def test_q5_k_one_pass_element_order_and_fifth_bits(gpu, oracle):
    """Unit activations pick single weights out of a Q5_K matrix: every element position of a super-block, so every bit of
    every qh byte meets its nibble (a fifth bit taken from the neighbouring sub-block or byte shifts a weight by 16 codes)."""
    in_dim, out_dim, tokens = 2048, 16, 8
    rng = np.random.default_rng(55)
    raw = synth.make_weights(rng, Q5_K, out_dim, in_dim)
    w = DevArray(raw)
    od = DevArray(nbytes=4 * tokens * out_dim)
    dense = oracle.dequantize(raw, Q5_K, out_dim * in_dim).reshape(out_dim, in_dim)
    for base in list(range(0, 256, 8)) + [256 + 64 + 9, 1024 + 200, 2040]:
        x = np.zeros((tokens, in_dim), dtype=np.float32)
        for m in range(tokens):                     # token m picks out column base + m
            x[m, base + m] = 1.0
        xd = DevArray(np.ascontiguousarray(x.reshape(-1)))
        quant.gemv_dev(w.ptr, Q5_K, xd.ptr, od.ptr, in_dim, out_dim, tokens)
        got = od.read(np.float32, tokens * out_dim).reshape(tokens, out_dim)
        for m in range(tokens):
            assert np.allclose(got[m], dense[:, base + m], rtol=0, atol=2e-6 * float(np.abs(dense).max())), (base, m)
        xd.close()
    for a in (w, od):
        a.close()


def test_q5_k_and_q4_k_read_one_image(gpu, oracle):
    """Q5_K takes the Q4_K activation image: one pack serves a Q4_K and a Q5_K matrix of the same input."""
    in_dim, tokens, d4, d5 = 4096, 7, 272, 1040
    rng = np.random.default_rng(45)
    raw4, raw5 = synth.make_weights(rng, Q4_K, d4, in_dim), synth.make_weights(rng, Q5_K, d5, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    w4, w5, xd = DevArray(raw4), DevArray(raw5), DevArray(x)
    assert quant.gemv_image_bytes(Q5_K, in_dim, tokens) == quant.gemv_image_bytes(Q4_K, in_dim, tokens)
    image = DevArray(nbytes=quant.gemv_image_bytes(Q4_K, in_dim, tokens))
    o4, o5 = DevArray(nbytes=4 * tokens * d4), DevArray(nbytes=4 * tokens * d5)
    quant.gemv_pack_dev(xd.ptr, Q4_K, in_dim, tokens, image.ptr)
    quant.gemv_packed_dev([w4.ptr], Q4_K, image.ptr, [o4.ptr], [d4], in_dim, tokens)
    quant.gemv_packed_dev([w5.ptr], Q5_K, image.ptr, [o5.ptr], [d5], in_dim, tokens)
    for raw, o, d, t in ((raw4, o4, d4, Q4_K), (raw5, o5, d5, Q5_K)):
        want, tol = oracle_rows(oracle, raw, x, in_dim, d, tokens, t)
        assert_bars(o.read(np.float32, tokens * d), want, tol, tokens, d, "type %d against the shared image" % t)
    for a in (w4, w5, xd, image, o4, o5):
        a.close()


def test_q6_k_one_pass_element_order_and_scale_positions(gpu, oracle):
    """Unit activations pick single weights out of a Q6_K matrix: a swapped quarter, half, nibble, high-bit pair, k-group or
    scale byte puts another weight there. Every element position of a super-block is visited, in an even and an odd block."""
    in_dim, out_dim, tokens = 2048, 16, 8
    rng = np.random.default_rng(6)
    raw = synth.make_weights(rng, Q6_K, out_dim, in_dim)
    w = DevArray(raw)
    od = DevArray(nbytes=4 * tokens * out_dim)
    dense = oracle.dequantize(raw, Q6_K, out_dim * in_dim).reshape(out_dim, in_dim)
    for base in range(0, 512, 8):
        x = np.zeros((tokens, in_dim), dtype=np.float32)
        for m in range(tokens):                     # token m picks out column base + m
            x[m, base + m] = 1.0
        xd = DevArray(np.ascontiguousarray(x.reshape(-1)))
        quant.gemv_dev(w.ptr, Q6_K, xd.ptr, od.ptr, in_dim, out_dim, tokens)
        got = od.read(np.float32, tokens * out_dim).reshape(tokens, out_dim)
        for m in range(tokens):
            assert np.allclose(got[m], dense[:, base + m], rtol=0, atol=2e-6 * float(np.abs(dense).max())), (base, m)
        xd.close()
    for a in (w, od):
        a.close()


@pytest.mark.parametrize("type_id,in_dim,dims,tokens", [(Q6_K, 4096, (1024, 272), 6), (Q5_K, 4096, (8192, 1024, 40), 2),
                                                        (Q5_K, 6144, (272, 16, 1040, 33), 8)])
def test_q5_k_and_q6_k_lists_share_one_image(gpu, oracle, type_id, in_dim, dims, tokens):
    """Q5_K and Q6_K matrices against one activation block through the list operator (one pack, up to three matrices per
    launch, from two tokens)."""
    rng = np.random.default_rng(66 + type_id)
    raws = [synth.make_weights(rng, type_id, d, in_dim) for d in dims]
    x = synth.make_activations(rng, tokens, in_dim)
    ws, xd = [DevArray(r) for r in raws], DevArray(x)
    outs = [DevArray(nbytes=4 * tokens * d) for d in dims]
    quant.gemv_many_dev([w_.ptr for w_ in ws], type_id, xd.ptr, [o.ptr for o in outs], list(dims), in_dim, tokens)
    for raw, o, d in zip(raws, outs, dims):
        want, tol = oracle_rows(oracle, raw, x, in_dim, d, tokens, type_id)
        assert_bars(o.read(np.float32, tokens * d), want, tol, tokens, d, "type %d list member %d" % (type_id, d))
    for a in ws + outs + [xd]:
        a.close()


@pytest.mark.parametrize("tokens", [1, 2, 4, 8])
def test_non_finite_activation_stays_in_its_token(gpu, oracle, tokens):
    """An infinite activation: the reference's sum for that token is +-Inf (or NaN where weights of both signs meet it).
    Every kernel must give non-finite values for that token's rows that use the element, and must leave the other tokens of
    the call within the bar (one token: vector ALU; two and four: matrix-core kernels; eight: one pass)."""
    rng = np.random.default_rng(700 + tokens)
    in_dim, out_dim = 4096, 64
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim).reshape(tokens, in_dim)
    bad = tokens - 1
    x[bad, 777] = np.float32(np.inf)
    x = np.ascontiguousarray(x.reshape(-1))
    w, xd, od = DevArray(raw), DevArray(x), DevArray(nbytes=4 * tokens * out_dim)
    quant.gemv_dev(w.ptr, Q4_K, xd.ptr, od.ptr, in_dim, out_dim, tokens)
    got = od.read(np.float32, tokens * out_dim).reshape(tokens, out_dim)
    with np.errstate(all="ignore"):
        ref = oracle.matmul_add(x, tokens, in_dim, raw, Q4_K, out_dim, np.zeros(out_dim, dtype=np.float32), threads=8).reshape(tokens, out_dim)
    assert not np.isfinite(ref[bad]).any() and not np.isfinite(got[bad]).any()
    if tokens > 1:
        good = [m for m in range(tokens) if m != bad]
        xs = np.ascontiguousarray(x.reshape(tokens, in_dim)[good].reshape(-1))
        want, tol = oracle_rows(oracle, raw, xs, in_dim, out_dim, len(good))
        assert np.all(np.abs(got[good].reshape(-1) - want) <= tol)
    for a in (w, xd, od):
        a.close()


def test_image_slots_return_when_streams_close(gpu, oracle):
    """The library keeps one activation image per stream, eight at most. A stream that is closed gives its image back, so
    the twelfth stream of a process still runs the one-pass kernel: its result is bit for bit that of the explicit
    pack + packed GEMV, which the per-token-group kernels' is not."""
    rng = np.random.default_rng(12)
    in_dim, out_dim, tokens = 4096, 256, 8
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    w, xd, od, o2 = DevArray(raw), DevArray(x), DevArray(nbytes=4 * tokens * out_dim), DevArray(nbytes=4 * tokens * out_dim)
    image = DevArray(nbytes=quant.gemv_image_bytes(Q4_K, in_dim, tokens))
    quant.gemv_pack_dev(xd.ptr, Q4_K, in_dim, tokens, image.ptr)
    quant.gemv_packed_dev([w.ptr], Q4_K, image.ptr, [o2.ptr], [out_dim], in_dim, tokens)
    explicit = o2.read(np.float32, tokens * out_dim)
    for i in range(12):
        st = hip.HIPStream()
        quant.gemv_dev(w.ptr, Q4_K, xd.ptr, od.ptr, in_dim, out_dim, tokens, 0, st.handle)
        st.synchronize()
        assert np.array_equal(od.read(np.float32, tokens * out_dim), explicit), i
        st.close()
    for a in (w, xd, od, o2, image):
        a.close()


def test_a_ninth_stream_is_counted_and_a_captured_image_stays_pinned(gpu, oracle):
    """Eight streams hold the eight images; a ninth stream's call runs the per-token-group kernels (within the bar, not
    the one-pass bits) and is counted. An image handed out under stream capture is pinned: closing the capture stream does
    not give it back, so a replay of the graph never shares it with another stream."""
    rng = np.random.default_rng(99)
    in_dim, out_dim, tokens = 4096, 256, 8
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    w, xd = DevArray(raw), DevArray(x)
    outs = [DevArray(nbytes=4 * tokens * out_dim) for _ in range(10)]
    want, tol = oracle_rows(oracle, raw, x, in_dim, out_dim, tokens)
    slots, used0, pinned0, missed0 = quant.gemv_image_stats()
    assert slots == 8
    streams = [hip.HIPStream() for _ in range(9)]
    try:
        held = []
        for i, st in enumerate(streams):
            before = quant.gemv_image_stats()
            quant.gemv_dev(w.ptr, Q4_K, xd.ptr, outs[i].ptr, in_dim, out_dim, tokens, 0, st.handle)
            st.synchronize()
            after = quant.gemv_image_stats()
            held.append(after[1] > before[1])
            assert_bars(outs[i].read(np.float32, tokens * out_dim), want, tol, tokens, out_dim, "stream %d" % i)
        free_at_start = slots - used0
        assert sum(held) == min(free_at_start, 9)
        assert quant.gemv_image_stats()[3] - missed0 == 9 - sum(held) >= 1
    finally:
        for st in streams:
            st.close()
    assert quant.gemv_image_stats()[1] == used0
    # capture on a fresh stream, close it, then make other streams take every free slot: the replay still gives the
    # one-pass bits
    cap = hip.HIPStream()
    cap.begin_capture(1)
    quant.gemv_dev(w.ptr, Q4_K, xd.ptr, outs[9].ptr, in_dim, out_dim, tokens, 0, cap.handle)
    graph = cap.end_capture()
    ex = graph.instantiate()
    assert quant.gemv_image_stats()[2] == pinned0 + 1
    cap.close()
    assert quant.gemv_image_stats()[2] == pinned0 + 1 and quant.gemv_image_stats()[1] == used0 + 1
    others = [hip.HIPStream() for _ in range(8)]
    run = hip.HIPStream()
    try:
        for i, st in enumerate(others):
            quant.gemv_dev(w.ptr, Q4_K, xd.ptr, outs[i].ptr, in_dim, out_dim, tokens, 0, st.handle)
        for rep in range(3):
            ex.launch(run)
            for st in others[:3]:   # eager work on the other streams between the replays
                quant.gemv_dev(w.ptr, Q4_K, xd.ptr, outs[0].ptr, in_dim, out_dim, tokens, 0, st.handle)
            run.synchronize()
            assert_bars(outs[9].read(np.float32, tokens * out_dim), want, tol, tokens, out_dim, "replay %d" % rep)
    finally:
        for st in others + [run]:
            st.synchronize()
            st.close()
        ex.close()
        graph.close()
    for a in [w, xd] + outs:
        a.close()


@pytest.mark.parametrize("t", [Q4_K, Q5_K, Q6_K, Q8_0])
@pytest.mark.parametrize("in_dim,dims,tokens", [(4096, [12288], 16), (4096, [4096, 1024, 1024], 9), (2048, [130], 12), (12288, [4096], 16),
                                                (1024, [48, 1000], 11), (5120, [257], 13), (256, [16], 1), (4096, [16 * 700], 10),
                                                (2048, [32, 64, 7, 4000], 15)])
def test_nine_to_sixteen_tokens_in_one_pass(gpu, oracle, t, in_dim, dims, tokens):
    """cogni_gemv_pack16_dev + cogni_gemv_packed16_dev: the one-pass kernels with sixteen single-term tokens. The activations
    are rounded to binary16 (the prefill GEMM's precision class) and everything behind that is exact codes and fp32 sums, so
    the result is held to the one-pass bars against the CPU form of the rounded activations (2e-5 of a token's largest output);
    resident and streamed operands, rows that do not fill their k-slices, lists, row counts that are no multiple of 16,
    workgroups that walk row groups, a single token."""
    rng = np.random.default_rng(in_dim + 31 * tokens + sum(dims) + int(t))
    raws = [synth.make_weights(rng, t, d, in_dim) for d in dims]
    x = synth.make_activations(rng, tokens, in_dim)
    x16 = x.astype(np.float16).astype(np.float32)
    image = DevArray(np.full(quant.gemv_image_bytes(t, in_dim, 8), 0xFF, dtype=np.uint8))
    xd, wd = DevArray(x), [DevArray(r) for r in raws]
    outs = [DevArray(np.full(tokens * d, np.float32(-9.0))) for d in dims]
    quant.gemv_pack16_dev(xd.ptr, t, in_dim, tokens, image.ptr)
    quant.gemv_packed16_dev([w.ptr for w in wd], t, image.ptr, [o.ptr for o in outs], dims, in_dim, tokens)
    for raw, o, d in zip(raws, outs, dims):
        want, tol = oracle_rows(oracle, raw, x16, in_dim, d, tokens, t)
        assert_bars(o.read(np.float32, tokens * d), want, tol, tokens, d, "type %d in=%d M=%d rows=%d" % (t, in_dim, tokens, d))
    with pytest.raises(quant.QuantError, match="1..16 tokens"):
        quant.gemv_pack16_dev(xd.ptr, t, in_dim, 17, image.ptr)
    with pytest.raises(quant.QuantError, match="Q4_K, Q5_K, Q6_K or Q8_0"):
        quant.gemv_packed16_dev([w.ptr for w in wd], 2, image.ptr, [o.ptr for o in outs], dims, in_dim, tokens)
    # a residual with a single matrix
    res = rng.standard_normal(tokens * dims[0]).astype(np.float32)
    rd, o2 = DevArray(res), DevArray(nbytes=4 * tokens * dims[0])
    quant.gemv_packed16_dev([wd[0].ptr], t, image.ptr, [o2.ptr], [dims[0]], in_dim, tokens, rd.ptr)
    assert np.array_equal(o2.read(np.float32, tokens * dims[0]), outs[0].read(np.float32, tokens * dims[0]) + res)
    if len(dims) > 1:
        with pytest.raises(quant.QuantError, match="a residual goes with a single matrix"):
            quant.gemv_packed16_dev([w.ptr for w in wd], t, image.ptr, [o.ptr for o in outs], dims, in_dim, tokens, rd.ptr)
    rd.close()
    o2.close()
    for a in [image, xd] + wd + outs:
        a.close()


def test_router_sends_nine_to_sixteen_tokens_to_the_one_pass_kernels(gpu):
    """cogni_matmul_dev between the GEMM threshold and sixteen tokens without a bias: the bits of cogni_gemv_pack16_dev +
    cogni_gemv_packed16_dev (Q4_K; Q6_K the same path); with a bias or with seventeen tokens it stays on the GEMM."""
    rng = np.random.default_rng(77)
    in_dim, out_dim = 2048, 520
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    raw6 = synth.make_weights(rng, Q6_K, out_dim, in_dim)
    bias = rng.standard_normal(out_dim).astype(np.float32)
    w, w6, bd = DevArray(raw), DevArray(raw6), DevArray(bias)
    for tokens in (9, 16, 17):
        x = synth.make_activations(rng, tokens, in_dim)
        xd = DevArray(x)
        wsb = quant.gemm_workspace_bytes(Q4_K, in_dim, tokens, out_dim)
        ws, img = DevArray(nbytes=wsb), DevArray(nbytes=quant.gemv_image_bytes(Q4_K, in_dim, 8))
        routed, direct, gemm, biased = (DevArray(nbytes=4 * tokens * out_dim) for _ in range(4))
        quant.matmul_dev(w.ptr, Q4_K, xd.ptr, routed.ptr, in_dim, out_dim, tokens, ws.ptr, wsb)
        quant.gemm_dev(w.ptr, Q4_K, xd.ptr, gemm.ptr, in_dim, out_dim, tokens, ws.ptr, wsb)
        r, g = routed.read(np.float32, tokens * out_dim), gemm.read(np.float32, tokens * out_dim)
        if tokens <= 16:
            quant.gemv_pack16_dev(xd.ptr, Q4_K, in_dim, tokens, img.ptr)
            quant.gemv_packed16_dev([w.ptr], Q4_K, img.ptr, [direct.ptr], [out_dim], in_dim, tokens)
            assert np.array_equal(r, direct.read(np.float32, tokens * out_dim))
            assert not np.array_equal(r, g) and np.max(np.abs(r - g)) <= 2e-3 * np.max(np.abs(g))
            quant.matmul_dev(w.ptr, Q4_K, xd.ptr, biased.ptr, in_dim, out_dim, tokens, ws.ptr, wsb, bd.ptr)
            want = (g.reshape(tokens, out_dim) + bias).reshape(-1)
            assert np.max(np.abs(biased.read(np.float32, tokens * out_dim) - want)) <= 1e-5 * np.max(np.abs(want))
        else:
            assert np.array_equal(r, g)
        quant.matmul_dev(w6.ptr, Q6_K, xd.ptr, routed.ptr, in_dim, out_dim, tokens, ws.ptr, wsb)
        quant.gemm_dev(w6.ptr, Q6_K, xd.ptr, gemm.ptr, in_dim, out_dim, tokens, ws.ptr, wsb)
        r6, g6 = routed.read(np.float32, tokens * out_dim), gemm.read(np.float32, tokens * out_dim)
        assert (not np.array_equal(r6, g6) and np.max(np.abs(r6 - g6)) <= 2e-3 * np.max(np.abs(g6))) if tokens <= 16 else np.array_equal(r6, g6)
        for a in (xd, ws, img, routed, direct, gemm, biased):
            a.close()
    for a in (w, w6, bd):
        a.close()


@pytest.mark.parametrize("in_dim,out_dim,tokens", [(4096, 12288, 16), (2048, 130, 9), (12288, 48, 12), (1024, 1000, 11), (6144, 40, 10)])
def test_swiglu_for_nine_to_sixteen_tokens(gpu, in_dim, out_dim, tokens):
    """cogni_gemv_packed16_swiglu_dev: gate | up | SwiGLU against a sixteen-token image - the bits of cogni_gemv_packed16_dev on
    the pair followed by cogni_swiglu_dev (resident and streamed operands, row counts that are no multiple of 16)."""
    rng = np.random.default_rng(in_dim + out_dim + tokens)
    raw_g, raw_u = synth.make_weights(rng, Q4_K, out_dim, in_dim), synth.make_weights(rng, Q4_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    n = tokens * out_dim
    wg, wu, xd = DevArray(raw_g), DevArray(raw_u), DevArray(x)
    image = DevArray(nbytes=quant.gemv_image_bytes(Q4_K, in_dim, 8))
    g, u, two_step, fused = DevArray(nbytes=4 * n), DevArray(nbytes=4 * n), DevArray(nbytes=4 * n), DevArray(np.full(n, np.float32(5.0)))
    quant.gemv_pack16_dev(xd.ptr, Q4_K, in_dim, tokens, image.ptr)
    quant.gemv_packed16_dev([wg.ptr, wu.ptr], Q4_K, image.ptr, [g.ptr, u.ptr], [out_dim, out_dim], in_dim, tokens)
    quant.swiglu_dev(g.ptr, u.ptr, two_step.ptr, n)
    quant.gemv_packed16_swiglu_dev(wg.ptr, wu.ptr, Q4_K, image.ptr, fused.ptr, in_dim, out_dim, tokens)
    assert np.array_equal(fused.read(np.float32, n), two_step.read(np.float32, n))
    with pytest.raises(quant.QuantError, match="Q4_K, 1..16 tokens"):
        quant.gemv_packed16_swiglu_dev(wg.ptr, wu.ptr, Q5_K, image.ptr, fused.ptr, in_dim, out_dim, tokens)
    for a in (wg, wu, xd, image, g, u, two_step, fused):
        a.close()
