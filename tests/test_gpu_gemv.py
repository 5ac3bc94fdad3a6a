"""GPU decode GEMV (M = 1..8, optional residual) vs the CPU oracle.

Tolerance (fp32 path): max|err| <= 1e-4 * ||x||_2 * max|w_row| per token and output row. The
reference's own probe gate (cos >= 0.99999 and max_diff <= 1e-3, bin/cuda_q4k_gemv_probe.cr:289)
is asserted as well where the output scale makes it meaningful.
"""
import numpy as np
import pytest

from cogni_ml_amd import quant, synth
from gpu_common import DevArray, gpu  # noqa: F401
from helpers import BLOCK, Q4_K, Q5_K, Q6_K, Q8_0, cosine, gemv_tolerance

pytestmark = pytest.mark.gpu
TYPES = [Q8_0, Q4_K, Q5_K, Q6_K]


def run_gemv(raw, type_id, x, in_dim, out_dim, tokens, residual=None):
    w, xd, od = DevArray(raw), DevArray(x), DevArray(nbytes=4 * tokens * out_dim)
    rd = DevArray(residual) if residual is not None else None
    quant.gemv_dev(w.ptr, type_id, xd.ptr, od.ptr, in_dim, out_dim, tokens, rd.ptr if rd else 0)
    out = od.read(np.float32, tokens * out_dim)
    for a in (w, xd, od, rd):
        if a:
            a.close()
    return out


def check(oracle, raw, type_id, x, in_dim, out_dim, tokens, residual=None, what=""):
    got = run_gemv(raw, type_id, x, in_dim, out_dim, tokens, residual)
    zero = np.zeros(out_dim, dtype=np.float32)
    want = oracle.matmul_add(x, tokens, in_dim, raw, type_id, out_dim, zero, threads=8).astype(np.float64)
    if residual is not None:
        want = (want.astype(np.float32) + residual).astype(np.float64)
    dense = np.abs(oracle.dequantize(raw, type_id, out_dim * (raw.size // out_dim // BLOCK[type_id][0]) * BLOCK[type_id][1])
                   ).reshape(out_dim, -1)
    tol = gemv_tolerance(x, dense, tokens, in_dim).reshape(-1)
    err = np.abs(got.astype(np.float64) - want)
    worst = int(np.argmax(err / np.maximum(tol, 1e-30)))
    assert np.all(err <= tol), "%s: err %.3e > tol %.3e at %d" % (what, err[worst], tol[worst], worst)
    # the bound above is loose for these kernels (they sit at a fraction of a per cent of it): every path also stays
    # within 2e-5 of each token's output scale (fp32 sums of exact weights; the kernels that feed the activations as two
    # binary16 terms carry 22 bits), so that a kernel a hundred times less accurate fails here
    e2, w2 = err.reshape(tokens, out_dim), np.abs(want).reshape(tokens, out_dim)
    for m in range(tokens):
        scale = float(w2[m].max())
        assert float(e2[m].max()) <= 2e-5 * scale + 1e-30, "%s: token %d err %.3e > 2e-5 * %.3e" % (what, m, e2[m].max(), scale)
    return got, want, float(np.max(err / np.maximum(tol, 1e-30)))


@pytest.mark.parametrize("type_id", TYPES)
@pytest.mark.parametrize("tokens", [1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("add", [False, True])
def test_small_shapes_all_token_counts(gpu, oracle, type_id, tokens, add):
    rng = np.random.default_rng(1000 * type_id + 10 * tokens + add)
    be = BLOCK[type_id][1]
    out_dim = 37                                  # not a multiple of the 16 rows a workgroup covers
    in_dim = be * 9 if be == 256 else 1024 + 96   # K-quants: 9 blocks = one full + one partial column set
    raw = synth.make_weights(rng, type_id, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    res = rng.standard_normal(tokens * out_dim).astype(np.float32) if add else None
    check(oracle, raw, type_id, x, in_dim, out_dim, tokens, res, "type %d M=%d add=%s" % (type_id, tokens, add))


@pytest.mark.parametrize("type_id,in_dim,short_rows", [(Q4_K, 4096, 1024), (Q4_K, 1024, 37), (Q5_K, 4096, 2040), (Q6_K, 4096, 1024),
                                                        (Q6_K, 12288, 130), (Q4_K, 12288, 64), (Q5_K, 8192, 300), (Q4_K, 26624, 33), (Q8_0, 1024, 3584), (Q8_0, 3584, 1024), (Q8_0, 1000, 2041),
                                                        (Q8_0, 4096, 5)])
@pytest.mark.parametrize("add", [False, True])
def test_one_token_of_a_short_matrix(gpu, oracle, type_id, in_dim, short_rows, add):
    """Matrices of few rows run the one-token kernel's variant with fewer rows per wavefront (one; Q8_0 two from 2041 rows):
    within the bars against the oracle, and - a row's arithmetic does not depend on how many rows its wavefront carries -
    bit for bit the values the plain kernel gives the same rows as the head of a matrix tall enough to be taken by it."""
    name = quant.gemv_plan(type_id, 1, in_dim, short_rows, add=add)[0]
    assert name.endswith("_r1") or name.endswith("_r2"), name
    tall_rows = 4096 + 16
    assert "_r" not in quant.gemv_plan(type_id, 1, in_dim, tall_rows)[0].rsplit("f32", 1)[1]
    rng = np.random.default_rng(type_id * 7919 + in_dim + short_rows)
    raw_tall = synth.make_weights(rng, type_id, tall_rows, in_dim)
    row_bytes = raw_tall.size // tall_rows
    raw_short = np.ascontiguousarray(raw_tall[:short_rows * row_bytes])
    x = synth.make_activations(rng, 1, in_dim)
    res_tall = rng.standard_normal(tall_rows).astype(np.float32) if add else None
    res_short = res_tall[:short_rows].copy() if add else None
    short = check(oracle, raw_short, type_id, x, in_dim, short_rows, 1, res_short, "%s %dx%d" % (name, short_rows, in_dim))[0]
    tall = run_gemv(raw_tall, type_id, x, in_dim, tall_rows, 1, res_tall)
    assert np.array_equal(short, tall[:short_rows])


@pytest.mark.parametrize("in_dim", [32, 80, 1000, 1024, 2048 + 32])
def test_q8_0_row_lengths_including_clipped_tail(gpu, oracle, in_dim):
    rng = np.random.default_rng(in_dim)
    raw = synth.make_weights(rng, Q8_0, 21, in_dim)
    x = synth.make_activations(rng, 2, in_dim)
    check(oracle, raw, Q8_0, x, in_dim, 21, 2, None, "Q8_0 in=%d" % in_dim)


@pytest.mark.parametrize("type_id", [Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("nb", [1, 7, 8, 16, 17, 33])
def test_k_quant_block_counts(gpu, oracle, type_id, nb):
    rng = np.random.default_rng(77 * type_id + nb)
    raw = synth.make_weights(rng, type_id, 16, 256 * nb)
    x = synth.make_activations(rng, 1, 256 * nb)
    check(oracle, raw, type_id, x, 256 * nb, 16, 1, None, "type %d nb=%d" % (type_id, nb))


def test_single_output_row_and_many_tokens(gpu, oracle):
    rng = np.random.default_rng(5)
    raw = synth.make_weights(rng, Q4_K, 1, 512)
    check(oracle, raw, Q4_K, synth.make_activations(rng, 1, 512), 512, 1, 1)
    raw = synth.make_weights(rng, Q6_K, 40, 512)
    res = rng.standard_normal(19 * 40).astype(np.float32)
    check(oracle, raw, Q6_K, synth.make_activations(rng, 19, 512), 512, 40, 19, res, "19 tokens in several launches")


CONFIGS = [
    ("cfg1 Q8_0 ffn_up 0.8B", Q8_0, 3584, 1024, [1]),
    ("cfg2 Q4_K gate/up", Q4_K, 12288, 4096, [1, 4, 8]),
    ("cfg2 Q4_K down", Q4_K, 4096, 12288, [1, 8]),
    ("cfg3 Q6_K down", Q6_K, 4096, 12288, [1, 4, 8]),
    ("cfg3 Q5_K", Q5_K, 4096, 4096, [1, 8]),
    ("cfg5 Q4_K k/v", Q4_K, 1024, 4096, [1, 8]),
]


@pytest.mark.parametrize("name,type_id,out_dim,in_dim,token_list", CONFIGS)
def test_configured_shapes(gpu, oracle, name, type_id, out_dim, in_dim, token_list):
    import zlib
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    raw = synth.make_weights(rng, type_id, out_dim, in_dim)
    for tokens in token_list:
        x = synth.make_activations(rng, tokens, in_dim)
        got, want, frac = check(oracle, raw, type_id, x, in_dim, out_dim, tokens, None, "%s M=%d" % (name, tokens))
        assert cosine(got, want) >= 0.99999
        assert np.max(np.abs(got - want)) <= 1e-3
        print("%s M=%d: max err / tolerance = %.4f" % (name, tokens, frac))


def test_q6_k_output_head_shape(gpu, oracle):
    """The 4096 -> 151936 Q6_K head (510 MB of weights): sampled rows against the oracle."""
    rng = np.random.default_rng(151936)
    out_dim, in_dim = 151936, 4096
    raw = synth.make_weights(rng, Q6_K, out_dim, in_dim)
    x = synth.make_activations(rng, 1, in_dim)
    got = run_gemv(raw, Q6_K, x, in_dim, out_dim, 1)
    rb = 16 * 210
    for lo in (0, 70000, out_dim - 4096):
        sub = raw[lo * rb:(lo + 4096) * rb]
        want = oracle.matmul_add(x, 1, in_dim, sub, Q6_K, 4096, np.zeros(4096, dtype=np.float32), threads=8)
        dense = np.abs(oracle.dequantize(sub, Q6_K, 4096 * in_dim)).reshape(4096, in_dim)
        tol = gemv_tolerance(x, dense, 1, in_dim).reshape(-1)
        assert np.all(np.abs(got[lo:lo + 4096].astype(np.float64) - want) <= tol)


def test_matmul_add_host_signature_with_bias(gpu, oracle):
    """QuantMatmul.matmul_add through the host-buffer entry point, with the reference spec's
    deterministic x and bias (spec/q4k_matmul_spec.cr:66-73)."""
    rng = np.random.default_rng(12)
    out_dim, in_dim, rows = 256, 1024, 2
    i = np.arange(rows * in_dim, dtype=np.uint64)
    x = (((i * 2654435761) % (1 << 32) % 2000).astype(np.int64) - 1000).astype(np.float32) / np.float32(1000.0)
    bias = ((np.arange(out_dim) % 10) / np.float32(100.0)).astype(np.float32)
    for t in TYPES:
        raw = synth.make_weights(rng, t, out_dim, in_dim)
        mine = quant.matmul_add(x, rows, in_dim, raw, t, out_dim, bias)
        ref = oracle.matmul_add(x, rows, in_dim, raw, t, out_dim, bias)
        assert cosine(mine, ref) >= 0.9999999
        assert np.max(np.abs(mine - ref)) / np.max(np.abs(ref)) <= 1e-5     # the reference's own gate
        qw = quant.QuantWeight(raw, t, out_dim, in_dim, "test")
        assert qw.device_ptr != 0
        assert np.array_equal(qw.matmul(x, rows, bias), mine)
        nobias = qw.matmul(x[:in_dim], 1)
        assert np.allclose(nobias, ref[:out_dim] - bias, rtol=0, atol=1e-4)
        qw.close()


def test_matvec_many_shares_one_activation_vector(gpu, oracle):
    """qmatvec_many (qwen35_cpu.cr:1419-1445): weights of different types and sizes against one x; each result equals the
    single-weight call bit for bit; no weights -> no results; a weight of another in_dim is refused."""
    rng = np.random.default_rng(1419)
    in_dim = 1024
    x = synth.make_activations(rng, 1, in_dim)
    shapes = [(Q4_K, 512), (Q4_K, 128), (Q6_K, 128), (Q5_K, 300), (Q8_0, 77)]
    qws = [quant.QuantWeight(synth.make_weights(rng, t, out_dim, in_dim), t, out_dim, in_dim) for t, out_dim in shapes]
    outs = quant.matvec_many(qws, x)
    assert [o.size for o in outs] == [out_dim for _, out_dim in shapes]
    for qw, o in zip(qws, outs):
        assert np.array_equal(o, qw.matmul(x, 1))
        ref = oracle.matmul_add(x, 1, in_dim, qw.raw, int(qw.type), qw.out_dim, np.zeros(qw.out_dim, dtype=np.float32))
        assert np.max(np.abs(o - ref)) <= 1e-5 * np.max(np.abs(ref))
    assert quant.matvec_many([], x) == []
    other = quant.QuantWeight(synth.make_weights(rng, Q4_K, 16, 512), Q4_K, 16, 512)
    with pytest.raises(quant.QuantError, match="in_dim"):
        quant.matvec_many([qws[0], other], x)
    for qw in qws + [other]:
        qw.close()


def test_linearity_and_determinism_at_full_size(gpu):
    """Size-independent properties at the headline shape: same input -> same bits; f(2a) == 2 f(a) exactly;
    f(a) + f(b) ~= f(a + b)."""
    rng = np.random.default_rng(99)
    out_dim, in_dim = 12288, 4096
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    a, b = synth.make_activations(rng, 1, in_dim), synth.make_activations(rng, 1, in_dim)
    fa = run_gemv(raw, Q4_K, a, in_dim, out_dim, 1)
    assert np.array_equal(fa, run_gemv(raw, Q4_K, a, in_dim, out_dim, 1))
    assert np.array_equal(run_gemv(raw, Q4_K, 2 * a, in_dim, out_dim, 1), 2 * fa)
    fb, fab = run_gemv(raw, Q4_K, b, in_dim, out_dim, 1), run_gemv(raw, Q4_K, a + b, in_dim, out_dim, 1)
    assert np.max(np.abs((fa + fb) - fab)) <= 1e-4 * np.max(np.abs(fab))
    # two tokens in one launch (the matrix-core kernel for this shape): reproducible, and the same values as
    # one launch per token up to the order of the fp32 additions
    both = run_gemv(raw, Q4_K, np.concatenate([a, b]), in_dim, out_dim, 2)
    assert np.array_equal(both, run_gemv(raw, Q4_K, np.concatenate([a, b]), in_dim, out_dim, 2))
    scale = np.max(np.abs(fab))
    assert np.max(np.abs(both[:out_dim] - fa)) <= 2e-5 * scale and np.max(np.abs(both[out_dim:] - fb)) <= 2e-5 * scale
    # a token's result does not depend on its neighbours in the launch
    swapped = run_gemv(raw, Q4_K, np.concatenate([b, a]), in_dim, out_dim, 2)
    assert np.array_equal(swapped[out_dim:], both[:out_dim]) and np.array_equal(swapped[:out_dim], both[out_dim:])


MFMA_SHAPES = [(256, 17), (512, 100), (768, 33), (1024, 3584), (2048, 48), (2304, 250), (4096, 1024), (8192, 300),
               (6144, 40), (12288, 530), (16384, 64), (26624, 33), (8448, 20), (2048, 20011), (512, 70003)]


@pytest.mark.parametrize("in_dim,out_dim", MFMA_SHAPES)
@pytest.mark.parametrize("tokens", [2, 3, 4, 7])
def test_q4_k_matrix_core_kernel_shapes(gpu, oracle, in_dim, out_dim, tokens):
    """2..4 tokens of a Q4_K matrix run on the matrix cores where the activations fit the staging buffer or the row is
    a multiple of 2048 values (staged a chunk at a time: whole chunks, a half-filled last chunk at 6144 and 26624, several
    row tiles per wavefront; 20011 x 2048 and 70003 x 512 have more row groups than the 256 workgroups launched, which
    walk them with the activations staged once): odd row counts, every k-slice split (1, 2, 3, 4, 8, 9, 16, 32 super-blocks), with and
    without residual. 8448 values (33 super-blocks) are neither: three and four tokens stay on the vector ALU."""
    rng = np.random.default_rng(in_dim * 131 + out_dim * 7 + tokens)
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    res = rng.standard_normal(tokens * out_dim).astype(np.float32)
    m = min(tokens, 4)
    name = quant.gemv_plan(Q4_K, m, in_dim, out_dim)[0]
    expect_mfma = m * (in_dim // 256) <= (64 if m >= 3 else 96) or in_dim % 2048 == 0
    assert ("mfma" in name) == expect_mfma, name
    check(oracle, raw, Q4_K, x, in_dim, out_dim, tokens, None, "%dx%d M=%d" % (in_dim, out_dim, tokens))
    check(oracle, raw, Q4_K, x, in_dim, out_dim, tokens, res, "%dx%d M=%d add" % (in_dim, out_dim, tokens))


@pytest.mark.parametrize("in_dim,out_dim", MFMA_SHAPES)
@pytest.mark.parametrize("tokens", [2, 3, 4, 7])
def test_q5_k_matrix_core_kernel_shapes(gpu, oracle, in_dim, out_dim, tokens):
    """Three and four tokens of a Q5_K matrix run through the Q4_K matrix-core kernel with the fifth bit or-ed in beside
    the nibble (two tokens stay on the vector ALU): the same shape rule, with and without residual."""
    rng = np.random.default_rng(in_dim * 139 + out_dim * 13 + tokens)
    raw = synth.make_weights(rng, Q5_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    res = rng.standard_normal(tokens * out_dim).astype(np.float32)
    m = min(tokens, 4)
    name = quant.gemv_plan(Q5_K, m, in_dim, out_dim)[0]
    expect_mfma = m >= 3 and (m * (in_dim // 256) <= 64 or in_dim % 2048 == 0)
    assert name == ("q5_k_gemv_mfma_f32_tbatch%d" % m if expect_mfma else "q5_k_gemv_f32_tbatch%d" % m), name
    check(oracle, raw, Q5_K, x, in_dim, out_dim, tokens, None, "%dx%d M=%d" % (in_dim, out_dim, tokens))
    check(oracle, raw, Q5_K, x, in_dim, out_dim, tokens, res, "%dx%d M=%d add" % (in_dim, out_dim, tokens))


def test_q5_k_matrix_core_kernel_element_order(gpu, oracle):
    """One-hot activations pick single weights out of every position of a super-block: a fifth bit taken from the wrong
    byte or bit position shows as a wrong value."""
    rng = np.random.default_rng(79)
    in_dim, out_dim, tokens = 512, 48, 4
    raw = synth.make_weights(rng, Q5_K, out_dim, in_dim)
    dense = oracle.dequantize(raw, Q5_K, out_dim * in_dim).reshape(out_dim, in_dim)
    for base in range(0, in_dim, tokens):
        x = np.zeros((tokens, in_dim), dtype=np.float32)
        for m in range(tokens):
            x[m, base + m] = 1.0
        got = run_gemv(raw, Q5_K, np.ascontiguousarray(x.reshape(-1)), in_dim, out_dim, tokens).reshape(tokens, out_dim)
        for m in range(tokens):
            assert np.allclose(got[m], dense[:, base + m], rtol=0, atol=1e-5 * np.max(np.abs(dense))), (base, m)


@pytest.mark.parametrize("in_dim,out_dim", MFMA_SHAPES)
@pytest.mark.parametrize("tokens", [3, 4, 7])
def test_q6_k_matrix_core_kernel_shapes(gpu, oracle, in_dim, out_dim, tokens):
    """Three and four tokens of a Q6_K matrix run on the matrix cores under the same shape rule as Q4_K (7 tokens:
    a group of four and one of three); two tokens stay on the vector ALU. With and without residual."""
    rng = np.random.default_rng(in_dim * 137 + out_dim * 11 + tokens)
    raw = synth.make_weights(rng, Q6_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    res = rng.standard_normal(tokens * out_dim).astype(np.float32)
    m = min(tokens, 4)
    name = quant.gemv_plan(Q6_K, m, in_dim, out_dim)[0]
    expect_mfma = m * (in_dim // 256) <= 64 or in_dim % 2048 == 0
    assert name == ("q6_k_gemv_mfma_f32_tbatch%d" % m if expect_mfma else "q6_k_gemv_f32_tbatch%d" % m), name
    assert quant.gemv_plan(Q6_K, 2, in_dim, out_dim)[0] == "q6_k_gemv_f32_tbatch2"
    check(oracle, raw, Q6_K, x, in_dim, out_dim, tokens, None, "%dx%d M=%d" % (in_dim, out_dim, tokens))
    check(oracle, raw, Q6_K, x, in_dim, out_dim, tokens, res, "%dx%d M=%d add" % (in_dim, out_dim, tokens))


def test_q6_k_matrix_core_kernel_element_order_and_ranges(gpu, oracle):
    """One-hot activations pick single weights out of every position of a super-block (a wrong quadrant, nibble or
    scale index shows as a wrong value, not as a small error); then activations far outside the binary16 range."""
    rng = np.random.default_rng(78)
    in_dim, out_dim, tokens = 512, 48, 4
    raw = synth.make_weights(rng, Q6_K, out_dim, in_dim)
    dense = oracle.dequantize(raw, Q6_K, out_dim * in_dim).reshape(out_dim, in_dim)
    for base in range(0, in_dim, tokens):
        x = np.zeros((tokens, in_dim), dtype=np.float32)
        for m in range(tokens):
            x[m, base + m] = 1.0
        got = run_gemv(raw, Q6_K, np.ascontiguousarray(x.reshape(-1)), in_dim, out_dim, tokens).reshape(tokens, out_dim)
        for m in range(tokens):
            assert np.allclose(got[m], dense[:, base + m], rtol=0, atol=1e-5 * np.max(np.abs(dense))), (base, m)
    in_dim, out_dim = 4096, 512
    raw = synth.make_weights(rng, Q6_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim).reshape(tokens, in_dim)
    x[0] *= np.float32(1e-30)
    x[1] *= np.float32(1e30)
    x[2, :256] = 0.0
    x[2, 700] = np.float32(3e7)
    x[3] = np.where(rng.random(in_dim) < 0.5, x[3] * np.float32(1e-6), x[3] * np.float32(1e4)).astype(np.float32)
    x = np.ascontiguousarray(x.reshape(-1))
    got, want, frac = check(oracle, raw, Q6_K, x, in_dim, out_dim, tokens, None, "activation ranges")
    g, w_ = got.reshape(tokens, out_dim).astype(np.float64), want.reshape(tokens, out_dim)
    for m in range(tokens):
        assert np.max(np.abs(g[m] - w_[m])) <= 2e-5 * np.max(np.abs(w_[m])), m


def test_q4_k_matrix_core_kernel_activation_ranges(gpu, oracle):
    """The matrix-core kernel feeds the activations as binary16 pairs scaled per token and super-block: values
    far outside the binary16 range, zeros and mixed magnitudes must come out as from fp32 arithmetic."""
    rng = np.random.default_rng(77)
    in_dim, out_dim, tokens = 4096, 512, 4
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim).reshape(tokens, in_dim)
    x[0] *= np.float32(1e-30)                       # far below the smallest binary16 subnormal
    x[1] *= np.float32(1e30)                        # far above the largest binary16 number
    x[2, :256] = 0.0                                # an all-zero super-block
    x[2, 256:512] *= np.float32(1e-12)
    x[2, 700] = np.float32(3e7)                     # one huge value among small ones
    x[3] = np.where(rng.random(in_dim) < 0.5, x[3] * np.float32(1e-6), x[3] * np.float32(1e4)).astype(np.float32)
    x = np.ascontiguousarray(x.reshape(-1))
    got, want, frac = check(oracle, raw, Q4_K, x, in_dim, out_dim, tokens, None, "activation ranges")
    # relative to each token's own output scale
    g, w_ = got.reshape(tokens, out_dim).astype(np.float64), want.reshape(tokens, out_dim)
    for m in range(tokens):
        assert np.max(np.abs(g[m] - w_[m])) <= 2e-5 * np.max(np.abs(w_[m])), m


@pytest.mark.parametrize("type_id,in_dim,out_dim,tokens", [(Q4_K, 4096, 12288, 1), (Q4_K, 512, 37, 1), (Q4_K, 1024, 1024, 3),
                                                            (Q6_K, 512, 40, 1), (Q4_K, 4096, 1024, 1), (Q4_K, 4096, 12288, 4),
                                                            (Q4_K, 4096, 1024, 8), (Q4_K, 12288, 48, 4), (Q4_K, 512, 40, 2),
                                                            (Q4_K, 2048, 8000, 5), (Q4_K, 768, 12304, 3)])
def test_dual_gemv_shares_activations(gpu, oracle, type_id, in_dim, out_dim, tokens):
    """Two matrices of one shape against the same x (gate | up, k | v): one launch for one token of a Q4_K pair,
    including a row count that puts the a | b boundary inside a wavefront's rows; several tokens of a Q4_K pair with a
    multiple of 16 rows go to the matrix-core kernel as one matrix of twice the rows (groups of four tokens and a last
    single one, activations staged in chunks, more row groups than workgroups), other shapes as two launches."""
    rng = np.random.default_rng(in_dim + 3 * out_dim + tokens)
    raw_a = synth.make_weights(rng, type_id, out_dim, in_dim)
    raw_b = synth.make_weights(rng, type_id, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    wa, wb, xd = DevArray(raw_a), DevArray(raw_b), DevArray(x)
    oa, ob = DevArray(nbytes=4 * tokens * out_dim), DevArray(nbytes=4 * tokens * out_dim)
    quant.gemv_dual_dev(wa.ptr, wb.ptr, type_id, xd.ptr, oa.ptr, ob.ptr, in_dim, out_dim, tokens)
    zero = np.zeros(out_dim, dtype=np.float32)
    for raw, o in ((raw_a, oa), (raw_b, ob)):
        got = o.read(np.float32, tokens * out_dim)
        want = oracle.matmul_add(x, tokens, in_dim, raw, type_id, out_dim, zero, threads=8).astype(np.float64)
        dense = np.abs(oracle.dequantize(raw, type_id, out_dim * in_dim)).reshape(out_dim, in_dim)
        tol = gemv_tolerance(x, dense, tokens, in_dim).reshape(-1)
        assert np.all(np.abs(got.astype(np.float64) - want) <= tol)
    if tokens == 1 and type_id == Q4_K:   # the pair in one launch gives the bits of the single-matrix kernel
        assert np.array_equal(oa.read(np.float32, out_dim), run_gemv(raw_a, type_id, x, in_dim, out_dim, 1))
        assert np.array_equal(ob.read(np.float32, out_dim), run_gemv(raw_b, type_id, x, in_dim, out_dim, 1))
    for d in (wa, wb, xd, oa, ob):
        d.close()


@pytest.mark.parametrize("type_id,in_dim,dims,tokens", [(Q4_K, 4096, (4096, 1024, 1024), 4), (Q4_K, 1024, (48, 16, 160), 7),
                                                        (Q4_K, 12288, (64, 32), 3), (Q4_K, 2048, (12288, 4096, 32), 2),
                                                        (Q4_K, 512, (40, 16, 16), 4), (Q6_K, 512, (32, 48, 16), 4),
                                                        (Q4_K, 1024, (64, 32, 16), 1), (Q4_K, 256, (16, 16, 16, 16), 3)])
def test_many_gemv_shares_activations(gpu, oracle, type_id, in_dim, dims, tokens):
    """Several matrices against one x in one call (q | k | v): two or three Q4_K matrices with multiples of 16 rows and
    two or more tokens run as one matrix-core launch per group of four tokens, everything else matrix by matrix. Either
    way the values are those of cogni_gemv_dev on each matrix, bit for bit where both take the matrix cores."""
    rng = np.random.default_rng(in_dim + sum(dims) + tokens)
    raws = [synth.make_weights(rng, type_id, d, in_dim) for d in dims]
    x = synth.make_activations(rng, tokens, in_dim)
    ws, xd = [DevArray(r) for r in raws], DevArray(x)
    outs = [DevArray(nbytes=4 * tokens * d) for d in dims]
    quant.gemv_many_dev([w.ptr for w in ws], type_id, xd.ptr, [o.ptr for o in outs], list(dims), in_dim, tokens)
    zero = {d: np.zeros(d, dtype=np.float32) for d in dims}
    for raw, o, d in zip(raws, outs, dims):
        got = o.read(np.float32, tokens * d)
        want = oracle.matmul_add(x, tokens, in_dim, raw, type_id, d, zero[d], threads=8).astype(np.float64)
        dense = np.abs(oracle.dequantize(raw, type_id, d * in_dim)).reshape(d, in_dim)
        assert np.all(np.abs(got.astype(np.float64) - want) <= gemv_tolerance(x, dense, tokens, in_dim).reshape(-1))
        single = run_gemv(raw, type_id, x, in_dim, d, tokens)
        # the list takes the one-pass kernel from two tokens on where there is one for the shape, a single matrix from five
        one_pass_list = quant.gemv_image_bytes(type_id, in_dim, min(tokens, 8)) > 0 and tokens >= 2
        one_pass_single = one_pass_list and tokens >= 5
        if one_pass_list != one_pass_single:
            assert np.max(np.abs(got - single)) <= 2e-5 * max(1e-30, float(np.abs(single).max()))
        elif one_pass_list or (all("mfma" in quant.gemv_plan(type_id, m, in_dim, d)[0] for m in {min(tokens, 4), tokens % 4 or 4} if m >= 2) and tokens % 4 != 1):
            assert np.array_equal(got, single)
        else:
            assert np.max(np.abs(got - single)) <= 2e-5 * max(1e-30, float(np.abs(single).max()))
    for a in ws + outs + [xd]:
        a.close()
    with pytest.raises(quant.QuantError):
        quant.gemv_many_dev([], type_id, 0, [], [], in_dim, tokens)


@pytest.mark.parametrize("in_dim,dims", [(4096, (4096, 1024, 1024)), (1024, (37, 5, 130)), (256, (3, 1)), (12288, (48, 77, 9)),
                                         (512, (8, 8, 8, 20, 7)), (256, (9000, 300, 2)), (2048, (16, 16, 16, 16, 16, 16, 16))])
def test_one_token_lists_in_one_launch(gpu, oracle, in_dim, dims):
    """One token against several Q4_K matrices (q | k | v): up to three per launch as one matrix of all their rows. Row counts
    that put a matrix boundary inside a wavefront's rows and inside a workgroup's, more rows than resident workgroups (the
    workgroups walk), rows of three column sets, five and seven matrices (launches of three, three and one). Every row must
    come out bit for bit as from the single-matrix call, and within the bar of the oracle."""
    rng = np.random.default_rng(in_dim + sum(dims))
    raws = [synth.make_weights(rng, Q4_K, d, in_dim) for d in dims]
    x = synth.make_activations(rng, 1, in_dim)
    ws, xd = [DevArray(r) for r in raws], DevArray(x)
    outs = [DevArray(nbytes=4 * d) for d in dims]
    quant.gemv_many_dev([w.ptr for w in ws], Q4_K, xd.ptr, [o.ptr for o in outs], list(dims), in_dim, 1)
    for raw, o, d in zip(raws, outs, dims):
        got = o.read(np.float32, d)
        assert np.array_equal(got, run_gemv(raw, Q4_K, x, in_dim, d, 1))
        want = oracle.matmul_add(x, 1, in_dim, raw, Q4_K, d, np.zeros(d, dtype=np.float32), threads=8).astype(np.float64)
        dense = np.abs(oracle.dequantize(raw, Q4_K, d * in_dim)).reshape(d, in_dim)
        assert np.all(np.abs(got.astype(np.float64) - want) <= gemv_tolerance(x, dense, 1, in_dim).reshape(-1))
    for a in ws + outs + [xd]:
        a.close()


def test_swiglu_kernel_and_fused_gate_up(gpu, oracle):
    """swiglu_f32 against the oracle's float32 form, and the fused gate/up + SwiGLU launch against the
    two-step composition (same bits: same GEMV arithmetic, same device function) and the oracle."""
    rng = np.random.default_rng(4242)
    g = (rng.standard_normal(5000) * 4).astype(np.float32)
    g[:6] = [0.0, -0.0, 100.0, -100.0, 1e-30, -20.0]
    u = rng.standard_normal(5000).astype(np.float32)
    gd, ud, od = DevArray(g), DevArray(u), DevArray(nbytes=g.nbytes)
    quant.swiglu_dev(gd.ptr, ud.ptr, od.ptr, g.size)
    got, want = od.read(np.float32, g.size), oracle.swiglu(g, u)
    assert np.all(np.abs(got - want) <= 4e-7 * np.abs(want) + 1e-37)          # a few ulp: the two exp differ in the last bit
    assert got[0] == 0.0 and got[3] == 0.0                                   # silu(0) = 0, silu(-100) * u underflows to -0 / 0
    for in_dim, out_dim, tokens in ((4096, 12288, 1), (512, 37, 1), (1024, 130, 3)):
        raw_g = synth.make_weights(rng, Q4_K, out_dim, in_dim)
        raw_u = synth.make_weights(rng, Q4_K, out_dim, in_dim)
        x = synth.make_activations(rng, tokens, in_dim)
        wg, wu, xd = DevArray(raw_g), DevArray(raw_u), DevArray(x)
        n = tokens * out_dim
        og, ou, o2, of = (DevArray(nbytes=4 * n) for _ in range(4))
        for t in range(tokens):   # two-step composition, one token per launch as the fused kernel works
            quant.gemv_dual_dev(wg.ptr, wu.ptr, Q4_K, xd.ptr + 4 * t * in_dim, og.ptr + 4 * t * out_dim, ou.ptr + 4 * t * out_dim,
                                in_dim, out_dim, 1)
        quant.swiglu_dev(og.ptr, ou.ptr, o2.ptr, n)
        quant.gemv_dual_swiglu_dev(wg.ptr, wu.ptr, Q4_K, xd.ptr, of.ptr, in_dim, out_dim, tokens)
        fused, two_step = of.read(np.float32, n), o2.read(np.float32, n)
        assert np.array_equal(fused, two_step)
        zero = np.zeros(out_dim, dtype=np.float32)
        ref = oracle.swiglu(oracle.matmul_add(x, tokens, in_dim, raw_g, Q4_K, out_dim, zero, threads=8),
                            oracle.matmul_add(x, tokens, in_dim, raw_u, Q4_K, out_dim, zero, threads=8))
        assert cosine(fused, ref) >= 0.999999
        assert np.max(np.abs(fused - ref)) <= 1e-4 * np.max(np.abs(ref))
        for d in (wg, wu, xd, og, ou, o2, of):
            d.close()
    # several tokens, a multiple of 16 rows: the matrix-core kernel with gate and up tiles side by side; the same bits as
    # the matrix-core pair kernel followed by swiglu_f32 on the same token groups (walking row groups, chunked activations,
    # a last single token)
    # (from two tokens on rows that are a multiple of 2048 long the one-pass kernel takes the call, with any out_dim: a
    # clipped last tile, and the rows above 4096 values whose operands are streamed)
    for in_dim, out_dim, tokens in ((4096, 12288, 4), (1024, 160, 7), (12288, 48, 3), (512, 48, 2), (2048, 8208, 5), (2048, 130, 5),
                                    (4096, 1000, 8), (6144, 40, 2), (8192, 100, 4), (12288, 200, 8), (10240, 7, 6)):
        raw_g = synth.make_weights(rng, Q4_K, out_dim, in_dim)
        raw_u = synth.make_weights(rng, Q4_K, out_dim, in_dim)
        x = synth.make_activations(rng, tokens, in_dim)
        wg, wu, xd = DevArray(raw_g), DevArray(raw_u), DevArray(x)
        n = tokens * out_dim
        og, ou, o2, of = (DevArray(nbytes=4 * n) for _ in range(4))
        quant.gemv_dual_dev(wg.ptr, wu.ptr, Q4_K, xd.ptr, og.ptr, ou.ptr, in_dim, out_dim, tokens)
        quant.swiglu_dev(og.ptr, ou.ptr, o2.ptr, n)
        quant.gemv_dual_swiglu_dev(wg.ptr, wu.ptr, Q4_K, xd.ptr, of.ptr, in_dim, out_dim, tokens)
        fused, two_step = of.read(np.float32, n), o2.read(np.float32, n)
        assert np.array_equal(fused, two_step), (in_dim, out_dim, tokens)
        zero = np.zeros(out_dim, dtype=np.float32)
        ref = oracle.swiglu(oracle.matmul_add(x, tokens, in_dim, raw_g, Q4_K, out_dim, zero, threads=8),
                            oracle.matmul_add(x, tokens, in_dim, raw_u, Q4_K, out_dim, zero, threads=8))
        assert cosine(fused, ref) >= 0.999999
        assert np.max(np.abs(fused - ref)) <= 1e-4 * np.max(np.abs(ref))
        for d in (wg, wu, xd, og, ou, o2, of):
            d.close()
    with pytest.raises(quant.QuantError, match="Unsupported quant type for the fused gate/up SwiGLU: Q6_K"):
        big = DevArray(nbytes=1 << 20)   # (real memory behind the pointers: a call accepted by mistake would stay inside it)
        quant.gemv_dual_swiglu_dev(big.ptr, big.ptr, Q6_K, big.ptr, big.ptr, 256, 16, 1)
    big.close()
    for d in (gd, ud, od):
        d.close()


@pytest.mark.parametrize("type_id,in_dim,out_dim", [(Q4_K, 4096, 64), (Q6_K, 12288, 40), (Q5_K, 1024, 33), (Q4_K, 16384, 24)])
@pytest.mark.parametrize("tokens", [1, 2])
def test_activations_at_any_float_alignment(gpu, oracle, type_id, in_dim, out_dim, tokens):
    """The activations are copied to LDS 16 bytes per lane; the pointer a caller passes is only float-aligned
    (one token of a longer buffer, an offset into a workspace). in_dim 16384 is staged in two chunks."""
    rng = np.random.default_rng(in_dim + tokens)
    raw = synth.make_weights(rng, type_id, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    wd, od = DevArray(raw), DevArray(nbytes=4 * tokens * out_dim)
    want = oracle.matmul_add(x, tokens, in_dim, raw, type_id, out_dim, np.zeros(out_dim, dtype=np.float32), threads=8)
    dense = np.abs(oracle.dequantize(raw, type_id, out_dim * in_dim)).reshape(out_dim, in_dim)
    tol = gemv_tolerance(x, dense, tokens, in_dim).reshape(-1)
    try:
        for shift in (1, 2, 3):                       # floats
            padded = np.concatenate([np.zeros(shift, dtype=np.float32), x.reshape(-1)])
            xd = DevArray(padded)
            quant.gemv_dev(wd.ptr, type_id, xd.ptr + 4 * shift, od.ptr, in_dim, out_dim, tokens)
            got = od.read(np.float32, tokens * out_dim)
            assert np.all(np.abs(got - want) <= tol), "shift %d" % shift
            xd.close()
    finally:
        wd.close()
        od.close()


@pytest.mark.parametrize("type_id,in_dim,out_dim", [(Q4_K, 256, 16 * 768 * 2 + 5), (Q6_K, 1024, 8 * 768 * 3 + 3),
                                                    (Q5_K, 512, 8 * 768 + 1), (Q4_K, 16384, 16 * 768 + 17)])
@pytest.mark.parametrize("add", [False, True])
def test_long_matrices_walk_row_groups(gpu, oracle, type_id, in_dim, out_dim, add):
    """One token of a K-quant matrix with more row groups than resident workgroups: every workgroup takes several
    groups. Rows are independent, so the result must equal, bit for bit, what the same kernel gives on slices of
    the matrix short enough for one group per workgroup; a few rows are also checked against the oracle.
    in_dim 16384 does not fit the staging buffer at once: the activations are staged again for every group."""
    rng = np.random.default_rng(out_dim)
    raw = synth.make_weights(rng, type_id, out_dim, in_dim)
    x = synth.make_activations(rng, 1, in_dim)
    res = rng.standard_normal(out_dim).astype(np.float32) if add else None
    row_bytes = raw.size // out_dim
    wd, xd, od = DevArray(raw), DevArray(x), DevArray(nbytes=4 * out_dim)
    rd = DevArray(res) if add else None
    try:
        grid = quant.gemv_launch_dims(type_id, 1, in_dim, out_dim)[0]
        assert grid <= {Q4_K: 1024, Q6_K: 768, Q5_K: 768}[type_id] and grid * 8 < out_dim      # 8 rows per workgroup: they walk
        quant.gemv_dev(wd.ptr, type_id, xd.ptr, od.ptr, in_dim, out_dim, 1, rd.ptr if add else 0)
        full = od.read(np.float32, out_dim)
        piece = 4096                                   # at most 512 row groups: one per workgroup
        parts = np.empty(out_dim, dtype=np.float32)
        for r0 in range(0, out_dim, piece):
            n = min(piece, out_dim - r0)
            quant.gemv_dev(wd.ptr + r0 * row_bytes, type_id, xd.ptr, od.ptr, in_dim, n, 1, rd.ptr + 4 * r0 if add else 0)
            parts[r0:r0 + n] = od.read(np.float32, n)
        assert np.array_equal(full, parts)
        rows = np.unique(np.concatenate([np.arange(3), rng.integers(0, out_dim, 24), np.arange(out_dim - 3, out_dim)]))
        for r in rows:
            bias = np.array([res[r] if add else 0.0], dtype=np.float32)
            want = oracle.matmul_add(x, 1, in_dim, raw[r * row_bytes:(r + 1) * row_bytes], type_id, 1, bias)[0]
            w_abs = np.abs(oracle.dequantize(raw[r * row_bytes:(r + 1) * row_bytes], type_id, in_dim)).max()
            assert abs(full[r] - want) <= 1e-4 * np.linalg.norm(x) * w_abs, "row %d" % r
    finally:
        for d in (wd, xd, od) + ((rd,) if add else ()):
            d.close()
