"""Pins QuantMatmul.matmul_add (quant_matmul.cr:20-368) through invariants and brute force."""
import numpy as np
import pytest

from cogni_ml_amd import synth
from oracle import numpy_restatement as npr
from helpers import BLOCK, F16, F32, IQ4_NL, Q4_K, Q5_K, Q6_K, Q8_0, cosine

ALL = [Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL, F16, F32]


def shape_for(type_id):
    be = BLOCK.get(type_id, (0, 1))[1]
    return 24, max(be * 2, 512)          # out_dim, in_dim


@pytest.mark.parametrize("type_id", ALL)
def test_fused_equals_bulk_dequant_f64_dot(oracle, type_id):
    """The invariant the reference tests (spec/q4k_matmul_spec.cr:66-88): cos >= 0.9999999, rel <= 1e-5."""
    rng = np.random.default_rng(type_id)
    out_dim, in_dim = shape_for(type_id)
    rows = 2
    w = synth.make_weights(rng, type_id, out_dim, in_dim)
    # the reference spec's deterministic x and bias
    i = np.arange(rows * in_dim, dtype=np.uint64)
    x = (((i * 2654435761) % (1 << 32) % 2000).astype(np.int64) - 1000).astype(np.float32) / np.float32(1000.0)
    bias = ((np.arange(out_dim) % 10) / np.float32(100.0)).astype(np.float32)
    mine = oracle.matmul_add(x, rows, in_dim, w, type_id, out_dim, bias)
    ref = npr.matmul_dense_f64(x, rows, in_dim, w, type_id, out_dim, bias)
    assert cosine(mine, ref) >= 0.9999999
    assert np.max(np.abs(mine - ref)) / np.max(np.abs(ref)) <= 1e-5
    # f64 accumulation makes the two agree far more tightly than the reference's gate
    assert np.max(np.abs(mine.astype(np.float64) - ref)) <= 2e-6 * np.max(np.abs(ref))


def brute_force(oracle, x, rows, in_dim, w, type_id, out_dim, bias):
    """Pure-Python float64 dot over the oracle's *bulk dequantized* weights in natural j order."""
    dense = oracle.dequantize(w, type_id, out_dim * in_dim).astype(np.float64).reshape(out_dim, in_dim)
    res = np.empty(rows * out_dim, dtype=np.float32)
    for r in range(rows):
        for o in range(out_dim):
            s = float(bias[o])
            for j in range(in_dim):
                s += float(x[r * in_dim + j]) * dense[o, j]
            res[r * out_dim + o] = np.float32(s)
    return res


@pytest.mark.parametrize("type_id", [Q8_0, Q4_K, Q5_K])
def test_tiny_brute_force_natural_order(oracle, type_id):
    """Q8_0/Q4_K/Q5_K sum in natural j order. With d a power of two and integer scales every
    float32 dequantized value equals the float64 one, so a float64 loop over the bulk-dequantized
    weights reproduces the fused result bit for bit."""
    rng = np.random.default_rng(40 + type_id)
    be = BLOCK[type_id][1]
    out_dim, in_dim, rows = 3, be * 2, 2
    w = synth.make_weights(rng, type_id, out_dim, in_dim)
    blocks = w.reshape(-1, BLOCK[type_id][0])
    blocks[:, 0:2] = [0x00, 0x30]                      # d = 0.125
    if type_id in (Q4_K, Q5_K):
        blocks[:, 2:4] = [0x00, 0x34]                  # dmin = 0.25
    x = synth.make_activations(rng, rows, in_dim)
    bias = rng.standard_normal(out_dim).astype(np.float32)
    got = oracle.matmul_add(x, rows, in_dim, w, type_id, out_dim, bias)
    assert np.array_equal(got, brute_force(oracle, x, rows, in_dim, w, type_id, out_dim, bias))


def test_q6_k_summation_order_is_interleaved(oracle):
    """Q6_K adds elements l, l+32, l+64, l+96 per l (quant_matmul.cr:215-218), not in natural order.
    Checked against a float64 loop in that order; it is bit-exact there and (on this input) not in natural order."""
    rng = np.random.default_rng(6)
    out_dim, in_dim, rows = 4, 512, 1
    w = synth.make_weights(rng, Q6_K, out_dim, in_dim)
    w.reshape(-1, 210)[:, 208:210] = [0x00, 0x30]      # d = 0.125: float32 products exact
    x = (synth.make_activations(rng, rows, in_dim) * 1000).astype(np.float32)
    bias = np.zeros(out_dim, dtype=np.float32)
    dense = oracle.dequantize(w, Q6_K, out_dim * in_dim).astype(np.float64).reshape(out_dim, in_dim)
    want = np.empty(out_dim, dtype=np.float32)
    natural = np.empty(out_dim, dtype=np.float32)
    for o in range(out_dim):
        s = 0.0
        for base in range(0, in_dim, 128):
            for l in range(32):
                for k in range(4):
                    j = base + l + 32 * k
                    s += float(x[j]) * dense[o, j]
        want[o] = np.float32(s)
        s = 0.0
        for j in range(in_dim):
            s += float(x[j]) * dense[o, j]
        natural[o] = np.float32(s)
    got = oracle.matmul_add(x, rows, in_dim, w, Q6_K, out_dim, bias)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("type_id", [F32, F16])
def test_dense_types_use_float32_products(oracle, type_id):
    """F32/F16 rows: x*w is rounded to float32 before it is added to the float64 sum (quant_matmul.cr:339,361)."""
    rng = np.random.default_rng(9)
    out_dim, in_dim = 5, 64
    w = synth.make_weights(rng, type_id, out_dim, in_dim)
    x = synth.make_activations(rng, 1, in_dim)
    bias = rng.standard_normal(out_dim).astype(np.float32)
    dense = npr.DEQUANT[type_id](w.tobytes(), out_dim * in_dim).reshape(out_dim, in_dim)
    want = np.empty(out_dim, dtype=np.float32)
    for o in range(out_dim):
        s = float(bias[o])
        for j in range(in_dim):
            s += float(np.float32(x[j] * dense[o, j]))
        want[o] = np.float32(s)
    assert np.array_equal(oracle.matmul_add(x, 1, in_dim, w, type_id, out_dim, bias), want)


@pytest.mark.parametrize("type_id", ALL)
def test_rows_are_independent_and_bias_is_added_once(oracle, type_id):
    rng = np.random.default_rng(20 + type_id)
    out_dim, in_dim = shape_for(type_id)
    w = synth.make_weights(rng, type_id, out_dim, in_dim)
    x = synth.make_activations(rng, 3, in_dim)
    bias = rng.standard_normal(out_dim).astype(np.float32)
    full = oracle.matmul_add(x, 3, in_dim, w, type_id, out_dim, bias).reshape(3, out_dim)
    for r in range(3):
        one = oracle.matmul_add(x[r * in_dim:(r + 1) * in_dim], 1, in_dim, w, type_id, out_dim, bias)
        assert np.array_equal(full[r], one)
    zero = oracle.matmul_add(np.zeros(in_dim, dtype=np.float32), 1, in_dim, w, type_id, out_dim, bias)
    assert np.array_equal(zero, bias)


@pytest.mark.parametrize("type_id", [Q8_0, Q4_K, Q5_K, Q6_K])
def test_linearity_in_x(oracle, type_id):
    rng = np.random.default_rng(30 + type_id)
    out_dim, in_dim = shape_for(type_id)
    w = synth.make_weights(rng, type_id, out_dim, in_dim)
    a, b = synth.make_activations(rng, 1, in_dim), synth.make_activations(rng, 1, in_dim)
    z = np.zeros(out_dim, dtype=np.float32)
    f = lambda v: oracle.matmul_add(v, 1, in_dim, w, type_id, out_dim, z).astype(np.float64)
    lhs, rhs = f((2 * a).astype(np.float32)) + f(b), f((2 * a + b).astype(np.float32))
    assert np.max(np.abs(lhs - rhs)) <= 1e-5 * np.max(np.abs(rhs))
    assert np.array_equal(f((4 * a).astype(np.float32)), 4 * f(a))    # power-of-two scaling is exact


def test_q8_0_partial_last_block(oracle):
    """Q8_0 rows may end inside a block: blocks_per_row = ceil(in/32), the tail is clipped (quant_matmul.cr:241,259)."""
    rng = np.random.default_rng(77)
    out_dim, in_dim = 6, 80
    w = synth.make_weights(rng, Q8_0, out_dim, in_dim)
    assert w.size == out_dim * 3 * 34
    x = synth.make_activations(rng, 1, in_dim)
    dense = np.stack([npr.dequantize_q8_0(w[o * 102:(o + 1) * 102].tobytes(), 96)[:80] for o in range(out_dim)])
    want = (dense.astype(np.float64) @ x.astype(np.float64)).astype(np.float32)
    got = oracle.matmul_add(x, 1, in_dim, w, Q8_0, out_dim, np.zeros(out_dim, dtype=np.float32))
    assert np.allclose(got, want, rtol=1e-6, atol=1e-7)


def test_threads_split_is_identical(oracle):
    rng = np.random.default_rng(3)
    w = synth.make_weights(rng, Q4_K, 37, 512)
    x = synth.make_activations(rng, 2, 512)
    bias = rng.standard_normal(37).astype(np.float32)
    assert np.array_equal(oracle.matmul_add(x, 2, 512, w, Q4_K, 37, bias),
                          oracle.matmul_add(x, 2, 512, w, Q4_K, 37, bias, threads=4))


def test_unsupported_type_raises(oracle):
    with pytest.raises(ValueError, match="Unsupported quant type for fused matmul"):
        oracle.matmul_add(np.zeros(256, dtype=np.float32), 1, 256, np.zeros(84, dtype=np.uint8), 10, 1,
                          np.zeros(1, dtype=np.float32))


def test_geometry_table(oracle):
    """block_bytes / block_elements (reader.cr:51-78) and data_bytes (reader.cr:119-127) at the configured shapes."""
    from cogni_ml_amd.types import TensorType
    for t in TensorType:
        assert oracle.block_bytes(int(t)) == t.block_bytes and oracle.block_elements(int(t)) == t.block_elements
    assert oracle.data_bytes(Q8_0, 3584 * 1024) == 3899392
    assert oracle.data_bytes(Q4_K, 12288 * 4096) == 28311552
    assert oracle.data_bytes(Q6_K, 151936 * 4096) == 510504960
    assert oracle.data_bytes(Q6_K, 4096 * 12288) == 41287680
    assert oracle.data_bytes(Q5_K, 4096 * 4096) == 11534336
    assert oracle.data_bytes(F16, 10) == 20 and oracle.data_bytes(IQ4_NL, 40) == 36
    assert oracle.block_bytes(99) == -1


def test_swiglu_closed_forms_and_float64():
    """silu(0) = 0; silu(x) - silu(-x) = x; silu(x) -> x for large x, -> 0 for very negative x; against float64."""
    from oracle import oracle
    x = np.array([0.0, 1.0, -1.0, 3.5, -3.5, 50.0, -50.0, 1e-4, -1e-4], dtype=np.float32)
    ones = np.ones_like(x)
    s = oracle.swiglu(x, ones)
    assert s[0] == 0.0
    assert np.allclose(s[1] - s[2], 1.0, atol=1e-7) and np.allclose(s[3] - s[4], 3.5, atol=1e-6)
    assert s[5] == np.float32(50.0) and abs(s[6]) < 1e-19
    rng = np.random.default_rng(5)
    g, u = (rng.standard_normal(4096) * 5).astype(np.float32), rng.standard_normal(4096).astype(np.float32)
    ref = g.astype(np.float64) / (1.0 + np.exp(-g.astype(np.float64))) * u.astype(np.float64)
    assert np.max(np.abs(oracle.swiglu(g, u) - ref)) <= 3e-7 * np.max(np.abs(ref))
    assert np.array_equal(oracle.swiglu(g, 2 * u), 2 * oracle.swiglu(g, u))      # exact: a power of two in the last product


def test_rms_norm_closed_forms_and_float64():
    """Constant vector c with unit weights -> c / sqrt(c^2 + eps); mean square of the output = ms / (ms + eps);
    invariance under scaling of x at eps = 0; weights enter linearly; against float64."""
    from oracle import oracle
    dim = 1024
    ones = np.ones(dim, dtype=np.float32)
    for c, eps in ((2.0, 1e-6), (-0.5, 1e-2), (1e-3, 1e-6)):
        out = oracle.rms_norm(np.full(dim, c, dtype=np.float32), ones, eps)
        assert np.allclose(out, c / np.sqrt(c * c + eps), rtol=2e-7, atol=0)
    rng = np.random.default_rng(6)
    x, w = rng.standard_normal(dim).astype(np.float32) * 3, rng.standard_normal(dim).astype(np.float32)
    ms = float(np.mean(x.astype(np.float64) ** 2))
    out = oracle.rms_norm(x, ones, 0.25)
    assert abs(float(np.mean(out.astype(np.float64) ** 2)) - ms / (ms + 0.25)) <= 1e-6
    assert np.array_equal(oracle.rms_norm(4 * x, w, 0.0), oracle.rms_norm(x, w, 0.0))     # power-of-two scale: exact
    assert np.array_equal(oracle.rms_norm(x, 2 * w, 1e-6), 2 * oracle.rms_norm(x, w, 1e-6))
    ref = x.astype(np.float64) / np.sqrt(ms + 1e-6) * w.astype(np.float64)
    assert np.max(np.abs(oracle.rms_norm(x, w, 1e-6) - ref)) <= 3e-7 * np.max(np.abs(ref))
    assert np.array_equal(oracle.rms_norm(np.zeros(8, dtype=np.float32), np.ones(8, dtype=np.float32), 1e-6), np.zeros(8, dtype=np.float32))
