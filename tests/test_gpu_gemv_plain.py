"""F32, F16 and IQ4_NL weights through the fused matmul (the arms of QuantMatmul.matmul_add beside the four block formats,
src/ml/gguf/quant_matmul.cr:30-32, 272-368) against the CPU oracle.

Tolerance: max|err| <= 1e-4 * ||x||_2 * max|w_row| per token and output row (fp32 accumulation against the reference's
float64), and the reference's own gate for its fused matmuls, max_diff / max|ref| <= 1e-5 (spec/q4k_matmul_spec.cr:87-96),
on the host-buffer entry point.
"""
import numpy as np
import pytest

from cogni_ml_amd import quant, synth
from gpu_common import DevArray, gpu  # noqa: F401
from helpers import cosine, gemv_tolerance

pytestmark = pytest.mark.gpu
F32, F16, IQ4_NL = 0, 1, 20


def dense_of(oracle, raw, t, out_dim, in_dim):
    """|w| per row, from the oracle's dequantize (IQ4_NL rows are padded to whole blocks: dequantize row by row)."""
    row_bytes = raw.size // out_dim
    return np.stack([np.abs(oracle.dequantize(raw[r * row_bytes:(r + 1) * row_bytes], t, in_dim)) for r in range(out_dim)])


def run(raw, t, x, in_dim, out_dim, tokens, residual=None):
    w, xd, od = DevArray(raw), DevArray(x), DevArray(nbytes=4 * tokens * out_dim)
    rd = DevArray(residual) if residual is not None else None
    try:
        quant.gemv_dev(w.ptr, t, xd.ptr, od.ptr, in_dim, out_dim, tokens, rd.ptr if rd else 0)
        return od.read(np.float32, tokens * out_dim)
    finally:
        for a in (w, xd, od, rd):
            if a:
                a.close()


@pytest.mark.parametrize("t", [F32, F16, IQ4_NL])
@pytest.mark.parametrize("in_dim,out_dim,tokens", [(1024, 37, 1), (1024, 300, 3), (4096, 64, 8), (1000, 9, 5), (33, 5, 2),
                                                   (40, 3, 1), (1, 1, 1), (2048 + 17, 130, 11), (4096, 4096, 1)])
def test_plain_types_against_oracle(gpu, oracle, t, in_dim, out_dim, tokens):
    """Row lengths that are and are not multiples of 4 and of the IQ4_NL block (clipped last block, a half block, a single
    element), row counts that are not multiples of the four rows of a workgroup, token counts on both sides of the four a
    lane holds, with and without residual."""
    rng = np.random.default_rng(in_dim * 7 + out_dim * 3 + tokens + t)
    raw = synth.make_weights(rng, t, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    res = rng.standard_normal(tokens * out_dim).astype(np.float32)
    zero = np.zeros(out_dim, dtype=np.float32)
    want = oracle.matmul_add(x, tokens, in_dim, raw, t, out_dim, zero, threads=8).astype(np.float64)
    tol = gemv_tolerance(x, dense_of(oracle, raw, t, out_dim, in_dim), tokens, in_dim).reshape(-1)
    got = run(raw, t, x, in_dim, out_dim, tokens)
    assert np.all(np.abs(got - want) <= tol), float(np.max(np.abs(got - want) / np.maximum(tol, 1e-30)))
    got = run(raw, t, x, in_dim, out_dim, tokens, res)
    assert np.all(np.abs(got - (want.astype(np.float32) + res)) <= tol + 1e-6 * np.abs(res))


def test_iq4_nl_element_order(gpu, oracle):
    """One-hot activations pick single weights: element e < 16 of a block is the low nibble of byte e, element 16 + e the
    high nibble; a swapped half or a wrong table entry shows as a wrong value."""
    rng = np.random.default_rng(20)
    in_dim, out_dim = 96, 6
    raw = synth.make_weights(rng, IQ4_NL, out_dim, in_dim)
    dense = np.stack([oracle.dequantize(raw[r * 54:(r + 1) * 54], IQ4_NL, in_dim) for r in range(out_dim)])
    for base in range(0, in_dim, 8):
        x = np.zeros((8, in_dim), dtype=np.float32)
        for m in range(8):
            x[m, base + m] = 1.0
        got = run(raw, IQ4_NL, np.ascontiguousarray(x.reshape(-1)), in_dim, out_dim, 8).reshape(8, out_dim)
        for m in range(8):
            assert np.array_equal(got[m], dense[:, base + m]), (base, m)


@pytest.mark.parametrize("t", [F32, F16, IQ4_NL])
def test_host_matmul_add_and_quant_weight(gpu, oracle, t):
    """QuantMatmul.matmul_add and QuantWeight through the host-buffer entry points with the reference spec's deterministic x
    and bias (spec/q4k_matmul_spec.cr:66-73), 2 rows and 12 rows (past the row count from which the block formats take the
    GEMM: these types stay on the row kernels)."""
    rng = np.random.default_rng(33 + t)
    out_dim, in_dim = 256, 1024
    for rows in (2, 12):
        i = np.arange(rows * in_dim, dtype=np.uint64)
        x = (((i * 2654435761) % (1 << 32) % 2000).astype(np.int64) - 1000).astype(np.float32) / np.float32(1000.0)
        bias = ((np.arange(out_dim) % 10) / np.float32(100.0)).astype(np.float32)
        raw = synth.make_weights(rng, t, out_dim, in_dim)
        mine = quant.matmul_add(x, rows, in_dim, raw, t, out_dim, bias)
        ref = oracle.matmul_add(x, rows, in_dim, raw, t, out_dim, bias)
        assert cosine(mine, ref) >= 0.9999999
        assert np.max(np.abs(mine - ref)) / np.max(np.abs(ref)) <= 1e-5
        qw = quant.QuantWeight(raw, t, out_dim, in_dim, "plain")
        assert np.array_equal(qw.matmul(x, rows, bias), mine)
        qw.close()


def test_other_ggml_types_are_still_refused(gpu):
    w = np.zeros(18 * 8, dtype=np.uint8)
    x = np.zeros(256, dtype=np.float32)
    with pytest.raises(quant.QuantError, match="Unsupported quant type for fused matmul: Q4_0") as e:
        quant.matmul_add(x, 1, 256, w, 2, 1, None)
    assert e.value.code == -2
