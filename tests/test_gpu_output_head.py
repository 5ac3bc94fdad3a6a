"""GEMV fused with the arg-max over the rows, and the resident output head (RMSNorm -> vocabulary projection -> top-1),
against the CPU form of the reference's probe (bin/cuda_mixed_stack_probe.cr:1479-1497): rms_norm, matmul_add with a zero
bias, then a scan that keeps the first of equal maxima."""
import numpy as np
import pytest

from cogni_ml_amd import hip, quant, synth
from cogni_ml_amd.output_head import QwenOutputHeadRunner, Weights
from gpu_common import DevArray, gpu  # noqa: F401

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14


def first_max(v):
    return int(np.argmax(v))        # numpy returns the first of equal maxima, as the reference's scan


def run_top1(raw, t, x, in_dim, out_dim, tokens):
    stride = quant.gemv_top1_partials(t, out_dim)
    wd, xd = DevArray(raw), DevArray(x)
    pi, pv = DevArray(nbytes=4 * tokens * stride), DevArray(nbytes=4 * tokens * stride)
    oi, ov, lo = DevArray(nbytes=4 * tokens), DevArray(nbytes=4 * tokens), DevArray(nbytes=4 * tokens * out_dim)
    try:
        quant.gemv_top1_dev(wd.ptr, t, xd.ptr, pi.ptr, pv.ptr, oi.ptr, ov.ptr, in_dim, out_dim, tokens)
        quant.gemv_dev(wd.ptr, t, xd.ptr, lo.ptr, in_dim, out_dim, tokens)
        return oi.read(np.uint32, tokens), ov.read(np.float32, tokens), lo.read(np.float32, tokens * out_dim).reshape(tokens, out_dim)
    finally:
        for d in (wd, xd, pi, pv, oi, ov, lo):
            d.close()


@pytest.mark.parametrize("t,in_dim,out_dim,tokens", [(Q6_K, 4096, 32003, 1), (Q6_K, 1024, 5000, 5), (Q6_K, 256, 7, 2),
                                                     (Q4_K, 1024, 4099, 1), (Q4_K, 512, 777, 7), (Q5_K, 512, 1001, 2),
                                                     (Q8_0, 1024, 3584, 3), (Q6_K, 256, 1, 1)])
def test_top1_matches_oracle_scan(gpu, oracle, t, in_dim, out_dim, tokens):
    rng = np.random.default_rng(out_dim + tokens)
    raw = synth.make_weights(rng, t, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    ids, vals, logits = run_top1(raw, t, x, in_dim, out_dim, tokens)
    want = oracle.matmul_add(x, tokens, in_dim, raw, t, out_dim, np.zeros(out_dim, dtype=np.float32), threads=8).reshape(tokens, out_dim)
    for tok in range(tokens):
        # the device's own logits decide ties and near-ties exactly; the oracle's winner must be within the GEMV tolerance
        assert ids[tok] == first_max(logits[tok]) or np.isclose(vals[tok], logits[tok].max(), rtol=2e-5, atol=0)
        top = float(want[tok].max())
        assert abs(float(vals[tok]) - top) <= 1e-4 * max(abs(top), float(np.abs(want[tok]).max()))
        assert want[tok][ids[tok]] >= top - 1e-4 * float(np.abs(want[tok]).max())


def test_top1_ties_take_the_lowest_row(gpu):
    """Rows with identical bytes give identical sums: the lowest row index must win, across wavefronts, workgroups and
    the strided final reduce."""
    rng = np.random.default_rng(1)
    in_dim, out_dim = 512, 20000          # 2500 row groups: every workgroup takes three or four of them
    base = synth.make_weights(rng, Q6_K, out_dim, in_dim).reshape(out_dim, -1)
    x = synth.make_activations(rng, 2, in_dim)
    _, _, logits = run_top1(np.ascontiguousarray(base).reshape(-1), Q6_K, x, in_dim, out_dim, 2)
    best = int(np.argmax(logits[0]))
    for dup in ([5, 2048 + 3, 5999], [4097, 1031], [19999, 12000], [best]):
        rows = base.copy()
        for r in dup:
            rows[r] = base[best]           # same bytes as the winning row
        ids, vals, lg = run_top1(np.ascontiguousarray(rows).reshape(-1), Q6_K, x, in_dim, out_dim, 2)
        assert ids[0] == min(dup + [best]) and vals[0] == lg[0].max()
        assert ids[1] == first_max(lg[1])
    # one row repeated everywhere: every partial result ties
    rows = np.repeat(base[:1], out_dim, axis=0)
    ids, _, _ = run_top1(np.ascontiguousarray(rows).reshape(-1), Q6_K, x, in_dim, out_dim, 2)
    assert list(ids) == [0, 0]


@pytest.mark.parametrize("t,in_dim,out_dim,tokens", [(Q6_K, 512, 70001, 4), (Q4_K, 2048, 20011, 3), (Q6_K, 1024, 3000, 4),
                                                     (Q4_K, 12288, 530, 3), (Q6_K, 256, 50, 3)])
def test_top1_on_the_matrix_cores(gpu, oracle, t, in_dim, out_dim, tokens):
    """Three and four tokens: the matrix-core kernel with the arg-max inside (where its workgroups fit the partial
    buffers), walking row groups for the tall shapes. Same bits as that kernel's logits, lowest row among equal values,
    winner within the GEMV tolerance of the oracle's."""
    rng = np.random.default_rng(out_dim * 3 + tokens)
    base = synth.make_weights(rng, t, out_dim, in_dim).reshape(out_dim, -1)
    x = synth.make_activations(rng, tokens, in_dim)
    ids, vals, logits = run_top1(np.ascontiguousarray(base).reshape(-1), t, x, in_dim, out_dim, tokens)
    assert "mfma" in quant.gemv_plan(t, tokens, in_dim, out_dim)[0]
    assert not 0 < quant.gemv_one_pass_from(t, in_dim, out_dim) <= tokens      # gemv_dev (the logits) runs that kernel too
    want = oracle.matmul_add(x, tokens, in_dim, base.reshape(-1), t, out_dim, np.zeros(out_dim, dtype=np.float32), threads=8).reshape(tokens, out_dim)
    for tok in range(tokens):
        assert ids[tok] == first_max(logits[tok]) and vals[tok] == logits[tok].max()
        top = float(want[tok].max())
        assert want[tok][ids[tok]] >= top - 1e-4 * float(np.abs(want[tok]).max())
    # ties: copies of token 0's winning row at lower and higher indices, in other tiles, row groups and workgroups
    best = int(ids[0])
    dup = sorted({out_dim - 1, out_dim // 2, min(best + 17, out_dim - 1), max(best - 1, 0), 3 % out_dim})
    rows = base.copy()
    for r in dup:
        rows[r] = base[best]
    ids2, vals2, lg2 = run_top1(np.ascontiguousarray(rows).reshape(-1), t, x, in_dim, out_dim, tokens)
    assert ids2[0] == min(dup + [best]) and vals2[0] == lg2[0].max()
    for tok in range(1, tokens):
        assert ids2[tok] == first_max(lg2[tok])
    rows = np.repeat(base[:1], out_dim, axis=0)
    ids3, _, _ = run_top1(np.ascontiguousarray(rows).reshape(-1), t, x, in_dim, out_dim, tokens)
    assert list(ids3) == [0] * tokens


@pytest.mark.parametrize("t,in_dim,out_dim,tokens", [(Q6_K, 2048, 70001, 8), (Q6_K, 4096, 3000, 3), (Q4_K, 4096, 20011, 5),
                                                     (Q4_K, 12288, 530, 4), (Q6_K, 6144, 50, 6), (Q4_K, 2048, 17, 8),
                                                     (Q6_K, 4096, 16 * 2 * 256 * 2 + 24, 7), (Q4_K, 4096, 4099, 13),
                                                     (Q6_K, 2048, 41000, 2), (Q4_K, 2048, 99001, 2), (Q4_K, 2048, 41000, 3)])
def test_top1_in_one_pass(gpu, oracle, t, in_dim, out_dim, tokens):
    """Up to eight tokens of a matrix the one-pass kernel takes: the weights once for the group, the arg-max inside
    (one, two and three tiles per wavefront, streamed long rows, workgroups that walk several row groups, a partial tile,
    13 tokens as eight and five, tall matrices from two and three tokens). Same bits as that kernel's logits, lowest row among equal values, winner within the GEMV
    tolerance of the oracle's."""
    rng = np.random.default_rng(out_dim * 5 + tokens)
    base = synth.make_weights(rng, t, out_dim, in_dim).reshape(out_dim, -1)
    x = synth.make_activations(rng, tokens, in_dim)
    ids, vals, logits = run_top1(np.ascontiguousarray(base).reshape(-1), t, x, in_dim, out_dim, tokens)
    assert 0 < quant.gemv_one_pass_from(t, in_dim, out_dim) <= min(tokens, 8)     # gemv_dev (the logits) goes one pass too
    want = oracle.matmul_add(x, tokens, in_dim, base.reshape(-1), t, out_dim, np.zeros(out_dim, dtype=np.float32), threads=8).reshape(tokens, out_dim)
    for tok in range(tokens):
        assert ids[tok] == first_max(logits[tok]) and vals[tok] == logits[tok].max(), tok
        top = float(want[tok].max())
        assert want[tok][ids[tok]] >= top - 1e-4 * float(np.abs(want[tok]).max())
    # ties: copies of token 0's winning row at lower and higher indices, in other tiles, row groups and workgroups
    best = int(ids[0])
    dup = sorted({out_dim - 1, out_dim // 2, min(best + 17, out_dim - 1), max(best - 1, 0), 3 % out_dim})
    rows = base.copy()
    for r in dup:
        rows[r] = base[best]
    ids2, vals2, lg2 = run_top1(np.ascontiguousarray(rows).reshape(-1), t, x, in_dim, out_dim, tokens)
    assert ids2[0] == min(dup + [best]) and vals2[0] == lg2[0].max()
    for tok in range(1, tokens):
        assert ids2[tok] == first_max(lg2[tok])
    rows = np.repeat(base[:1], out_dim, axis=0)
    ids3, _, _ = run_top1(np.ascontiguousarray(rows).reshape(-1), t, x, in_dim, out_dim, tokens)
    assert list(ids3) == [0] * tokens


@pytest.mark.parametrize("out_dim", [151936, 248320])
def test_full_size_heads(gpu, oracle, out_dim):
    """The vocabulary projections at their real sizes, Q6_K x 4096 columns: 151 936 rows (the configured head) and 248 320
    (Qwen3.5's, src/ml/gguf/qwen_output_head_runner.cr:895): one token on the vector ALU and eight in one pass, the
    arg-max inside. The winner is the first maximum of the same kernels' logits, the logits agree with the oracle on every
    row to the GEMV bars, and the oracle's value at the winner is its maximum up to the tolerance."""
    rng = np.random.default_rng(out_dim)
    in_dim = 4096
    raw = synth.make_weights(rng, Q6_K, out_dim, in_dim)
    dense_max = float(np.abs(oracle.dequantize(raw[:4096 * 16 * 210], Q6_K, 4096 * in_dim)).max())
    for tokens in (1, 8):
        x = synth.make_activations(rng, tokens, in_dim)
        ids, vals, logits = run_top1(raw, Q6_K, x, in_dim, out_dim, tokens)
        assert quant.gemv_passes(Q6_K, tokens, in_dim, out_dim) == 1
        want = oracle.matmul_add(x, tokens, in_dim, raw, Q6_K, out_dim, np.zeros(out_dim, dtype=np.float32), threads=16).reshape(tokens, out_dim)
        for tok in range(tokens):
            assert ids[tok] == first_max(logits[tok]) and vals[tok] == logits[tok].max(), (tokens, tok)
            scale = float(np.abs(want[tok]).max())
            err = float(np.abs(logits[tok].astype(np.float64) - want[tok]).max())
            assert err <= 1e-4 * float(np.linalg.norm(x[tok * in_dim:(tok + 1) * in_dim])) * dense_max
            assert err <= 2e-5 * scale, (tokens, tok, err, scale)
            assert want[tok][ids[tok]] >= float(want[tok].max()) - 2e-5 * scale


@pytest.mark.parametrize("hidden,vocab,tokens", [(1024, 20011, 4), (2048, 41003, 6), (4096, 3001, 8)])
def test_output_head_runner(gpu, oracle, hidden, vocab, tokens):
    """(1024 hidden values: the matrix-core kernel for the group of four; 2048 and 4096: the norm writes the activation image
    and the group goes through the one-pass kernel with the arg-max inside.)"""
    rng = np.random.default_rng(3 + hidden)
    w = Weights((1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float32), synth.make_weights(rng, Q6_K, vocab, hidden),
                Q6_K, hidden, vocab)
    xs = (rng.standard_normal(tokens * hidden) * 3).astype(np.float32)
    runner = QwenOutputHeadRunner.from_weights(w, tokens, xs, 1e-6, read_logits=True)
    stream = hip.HIPStream()
    try:
        runner.upload_weights()
        runner.reset_sequence()
        with hip.with_stream(stream):
            assert runner.run_repeated(2) == 2 * tokens
        stream.synchronize()
        runner.read_outputs()
        for tok in range(tokens):
            normed = oracle.rms_norm(xs[tok * hidden:(tok + 1) * hidden], w.norm, 1e-6)
            logits = oracle.matmul_add(normed, 1, hidden, w.output_raw, Q6_K, vocab, np.zeros(vocab, dtype=np.float32), threads=8)
            assert runner.top1_ids[tok] == first_max(logits)
            assert abs(runner.top1_values[tok] - logits.max()) <= 1e-4 * np.abs(logits).max()
            dev = runner.logits[tok * vocab:(tok + 1) * vocab]
            # (logits and top-1 of a group come from the same kernel family on the same operands: the same sums)
            assert runner.top1_ids[tok] == first_max(dev) and runner.top1_values[tok] == dev.max()
        # token-local path gives the same ids
        grouped = runner.top1_ids.copy()
        for tok in range(tokens):
            runner._run_token(tok)
        runner.read_outputs()
        assert np.array_equal(runner.top1_ids, grouped)
        with pytest.raises(ValueError, match="xs size mismatch"):
            runner.replace_sequence_input(xs[:-1])
    finally:
        runner.close()
        stream.close()


@pytest.mark.parametrize("t", [Q4_K, Q6_K])
def test_embedding_row_from_a_device_token_id(gpu, oracle, t):
    """The reference's token embedder (bin/cuda_mixed_stack_probe.cr:900-947): row token_ids[0] of the embedding matrix,
    bit-exact with the bulk dequantize; the id goes into the history; an id outside the vocabulary gives zeros."""
    hidden, vocab = 1024, 300
    rng = np.random.default_rng(int(t))
    raw = synth.make_weights(rng, t, vocab, hidden)
    table = oracle.dequantize(raw, t, vocab * hidden).reshape(vocab, hidden)
    wd, idd = DevArray(raw), DevArray(np.zeros(1, dtype=np.uint32))
    od, hd = DevArray(nbytes=4 * hidden), DevArray(np.full(8, 0xFFFFFFFF, dtype=np.uint32))
    try:
        for pos, tok in enumerate((0, 299, 17, 300, 4000000000)):
            hip.copy_htod(idd.ptr, np.array([tok], dtype=np.uint32), 4, "token id")
            quant.embed_dev(wd.ptr, t, idd.ptr, od.ptr, hd.ptr, pos, hidden, vocab)
            got = od.read(np.float32, hidden)
            want = table[tok] if tok < vocab else np.zeros(hidden, dtype=np.float32)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "token %d" % tok
        assert list(hd.read(np.uint32, 8)) == [0, 299, 17, 300, 4000000000, 0xFFFFFFFF, 0xFFFFFFFF, 0xFFFFFFFF]
        with pytest.raises(quant.QuantError, match="requires Q4_K or Q6_K token embeddings, got Q8_0"):
            quant.embed_dev(wd.ptr, Q8_0, idd.ptr, od.ptr, hd.ptr, 0, hidden, vocab)
        with pytest.raises(quant.QuantError, match="embedding dim 1000 must be divisible by 256"):
            quant.embed_dev(wd.ptr, t, idd.ptr, od.ptr, hd.ptr, 0, 1000, vocab)
    finally:
        for d in (wd, idd, od, hd):
            d.close()
