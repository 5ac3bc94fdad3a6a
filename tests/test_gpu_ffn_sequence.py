"""The resident FFN sequence (Q4_K gate/up -> SwiGLU -> Q6_K down, optional residual add) against the CPU form the
reference's probe checks it with (bin/cuda_ffn_sequence_probe.cr:254-266): per token, gate and up through
QuantMatmul.matmul_add, silu(gate) * up in float32, down through matmul_add with the residual row as bias."""
import numpy as np
import pytest

from cogni_ml_amd import hip, quant, synth
from cogni_ml_amd.ffn_sequence import FFNSequenceRunner
from gpu_common import gpu  # noqa: F401
from helpers import cosine

pytestmark = pytest.mark.gpu
Q4_K, Q6_K = 12, 14


@pytest.mark.parametrize("hidden,ffn_dim,tokens,residual_add", [(4096, 12288, 1, True), (4096, 12288, 4, True),
                                                               (512, 768, 1, False), (512, 768, 3, True), (1024, 256, 9, True)])
def test_ffn_sequence_matches_cpu_form(gpu, oracle, hidden, ffn_dim, tokens, residual_add):
    rng = np.random.default_rng(hidden + ffn_dim + tokens)
    gate_raw = synth.make_weights(rng, Q4_K, ffn_dim, hidden)
    up_raw = synth.make_weights(rng, Q4_K, ffn_dim, hidden)
    down_raw = synth.make_weights(rng, Q6_K, hidden, ffn_dim)
    xs = rng.uniform(-1.0, 1.0, tokens * hidden).astype(np.float32)            # the probe's input distribution
    residual = rng.uniform(-1.0, 1.0, tokens * hidden).astype(np.float32) if residual_add else None
    runner = FFNSequenceRunner(gate_raw, up_raw, down_raw, hidden, ffn_dim, tokens, xs, residual)
    stream = hip.HIPStream()
    try:
        runner.upload_weights()
        runner.reset_sequence()
        with hip.with_stream(stream):
            assert runner.run_repeated(2) == 2 * tokens
        stream.synchronize()
        runner.read_outputs()
        zero_f, zero_h = np.zeros(ffn_dim, dtype=np.float32), np.zeros(hidden, dtype=np.float32)
        for tok in range(tokens):
            x = xs[tok * hidden:(tok + 1) * hidden]
            gate = oracle.matmul_add(x, 1, hidden, gate_raw, Q4_K, ffn_dim, zero_f, threads=8)
            up = oracle.matmul_add(x, 1, hidden, up_raw, Q4_K, ffn_dim, zero_f, threads=8)
            combined = oracle.swiglu(gate, up)
            bias = residual[tok * hidden:(tok + 1) * hidden] if residual_add else zero_h
            want = oracle.matmul_add(combined, 1, ffn_dim, down_raw, Q6_K, hidden, bias, threads=8)
            got_c = runner.combined[tok * ffn_dim:(tok + 1) * ffn_dim]
            got = runner.out[tok * hidden:(tok + 1) * hidden]
            # more tokens than the router's threshold: the prefill GEMMs (operands rounded to binary16), else fp32 GEMVs
            bar = 4e-3 if tokens > quant.get_gemm_threshold() else 1e-4
            assert np.max(np.abs(got_c - combined)) <= bar * np.max(np.abs(combined)), "combined, token %d" % tok
            assert cosine(got, want) >= (0.9999 if bar > 1e-4 else 0.99999) and np.max(np.abs(got - want)) <= bar * np.max(np.abs(want)), "out, token %d" % tok
    finally:
        runner.close()
        stream.close()


@pytest.mark.parametrize("hidden,ffn_dim,tokens", [(1024, 1536, 1), (1024, 1536, 3), (2048, 2304, 5), (4096, 1024, 8),
                                                   (2048, 512, 11)])
def test_ffn_half_of_a_layer(gpu, oracle, hidden, ffn_dim, tokens):
    """r = x + attn_out; h = rmsnorm(r); out = r + down(silu(gate h) * up h) - src/ml/gguf/qwen35_cpu.cr:1705-1725.
    With 2048 or 4096 hidden values and several tokens the norm writes the activation image of gate | up itself."""
    rng = np.random.default_rng(77 + tokens + hidden)
    gate_raw = synth.make_weights(rng, Q4_K, ffn_dim, hidden)
    up_raw = synth.make_weights(rng, Q4_K, ffn_dim, hidden)
    down_raw = synth.make_weights(rng, Q6_K, hidden, ffn_dim)
    xs = rng.standard_normal(tokens * hidden).astype(np.float32)
    attn = rng.standard_normal(tokens * hidden).astype(np.float32)
    norm = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    runner = FFNSequenceRunner(gate_raw, up_raw, down_raw, hidden, ffn_dim, tokens, xs, norm=norm, add=attn, eps=1e-6)
    try:
        runner.upload_weights()
        runner.reset_sequence()
        runner.run_sequence()
        runner.read_outputs()
        zero_f = np.zeros(ffn_dim, dtype=np.float32)
        for tok in range(tokens):
            r = xs[tok * hidden:(tok + 1) * hidden] + attn[tok * hidden:(tok + 1) * hidden]
            h = oracle.rms_norm(r, norm, 1e-6)
            gate = oracle.matmul_add(h, 1, hidden, gate_raw, Q4_K, ffn_dim, zero_f, threads=8)
            up = oracle.matmul_add(h, 1, hidden, up_raw, Q4_K, ffn_dim, zero_f, threads=8)
            want = oracle.matmul_add(oracle.swiglu(gate, up), 1, ffn_dim, down_raw, Q6_K, hidden, r, threads=8)
            got = runner.out[tok * hidden:(tok + 1) * hidden]
            bar = 4e-3 if tokens > quant.get_gemm_threshold() else 1e-4
            assert cosine(got, want) >= (0.9999 if bar > 1e-4 else 0.99999) and np.max(np.abs(got - want)) <= bar * np.max(np.abs(want)), "token %d" % tok
        with pytest.raises(ValueError, match="norm and add go together"):
            FFNSequenceRunner(gate_raw, up_raw, down_raw, hidden, ffn_dim, tokens, xs, norm=norm)
    finally:
        runner.close()


@pytest.mark.parametrize("hidden,ffn_dim,tokens,block", [(1024, 1536, 64, False), (2048, 768, 130, True), (4096, 12288, 64, True),
                                                         (4096, 12288, 512, True), (4096, 12288, 512, False),
                                                         (4096, 12288, 16, True), (2048, 768, 9, False), (1024, 1536, 13, True)])
def test_prefill_form_of_the_ffn_block(gpu, oracle, hidden, ffn_dim, tokens, block):
    """More tokens than the GEMM threshold: pack, gate | up GEMM with SwiGLU inside, pack, down GEMM with the residual inside
    (block: add + RMSNorm in front, as in a decoder layer). A sample of tokens against the CPU form to the fp16-path bar, and
    the first eight tokens against the decode path of the same runner class (fp32 GEMVs) to the same bar. Up to sixteen tokens
    the block runs on the one-pass decode kernels with sixteen single-term tokens: the same bars."""
    rng = np.random.default_rng(5 * tokens + hidden)
    gate_raw = synth.make_weights(rng, Q4_K, ffn_dim, hidden)
    up_raw = synth.make_weights(rng, Q4_K, ffn_dim, hidden)
    down_raw = synth.make_weights(rng, Q6_K, hidden, ffn_dim)
    # (magnitudes that keep silu(gate) * up inside the binary16 range: the down GEMM takes its input as binary16, as the
    # reference's Metal prefill kernels do)
    xs = rng.uniform(-0.1, 0.1, tokens * hidden).astype(np.float32)
    other = rng.uniform(-1.0, 1.0, tokens * hidden).astype(np.float32)        # the residual, or the attention output
    norm = (0.1 + 0.01 * rng.standard_normal(hidden)).astype(np.float32)
    kw = dict(norm=norm, add=other) if block else dict(residual=other)
    runner = FFNSequenceRunner(gate_raw, up_raw, down_raw, hidden, ffn_dim, tokens, xs, **kw)
    small = FFNSequenceRunner(gate_raw, up_raw, down_raw, hidden, ffn_dim, 8, xs[:8 * hidden],
                              **{k: (v if k == "norm" else v[:8 * hidden]) for k, v in kw.items()})
    try:
        for r_ in (runner, small):
            r_.upload_weights()
            r_.reset_sequence()
            r_.run_sequence()
            r_.read_outputs()
        assert runner._ws_x is not None and small._ws_x is None
        zero_f = np.zeros(ffn_dim, dtype=np.float32)
        for tok in sorted(t_ for t_ in {0, 1, 7, 31, 32, tokens // 2, tokens - 1} if t_ < tokens):
            x = xs[tok * hidden:(tok + 1) * hidden]
            o = other[tok * hidden:(tok + 1) * hidden]
            r = x + o if block else o
            h = oracle.rms_norm(r, norm, 1e-6) if block else x
            gate = oracle.matmul_add(h, 1, hidden, gate_raw, Q4_K, ffn_dim, zero_f, threads=16)
            up = oracle.matmul_add(h, 1, hidden, up_raw, Q4_K, ffn_dim, zero_f, threads=16)
            want = oracle.matmul_add(oracle.swiglu(gate, up), 1, ffn_dim, down_raw, Q6_K, hidden, r, threads=16)
            got = runner.out[tok * hidden:(tok + 1) * hidden]
            assert cosine(got, want) >= 0.9999, tok
            assert np.max(np.abs(got - want)) <= 4e-3 * np.max(np.abs(want)), tok
        a, b = runner.out[:8 * hidden], small.out
        assert np.max(np.abs(a - b)) <= 4e-3 * np.max(np.abs(b))
        # without the fp32 products stored (they leave the gate | up GEMM as the down GEMM's packed input only): same bits
        lean = FFNSequenceRunner(gate_raw, up_raw, down_raw, hidden, ffn_dim, tokens, xs, keep_combined=False, **kw)
        try:
            lean.upload_weights()
            lean.reset_sequence()
            lean.run_sequence()
            lean.read_outputs()
            assert (lean.combined is None) == (tokens > 16) and runner.combined is not None
            assert np.array_equal(lean.out, runner.out)
        finally:
            lean.close()
    finally:
        runner.close()
        small.close()
