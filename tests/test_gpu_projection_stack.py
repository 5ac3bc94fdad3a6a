"""The resident projection stack (q,k,v,o,gate,up Q4_K + down Q6_K at hidden 4096 / FFN 12288), M in {1,4,8}:
every projection's output against the oracle applied to the input that projection actually consumed."""
import numpy as np
import pytest

from cogni_ml_amd import hip, quant, synth
from cogni_ml_amd.projection_stack import QWEN_LAYER_4096, QwenProjectionStackRunner, Weights
from gpu_common import gpu  # noqa: F401
from helpers import cosine, gemv_tolerance

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def weights():
    return Weights.synthetic(np.random.default_rng(55))


@pytest.mark.parametrize("tokens,threshold", [(1, 8), (4, 8), (8, 8), (11, 64)])
def test_stack_matches_oracle(gpu, oracle, weights, tokens, threshold):
    """(11 tokens with the router's threshold raised: a group of eight and a group of three on the decode kernels)"""
    rng = np.random.default_rng(tokens)
    xs = synth.make_activations(rng, tokens, weights.hidden)
    quant.set_gemm_threshold(threshold)
    runner = QwenProjectionStackRunner.from_weights(weights, tokens, xs)
    stream = hip.HIPStream()
    try:
        assert not runner._prefill_ws
        runner.upload_weights()
        runner.reset_sequence()
        with hip.with_stream(stream):
            assert runner.run_repeated(2) == 2 * tokens
        stream.synchronize()
        runner.read_outputs()
        acts = {"x": xs}
        acts.update(runner.outputs)
        for name, src, t, out_dim, in_dim, raw in weights.entries:
            x_in = acts[src]
            want = oracle.matmul_add(x_in, tokens, in_dim, raw, int(t), out_dim, np.zeros(out_dim, dtype=np.float32), threads=16)
            dense = np.abs(oracle.dequantize(raw, int(t), out_dim * in_dim)).reshape(out_dim, in_dim)
            tol = gemv_tolerance(x_in, dense, tokens, in_dim).reshape(-1)
            err = np.abs(runner.outputs[name].astype(np.float64) - want)
            assert np.all(err <= tol), "%s M=%d: %g > %g" % (name, tokens, err.max(), tol[np.argmax(err)])
            assert cosine(runner.outputs[name], want) >= 0.99999
    finally:
        quant.set_gemm_threshold(8)
        runner.close()
        stream.close()


@pytest.mark.parametrize("tokens", [11, 16, 64, 200])
def test_prefill_route_of_the_stack(gpu, oracle, weights, tokens):
    """More tokens than the router's threshold: every distinct input packed once, every projection one GEMM over all the
    tokens (k-split where a projection has few tiles; lists of projections that share their input in one launch; up to sixteen
    tokens the Q4_K projections on the one-pass kernels with sixteen single-term tokens). Each projection against the oracle on the input it consumed, to
    the fp16-path bar; the active-token prefix below the threshold falls back to the decode kernels."""
    rng = np.random.default_rng(1000 + tokens)
    xs = synth.make_activations(rng, tokens, weights.hidden)
    runner = QwenProjectionStackRunner.from_weights(weights, tokens, xs)
    try:
        assert set(runner._prefill_ws) == {("x", "q45"), ("q", "q45"), ("gate", "q6")}
        runner.upload_weights()
        runner.reset_sequence()
        runner.run_sequence()
        runner.read_outputs()
        acts = {"x": xs}
        acts.update(runner.outputs)
        sample = sorted({0, 1, tokens // 2, tokens - 1})
        for name, src, t, out_dim, in_dim, raw in weights.entries:
            x_in = np.ascontiguousarray(acts[src].reshape(tokens, in_dim)[sample].reshape(-1))
            want = oracle.matmul_add(x_in, len(sample), in_dim, raw, int(t), out_dim, np.zeros(out_dim, dtype=np.float32), threads=16)
            got = runner.outputs[name].reshape(tokens, out_dim)[sample].reshape(-1)
            assert cosine(got, want) >= 0.9999, name
            assert np.max(np.abs(got - want)) <= 2e-3 * np.max(np.abs(want)), name
        prefill_k = runner.outputs["k"].copy()
        runner.active_tokens = 5
        runner.run_sequence()
        runner.read_outputs()
        k5 = runner.outputs["k"][:5 * 1024]
        assert not np.array_equal(k5, prefill_k[:5 * 1024])                         # other kernels: fp32 sums
        assert np.max(np.abs(k5 - prefill_k[:5 * 1024])) <= 2e-3 * np.max(np.abs(k5))
        assert runner.bytes_per_sequence(tokens) == weights.raw_bytes + 4 * tokens * sum(e[3] + e[4] for e in weights.entries)
    finally:
        runner.close()


def test_active_token_prefix_and_per_token_path(gpu, oracle, weights):
    tokens = 6
    xs = synth.make_activations(np.random.default_rng(9), tokens, weights.hidden)
    runner = QwenProjectionStackRunner.from_weights(weights, tokens, xs)
    try:
        runner.upload_weights()
        runner.reset_sequence()
        runner.active_tokens = 3
        runner.run_sequence()
        runner.read_outputs()
        grouped = runner.outputs["k"].copy()
        # token-local path: one launch per token gives the same values for the active prefix (another kernel
        # than the three-token launch, so up to the order of the fp32 additions)
        for tok in range(3):
            runner._run_token(tok)
        runner.read_outputs()
        single = runner.outputs["k"][:3 * 1024]
        assert np.max(np.abs(single - grouped[:3 * 1024])) <= 2e-5 * np.max(np.abs(single))
        with pytest.raises(ValueError, match="active_tokens must be <= tokens"):
            runner.active_tokens = 7
        runner.reset_active_tokens()
        assert runner.active_tokens == 6
        assert runner.bytes_per_sequence(1) == weights.raw_bytes + 4 * sum(e[3] + e[4] for e in weights.entries)
    finally:
        runner.close()


def test_layout_is_the_configured_layer():
    assert [(n, int(t), o, i) for n, s, t, o, i in QWEN_LAYER_4096] == [
        ("q", 12, 4096, 4096), ("k", 12, 1024, 4096), ("v", 12, 1024, 4096), ("o", 12, 4096, 4096),
        ("gate", 12, 12288, 4096), ("up", 12, 12288, 4096), ("down", 14, 4096, 12288)]
