"""Weights out of a GGUF file into the operators: load_qw / load_f32 (src/ml/gguf/qwen35_weights.cr:203-218) and
read_tensor_f32 (reader.cr:162-166) against the oracle on the same bytes."""
import numpy as np
import pytest

import gguf_writer as gw
from cogni_ml_amd import gguf, synth
from gpu_common import gpu  # noqa: F401
from helpers import gemv_tolerance

pytestmark = pytest.mark.gpu


def test_quant_weights_and_norms_from_a_gguf_file(gpu, oracle, tmp_path):
    rng = np.random.default_rng(8)
    hidden, ffn = 512, 768
    gate = synth.make_weights(rng, 12, ffn, hidden)
    down = synth.make_weights(rng, 14, hidden, ffn)
    head = synth.make_weights(rng, 8, 300, hidden)
    norm = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    half = rng.standard_normal(96).astype(np.float16)
    path = str(tmp_path / "layer.gguf")
    gw.write_gguf(path, [("general.architecture", gw.STRING, "qwen35")],
                  [("blk.0.ffn_gate.weight", [hidden, ffn], 12, gate.tobytes()),
                   ("blk.0.ffn_down.weight", [ffn, hidden], 14, down.tobytes()),
                   ("output.weight", [hidden, 300], 8, head.tobytes()),
                   ("blk.0.post_attention_norm.weight", [hidden], 0, norm.tobytes()),
                   ("half.weight", [96], 1, half.tobytes())])
    with gguf.GGUFFile(path) as g:
        assert np.array_equal(gguf.load_f32(g, "blk.0.post_attention_norm.weight"), norm)
        assert np.array_equal(gguf.load_f32(g, "half.weight"), half.astype(np.float32))
        info = g.tensor("blk.0.ffn_down.weight")
        assert np.array_equal(g.read_tensor_f32(info), oracle.dequantize(down, 14, hidden * ffn))     # bit-exact
        x = synth.make_activations(rng, 2, hidden)
        for name, raw, t, out_dim, in_dim in (("blk.0.ffn_gate.weight", gate, 12, ffn, hidden),
                                              ("output.weight", head, 8, 300, hidden)):
            qw = gguf.load_qw(g, name)
            try:
                assert (int(qw.type), qw.out_dim, qw.in_dim, qw.route_tag) == (t, out_dim, in_dim, "qwen35:" + name)
                got = qw.matmul(x, rows=2)
                want = oracle.matmul_add(x, 2, in_dim, raw, t, out_dim, np.zeros(out_dim, dtype=np.float32))
                dense = np.abs(oracle.dequantize(raw, t, out_dim * in_dim)).reshape(out_dim, in_dim)
                assert np.all(np.abs(got - want) <= gemv_tolerance(x, dense, 2, in_dim).reshape(-1))
            finally:
                qw.close()
        with pytest.raises(gguf.GGUFError, match="missing tensor"):
            gguf.load_qw(g, "blk.1.ffn_gate.weight")
