"""GPU dequantize kernels vs the CPU oracle: bit-exact float32 (NaN compares as NaN)."""
import numpy as np
import pytest

from cogni_ml_amd import hip, quant, synth
from gpu_common import DevArray, gpu  # noqa: F401
from helpers import (BLOCK, F16, F32, IQ4_NL, NONFINITE_F16, Q4_K, Q5_K, Q6_K, Q8_0, SPECIAL_F16, assert_bits_equal,
                     f16_bytes, inject_special_scales)

pytestmark = pytest.mark.gpu
BLOCKED = [Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL]


@pytest.mark.parametrize("type_id", BLOCKED)
def test_random_and_special_blocks_bit_exact(gpu, oracle, type_id):
    rng = np.random.default_rng(500 + type_id)
    bb, be = BLOCK[type_id]
    rows, in_dim = 96, be * 24
    raw = synth.make_weights(rng, type_id, rows, in_dim)
    raw = inject_special_scales(raw, type_id, SPECIAL_F16 + NONFINITE_F16, rng)
    n = rows * in_dim
    assert_bits_equal(quant.dequantize(raw, type_id, n), oracle.dequantize(raw, type_id, n), "type %d" % type_id)


@pytest.mark.parametrize("type_id", BLOCKED)
@pytest.mark.parametrize("n_blocks,extra", [(1, 0), (3, 1), (5, 17), (9, 255), (0, 7)])
def test_ragged_lengths(gpu, oracle, type_id, n_blocks, extra):
    """n that ends inside a block: the K-quants leave the partial block zero, Q8_0/IQ4_NL clip it."""
    rng = np.random.default_rng(n_blocks * 31 + extra)
    bb, be = BLOCK[type_id]
    extra = extra % be
    n = n_blocks * be + extra
    raw = synth.make_weights(rng, type_id, 1, (n_blocks + 1) * be)
    got = quant.dequantize(raw, type_id, n)
    assert got.size == n
    assert_bits_equal(got, oracle.dequantize(raw, type_id, n), "type %d n=%d" % (type_id, n))


def test_empty_input(gpu):
    for t in BLOCKED + [F16, F32]:
        assert quant.dequantize(np.zeros(0, dtype=np.uint8), t, 0).size == 0


def test_f16_every_bit_pattern_and_f32_copy(gpu, oracle):
    h = np.arange(65536, dtype=np.uint16)
    assert_bits_equal(quant.dequantize(h.view(np.uint8), F16, 65536), oracle.dequantize(h.view(np.uint8), F16, 65536))
    # canonical NaN, as the reference's fp16_to_f32 returns Float32::NAN for every NaN input
    got = quant.dequantize(h.view(np.uint8), F16, 65536)
    nan = np.isnan(got)
    assert np.all(got[nan].view(np.uint32) == 0x7FC00000)
    assert_bits_equal(quant.dequantize(h[:1001].view(np.uint8), F16, 1001), oracle.dequantize(h[:1001].view(np.uint8), F16, 1001))
    v = np.random.default_rng(1).standard_normal(1003).astype(np.float32)
    assert np.array_equal(quant.dequantize(v.view(np.uint8), F32, 1003), v)


def test_reference_iq4_nl_vectors(gpu):
    """spec/iq4_nl_dequant_spec.cr:34-68 on the GPU kernel."""
    kv = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=np.float32)
    blk = lambda bits, rule: f16_bytes(bits, bits=True) + [rule(j) for j in range(16)]
    raw = np.array(blk(0x3C00, lambda j: j | ((15 - j) << 4)) + blk(0xB800, lambda j: 0x08), dtype=np.uint8)
    out = quant.dequantize(raw, IQ4_NL, 32)
    assert np.array_equal(out[:16], kv) and np.array_equal(out[16:], kv[::-1])
    out = quant.dequantize(raw, IQ4_NL, 40)
    assert out.size == 40 and (out[0], out[15], out[16], out[31]) == (-127.0, 113.0, 113.0, -127.0)
    assert np.array_equal(out[32:], np.full(8, -0.5, dtype=np.float32))


def test_size_check_and_unsupported_type(gpu):
    with pytest.raises(quant.QuantError, match="needs 288") as e:
        quant.dequantize(np.zeros(144, dtype=np.uint8), Q4_K, 512)
    assert e.value.code == -1
    with pytest.raises(quant.QuantError, match="Unsupported dequantization type"):
        quant.dequantize(np.zeros(84, dtype=np.uint8), 10, 256)


@pytest.mark.parametrize("type_id,out_dim,in_dim", [(Q8_0, 3584, 1024), (Q4_K, 12288, 4096), (Q5_K, 4096, 4096),
                                                     (Q6_K, 4096, 12288)])
def test_configured_shapes_bit_exact(gpu, oracle, type_id, out_dim, in_dim):
    """Whole weight matrices at the benchmark's shapes, bit-exact against the oracle."""
    rng = np.random.default_rng(900 + type_id)
    raw = synth.make_weights(rng, type_id, out_dim, in_dim)
    n = out_dim * in_dim
    assert_bits_equal(quant.dequantize(raw, type_id, n), oracle.dequantize(raw, type_id, n))


def test_kernel_by_name_through_the_driver_layer(gpu, oracle):
    """The path a Crystal ML::HIP binding takes: module -> function by name -> boxed params -> launch."""
    import ctypes
    rng = np.random.default_rng(3)
    raw = synth.make_weights(rng, Q4_K, 8, 1024)
    n = 8 * 1024
    mod = hip.HIPModule.load_builtin()
    fn = mod.function(quant.dequantize_kernel_name(Q4_K))
    assert fn.attribute(hip.FunctionAttribute.NumRegs) > 0
    assert fn.attribute(hip.FunctionAttribute.LocalSizeBytes) == 0     # no register spills
    w, out = DevArray(raw), DevArray(nbytes=4 * n)
    params = hip.KernelParams(ctypes.c_uint64(w.ptr), ctypes.c_uint64(out.ptr), ctypes.c_uint64(n))
    stream = hip.HIPStream()
    with hip.with_stream(stream):
        hip.launch(fn, 8, 1, 1, 256, 1, 1, params, fn.name)
    stream.synchronize()
    assert_bits_equal(out.read(np.float32, n), oracle.dequantize(raw, Q4_K, n))
    with pytest.raises(hip.HIPError, match="hipModuleGetFunction\\(no_such_kernel\\) failed with HIP error"):
        mod.function("no_such_kernel")
    for o in (w, out, stream, mod):
        o.close()
    mod.close()      # close is idempotent
