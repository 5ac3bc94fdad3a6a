"""Pins fp16_to_f32 (dequant.cr:252-283) and get_scale_min_k4 (dequant.cr:240-249)."""
import json
import os

import numpy as np

from oracle import numpy_restatement as npr

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "iq4_nl_vectors.json")))


def test_fp16_exhaustive_against_ieee(oracle):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([oracle.fp16_to_f32(int(v)) for v in h], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))  # bit exact incl. -0.0, subnormals
    # the reference canonicalises every NaN to Float32::NAN: sign and payload are dropped
    assert np.all(got[nan].view(np.uint32) == 0x7FC00000)


def test_fp16_reference_constants(oracle):
    for hx, val in GOLD["fp16_constants"].items():
        assert oracle.fp16_to_f32(int(hx, 16)) == np.float32(val)
    assert oracle.fp16_to_f32(0x0001) == np.float32(2.0 ** -24)       # smallest subnormal
    assert oracle.fp16_to_f32(0x03FF) == np.float32(1023 * 2.0 ** -24)
    assert oracle.fp16_to_f32(0x7BFF) == np.float32(65504.0)
    assert np.signbit(oracle.fp16_to_f32(0x8000)) and oracle.fp16_to_f32(0x8000) == 0.0


def pack_scales(sc, m):
    """Inverse of the K-quant 6-bit packing: 8 (sc, m) pairs in [0, 63] -> 12 bytes."""
    s = np.zeros(12, dtype=np.uint8)
    for j in range(4):
        s[j] = (sc[j] & 63) | ((sc[j + 4] >> 4) << 6)
        s[j + 4] = (m[j] & 63) | ((m[j + 4] >> 4) << 6)
        s[j + 8] = (sc[j + 4] & 0x0F) | ((m[j + 4] & 0x0F) << 4)
    return s


def test_scale_min_inverse_packing(oracle):
    rng = np.random.default_rng(7)
    cases = [rng.integers(0, 64, size=(2, 8)) for _ in range(300)]
    # walking ones / single-field cases: every field alone takes every 6-bit value
    for field in range(16):
        for v in (1, 2, 4, 8, 16, 32, 63):
            c = np.zeros((2, 8), dtype=np.int64)
            c[field // 8, field % 8] = v
            cases.append(c)
    for c in cases:
        sc, m = c[0], c[1]
        s = pack_scales(sc, m)
        for j in range(8):
            a, b = oracle.get_scale_min_k4(j, s)
            assert (a, b) == (np.float32(sc[j]), np.float32(m[j])), (j, c)


def test_scale_min_matches_16bit_word_form(oracle):
    rng = np.random.default_rng(11)
    s = rng.integers(0, 256, size=(500, 12), dtype=np.uint8)
    sc, m = npr.scale_min_k4(s)
    for i in range(s.shape[0]):
        for j in range(8):
            a, b = oracle.get_scale_min_k4(j, s[i])
            assert a == sc[i, j] and b == m[i, j]
