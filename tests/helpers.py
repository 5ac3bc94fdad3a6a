"""Shared helpers for the parity tests: hand-built blocks, comparison, special fp16 values."""
import numpy as np

F32, F16, Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL = 0, 1, 8, 12, 13, 14, 20
QUANT_TYPES = [Q8_0, Q4_K, Q5_K, Q6_K]
BLOCK = {Q8_0: (34, 32), Q4_K: (144, 256), Q5_K: (176, 256), Q6_K: (210, 256), IQ4_NL: (18, 32)}
D_OFFSET = {Q8_0: 0, Q4_K: 0, Q5_K: 0, Q6_K: 208, IQ4_NL: 0}
# zero, subnormals, smallest normal, largest finite, negative values
SPECIAL_F16 = [0x0000, 0x8000, 0x0001, 0x03FF, 0x8155, 0x0400, 0x7BFF, 0xFBFF, 0x3C00, 0xBC00]
NONFINITE_F16 = [0x7C00, 0xFC00, 0x7E00, 0xFE01, 0x7C01]


def f16_bytes(value_or_bits, bits=False):
    if bits:
        h = np.uint16(value_or_bits)
    else:
        h = np.array([value_or_bits], dtype=np.float16).view(np.uint16)[0]
    return [int(h) & 0xFF, int(h) >> 8]


def pack_scales(sc, m):
    """Inverse of the K-quant 6-bit packing: 8 (sc, m) pairs in [0, 63] -> 12 bytes."""
    s = np.zeros(12, dtype=np.uint8)
    for j in range(4):
        s[j] = (sc[j] & 63) | ((sc[j + 4] >> 4) << 6)
        s[j + 4] = (m[j] & 63) | ((m[j + 4] >> 4) << 6)
        s[j + 8] = (sc[j + 4] & 0x0F) | ((m[j + 4] & 0x0F) << 4)
    return s


def assert_bits_equal(got, want, what=""):
    """Bit-exact float32 comparison; NaN matches NaN regardless of sign and payload."""
    got = np.asarray(got, dtype=np.float32).reshape(-1)
    want = np.asarray(want, dtype=np.float32).reshape(-1)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    gn, wn = np.isnan(got), np.isnan(want)
    assert np.array_equal(gn, wn), "%s: NaN positions differ" % what
    a, b = got[~gn].view(np.uint32), want[~wn].view(np.uint32)
    if not np.array_equal(a, b):
        bad = np.flatnonzero(a != b)
        raise AssertionError("%s: %d of %d values differ, first at %d: got %r want %r" % (
            what, bad.size, a.size, bad[0], got[~gn][bad[0]], want[~wn][bad[0]]))


def inject_special_scales(raw, type_id, bits_list, rng):
    """Overwrite the fp16 d (and dmin) of randomly chosen blocks with the given bit patterns."""
    bb, _ = BLOCK[type_id]
    blocks = raw.reshape(-1, bb)
    idx = rng.choice(blocks.shape[0], size=min(len(bits_list) * 2, blocks.shape[0]), replace=False)
    for k, i in enumerate(idx):
        bits = bits_list[k % len(bits_list)]
        off = D_OFFSET[type_id] + (2 if (type_id in (Q4_K, Q5_K) and k >= len(bits_list)) else 0)
        blocks[i, off] = bits & 0xFF
        blocks[i, off + 1] = bits >> 8
    return raw


def cosine(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(a @ b / np.sqrt((a @ a) * (b @ b)))


def gemv_tolerance(x, w_dense, rows, in_dim):
    """Per-token bound 1e-4 * ||x||_2 * max|w_row| (max over the matrix's rows of max |w|)."""
    xx = np.asarray(x, dtype=np.float64).reshape(rows, in_dim)
    wmax = np.max(np.abs(w_dense), axis=1)          # (out_dim,)
    return 1e-4 * np.linalg.norm(xx, axis=1)[:, None] * wmax[None, :]
