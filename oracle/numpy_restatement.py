"""Independent vectorised numpy restatement of the GGUF block formats.

Test infrastructure. Written from the block-layout descriptions
(src/ml/gguf/dequant.cr:52, 103-104, 144-145, 195-196 and
src/ml/gguf/kernels/gemm_q56k.metal:8-9), not from oracle/quant_oracle.c, so
that an indexing slip in one of the two shows up as a mismatch. Every float32
operation below rounds once (numpy never fuses multiply and add).
"""
import numpy as np

f32 = np.float32
np_err = np.errstate(invalid="ignore", over="ignore")  # inf * 0 in blocks with non-finite scales is expected


def _f16(col_pair):
    """(nb, 2) uint8 little-endian binary16 -> (nb,) float32 (IEEE exact)."""
    return np.ascontiguousarray(col_pair).view("<f2").astype(f32).reshape(-1)


def scale_min_k4(scales):
    """(nb, 12) uint8 -> (sc, m) each (nb, 8) uint8.

    Uses the 16-bit-word formulation of the packing (pairs of 6-bit fields
    handled as one uint16, as in gemm_q4k.metal:180-183) instead of the
    byte-wise form in dequant.cr:240-249.
    """
    s16 = np.ascontiguousarray(scales).view("<u2").astype(np.uint32)  # (nb, 6): bytes (0,1)(2,3)...(10,11)
    sc = np.empty((scales.shape[0], 8), dtype=np.uint8)
    m = np.empty_like(sc)
    for p in range(2):  # sub-block pairs (0,1), (2,3): plain low 6 bits
        w_sc = s16[:, p] & 0x3F3F
        w_m = s16[:, p + 2] & 0x3F3F
        sc[:, 2 * p], sc[:, 2 * p + 1] = w_sc & 0xFF, w_sc >> 8
        m[:, 2 * p], m[:, 2 * p + 1] = w_m & 0xFF, w_m >> 8
    for p in range(2):  # sub-block pairs (4,5), (6,7): 4 bits from bytes 8..11, top 2 bits from bytes 0..7
        w_sc = (s16[:, p + 4] & 0x0F0F) | ((s16[:, p] & 0xC0C0) >> 2)
        w_m = ((s16[:, p + 4] & 0xF0F0) >> 4) | ((s16[:, p + 2] & 0xC0C0) >> 2)
        sc[:, 4 + 2 * p], sc[:, 5 + 2 * p] = w_sc & 0xFF, w_sc >> 8
        m[:, 4 + 2 * p], m[:, 5 + 2 * p] = w_m & 0xFF, w_m >> 8
    return sc, m


@np_err
def dequantize_q8_0(data, n):
    nb = (n + 31) // 32
    b = np.frombuffer(data, dtype=np.uint8, count=nb * 34).reshape(nb, 34)
    d = _f16(b[:, 0:2])[:, None]
    q = b[:, 2:34].view(np.int8).astype(f32)
    return (d * q).reshape(-1)[:n].copy()


@np_err
def dequantize_q4_k(data, n):
    nb = n // 256
    b = np.frombuffer(data, dtype=np.uint8, count=nb * 144).reshape(nb, 144)
    d, dmin = _f16(b[:, 0:2])[:, None], _f16(b[:, 2:4])[:, None]
    sc, m = scale_min_k4(b[:, 4:16])
    dsc = d * sc.astype(f32)      # (nb, 8), rounded once
    dm = dmin * m.astype(f32)
    qs = b[:, 16:144].reshape(nb, 4, 32)
    y = np.zeros((nb, 4, 2, 32), dtype=f32)
    y[:, :, 0, :] = dsc[:, 0::2, None] * (qs & 0x0F).astype(f32) - dm[:, 0::2, None]
    y[:, :, 1, :] = dsc[:, 1::2, None] * (qs >> 4).astype(f32) - dm[:, 1::2, None]
    out = np.zeros(n, dtype=f32)
    out[: nb * 256] = y.reshape(-1)
    return out


@np_err
def dequantize_q5_k(data, n):
    nb = n // 256
    b = np.frombuffer(data, dtype=np.uint8, count=nb * 176).reshape(nb, 176)
    d, dmin = _f16(b[:, 0:2])[:, None], _f16(b[:, 2:4])[:, None]
    sc, m = scale_min_k4(b[:, 4:16])
    dsc = d * sc.astype(f32)
    dm = dmin * m.astype(f32)
    qh = b[:, 16:48]                       # (nb, 32): bit 2g -> low half of group g, bit 2g+1 -> high half
    ql = b[:, 48:176].reshape(nb, 4, 32)
    g = np.arange(4)[None, :, None]
    bit_lo = ((qh[:, None, :] >> (2 * g)) & 1).astype(np.uint8)
    bit_hi = ((qh[:, None, :] >> (2 * g + 1)) & 1).astype(np.uint8)
    q_lo = (ql & 0x0F) + 16 * bit_lo
    q_hi = (ql >> 4) + 16 * bit_hi
    y = np.zeros((nb, 4, 2, 32), dtype=f32)
    y[:, :, 0, :] = dsc[:, 0::2, None] * q_lo.astype(f32) - dm[:, 0::2, None]
    y[:, :, 1, :] = dsc[:, 1::2, None] * q_hi.astype(f32) - dm[:, 1::2, None]
    out = np.zeros(n, dtype=f32)
    out[: nb * 256] = y.reshape(-1)
    return out


@np_err
def dequantize_q6_k(data, n):
    nb = n // 256
    b = np.frombuffer(data, dtype=np.uint8, count=nb * 210).reshape(nb, 210)
    ql = b[:, 0:128].reshape(nb, 2, 2, 32)    # [half][byte row 0/1][l]
    qh = b[:, 128:192].reshape(nb, 2, 32)     # [half][l]
    sc = b[:, 192:208].view(np.int8).reshape(nb, 2, 4, 2).astype(f32)  # [half][quarter][l // 16]
    d = _f16(b[:, 208:210])[:, None, None, None]
    y = np.zeros((nb, 2, 4, 32), dtype=f32)
    for k in range(4):                         # quarter k: elements 128*half + 32*k + l
        nib = ql[:, :, k % 2, :]
        low4 = (nib & 0x0F) if k < 2 else (nib >> 4)
        hi2 = (qh >> (2 * k)) & 3
        q = (low4 | (hi2 << 4)).astype(np.int32) - 32
        s = np.repeat(sc[:, :, k, :], 16, axis=-1)              # (nb, 2, 32)
        y[:, :, k, :] = (d[:, :, 0, :] * s) * q.astype(f32)
    out = np.zeros(n, dtype=f32)
    out[: nb * 256] = y.reshape(-1)
    return out


_IQ4_NL = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], dtype=f32)


@np_err
def dequantize_iq4_nl(data, n):
    nb = (n + 31) // 32
    b = np.frombuffer(data, dtype=np.uint8, count=nb * 18).reshape(nb, 18)
    d = _f16(b[:, 0:2])[:, None]
    qs = b[:, 2:18]
    y = np.concatenate([d * _IQ4_NL[qs & 0x0F], d * _IQ4_NL[qs >> 4]], axis=1)
    return y.reshape(-1)[:n].copy()


def dequantize_f16(data, n):
    return np.frombuffer(data, dtype="<f2", count=n).astype(f32)


def dequantize_f32(data, n):
    return np.frombuffer(data, dtype="<f4", count=n).copy()


DEQUANT = {0: dequantize_f32, 1: dequantize_f16, 8: dequantize_q8_0, 12: dequantize_q4_k,
           13: dequantize_q5_k, 14: dequantize_q6_k, 20: dequantize_iq4_nl}


def matmul_dense_f64(x, rows, in_dim, w_raw, w_type, out_dim, bias):
    """Bulk dequantize, then a float64 dense product (the invariant of spec/q4k_matmul_spec.cr:15-34)."""
    w = DEQUANT[w_type](np.ascontiguousarray(w_raw, dtype=np.uint8).tobytes(), out_dim * in_dim)
    w = w.reshape(out_dim, in_dim).astype(np.float64)
    xx = np.asarray(x, dtype=np.float32).reshape(rows, in_dim).astype(np.float64)
    return (xx @ w.T + np.asarray(bias, dtype=np.float32).astype(np.float64)[None, :]).astype(f32).reshape(-1)
