"""ctypes binding of oracle/liboracle.so (quant_oracle.c).

Test infrastructure: imported only by tests/, the smoke check and the
benchmark's cpu_baseline leg. Function names follow the reference:
Dequant.dequantize (src/ml/gguf/dequant.cr:19) and
QuantMatmul.matmul_add (src/ml/gguf/quant_matmul.cr:20).
"""
import ctypes
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

# ggml tensor type ids (src/ml/gguf/reader.cr:34-49)
F32, F16, Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL = 0, 1, 8, 12, 13, 14, 20
TYPE_NAMES = {F32: "F32", F16: "F16", Q8_0: "Q8_0", Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K", IQ4_NL: "IQ4_NL"}


def build(force=False):
    """Compile liboracle.so with oracle/Makefile."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        u8p, f32p = ctypes.c_void_p, ctypes.c_void_p
        L.oracle_fp16_to_f32.restype = ctypes.c_float
        L.oracle_fp16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_get_scale_min_k4.restype = None
        L.oracle_get_scale_min_k4.argtypes = [ctypes.c_int, u8p, ctypes.POINTER(ctypes.c_float),
                                              ctypes.POINTER(ctypes.c_float)]
        L.oracle_dequantize.restype = ctypes.c_int
        L.oracle_dequantize.argtypes = [u8p, ctypes.c_uint32, ctypes.c_int, f32p]
        L.oracle_matmul_add.restype = ctypes.c_int
        L.oracle_matmul_add.argtypes = [f32p, ctypes.c_int, ctypes.c_int, u8p, ctypes.c_uint32, ctypes.c_int,
                                        f32p, f32p]
        L.oracle_matmul_add_range.restype = ctypes.c_int
        L.oracle_matmul_add_range.argtypes = L.oracle_matmul_add.argtypes + [ctypes.c_int, ctypes.c_int]
        for name in ("oracle_block_bytes", "oracle_block_elements"):
            getattr(L, name).restype = ctypes.c_int
            getattr(L, name).argtypes = [ctypes.c_uint32]
        L.oracle_swiglu.restype = None
        L.oracle_swiglu.argtypes = [f32p, f32p, ctypes.c_void_p, ctypes.c_int64]
        L.oracle_rms_norm.restype = None
        L.oracle_rms_norm.argtypes = [f32p, f32p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_float]
        L.oracle_data_bytes.restype = ctypes.c_int64
        L.oracle_data_bytes.argtypes = [ctypes.c_uint32, ctypes.c_int64]
        _lib = L
    return _lib


def _u8(a):
    a = np.ascontiguousarray(a, dtype=np.uint8)
    return a, a.ctypes.data


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data


def fp16_to_f32(h):
    return np.float32(lib().oracle_fp16_to_f32(int(h) & 0xFFFF))


def get_scale_min_k4(j, scales):
    s, sp = _u8(scales)
    sc, m = ctypes.c_float(), ctypes.c_float()
    lib().oracle_get_scale_min_k4(int(j), sp, ctypes.byref(sc), ctypes.byref(m))
    return np.float32(sc.value), np.float32(m.value)


def block_bytes(t):
    return lib().oracle_block_bytes(t)


def block_elements(t):
    return lib().oracle_block_elements(t)


def data_bytes(t, n):
    return lib().oracle_data_bytes(t, n)


def dequantize(data, type_id, n_elements):
    """Dequant.dequantize(data, type, n_elements) -> float32[n]."""
    d, dp = _u8(data)
    out = np.empty(int(n_elements), dtype=np.float32)
    rc = lib().oracle_dequantize(dp, type_id, int(n_elements), out.ctypes.data)
    if rc != 0:
        raise ValueError("Unsupported dequantization type: %s" % type_id)
    return out


def matmul_add(x, rows, in_dim, w_raw, w_type, out_dim, bias, threads=1):
    """QuantMatmul.matmul_add(x, rows, in_dim, w_raw, w_type, out_dim, bias) -> float32[rows*out_dim].

    threads > 1 splits the output rows over host threads (same arithmetic per
    output element; used only to time a multi-core CPU baseline).
    """
    xa, xp = _f32(x)
    wa, wp = _u8(w_raw)
    ba, bp = _f32(bias)
    assert xa.size >= rows * in_dim and ba.size >= out_dim
    res = np.empty(rows * out_dim, dtype=np.float32)
    L = lib()
    if threads <= 1:
        rc = L.oracle_matmul_add(xp, rows, in_dim, wp, w_type, out_dim, bp, res.ctypes.data)
    else:
        bounds = np.linspace(0, out_dim, threads + 1).astype(int)
        with ThreadPoolExecutor(threads) as ex:
            rcs = list(ex.map(lambda i: L.oracle_matmul_add_range(
                xp, rows, in_dim, wp, w_type, out_dim, bp, res.ctypes.data, int(bounds[i]), int(bounds[i + 1])),
                range(threads)))
        rc = min(rcs)
    if rc != 0:
        raise ValueError("Unsupported quant type for fused matmul: %s" % w_type)
    return res


def swiglu(gate, up):
    """silu(gate) * up in float32, as the reference's FFN probe checks it (bin/cuda_ffn_sequence_probe.cr:189-191)."""
    ga, gp = _f32(gate)
    ua, up_p = _f32(up)
    assert ga.size == ua.size
    out = np.empty(ga.size, dtype=np.float32)
    lib().oracle_swiglu(gp, up_p, out.ctypes.data, ctypes.c_int64(ga.size))
    return out


def rms_norm(x, w, eps=1.0e-6):
    """RMSNorm of one vector (src/ml/gguf/qwen35_cpu.cr:484-490): float64 sum of squares, float32 scaling."""
    xa, xp = _f32(x)
    wa, wp = _f32(w)
    assert xa.size == wa.size
    out = np.empty(xa.size, dtype=np.float32)
    lib().oracle_rms_norm(xp, wp, out.ctypes.data, ctypes.c_int64(xa.size), ctypes.c_float(eps))
    return out
