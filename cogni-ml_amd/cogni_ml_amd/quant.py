"""QuantMatmul / Dequant on the GPU: Python (ctypes) binding of the operator layer in libcogni_hip.so.

Signatures follow the reference's CPU operators so a caller switches by renaming the module:
  dequantize(data, type, n_elements)                              src/ml/gguf/dequant.cr:19
  matmul_add(x, rows, in_dim, w_raw, w_type, out_dim, bias)       src/ml/gguf/quant_matmul.cr:20
  QuantWeight(raw, type, out_dim, in_dim, route_tag)              src/ml/gguf/compute.cr:20-30
"""
import ctypes

import numpy as np

from . import hip
from .types import TensorType

MAX_GEMV_TOKENS = 8


class QuantError(RuntimeError):
    def __init__(self, code):
        self.code = code
        super().__init__(hip.lib().cogni_last_error().decode())


def _check(code):
    if code != 0:
        raise QuantError(code)


def init(ordinal=0):
    """Load the gfx950 code object on device `ordinal`. Raises if there is no such GPU."""
    _check(hip.lib().cogni_quant_init(ordinal))


def shutdown():
    _check(hip.lib().cogni_quant_shutdown())


def gemv_kernel_name(w_type, tokens=1, add=False):
    n = hip.lib().cogni_gemv_kernel_name(int(w_type), tokens, int(add))
    return n.decode() if n else None


def dequantize_kernel_name(w_type):
    n = hip.lib().cogni_dequantize_kernel_name(int(w_type))
    return n.decode() if n else None


def gemv_launch_dims(w_type, tokens, in_dim, out_dim):
    """(grid_x, block_x, shared_mem_bytes) of the GEMV kernel for this type, token count and shape."""
    g, b, s = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint32()
    _check(hip.lib().cogni_gemv_launch_dims(int(w_type), tokens, in_dim, out_dim, ctypes.byref(g), ctypes.byref(b),
                                            ctypes.byref(s)))
    return g.value, b.value, s.value


def gemv_plan(w_type, tokens, in_dim, out_dim, add=False):
    """(kernel_name, grid_x, block_x, shared_mem_bytes) the library launches for this shape."""
    k = ctypes.c_char_p()
    g, b, s = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint32()
    _check(hip.lib().cogni_gemv_plan(int(w_type), tokens, int(add), in_dim, out_dim, ctypes.byref(k), ctypes.byref(g),
                                     ctypes.byref(b), ctypes.byref(s)))
    return k.value.decode(), g.value, b.value, s.value


def dequantize_dev(w_ptr, w_type, n_elements, out_ptr, stream=None):
    _check(hip.lib().cogni_dequantize_dev(ctypes.c_uint64(w_ptr), ctypes.c_uint32(int(w_type)),
                                          ctypes.c_uint64(n_elements), ctypes.c_uint64(out_ptr), stream))


def gemv_dev(w_ptr, w_type, x_ptr, out_ptr, in_dim, out_dim, tokens=1, residual_ptr=0, stream=None):
    _check(hip.lib().cogni_gemv_dev(ctypes.c_uint64(w_ptr), ctypes.c_uint32(int(w_type)), ctypes.c_uint64(x_ptr),
                                    ctypes.c_uint64(residual_ptr), ctypes.c_uint64(out_ptr), ctypes.c_uint32(in_dim),
                                    ctypes.c_uint32(out_dim), ctypes.c_uint32(tokens), stream))


def gemv_many_dev(w_ptrs, w_type, x_ptr, out_ptrs, out_dims, in_dim, tokens=1, stream=None):
    """Several matrices of one type and in_dim against the same activations (q | k | v): the qmatvec_many seam on
    device pointers."""
    n = len(w_ptrs)
    if len(out_ptrs) != n or len(out_dims) != n:
        raise ValueError("w_ptrs, out_ptrs and out_dims must have the same length")
    U64, U32 = ctypes.c_uint64 * n, ctypes.c_uint32 * n
    _check(hip.lib().cogni_gemv_many_dev(U64(*w_ptrs), ctypes.c_uint32(int(w_type)), ctypes.c_uint64(x_ptr), U64(*out_ptrs),
                                         U32(*out_dims), ctypes.c_uint32(n), ctypes.c_uint32(in_dim), ctypes.c_uint32(tokens),
                                         stream))


def gemv_one_pass_from(w_type, in_dim, out_dim):
    """Token count from which gemv_dev packs the activations and reads the weights once (0: never for this shape)."""
    f = hip.lib().cogni_gemv_one_pass_from
    f.restype = ctypes.c_uint32
    return int(f(ctypes.c_uint32(int(w_type)), ctypes.c_uint32(in_dim), ctypes.c_uint32(out_dim)))


def gemv_one_pass_multi_from(w_type, in_dim):
    """The same for pairs, lists and the fused gate | up | SwiGLU (0: never for this row length)."""
    f = hip.lib().cogni_gemv_one_pass_multi_from
    f.restype = ctypes.c_uint32
    return int(f(ctypes.c_uint32(int(w_type)), ctypes.c_uint32(in_dim)))


def gemv_image_stats():
    """(slots, in use, pinned by a capture, multi-token calls that found no slot) of the library's activation images."""
    a, b, c, d = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint64()
    _check(hip.lib().cogni_gemv_image_stats(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c), ctypes.byref(d)))
    return a.value, b.value, c.value, d.value


def gemv_passes(w_type, tokens, in_dim, out_dim):
    """Passes over the weights gemv_dev makes for such a call (-1: refused)."""
    f = hip.lib().cogni_gemv_passes
    f.restype = ctypes.c_int32
    return f(ctypes.c_uint32(int(w_type)), ctypes.c_uint32(tokens), ctypes.c_uint32(in_dim), ctypes.c_uint32(out_dim))


def gemv_image_bytes(w_type, in_dim, tokens):
    """Bytes of the activation image of the one-pass multi-token GEMV; 0 = no such kernel for the combination."""
    f = hip.lib().cogni_gemv_image_bytes
    f.restype = ctypes.c_size_t
    return f(ctypes.c_uint32(int(w_type)), ctypes.c_uint32(in_dim), ctypes.c_uint32(tokens))


def gemv_packed_launch_dims(w_type, in_dim, total_rows):
    """(grid_x, block_x, shared_mem_bytes) of the one-pass kernel for a launch of total_rows rows."""
    g, b, sh = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint32()
    _check(hip.lib().cogni_gemv_packed_launch_dims(ctypes.c_uint32(int(w_type)), ctypes.c_uint32(in_dim), ctypes.c_uint32(total_rows),
                                                   ctypes.byref(g), ctypes.byref(b), ctypes.byref(sh)))
    return g.value, b.value, sh.value


def gemv_pack_dev(x_ptr, w_type, in_dim, tokens, image_ptr, stream=None):
    """x[tokens][in_dim] (fp32) -> the image gemv_packed_dev reads."""
    _check(hip.lib().cogni_gemv_pack_dev(ctypes.c_uint64(x_ptr), ctypes.c_uint32(int(w_type)), ctypes.c_uint32(in_dim),
                                         ctypes.c_uint32(tokens), ctypes.c_uint64(image_ptr), stream))


def gemv_packed_dev(w_ptrs, w_type, image_ptr, out_ptrs, out_dims, in_dim, tokens, residual_ptr=0, stream=None):
    """Up to 8 matrices against one packed activation block of 2..8 tokens, the weights read once for all tokens."""
    n = len(w_ptrs)
    if len(out_ptrs) != n or len(out_dims) != n:
        raise ValueError("w_ptrs, out_ptrs and out_dims must have the same length")
    U64, U32 = ctypes.c_uint64 * n, ctypes.c_uint32 * n
    _check(hip.lib().cogni_gemv_packed_dev(U64(*w_ptrs), ctypes.c_uint32(int(w_type)), ctypes.c_uint64(image_ptr),
                                           ctypes.c_uint64(residual_ptr), U64(*out_ptrs), U32(*out_dims), ctypes.c_uint32(n),
                                           ctypes.c_uint32(in_dim), ctypes.c_uint32(tokens), stream))


def gemv_packed_swiglu_dev(w_gate_ptr, w_up_ptr, w_type, image_ptr, out_ptr, in_dim, out_dim, tokens, stream=None):
    """out = silu(x W_gate^T) * (x W_up^T) against a packed activation block of 2..8 tokens, one launch."""
    _check(hip.lib().cogni_gemv_packed_swiglu_dev(ctypes.c_uint64(w_gate_ptr), ctypes.c_uint64(w_up_ptr),
                                                  ctypes.c_uint32(int(w_type)), ctypes.c_uint64(image_ptr),
                                                  ctypes.c_uint64(out_ptr), ctypes.c_uint32(in_dim), ctypes.c_uint32(out_dim),
                                                  ctypes.c_uint32(tokens), stream))


def gemv_dual_dev(w_a_ptr, w_b_ptr, w_type, x_ptr, out_a_ptr, out_b_ptr, in_dim, out_dim, tokens=1, stream=None):
    """Two matrices of one shape against the same activations (gate | up, k | v)."""
    _check(hip.lib().cogni_gemv_dual_dev(ctypes.c_uint64(w_a_ptr), ctypes.c_uint64(w_b_ptr), ctypes.c_uint32(int(w_type)),
                                         ctypes.c_uint64(x_ptr), ctypes.c_uint64(out_a_ptr), ctypes.c_uint64(out_b_ptr),
                                         ctypes.c_uint32(in_dim), ctypes.c_uint32(out_dim), ctypes.c_uint32(tokens), stream))


def swiglu_dev(gate_ptr, up_ptr, out_ptr, n, stream=None):
    _check(hip.lib().cogni_swiglu_dev(ctypes.c_uint64(gate_ptr), ctypes.c_uint64(up_ptr), ctypes.c_uint64(out_ptr),
                                      ctypes.c_uint32(n), stream))


def gemv_dual_swiglu_dev(w_gate_ptr, w_up_ptr, w_type, x_ptr, out_ptr, in_dim, out_dim, tokens=1, stream=None):
    """out = silu(x W_gate^T) * (x W_up^T) in one launch (Q4_K)."""
    _check(hip.lib().cogni_gemv_dual_swiglu_dev(ctypes.c_uint64(w_gate_ptr), ctypes.c_uint64(w_up_ptr),
                                                ctypes.c_uint32(int(w_type)), ctypes.c_uint64(x_ptr), ctypes.c_uint64(out_ptr),
                                                ctypes.c_uint32(in_dim), ctypes.c_uint32(out_dim), ctypes.c_uint32(tokens),
                                                stream))


def embed_dev(w_ptr, w_type, token_ids_ptr, output_ptr, history_ptr, token_index, hidden_dim, vocab_size, stream=None):
    """output = dequantized embedding row token_ids[0]; history[token_index] = token_ids[0] (Q4_K, Q6_K)."""
    _check(hip.lib().cogni_embed_dev(ctypes.c_uint64(w_ptr), ctypes.c_uint32(int(w_type)), ctypes.c_uint64(token_ids_ptr),
                                     ctypes.c_uint64(output_ptr), ctypes.c_uint64(history_ptr), ctypes.c_uint32(token_index),
                                     ctypes.c_uint32(hidden_dim), ctypes.c_uint32(vocab_size), stream))


def gemv_top1_partials(w_type, out_dim):
    f = hip.lib().cogni_gemv_top1_partials
    f.restype = ctypes.c_uint32
    return f(ctypes.c_uint32(int(w_type)), ctypes.c_uint32(out_dim))


def gemv_top1_dev(w_ptr, w_type, x_ptr, partial_ids_ptr, partial_values_ptr, top1_ids_ptr, top1_values_ptr, in_dim, out_dim,
                  tokens=1, stream=None):
    """Index and value of the largest element of W x per token; partial_* hold tokens * gemv_top1_partials() elements."""
    _check(hip.lib().cogni_gemv_top1_dev(ctypes.c_uint64(w_ptr), ctypes.c_uint32(int(w_type)), ctypes.c_uint64(x_ptr),
                                         ctypes.c_uint64(partial_ids_ptr), ctypes.c_uint64(partial_values_ptr),
                                         ctypes.c_uint64(top1_ids_ptr), ctypes.c_uint64(top1_values_ptr),
                                         ctypes.c_uint32(in_dim), ctypes.c_uint32(out_dim), ctypes.c_uint32(tokens), stream))


TOP1_NOALLOC_MAX_PARTIALS = 65536


def gemv_packed_top1_dev(w_ptr, w_type, image_ptr, partial_ids_ptr, partial_values_ptr, top1_ids_ptr, top1_values_ptr, in_dim, out_dim,
                         tokens, stream=None):
    """Top-1 of up to 8 tokens against a packed activation image (one pass over the weights, arg-max inside, reduce)."""
    _check(hip.lib().cogni_gemv_packed_top1_dev(ctypes.c_uint64(w_ptr), ctypes.c_uint32(int(w_type)), ctypes.c_uint64(image_ptr),
                                                ctypes.c_uint64(partial_ids_ptr), ctypes.c_uint64(partial_values_ptr),
                                                ctypes.c_uint64(top1_ids_ptr), ctypes.c_uint64(top1_values_ptr),
                                                ctypes.c_uint32(in_dim), ctypes.c_uint32(out_dim), ctypes.c_uint32(tokens), stream))


def gemv_top1_noalloc_dev(w_ptr, w_type, x_ptr, top1_ids_ptr, top1_values_ptr, in_dim, out_dim, tokens=1, stream=None):
    """gemv_top1_dev with the partial results in the library's static device array: allocates nothing. Fails when
    tokens * gemv_top1_partials() exceeds TOP1_NOALLOC_MAX_PARTIALS; calls that overlap on one GPU race."""
    _check(hip.lib().cogni_gemv_top1_noalloc_dev(ctypes.c_uint64(w_ptr), ctypes.c_uint32(int(w_type)), ctypes.c_uint64(x_ptr),
                                                 ctypes.c_uint64(top1_ids_ptr), ctypes.c_uint64(top1_values_ptr),
                                                 ctypes.c_uint32(in_dim), ctypes.c_uint32(out_dim), ctypes.c_uint32(tokens),
                                                 stream))


def rmsnorm_dev(x_ptr, norm_ptr, out_ptr, dim, tokens=1, eps=1.0e-6, stream=None):
    _check(hip.lib().cogni_rmsnorm_dev(ctypes.c_uint64(x_ptr), ctypes.c_uint64(norm_ptr), ctypes.c_uint64(out_ptr),
                                       ctypes.c_uint32(dim), ctypes.c_uint32(tokens), ctypes.c_float(eps), stream))


def add_rmsnorm_dev(x_ptr, add_ptr, norm_ptr, residual_out_ptr, normed_out_ptr, dim, tokens=1, eps=1.0e-6, stream=None):
    """residual_out = x + add; normed_out = rmsnorm(residual_out)."""
    _check(hip.lib().cogni_add_rmsnorm_dev(ctypes.c_uint64(x_ptr), ctypes.c_uint64(add_ptr), ctypes.c_uint64(norm_ptr),
                                           ctypes.c_uint64(residual_out_ptr), ctypes.c_uint64(normed_out_ptr),
                                           ctypes.c_uint32(dim), ctypes.c_uint32(tokens), ctypes.c_float(eps), stream))


def rmsnorm_pack_dev(x_ptr, norm_ptr, out_ptr, w_type, image_ptr, dim, tokens, eps=1.0e-6, stream=None):
    """rmsnorm_dev that also writes the normalised rows as the one-pass GEMV's activation image (out_ptr may be 0)."""
    _check(hip.lib().cogni_rmsnorm_pack_dev(ctypes.c_uint64(x_ptr), ctypes.c_uint64(norm_ptr), ctypes.c_uint64(out_ptr),
                                            ctypes.c_uint32(int(w_type)), ctypes.c_uint64(image_ptr), ctypes.c_uint32(dim),
                                            ctypes.c_uint32(tokens), ctypes.c_float(eps), stream))


def add_rmsnorm_pack_dev(x_ptr, add_ptr, norm_ptr, residual_out_ptr, normed_out_ptr, w_type, image_ptr, dim, tokens, eps=1.0e-6,
                         stream=None):
    """add_rmsnorm_dev that also writes the normalised rows as the one-pass GEMV's activation image (normed_out_ptr may be 0)."""
    _check(hip.lib().cogni_add_rmsnorm_pack_dev(ctypes.c_uint64(x_ptr), ctypes.c_uint64(add_ptr), ctypes.c_uint64(norm_ptr),
                                                ctypes.c_uint64(residual_out_ptr), ctypes.c_uint64(normed_out_ptr),
                                                ctypes.c_uint32(int(w_type)), ctypes.c_uint64(image_ptr), ctypes.c_uint32(dim),
                                                ctypes.c_uint32(tokens), ctypes.c_float(eps), stream))


def rmsnorm_pack16_dev(x_ptr, norm_ptr, out_ptr, w_type, image_ptr, dim, tokens, eps=1.0e-6, stream=None):
    """rmsnorm_dev that writes the normalised rows as the image of the sixteen-token one-pass kernels (out_ptr may be 0)."""
    _check(hip.lib().cogni_rmsnorm_pack16_dev(ctypes.c_uint64(x_ptr), ctypes.c_uint64(norm_ptr), ctypes.c_uint64(out_ptr),
                                              ctypes.c_uint32(int(w_type)), ctypes.c_uint64(image_ptr), ctypes.c_uint32(dim),
                                              ctypes.c_uint32(tokens), ctypes.c_float(eps), stream))


def add_rmsnorm_pack16_dev(x_ptr, add_ptr, norm_ptr, residual_out_ptr, normed_out_ptr, w_type, image_ptr, dim, tokens, eps=1.0e-6,
                           stream=None):
    """add_rmsnorm_dev that writes the normalised rows as the image of the sixteen-token one-pass kernels (normed_out_ptr may be 0)."""
    _check(hip.lib().cogni_add_rmsnorm_pack16_dev(ctypes.c_uint64(x_ptr), ctypes.c_uint64(add_ptr), ctypes.c_uint64(norm_ptr),
                                                  ctypes.c_uint64(residual_out_ptr), ctypes.c_uint64(normed_out_ptr),
                                                  ctypes.c_uint32(int(w_type)), ctypes.c_uint64(image_ptr), ctypes.c_uint32(dim),
                                                  ctypes.c_uint32(tokens), ctypes.c_float(eps), stream))


def rmsnorm_gemm_pack_dev(x_ptr, norm_ptr, out_ptr, w_type, workspace_ptr, workspace_bytes, dim, tokens, eps=1.0e-6, stream=None):
    """rmsnorm_dev whose rows leave as the packed activations of the prefill GEMMs (what gemm_pack_dev would write); out_ptr may be 0."""
    _check(hip.lib().cogni_rmsnorm_gemm_pack_dev(ctypes.c_uint64(x_ptr), ctypes.c_uint64(norm_ptr), ctypes.c_uint64(out_ptr),
                                                 ctypes.c_uint32(int(w_type)), ctypes.c_uint64(workspace_ptr), ctypes.c_size_t(workspace_bytes),
                                                 ctypes.c_uint32(dim), ctypes.c_uint32(tokens), ctypes.c_float(eps), stream))


def add_rmsnorm_gemm_pack_dev(x_ptr, add_ptr, norm_ptr, residual_out_ptr, normed_out_ptr, w_type, workspace_ptr, workspace_bytes, dim,
                              tokens, eps=1.0e-6, stream=None):
    """add_rmsnorm_dev whose normalised rows leave as the packed activations of the prefill GEMMs; normed_out_ptr may be 0."""
    _check(hip.lib().cogni_add_rmsnorm_gemm_pack_dev(
        ctypes.c_uint64(x_ptr), ctypes.c_uint64(add_ptr), ctypes.c_uint64(norm_ptr), ctypes.c_uint64(residual_out_ptr),
        ctypes.c_uint64(normed_out_ptr), ctypes.c_uint32(int(w_type)), ctypes.c_uint64(workspace_ptr), ctypes.c_size_t(workspace_bytes),
        ctypes.c_uint32(dim), ctypes.c_uint32(tokens), ctypes.c_float(eps), stream))

def gemm_workspace_bytes(w_type, in_dim, tokens, out_dim=None):
    """Bytes of caller-owned scratch for gemm_dev: the packed activations, and with `out_dim` given also the planes of
    a k-split launch (few tiles), which gemm_dev uses when the workspace has room for them."""
    if out_dim is None:
        f = hip.lib().cogni_gemm_workspace_bytes
        f.restype = ctypes.c_size_t
        return f(ctypes.c_uint32(int(w_type)), ctypes.c_uint32(in_dim), ctypes.c_uint32(tokens))
    f = hip.lib().cogni_gemm_workspace_bytes_split
    f.restype = ctypes.c_size_t
    return f(ctypes.c_uint32(int(w_type)), ctypes.c_uint32(in_dim), ctypes.c_uint32(out_dim), ctypes.c_uint32(tokens))


def gemm_dev(w_ptr, w_type, x_ptr, out_ptr, in_dim, out_dim, tokens, workspace_ptr, workspace_bytes, bias_ptr=0,
             stream=None):
    _check(hip.lib().cogni_gemm_dev(ctypes.c_uint64(w_ptr), ctypes.c_uint32(int(w_type)), ctypes.c_uint64(x_ptr),
                                    ctypes.c_uint64(bias_ptr), ctypes.c_uint64(out_ptr), ctypes.c_uint32(in_dim),
                                    ctypes.c_uint32(out_dim), ctypes.c_uint32(tokens), ctypes.c_uint64(workspace_ptr),
                                    ctypes.c_size_t(workspace_bytes), stream))


def gemm_plan(w_type, in_dim, out_dim, tokens, workspace_bytes):
    """(kernel name, grid_x, k splits, block) of the launch gemm_packed_dev makes for this shape and workspace size."""
    name = ctypes.c_char_p()
    gx, gy, bx = ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint32()
    _check(hip.lib().cogni_gemm_plan(ctypes.c_uint32(int(w_type)), ctypes.c_uint32(in_dim), ctypes.c_uint32(out_dim),
                                     ctypes.c_uint32(tokens), ctypes.c_size_t(workspace_bytes), ctypes.byref(name),
                                     ctypes.byref(gx), ctypes.byref(gy), ctypes.byref(bx)))
    return name.value.decode(), gx.value, gy.value, bx.value


def gemm_pack_dev(x_ptr, w_type, in_dim, tokens, workspace_ptr, workspace_bytes, stream=None):
    """The first half of gemm_dev: the activations as packed fp16 at the head of the workspace (shared by every projection of
    one type family that reads them)."""
    _check(hip.lib().cogni_gemm_pack_dev(ctypes.c_uint64(x_ptr), ctypes.c_uint32(int(w_type)), ctypes.c_uint32(in_dim),
                                         ctypes.c_uint32(tokens), ctypes.c_uint64(workspace_ptr), ctypes.c_size_t(workspace_bytes),
                                         stream))


def gemm_packed_dev(w_ptr, w_type, workspace_ptr, workspace_bytes, out_ptr, in_dim, out_dim, tokens, bias_ptr=0, stream=None):
    """The second half of gemm_dev: one matrix against activations gemm_pack_dev has packed."""
    _check(hip.lib().cogni_gemm_packed_dev(ctypes.c_uint64(w_ptr), ctypes.c_uint32(int(w_type)), ctypes.c_uint64(workspace_ptr),
                                           ctypes.c_size_t(workspace_bytes), ctypes.c_uint64(bias_ptr), ctypes.c_uint64(out_ptr),
                                           ctypes.c_uint32(in_dim), ctypes.c_uint32(out_dim), ctypes.c_uint32(tokens), stream))


def gemm_packed_add_dev(w_ptr, w_type, workspace_ptr, workspace_bytes, residual_ptr, out_ptr, in_dim, out_dim, tokens, stream=None):
    """gemm_packed_dev with a [tokens][out_dim] residual added (it may be the output buffer itself)."""
    _check(hip.lib().cogni_gemm_packed_add_dev(ctypes.c_uint64(w_ptr), ctypes.c_uint32(int(w_type)), ctypes.c_uint64(workspace_ptr),
                                               ctypes.c_size_t(workspace_bytes), ctypes.c_uint64(residual_ptr), ctypes.c_uint64(out_ptr),
                                               ctypes.c_uint32(in_dim), ctypes.c_uint32(out_dim), ctypes.c_uint32(tokens), stream))


def gemm_packed_swiglu_dev(w_gate_ptr, w_up_ptr, w_type, workspace_ptr, workspace_bytes, out_ptr, in_dim, out_dim, tokens, stream=None):
    """silu(x W_gate^T) * (x W_up^T) in one GEMM launch against packed activations (Q4_K)."""
    _check(hip.lib().cogni_gemm_packed_swiglu_dev(ctypes.c_uint64(w_gate_ptr), ctypes.c_uint64(w_up_ptr), ctypes.c_uint32(int(w_type)),
                                                  ctypes.c_uint64(workspace_ptr), ctypes.c_size_t(workspace_bytes), ctypes.c_uint64(out_ptr),
                                                  ctypes.c_uint32(in_dim), ctypes.c_uint32(out_dim), ctypes.c_uint32(tokens), stream))


def gemv_pack16_dev(x_ptr, w_type, in_dim, tokens, image_ptr, stream=None):
    """The activation image of the sixteen-token one-pass kernels (one binary16 term per token), gemv_image_bytes(type, in_dim, 8) bytes."""
    _check(hip.lib().cogni_gemv_pack16_dev(ctypes.c_uint64(x_ptr), ctypes.c_uint32(int(w_type)), ctypes.c_uint32(in_dim),
                                           ctypes.c_uint32(tokens), ctypes.c_uint64(image_ptr), stream))


def gemv_packed16_dev(w_ptrs, w_type, image_ptr, out_ptrs, out_dims, in_dim, tokens, residual_ptr=0, stream=None):
    """Up to eight Q4_K, Q5_K or Q6_K matrices against a sixteen-token image, 1..16 tokens in one pass over the weights (a
    [tokens][out_dim] residual with a single matrix)."""
    n = len(w_ptrs)
    if not (n == len(out_ptrs) == len(out_dims)):
        raise ValueError("w_ptrs, out_ptrs and out_dims must have one entry per matrix")
    _check(hip.lib().cogni_gemv_packed16_dev((ctypes.c_uint64 * n)(*w_ptrs), ctypes.c_uint32(int(w_type)), ctypes.c_uint64(image_ptr),
                                             ctypes.c_uint64(residual_ptr), (ctypes.c_uint64 * n)(*out_ptrs), (ctypes.c_uint32 * n)(*out_dims), ctypes.c_uint32(n),
                                             ctypes.c_uint32(in_dim), ctypes.c_uint32(tokens), stream))


def gemv_packed16_swiglu_dev(w_gate_ptr, w_up_ptr, w_type, image_ptr, out_ptr, in_dim, out_dim, tokens, stream=None):
    """silu(gate . x) * (up . x) for up to sixteen tokens against a sixteen-token image (Q4_K), one pass over both matrices."""
    _check(hip.lib().cogni_gemv_packed16_swiglu_dev(ctypes.c_uint64(w_gate_ptr), ctypes.c_uint64(w_up_ptr), ctypes.c_uint32(int(w_type)),
                                                    ctypes.c_uint64(image_ptr), ctypes.c_uint64(out_ptr), ctypes.c_uint32(in_dim),
                                                    ctypes.c_uint32(out_dim), ctypes.c_uint32(tokens), stream))


def gemm_packed_many_dev(w_ptrs, w_type, workspace_ptr, workspace_bytes, out_ptrs, out_dims, in_dim, tokens, stream=None):
    """One GEMM launch for up to six matrices of one type and row length against the same packed activations (no k split)."""
    n = len(w_ptrs)
    if not (n == len(out_ptrs) == len(out_dims)):
        raise ValueError("w_ptrs, out_ptrs and out_dims must have one entry per matrix")
    _check(hip.lib().cogni_gemm_packed_many_dev((ctypes.c_uint64 * n)(*w_ptrs), ctypes.c_uint32(int(w_type)), ctypes.c_uint64(workspace_ptr),
                                                ctypes.c_size_t(workspace_bytes), (ctypes.c_uint64 * n)(*out_ptrs),
                                                (ctypes.c_uint32 * n)(*out_dims), ctypes.c_uint32(n), ctypes.c_uint32(in_dim),
                                                ctypes.c_uint32(tokens), stream))


def gemm_packed_swiglu_pack_dev(w_gate_ptr, w_up_ptr, w_type, workspace_ptr, workspace_bytes, out_ptr, next_type, next_workspace_ptr,
                                next_workspace_bytes, in_dim, out_dim, tokens, stream=None):
    """gemm_packed_swiglu_dev whose products also (out_ptr 0: only) leave as the packed activations of the next GEMM."""
    _check(hip.lib().cogni_gemm_packed_swiglu_pack_dev(
        ctypes.c_uint64(w_gate_ptr), ctypes.c_uint64(w_up_ptr), ctypes.c_uint32(int(w_type)), ctypes.c_uint64(workspace_ptr),
        ctypes.c_size_t(workspace_bytes), ctypes.c_uint64(out_ptr), ctypes.c_uint32(int(next_type)), ctypes.c_uint64(next_workspace_ptr),
        ctypes.c_size_t(next_workspace_bytes), ctypes.c_uint32(in_dim), ctypes.c_uint32(out_dim), ctypes.c_uint32(tokens), stream))


def matmul_dev(w_ptr, w_type, x_ptr, out_ptr, in_dim, out_dim, tokens, workspace_ptr=0, workspace_bytes=0, bias_ptr=0,
               stream=None):
    """The GEMV/GEMM router (tokens > threshold and Q4_K -> GEMM)."""
    _check(hip.lib().cogni_matmul_dev(ctypes.c_uint64(w_ptr), ctypes.c_uint32(int(w_type)), ctypes.c_uint64(x_ptr),
                                      ctypes.c_uint64(bias_ptr), ctypes.c_uint64(out_ptr), ctypes.c_uint32(in_dim),
                                      ctypes.c_uint32(out_dim), ctypes.c_uint32(tokens),
                                      ctypes.c_uint64(workspace_ptr), ctypes.c_size_t(workspace_bytes), stream))


def set_gemm_threshold(tokens):
    _check(hip.lib().cogni_set_gemm_threshold(ctypes.c_int32(tokens)))


def get_gemm_threshold():
    return hip.lib().cogni_get_gemm_threshold()


def dequantize(data, w_type, n_elements):
    """Dequant.dequantize: raw bytes -> float32[n_elements], computed on the GPU."""
    d = np.ascontiguousarray(np.frombuffer(data, dtype=np.uint8) if not isinstance(data, np.ndarray) else data,
                             dtype=np.uint8)
    out = np.empty(int(n_elements), dtype=np.float32)
    _check(hip.lib().cogni_dequantize(ctypes.c_void_p(d.ctypes.data), ctypes.c_size_t(d.size),
                                      ctypes.c_uint32(int(w_type)), ctypes.c_int64(int(n_elements)),
                                      ctypes.c_void_p(out.ctypes.data)))
    return out


def matmul_add(x, rows, in_dim, w_raw, w_type, out_dim, bias):
    """QuantMatmul.matmul_add: float32[rows*out_dim] = bias + x @ deq(W)^T, computed on the GPU."""
    xa = np.ascontiguousarray(x, dtype=np.float32)
    wa = np.ascontiguousarray(w_raw, dtype=np.uint8)
    ba = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
    if xa.size < rows * in_dim:
        raise ValueError("x has %d elements, rows*in_dim is %d" % (xa.size, rows * in_dim))
    if ba is not None and ba.size < out_dim:
        raise ValueError("bias has %d elements, out_dim is %d" % (ba.size, out_dim))
    res = np.empty(rows * out_dim, dtype=np.float32)
    _check(hip.lib().cogni_matmul_add(ctypes.c_void_p(xa.ctypes.data), ctypes.c_int32(rows), ctypes.c_int32(in_dim),
                                      ctypes.c_void_p(wa.ctypes.data), ctypes.c_size_t(wa.size),
                                      ctypes.c_uint32(int(w_type)), ctypes.c_int32(out_dim),
                                      ctypes.c_void_p(ba.ctypes.data if ba is not None else None),
                                      ctypes.c_void_p(res.ctypes.data)))
    return res


class QuantWeight:
    """compute.cr:20-45: {raw, type, out_dim, in_dim, route_tag} plus the resident device copy."""

    def __init__(self, raw, w_type, out_dim, in_dim, route_tag=None):
        self.raw = np.ascontiguousarray(raw, dtype=np.uint8)
        self.type, self.out_dim, self.in_dim, self.route_tag = TensorType(int(w_type)), out_dim, in_dim, route_tag
        self._handle = ctypes.c_void_p()
        _check(hip.lib().cogni_weight_create(ctypes.byref(self._handle), ctypes.c_void_p(self.raw.ctypes.data),
                                             ctypes.c_size_t(self.raw.size), ctypes.c_uint32(int(w_type)),
                                             ctypes.c_int32(out_dim), ctypes.c_int32(in_dim)))

    @property
    def device_ptr(self):
        return hip.lib().cogni_weight_device_ptr(self._handle)

    def matmul(self, x, rows=1, bias=None):
        xa = np.ascontiguousarray(x, dtype=np.float32)
        ba = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        if rows <= 0:
            raise ValueError("rows must be positive, got %d" % rows)
        if xa.size < rows * self.in_dim:   # the library copies rows*in_dim floats from this buffer
            raise ValueError("x has %d elements, rows*in_dim is %d" % (xa.size, rows * self.in_dim))
        if ba is not None and ba.size < self.out_dim:
            raise ValueError("bias has %d elements, out_dim is %d" % (ba.size, self.out_dim))
        res = np.empty(rows * self.out_dim, dtype=np.float32)
        _check(hip.lib().cogni_weight_matmul(self._handle, ctypes.c_void_p(xa.ctypes.data), ctypes.c_int32(rows),
                                             ctypes.c_void_p(ba.ctypes.data if ba is not None else None),
                                             ctypes.c_void_p(res.ctypes.data)))
        return res

    def close(self):
        if self._handle:
            hip.lib().cogni_weight_destroy(self._handle)
            self._handle = None


def matvec_many(qws, x):
    """qmatvec_many(qws, x) (qwen35_cpu.cr:1419-1445): every weight against the same one-token x in one call; a list of
    float32 arrays, one per weight, [] for no weights."""
    qws = list(qws)
    if not qws:
        return []
    xa = np.ascontiguousarray(x, dtype=np.float32)
    if xa.size != qws[0].in_dim:
        raise ValueError("matvec_many x size mismatch: expected %d, got %d" % (qws[0].in_dim, xa.size))
    outs = [np.empty(q.out_dim, dtype=np.float32) for q in qws]
    handles = (ctypes.c_void_p * len(qws))(*[q._handle for q in qws])
    ptrs = (ctypes.c_void_p * len(qws))(*[o.ctypes.data for o in outs])
    _check(hip.lib().cogni_weight_matvec_many(handles, ctypes.c_int32(len(qws)), ctypes.c_void_p(xa.ctypes.data), ptrs))
    return outs
