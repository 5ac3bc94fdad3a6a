"""Resident FFN sequence on one HIP stream: Q4_K gate and up GEMVs -> SwiGLU -> Q6_K down GEMV (+ residual).

The HIP counterpart of the reference's FFN sequence probe (bin/cuda_ffn_sequence_probe.cr:3, 254-266 for the
CPU form, 314-440 for the launches): weights and activations stay on the device, the lifecycle goes through
ResidentSequenceRunner. Where the reference launches gate, up, the activation and down as four kernels per token,
a group of up to four tokens here is two launches (gate | up | SwiGLU fused, then down with the residual add); an FFN width
that is not a multiple of 16 goes through the weight-stationary kernels for several tokens (gate | up pair, swiglu_f32, down).

A sequence of more tokens than the GEMM threshold (quant.get_gemm_threshold()) is the prefill form of the same block, all
tokens at once in three launches: the activations packed (by the add + RMSNorm in front, where there is one), gate | up as
one GEMM with SwiGLU in its epilogue, which also writes its products as the packed fp16 activations of the down matrix's
layout, and the down GEMM with the residual added in its epilogue (src/ml/gguf/qwen35_cpu.cr:1711-1722; the reference's Metal kernels gemm_q4k.metal:1233 and gemm_mm.metal:651).
Up to sixteen tokens take the one-pass decode kernels with sixteen single-term tokens instead (gate | up as one list, SwiGLU,
down with the residual: every matrix read once, at the GEMM's precision class).
`keep_combined=False` leaves the fp32 products (`combined`, the probe's second output) unwritten on that route: they then
exist only as the down GEMM's input.

With `norm` and `add` the sequence is the whole FFN half of a decoder layer (src/ml/gguf/qwen35_cpu.cr:1705-1725):
r = x + add (the attention output joining the residual stream), h = rmsnorm(r, norm), out = r + down(silu(gate h) * up h).
"""
import numpy as np

from . import hip, quant
from .types import TensorType


class FFNSequenceRunner:
    def __init__(self, gate_raw, up_raw, down_raw, hidden, ffn_dim, tokens, xs, residual=None, down_type=TensorType.Q6_K,
                 norm=None, add=None, eps=1.0e-6, keep_combined=True):
        if not tokens > 0:
            raise ValueError("tokens must be positive")
        if len(xs) != tokens * hidden:
            raise ValueError("xs size mismatch")
        if residual is not None and len(residual) != tokens * hidden:
            raise ValueError("residual size mismatch")
        if (norm is None) != (add is None):
            raise ValueError("norm and add go together")
        if norm is not None and (residual is not None or len(norm) != hidden or len(add) != tokens * hidden):
            raise ValueError("norm/add size mismatch, or a residual given besides them")
        self.hidden, self.ffn_dim, self.tokens, self.down_type = hidden, ffn_dim, tokens, down_type
        self.keep_combined = keep_combined
        self._raw = {"gate": gate_raw, "up": up_raw, "down": down_raw}
        self._xs = np.ascontiguousarray(xs, dtype=np.float32)
        self._residual = None if residual is None else np.ascontiguousarray(residual, dtype=np.float32)
        self._buffers = []
        self._w = {k: self._alloc(v.size) for k, v in self._raw.items()}
        self._x = self._alloc(4 * tokens * hidden)
        self._res = self._alloc(4 * tokens * hidden) if residual is not None or norm is not None else None
        self._eps = eps
        self._norm_w = None if norm is None else np.ascontiguousarray(norm, dtype=np.float32)
        self._add_h = None if add is None else np.ascontiguousarray(add, dtype=np.float32)
        self._norm = self._alloc(4 * hidden) if norm is not None else None
        self._add = self._alloc(4 * tokens * hidden) if norm is not None else None
        self._normed = self._alloc(4 * tokens * hidden) if norm is not None else None
        # several tokens behind the norm: the norm itself writes the activation image gate | up read (no pack launch)
        image_bytes = quant.gemv_image_bytes(TensorType.Q4_K, hidden, quant.MAX_GEMV_TOKENS) if hidden <= 4096 else 0
        self._image = self._alloc(image_bytes) if norm is not None and image_bytes and ffn_dim % 16 == 0 else None
        self._image_from = quant.gemv_one_pass_multi_from(TensorType.Q4_K, hidden)   # token count from which it is used
        self._gate = self._alloc(4 * tokens * ffn_dim)      # only used when several tokens run together
        self._up = self._alloc(4 * tokens * ffn_dim)
        self._act = self._alloc(4 * tokens * ffn_dim)
        self._out = self._alloc(4 * tokens * hidden)
        # prefill: workspaces for x (Q4_K layout) and for the SwiGLU output (the down matrix's layout, with its k-split planes)
        self._ws_x = self._ws_act = None
        gemm_types = (int(TensorType.Q4_K), int(TensorType.Q5_K), int(TensorType.Q6_K))
        if tokens > quant.get_gemm_threshold() and hidden % 256 == 0 and ffn_dim % 256 == 0 and int(down_type) in gemm_types:
            self._ws_x_bytes = quant.gemm_workspace_bytes(TensorType.Q4_K, hidden, tokens)
            self._ws_act_bytes = quant.gemm_workspace_bytes(down_type, ffn_dim, tokens, hidden)
            self._ws_x, self._ws_act = self._alloc(self._ws_x_bytes), self._alloc(self._ws_act_bytes)
        # up to sixteen tokens: the images of the one-pass kernels with sixteen single-term tokens (x for gate | up, the
        # SwiGLU products for down)
        self._img16_x = self._img16_act = None
        if self._ws_x is not None:
            nx = quant.gemv_image_bytes(TensorType.Q4_K, hidden, quant.MAX_GEMV_TOKENS)
            na = quant.gemv_image_bytes(down_type, ffn_dim, quant.MAX_GEMV_TOKENS)
            if nx and na:
                self._img16_x, self._img16_act = self._alloc(nx), self._alloc(na)
        self.combined = self.out = None
        self._runner = hip.ResidentSequenceRunner(tokens, self._upload_weights, self._reset_sequence, self._run_token,
                                                  self._read_outputs, self._run_sequence)

    def _alloc(self, nbytes):
        b = hip.DeviceBuffer(nbytes)
        self._buffers.append(b)
        return b

    def _upload_weights(self):
        for k, raw in self._raw.items():
            hip.copy_htod(self._w[k].ptr, raw, raw.size, "%s weights" % k)
        if self._norm is not None:
            hip.copy_htod(self._norm.ptr, self._norm_w, self._norm_w.nbytes, "norm weights")

    def _reset_sequence(self):
        hip.copy_htod(self._x.ptr, self._xs, self._xs.nbytes, "sequence input")
        if self._residual is not None:
            hip.copy_htod(self._res.ptr, self._residual, self._residual.nbytes, "residual")
        if self._add is not None:
            hip.copy_htod(self._add.ptr, self._add_h, self._add_h.nbytes, "add")

    def _launch(self, tok0, count):
        st = hip.current_stream_handle()
        h, f = self.hidden, self.ffn_dim
        x, act = self._x.ptr + 4 * tok0 * h, self._act.ptr + 4 * tok0 * f
        fused_norm = self._image is not None and count >= self._image_from
        if fused_norm:
            # r = x + add, and rmsnorm(r) written straight as the activation image gate | up | SwiGLU read
            quant.add_rmsnorm_pack_dev(x, self._add.ptr + 4 * tok0 * h, self._norm.ptr, self._res.ptr + 4 * tok0 * h, 0,
                                       TensorType.Q4_K, self._image.ptr, h, count, self._eps, st)
            quant.gemv_packed_swiglu_dev(self._w["gate"].ptr, self._w["up"].ptr, TensorType.Q4_K, self._image.ptr, act, h, f,
                                         count, st)
        elif self._norm is not None:
            normed = self._normed.ptr + 4 * tok0 * h
            quant.add_rmsnorm_dev(x, self._add.ptr + 4 * tok0 * h, self._norm.ptr, self._res.ptr + 4 * tok0 * h, normed, h,
                                  count, self._eps, st)
            x = normed
        if fused_norm:
            pass
        elif count == 1 or f % 16 == 0:
            # gate | up | SwiGLU in one launch (several tokens: one pass over both matrices per group of up to eight)
            quant.gemv_dual_swiglu_dev(self._w["gate"].ptr, self._w["up"].ptr, TensorType.Q4_K, x, act, h, f, count, st)
        else:
            g, u = self._gate.ptr + 4 * tok0 * f, self._up.ptr + 4 * tok0 * f
            quant.gemv_dual_dev(self._w["gate"].ptr, self._w["up"].ptr, TensorType.Q4_K, x, g, u, h, f, count, st)
            quant.swiglu_dev(g, u, act, count * f, st)
        res = self._res.ptr + 4 * tok0 * h if self._res is not None else 0
        quant.gemv_dev(self._w["down"].ptr, self.down_type, act, self._out.ptr + 4 * tok0 * h, f, h, count, res, st)

    def _launch_prefill16(self, count):
        """9..16 tokens: every projection in one pass over its weights on the decode kernels with sixteen single-term tokens
        (the GEMM's precision class at half its time): norm, image of x, gate | up | SwiGLU in one launch, image of the products
        in the down matrix's order, down with the residual."""
        st = hip.current_stream_handle()
        h, f = self.hidden, self.ffn_dim
        x = self._x.ptr
        if self._norm is not None and h <= 4096:
            # r = x + add, and rmsnorm(r) written straight as the image gate | up read
            quant.add_rmsnorm_pack16_dev(x, self._add.ptr, self._norm.ptr, self._res.ptr, 0, TensorType.Q4_K, self._img16_x.ptr, h,
                                         count, self._eps, st)
        else:
            if self._norm is not None:
                quant.add_rmsnorm_dev(x, self._add.ptr, self._norm.ptr, self._res.ptr, self._normed.ptr, h, count, self._eps, st)
                x = self._normed.ptr
            quant.gemv_pack16_dev(x, TensorType.Q4_K, h, count, self._img16_x.ptr, st)
        if f % 16 == 0:
            quant.gemv_packed16_swiglu_dev(self._w["gate"].ptr, self._w["up"].ptr, TensorType.Q4_K, self._img16_x.ptr, self._act.ptr,
                                           h, f, count, st)
        else:
            quant.gemv_packed16_dev([self._w["gate"].ptr, self._w["up"].ptr], TensorType.Q4_K, self._img16_x.ptr,
                                    [self._gate.ptr, self._up.ptr], [f, f], h, count, 0, st)
            quant.swiglu_dev(self._gate.ptr, self._up.ptr, self._act.ptr, count * f, st)
        quant.gemv_pack16_dev(self._act.ptr, self.down_type, f, count, self._img16_act.ptr, st)
        quant.gemv_packed16_dev([self._w["down"].ptr], self.down_type, self._img16_act.ptr, [self._out.ptr], [h], f, count,
                                self._res.ptr if self._res is not None else 0, st)

    def _launch_prefill(self, count):
        if count <= 16 and self._img16_x is not None:
            return self._launch_prefill16(count)
        st = hip.current_stream_handle()
        h, f = self.hidden, self.ffn_dim
        x = self._x.ptr
        if self._norm is not None and h <= 4096:
            # r = x + add, and rmsnorm(r) written straight as the packed activations gate | up read
            quant.add_rmsnorm_gemm_pack_dev(x, self._add.ptr, self._norm.ptr, self._res.ptr, 0, TensorType.Q4_K, self._ws_x.ptr,
                                            self._ws_x_bytes, h, count, self._eps, st)
        else:
            if self._norm is not None:
                quant.add_rmsnorm_dev(x, self._add.ptr, self._norm.ptr, self._res.ptr, self._normed.ptr, h, count, self._eps, st)
                x = self._normed.ptr
            quant.gemm_pack_dev(x, TensorType.Q4_K, h, count, self._ws_x.ptr, self._ws_x_bytes, st)
        # silu(gate) * up leaves the GEMM as the down GEMM's packed input (and as fp32 only when `combined` is wanted)
        quant.gemm_packed_swiglu_pack_dev(self._w["gate"].ptr, self._w["up"].ptr, TensorType.Q4_K, self._ws_x.ptr, self._ws_x_bytes,
                                          self._act.ptr if self.keep_combined else 0, self.down_type, self._ws_act.ptr,
                                          self._ws_act_bytes, h, f, count, st)
        if self._res is not None:
            quant.gemm_packed_add_dev(self._w["down"].ptr, self.down_type, self._ws_act.ptr, self._ws_act_bytes, self._res.ptr,
                                      self._out.ptr, f, h, count, st)
        else:
            quant.gemm_packed_dev(self._w["down"].ptr, self.down_type, self._ws_act.ptr, self._ws_act_bytes, self._out.ptr, f, h,
                                  count, 0, st)

    def _run_token(self, tok):
        self._launch(tok, 1)

    def _run_sequence(self, active_tokens):
        if self._ws_x is not None and active_tokens > quant.get_gemm_threshold():
            self._launch_prefill(active_tokens)
            return
        for tok0 in range(0, active_tokens, quant.MAX_GEMV_TOKENS):
            self._launch(tok0, min(quant.MAX_GEMV_TOKENS, active_tokens - tok0))

    def _read_outputs(self):
        hip.synchronize("hipDeviceSynchronize(read_outputs)")
        active = self._runner.active_tokens
        prefill = self._ws_x is not None and active > quant.get_gemm_threshold() and not (active <= 16 and self._img16_x is not None)
        self.combined = None
        if self.keep_combined or not prefill:
            self.combined = np.empty(self.tokens * self.ffn_dim, dtype=np.float32)
            hip.copy_dtoh(self.combined, self._act.ptr, self.combined.nbytes, "combined")
        self.out = np.empty(self.tokens * self.hidden, dtype=np.float32)
        hip.copy_dtoh(self.out, self._out.ptr, self.out.nbytes, "out")

    # lifecycle
    def upload_weights(self):
        self._runner.upload_weights()

    def reset_sequence(self):
        self._runner.reset_sequence()

    def run_sequence(self):
        self._runner.run_sequence()

    def run_repeated(self, reps):
        return self._runner.run_repeated(reps)

    def read_outputs(self):
        self._runner.read_outputs()

    def bytes_per_sequence(self):
        """Algorithmic bytes: the three matrices once per group of up to 8 tokens, x and residual in, out out."""
        groups = 1 if (self._ws_x is not None and self.tokens > quant.get_gemm_threshold()) else -(-self.tokens // quant.MAX_GEMV_TOKENS)
        vec = 4 * self.tokens * self.hidden * (4 if self._norm is not None else 3 if self._res is not None else 2)
        return groups * sum(r.size for r in self._raw.values()) + vec

    def flops_per_sequence(self):
        """Multiply-adds x 2 of the three projections for every token."""
        return 2.0 * self.tokens * 3 * self.hidden * self.ffn_dim

    def close(self):
        for b in self._buffers:
            b.close()
        self._buffers = []
