"""Resident output head: RMSNorm -> quantized vocabulary projection -> top-1, on one HIP stream.

The HIP counterpart of the reference's QwenOutputHeadRunner (src/ml/cuda/qwen_output_head_runner.cr:6-7, 659-760; launches
:937-940): the default decode-facing path reads back only the top-1 id and value per token; the full logits are read
only on request (read_logits), through the plain GEMV. Groups of up to eight tokens share one pass over the weights.
"""
import numpy as np

from . import hip, quant
from .types import TensorType


class Weights:
    def __init__(self, norm, output_raw, output_type, hidden, vocab):
        self.norm = np.ascontiguousarray(norm, dtype=np.float32)
        self.output_raw, self.output_type, self.hidden, self.vocab = output_raw, TensorType(int(output_type)), hidden, vocab


class QwenOutputHeadRunner:
    GROUP = quant.MAX_GEMV_TOKENS    # tokens handed to the library at a time: up to eight share one pass over the weights

    def __init__(self, weights, tokens, xs, eps, read_logits=False):
        if not tokens > 0:
            raise ValueError("tokens must be positive")
        if len(xs) != tokens * weights.hidden:
            raise ValueError("xs size mismatch")
        if weights.norm.size != weights.hidden:
            raise ValueError("norm size mismatch")
        self.weights, self.tokens, self.eps, self.read_logits = weights, tokens, eps, read_logits
        self.hidden, self.vocab = weights.hidden, weights.vocab
        self._xs = np.ascontiguousarray(xs, dtype=np.float32)
        self._buffers = []
        self._w = self._alloc(weights.output_raw.size)
        self._norm = self._alloc(4 * self.hidden)
        self._x = self._alloc(4 * tokens * self.hidden)
        self._normed = self._alloc(4 * tokens * self.hidden)
        self._stride = quant.gemv_top1_partials(weights.output_type, self.vocab)
        self._partial_ids = self._alloc(4 * tokens * self._stride)
        self._partial_values = self._alloc(4 * tokens * self._stride)
        self._top1_ids = self._alloc(4 * tokens)
        self._top1_values = self._alloc(4 * tokens)
        self._logits = self._alloc(4 * tokens * self.vocab) if read_logits else None
        # token groups that go through the one-pass kernel: the norm writes that kernel's activation image itself
        t = weights.output_type
        self._from = quant.gemv_one_pass_from(t, self.hidden, self.vocab) if int(t) in (12, 14) and self.hidden <= 4096 else 0
        self._image = self._alloc(quant.gemv_image_bytes(t, self.hidden, quant.MAX_GEMV_TOKENS)) if self._from else None
        self.top1_ids = np.zeros(tokens, dtype=np.int32)
        self.top1_values = np.zeros(tokens, dtype=np.float32)
        self.logits = None
        self._runner = hip.ResidentSequenceRunner(tokens, self._upload_weights, self._reset_sequence, self._run_token,
                                                  self._read_outputs, self._run_sequence)

    @classmethod
    def from_weights(cls, weights, tokens, xs, eps, read_logits=False):
        return cls(weights, tokens, xs, eps, read_logits)

    @property
    def top1_ids_device_ptr(self):
        return self._top1_ids.ptr

    def _alloc(self, nbytes):
        b = hip.DeviceBuffer(nbytes)
        self._buffers.append(b)
        return b

    def _upload_weights(self):
        raw = self.weights.output_raw
        hip.copy_htod(self._w.ptr, raw, raw.size, "output weights")
        hip.copy_htod(self._norm.ptr, self.weights.norm, self.weights.norm.nbytes, "output norm")

    def _reset_sequence(self):
        hip.copy_htod(self._x.ptr, self._xs, self._xs.nbytes, "sequence input")

    def _launch(self, tok0, count):
        st = hip.current_stream_handle()
        h, t = self.hidden, self.weights.output_type
        normed = self._normed.ptr + 4 * tok0 * h
        if self._from and count >= self._from:
            quant.rmsnorm_pack_dev(self._x.ptr + 4 * tok0 * h, self._norm.ptr, normed if self._logits is not None else 0, t,
                                   self._image.ptr, h, count, self.eps, st)
            quant.gemv_packed_top1_dev(self._w.ptr, t, self._image.ptr, self._partial_ids.ptr + 4 * tok0 * self._stride,
                                       self._partial_values.ptr + 4 * tok0 * self._stride, self._top1_ids.ptr + 4 * tok0,
                                       self._top1_values.ptr + 4 * tok0, h, self.vocab, count, st)
        else:
            quant.rmsnorm_dev(self._x.ptr + 4 * tok0 * h, self._norm.ptr, normed, h, count, self.eps, st)
            quant.gemv_top1_dev(self._w.ptr, t, normed, self._partial_ids.ptr + 4 * tok0 * self._stride,
                                self._partial_values.ptr + 4 * tok0 * self._stride, self._top1_ids.ptr + 4 * tok0,
                                self._top1_values.ptr + 4 * tok0, h, self.vocab, count, st)
        if self._logits is not None:
            quant.gemv_dev(self._w.ptr, t, normed, self._logits.ptr + 4 * tok0 * self.vocab, h, self.vocab, count, 0, st)

    def _run_token(self, tok):
        self._launch(tok, 1)

    def _run_sequence(self, active_tokens):
        for tok0 in range(0, active_tokens, self.GROUP):
            self._launch(tok0, min(self.GROUP, active_tokens - tok0))

    def _read_outputs(self):
        hip.synchronize("hipDeviceSynchronize(read_outputs)")
        ids = np.empty(self.tokens, dtype=np.uint32)
        hip.copy_dtoh(ids, self._top1_ids.ptr, ids.nbytes, "top1 ids")
        self.top1_ids = ids.astype(np.int32)
        hip.copy_dtoh(self.top1_values, self._top1_values.ptr, self.top1_values.nbytes, "top1 values")
        if self._logits is not None:
            self.logits = np.empty(self.tokens * self.vocab, dtype=np.float32)
            hip.copy_dtoh(self.logits, self._logits.ptr, self.logits.nbytes, "logits")

    # lifecycle
    def upload_weights(self):
        self._runner.upload_weights()

    def replace_sequence_input(self, xs):
        if len(xs) != self.tokens * self.hidden:
            raise ValueError("xs size mismatch")
        self._xs = np.ascontiguousarray(xs, dtype=np.float32)

    def reset_sequence(self):
        self._runner.reset_sequence()

    def run_sequence(self):
        self._runner.run_sequence()

    def run_repeated(self, reps):
        return self._runner.run_repeated(reps)

    @property
    def active_tokens(self):
        return self._runner.active_tokens

    @active_tokens.setter
    def active_tokens(self, count):
        self._runner.active_tokens = count

    def reset_active_tokens(self):
        self._runner.reset_active_tokens()

    def read_outputs(self):
        self._runner.read_outputs()

    def bytes_per_sequence(self):
        groups = -(-self.tokens // self.GROUP)
        return groups * self.weights.output_raw.size + 4 * self.tokens * self.hidden * 3

    def close(self):
        for b in self._buffers:
            b.close()
        self._buffers = []
