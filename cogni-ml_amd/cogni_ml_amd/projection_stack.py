"""Resident decoder-layer projection stack on one HIP stream.

The HIP counterpart of the reference's resident projection runners
(src/ml/cuda/qwen_full_attn_projection_runner.cr: q/k/v bundle; bin/cuda_ffn_sequence_probe.cr:
gate/up/down): weights and activations stay on the device, every projection of every token group is
launched back to back into the current stream, and the lifecycle goes through ResidentSequenceRunner
(upload_weights -> reset_sequence -> run_sequence x reps -> synchronize -> read_outputs).

Where the reference runs either one launch per token or weight-stationary groups of 4 tokens
(`tbatch4`, qwen_full_attn_projection_runner.cr:274-301), this runner hands groups of up to 8 tokens
to one weight-stationary launch. A sequence of more tokens than the GEMM threshold (quant.get_gemm_threshold(), 8 as
in the reference's router) goes through the prefill GEMMs instead, all tokens at once: every distinct input is packed
once (q | k | v and gate | up share x) and each projection is one GEMM against it - the reference's
`qmatmul_nobias(qw, x, batch)` calls of a prefill layer (src/ml/gguf/qwen35_cpu.cr:1478-1490).
"""
import numpy as np

from . import hip, quant
from .types import TensorType

# (name, input, weight type, out_dim, in_dim) at the shapes of the benchmark's mixed-quant layer:
# hidden 4096, 32 query / 8 KV heads of 128, FFN 12288; q/k/v/o/gate/up Q4_K, down Q6_K
QWEN_LAYER_4096 = [
    ("q", "x", TensorType.Q4_K, 4096, 4096),
    ("k", "x", TensorType.Q4_K, 1024, 4096),
    ("v", "x", TensorType.Q4_K, 1024, 4096),
    ("o", "q", TensorType.Q4_K, 4096, 4096),
    ("gate", "x", TensorType.Q4_K, 12288, 4096),
    ("up", "x", TensorType.Q4_K, 12288, 4096),
    ("down", "gate", TensorType.Q6_K, 4096, 12288),
]


class Weights:
    """Raw GGUF bytes per projection: {name: (raw, type, out_dim, in_dim, input name)}."""

    def __init__(self, hidden, entries):
        self.hidden = hidden
        self.entries = entries        # ordered list of (name, input, type, out_dim, in_dim, raw)

    @classmethod
    def synthetic(cls, rng, layout=QWEN_LAYER_4096):
        from . import synth
        hidden = layout[0][4]
        return cls(hidden, [(n, src, t, o, i, synth.make_weights(rng, t, o, i)) for n, src, t, o, i in layout])

    @property
    def raw_bytes(self):
        return sum(e[5].size for e in self.entries)


class QwenProjectionStackRunner:
    def __init__(self, weights, tokens, xs):
        if not tokens > 0:
            raise ValueError("tokens must be positive")
        if len(xs) != tokens * weights.hidden:
            raise ValueError("xs size mismatch")
        self.weights, self.tokens, self.hidden = weights, tokens, weights.hidden
        self._xs = np.ascontiguousarray(xs, dtype=np.float32)
        self._buffers = []
        self._w = {}
        self._images = {}   # (input name, weight type) -> packed activation image shared by every list that reads that input
        self._act = {"x": self._alloc(4 * tokens * self.hidden)}
        for name, src, t, out_dim, in_dim, raw in weights.entries:
            self._w[name] = self._alloc(raw.size)
            self._act[name] = self._alloc(4 * tokens * out_dim)
            # (allocated here, not at first use: the sequence may be issued under stream capture)
            nbytes = quant.gemv_image_bytes(t, in_dim, quant.MAX_GEMV_TOKENS)
            if nbytes and (src, int(t)) not in self._images:
                self._images[(src, int(t))] = self._alloc(nbytes)
        # prefill: one workspace per (input, packed layout) - Q4_K and Q5_K read one layout, Q6_K its own - large enough
        # for the k-split planes of the projection that needs the most
        self._prefill_ws = {}
        self._images16 = {}   # input name -> the image of the sixteen-token one-pass kernels (Q4_K / Q5_K projections, 9..16 tokens)
        if tokens > quant.get_gemm_threshold() and all(self._gemm_capable(e) for e in weights.entries):
            need = {}
            for name, src, t, out_dim, in_dim, raw in weights.entries:
                key = (src, self._family(t))
                need[key] = max(need.get(key, 0), quant.gemm_workspace_bytes(t, in_dim, tokens, out_dim))
                if self._one_pass16(t, in_dim) and key not in self._images16:
                    self._images16[key] = self._alloc(quant.gemv_image_bytes(t, in_dim, quant.MAX_GEMV_TOKENS))
            self._prefill_ws = {k: (self._alloc(n), n) for k, n in need.items()}
        self.outputs = {}
        self._runner = hip.ResidentSequenceRunner(
            tokens, self._upload_weights, self._reset_sequence, self._run_token, self._read_outputs,
            self._run_sequence)

    @classmethod
    def from_weights(cls, weights, tokens, xs):
        return cls(weights, tokens, xs)

    def _alloc(self, nbytes):
        b = hip.DeviceBuffer(nbytes)
        self._buffers.append(b)
        return b

    # ---- closures handed to ResidentSequenceRunner -------------------------------------------------
    def _upload_weights(self):
        for name, src, t, out_dim, in_dim, raw in self.weights.entries:
            hip.copy_htod(self._w[name].ptr, raw, raw.size, "%s weights" % name)

    def _reset_sequence(self):
        hip.copy_htod(self._act["x"].ptr, self._xs, self._xs.nbytes, "sequence input")

    def _launch(self, tok0, count):
        stream = hip.current_stream_handle()
        ents = self.weights.entries
        packed = set()
        i = 0
        while i < len(ents):
            name, src, t, out_dim, in_dim, raw = ents[i]
            nxt = ents[i + 1] if i + 1 < len(ents) else None
            # up to three consecutive projections of one input, type and row length (q | k | v, gate | up) go to the
            # library as one list (the qmatvec_many seam), which stages the input once for them
            j = i + 1
            while j < len(ents) and j - i < 3 and (ents[j][1], ents[j][2], ents[j][4]) == (src, t, in_dim):
                j += 1
            if j - i >= 2 and 0 < quant.gemv_one_pass_multi_from(t, in_dim) <= count:
                # several tokens of a shape the one-pass kernel takes: the input is packed once per sequence step and
                # every list that reads it (q | k | v, then gate | up) goes against that one image
                grp = ents[i:j]
                key = (src, int(t))
                if key not in packed:
                    quant.gemv_pack_dev(self._act[src].ptr + 4 * tok0 * in_dim, t, in_dim, count, self._images[key].ptr, stream)
                    packed.add(key)
                quant.gemv_packed_dev([self._w[e[0]].ptr for e in grp], t, self._images[key].ptr,
                                      [self._act[e[0]].ptr + 4 * tok0 * e[3] for e in grp], [e[3] for e in grp], in_dim,
                                      count, 0, stream)
                i = j
                continue
            if j - i >= 2:
                grp = ents[i:j]
                quant.gemv_many_dev([self._w[e[0]].ptr for e in grp], t, self._act[src].ptr + 4 * tok0 * in_dim,
                                    [self._act[e[0]].ptr + 4 * tok0 * e[3] for e in grp], [e[3] for e in grp], in_dim,
                                    count, stream)
                i = j
                continue
            if nxt is not None and nxt[1:5] == (src, t, out_dim, in_dim):
                # two projections of one shape on the same input (k | v, gate | up) share one launch
                quant.gemv_dual_dev(self._w[name].ptr, self._w[nxt[0]].ptr, t, self._act[src].ptr + 4 * tok0 * in_dim,
                                    self._act[name].ptr + 4 * tok0 * out_dim, self._act[nxt[0]].ptr + 4 * tok0 * out_dim,
                                    in_dim, out_dim, count, stream)
                i += 2
                continue
            quant.gemv_dev(self._w[name].ptr, t, self._act[src].ptr + 4 * tok0 * in_dim,
                           self._act[name].ptr + 4 * tok0 * out_dim, in_dim, out_dim, count, 0, stream)
            i += 1

    @staticmethod
    def _family(t):
        return "q6" if int(t) == int(TensorType.Q6_K) else "q45"

    @staticmethod
    def _gemm_capable(entry):
        return int(entry[2]) in (int(TensorType.Q4_K), int(TensorType.Q5_K), int(TensorType.Q6_K)) and entry[4] % 256 == 0

    @staticmethod
    def _one_pass16(t, in_dim):
        return int(t) in (int(TensorType.Q4_K), int(TensorType.Q5_K), int(TensorType.Q6_K)) and \
            quant.gemv_image_bytes(t, in_dim, quant.MAX_GEMV_TOKENS) > 0

    def _launch_prefill(self, count):
        """All `count` tokens through the GEMMs: one pack per (input, layout), one GEMM per list of projections that share
        their input, type and row length (or per projection)."""
        stream = hip.current_stream_handle()
        ents = self.weights.entries
        packed, done = set(), set()
        list_types = (int(TensorType.Q4_K), int(TensorType.Q5_K))
        for idx, (name, src, t, out_dim, in_dim, raw) in enumerate(ents):
            if name in done:
                continue
            if count <= 16 and self._one_pass16(t, in_dim):
                # up to sixteen tokens: the one-pass decode kernels with sixteen single-term tokens, one image per input,
                # every projection of that input, type and row length in the same call
                key16 = (src, self._family(t))
                img = self._images16[key16]
                if key16 + ("x16",) not in packed:
                    quant.gemv_pack16_dev(self._act[src].ptr, t, in_dim, count, img.ptr, stream)
                    packed.add(key16 + ("x16",))
                grp = [e for e in ents[idx:] if e[0] not in done and (e[1], int(e[2]), e[4]) == (src, int(t), in_dim)][:8]
                quant.gemv_packed16_dev([self._w[e[0]].ptr for e in grp], t, img.ptr, [self._act[e[0]].ptr for e in grp],
                                        [e[3] for e in grp], in_dim, count, 0, stream)
                done.update(e[0] for e in grp)
                continue
            key = (src, self._family(t))
            ws, nbytes = self._prefill_ws[key]
            if key not in packed:
                quant.gemm_pack_dev(self._act[src].ptr, t, in_dim, count, ws.ptr, nbytes, stream)
                packed.add(key)
            # every projection still to come of the same input, type and row length joins this launch (q | k | v | gate | up:
            # their input is this one's, so it exists already) - the prefill counterpart of the qmatvec_many seam
            grp = [e for e in ents[idx:] if e[0] not in done and (e[1], int(e[2]), e[4]) == (src, int(t), in_dim)][:6]
            if len(grp) >= 2 and int(t) in list_types:
                quant.gemm_packed_many_dev([self._w[e[0]].ptr for e in grp], t, ws.ptr, nbytes, [self._act[e[0]].ptr for e in grp],
                                           [e[3] for e in grp], in_dim, count, stream)
                done.update(e[0] for e in grp)
            else:
                quant.gemm_packed_dev(self._w[name].ptr, t, ws.ptr, nbytes, self._act[name].ptr, in_dim, out_dim, count, 0, stream)
                done.add(name)

    def _run_token(self, tok):
        self._launch(tok, 1)

    def _run_sequence(self, active_tokens):
        if self._prefill_ws and active_tokens > quant.get_gemm_threshold():
            self._launch_prefill(active_tokens)
            return
        for tok0 in range(0, active_tokens, quant.MAX_GEMV_TOKENS):
            self._launch(tok0, min(quant.MAX_GEMV_TOKENS, active_tokens - tok0))

    def _read_outputs(self):
        hip.synchronize("hipDeviceSynchronize(read_outputs)")
        for name, src, t, out_dim, in_dim, raw in self.weights.entries:
            out = np.empty(self.tokens * out_dim, dtype=np.float32)
            hip.copy_dtoh(out, self._act[name].ptr, out.nbytes, "%s output" % name)
            self.outputs[name] = out

    # ---- public lifecycle, as the reference runner's (qwen_full_attn_projection_runner.cr:111-165) ----
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

    def device_ptr(self, name):
        return self._act[name].ptr

    def bytes_per_sequence(self, active_tokens=None):
        """Algorithmic bytes of one run_sequence: every weight once per group of up to 8 tokens, x in, out out."""
        m = self.tokens if active_tokens is None else active_tokens
        groups = 1 if (self._prefill_ws and m > quant.get_gemm_threshold()) else -(-m // quant.MAX_GEMV_TOKENS)
        total = 0
        for name, src, t, out_dim, in_dim, raw in self.weights.entries:
            total += groups * raw.size + 4 * m * (in_dim + out_dim)
        return total

    def close(self):
        for b in self._buffers:
            b.close()
        self._buffers = []
