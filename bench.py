#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

Headline (the JSON line on stdout): Q4_K decode GEMV, W = 12288 x 4096 (in_dim 4096 -> out_dim 12288,
the ffn_gate/ffn_up shape), M = 1, fp32 activations and accumulation. One "step" is one GEMV launch.
Weights are seeded synthetic super-blocks, already resident in HBM; consecutive steps read different
copies of the matrix, and a copy comes round again only after more bytes than the 256 MB last-level
cache holds, so every step streams its 28 MB from HBM.

How a workload is timed (`measure`): the K = --steps launches are captured into HIP graphs; after the
--warmup launches the graphs are replayed untimed for a fixed wall time (the clocks of an idle GPU take
tens of milliseconds to come up, however few warm-up steps the caller asks for); then R samples are
taken back to back, each one exactly K steps (or a whole number of replays of them when K steps are
shorter than a couple of milliseconds), bracketed by HIP events on the launch stream. The figure
reported is the median sample; min, max, R and the length of the timed region go into the line as well.
The CPU baseline runs after the GPU work, so the GPU never waits idle in front of a timed region.

The same line carries, under "cases", every other configuration (Q8_0 and the other K-quant GEMVs, the
510 MB output head, the prefill GEMM at M = 64 / 512 / 2048, the projection stack at M = 1 / 4 / 8), each
with its fraction of the roofline that bounds it and, for matrices under 16 MB, the time a kernel that
only reads the same bytes takes.

  python bench.py [--gpus 1] [--steps K] [--warmup W]
  python bench.py --mode cases      more shapes and fused sequences in the same line
  python bench.py --mode pmc        plain launches of the dominant kernels (one-token and one-pass GEMV, prefill GEMM)
                                    and of a copy kernel of known size, for rocprofv3 --pmc / --kernel-trace runs
  python bench.py --mode pmc-gemm   plain launches of the M = 512 prefill GEMM alone
  python bench.py --mode ceiling    empty launch, read-only stream, matrix-core-only loop
  python bench.py --launch direct   the same work without HIP graphs (for rocprofv3 --kernel-trace)
"""
import argparse
import ctypes
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "cogni-ml_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

import numpy as np  # noqa: E402

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0   # MI355X dense fp16 matrix peak, published
LLC_BYTES = 256 << 20           # last-level (Infinity) cache
Q4_K, Q5_K, Q6_K, Q8_0 = 12, 13, 14, 8
TYPE_NAME = {Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K", Q8_0: "Q8_0"}
MEASURE_HSACO = os.path.join(ROOT, "cogni-ml_amd", "lib", "measure_kernels_gfx950.hsaco")
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "traffic.json")

RAMP_MS = 150.0        # untimed replays right before the timed samples
MIN_SAMPLE_MS = 2.0    # a sample is at least this long (whole replays of the K steps)
MIN_TIMED_MS = 20.0    # all samples together
MIN_SAMPLES, MAX_SAMPLES = 5, 60


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def gemv_bytes(w_bytes, in_dim, out_dim, tokens):
    """Algorithmic bytes of one GEMV: weights once + activations in + results out."""
    return w_bytes + 4 * tokens * in_dim + 4 * tokens * out_dim


def rotation(steps, copies, needed):
    """How `copies` buffers are walked by consecutive steps so that a buffer is read again only after `needed` others:
    returns (C, G): step number n (counted across replays) reads buffer n % C, and G = C / gcd(steps, C) graphs of
    `steps` launches each, replayed in turn, continue that sequence without a seam."""
    best = None
    for c in range(min(copies, max(1, needed)), copies + 1):
        g = c // math.gcd(steps, c)
        if best is None or g < best[1] or (g == best[1] and c > best[0]):
            best = (c, g)
    return best


class Rotating:
    """Launches that walk a set of equivalent buffers (weight copies, runner instances)."""

    def __init__(self, launch, copies, bytes_per_copy):
        self.launch, self.copies = launch, copies
        # buffers that must be read in between before one comes round again: more than the last-level cache holds
        self.needed = min(copies, max(2, int(math.ceil(1.1 * LLC_BYTES / max(1, bytes_per_copy)))))


USE_GRAPHS = True   # --launch direct clears it: every launch goes to the stream one by one (profiler runs)


def measure(hip, stream, rot, steps, warmup, graph=True):
    """Time `steps` launches of rot.launch(copy_index, stream) per sample; see the module docstring.
    Returns a dict: us (median per step), us_min, us_max, samples, replays_per_sample, timed_region_ms, graphed."""
    C, G = rotation(steps, rot.copies, rot.needed)
    graphs, execs = [], []
    if graph and USE_GRAPHS:
        try:
            for g in range(G):
                stream.begin_capture(1)
                for i in range(steps):
                    rot.launch((g * steps + i) % C, stream)
                gr = stream.end_capture()
                graphs.append(gr)
                ex = gr.instantiate()   # (no hipGraphUpload: the ramp below replays every graph before anything is timed,
                execs.append(ex)        #  and a profiler that reads kernel arguments cannot follow them into device memory)
            stream.synchronize()
        except Exception as e:   # stream capture unavailable: direct launches
            log("graph capture failed (%s); timing direct launches" % e)
            for o in execs + graphs:
                o.close()
            graphs, execs = [], []
    counter = [0]   # replays so far: each is `steps` launches (warm-up launches come on top)

    def replay():
        if execs:
            execs[counter[0] % G].launch(stream)
        else:
            for i in range(steps):
                rot.launch((counter[0] * steps + i) % C, stream)
        counter[0] += 1

    for i in range(warmup):
        rot.launch(i % C, stream)
    # a first estimate of one replay, then untimed replays for RAMP_MS
    e0, e1 = hip.Event(), hip.Event()
    stream.synchronize()
    e0.record(stream)
    replay()
    e1.record(stream)
    e1.synchronize()
    est_ms = max(e0.elapsed_ms(e1), 1e-3)
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < RAMP_MS:
        for _ in range(max(1, min(64, int(5.0 / est_ms)))):
            replay()
        stream.synchronize()
    e0.record(stream)
    replay()
    e1.record(stream)
    e1.synchronize()
    est_ms = max(e0.elapsed_ms(e1), 1e-3)
    inner = max(1, int(math.ceil(MIN_SAMPLE_MS / est_ms)))
    samples = int(min(MAX_SAMPLES, max(MIN_SAMPLES, math.ceil(MIN_TIMED_MS / (inner * est_ms)))))
    # keep the GPU busy between the estimate and the samples, then enqueue every sample without a host wait in between
    events = [hip.Event() for _ in range(samples + 1)]
    for _ in range(inner):
        replay()
    events[0].record(stream)
    for s in range(samples):
        for _ in range(inner):
            replay()
        events[s + 1].record(stream)
    events[-1].synchronize()
    hip.synchronize()
    per_step_us = sorted(events[s].elapsed_ms(events[s + 1]) * 1e3 / (inner * steps) for s in range(samples))
    region_ms = events[0].elapsed_ms(events[-1])
    for o in execs + graphs + events + [e0, e1]:
        o.close()
    return {"us": per_step_us[len(per_step_us) // 2], "us_min": per_step_us[0], "us_max": per_step_us[-1],
            "samples": samples, "replays_per_sample": inner, "timed_region_ms": region_ms, "graphed": bool(execs),
            "buffers_rotated": C, "launches": warmup + counter[0] * steps}


class GemvCase:
    """Rotating weight copies + activations + output for one (type, shape, tokens)."""

    def __init__(self, hip, quant, synth, rng, w_type, out_dim, in_dim, tokens, min_total_bytes=2 * LLC_BYTES + (32 << 20),
                 max_copies=96):
        from cogni_ml_amd.types import TensorType
        self.hip, self.quant = hip, quant
        self.w_type, self.out_dim, self.in_dim, self.tokens = w_type, out_dim, in_dim, tokens
        self.w_bytes = TensorType(w_type).data_bytes(in_dim) * out_dim
        self.copies = int(max(2, min(max_copies, -(-min_total_bytes // self.w_bytes))))
        self.host_w = synth.make_weights(rng, w_type, out_dim, in_dim)
        self.host_x = synth.make_activations(rng, tokens, in_dim)
        self.w = []
        for c in range(self.copies):
            buf = hip.DeviceBuffer(self.w_bytes)
            # copy 0 is the matrix checked against the oracle; the others are the same bytes rotated, so that
            # every copy holds different data at every address
            src = self.host_w if c == 0 else np.roll(self.host_w, 4096 * c + 17)
            hip.copy_htod(buf.ptr, src, self.w_bytes, "weights")
            self.w.append(buf)
        self.x = hip.DeviceBuffer(self.host_x.nbytes)
        hip.copy_htod(self.x.ptr, self.host_x, self.host_x.nbytes, "x")
        self.out = hip.DeviceBuffer(4 * tokens * out_dim)
        self.bytes_per_step = gemv_bytes(self.w_bytes, in_dim, out_dim, tokens)

    def launch(self, copy, stream):
        self.quant.gemv_dev(self.w[copy].ptr, self.w_type, self.x.ptr, self.out.ptr, self.in_dim,
                            self.out_dim, self.tokens, 0, stream.handle)

    def rotating(self):
        return Rotating(self.launch, self.copies, self.w_bytes)

    def read_out(self):
        out = np.empty(self.tokens * self.out_dim, dtype=np.float32)
        self.hip.synchronize()
        self.hip.copy_dtoh(out, self.out.ptr, out.nbytes, "out")
        return out

    def close(self):
        for b in self.w + [self.x, self.out]:
            b.close()


class MeasureKernels:
    """The bench-only code object: copy, read-only stream, matrix-core loop."""

    def __init__(self, hip):
        if not os.path.exists(MEASURE_HSACO):
            raise RuntimeError("%s is missing: run __graft_entry__.build() first" % MEASURE_HSACO)
        self.hip = hip
        self.mod = hip.HIPModule.load(open(MEASURE_HSACO, "rb").read(), "measure_kernels_gfx950")
        self.sink = hip.DeviceBuffer(4 * 65536)

    def fn(self, name):
        return self.mod.function(name)

    def read_floor(self, stream, case, steps, warmup):
        """Best time of a kernel that only reads the weight bytes of `case` (same rotating buffers): (us, grid)."""
        read_fn = self.fn("read_bytes_16")
        best = None
        for grid in (256, 512, 1024, 2048, 4096):
            if grid * 256 * 16 > 2 * case.w_bytes and grid > 256:
                break
            boxes = [self.hip.KernelParams(ctypes.c_uint64(b.ptr), ctypes.c_uint64(self.sink.ptr),
                                           ctypes.c_uint64(case.w_bytes & ~15)) for b in case.w]

            def rd(copy, st, grid=grid, boxes=boxes):
                with self.hip.with_stream(st):
                    self.hip.launch(read_fn, grid, 1, 1, 256, 1, 1, boxes[copy], "read")
            r = measure(self.hip, stream, Rotating(rd, case.copies, case.w_bytes), steps, warmup)
            if best is None or r["us"] < best[0]:
                best = (r["us"], grid)
        return best


def gemv_record(r, bytes_per_step):
    gbps = bytes_per_step / r["us"] / 1e3
    return {"us": round(r["us"], 3), "us_min": round(r["us_min"], 3), "us_max": round(r["us_max"], 3),
            "gbps": round(gbps, 1), "frac_hbm": round(gbps / HBM_PEAK_GBPS, 4), "bytes": bytes_per_step,
            "samples": r["samples"], "timed_region_ms": round(r["timed_region_ms"], 2)}


def bench_gemm(hip, quant, synth, rng, stream, w_type, tokens, out_dim, in_dim, steps, warmup, graph=True, packed=False):
    """Prefill GEMM (x repack + MFMA kernel, every launch of the call) at `tokens`; returns the case record. Consecutive
    steps read different copies of the weights, as the GEMV cases do, so that a step's weights come from HBM and not from
    the last-level cache the previous step left them in. packed: the activations are packed once, outside the timed
    region - the GEMM as it runs behind a producer that writes them packed (cogni_rmsnorm_gemm_pack_dev, the SwiGLU GEMM)."""
    raw = synth.make_weights(rng, w_type, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    wsb = quant.gemm_workspace_bytes(w_type, in_dim, tokens, out_dim)
    copies = int(max(2, min(24, -(-int(1.2 * LLC_BYTES) // raw.nbytes))))
    wbufs = []
    for c in range(copies):
        b = hip.DeviceBuffer(raw.nbytes)
        hip.copy_htod(b.ptr, raw if c == 0 else np.roll(raw, 4096 * c + 17), raw.nbytes, "w")
        wbufs.append(b)
    bufs = [hip.DeviceBuffer(n) for n in (x.nbytes, 4 * tokens * out_dim, wsb)]
    hip.copy_htod(bufs[0].ptr, x, x.nbytes, "x")

    if packed:
        quant.gemm_pack_dev(bufs[0].ptr, w_type, in_dim, tokens, bufs[2].ptr, wsb, stream.handle)
        stream.synchronize()

    def launch(copy, st):
        if packed:
            quant.gemm_packed_dev(wbufs[copy].ptr, w_type, bufs[2].ptr, wsb, bufs[1].ptr, in_dim, out_dim, tokens, 0, st.handle)
        else:
            quant.gemm_dev(wbufs[copy].ptr, w_type, bufs[0].ptr, bufs[1].ptr, in_dim, out_dim, tokens, bufs[2].ptr, wsb, 0,
                           st.handle)
    r = measure(hip, stream, Rotating(launch, copies, raw.nbytes), steps, warmup, graph)
    kernel, grid_x, splits, block = quant.gemm_plan(w_type, in_dim, out_dim, tokens, wsb)
    for b in bufs + wbufs:
        b.close()
    flops = 2.0 * tokens * out_dim * in_dim
    tf = flops / r["us"] / 1e6
    return {"us": round(r["us"], 2), "us_min": round(r["us_min"], 2), "us_max": round(r["us_max"], 2),
            "tflops": round(tf, 1), "frac_mfma_f16": round(tf / MFMA_F16_PEAK_TFLOPS, 4), "flops": flops,
            "samples": r["samples"], "timed_region_ms": round(r["timed_region_ms"], 2),
            "kernel": kernel, "grid": [grid_x, splits], "block": block, "weight_copies_rotated": r["buffers_rotated"],
            "includes": ("GEMM against activations packed by their producer" if packed else "activation repack + GEMM") +
                        " (+ plane sum where the k range is split)"}


def raw_gemm_bytes(tokens, out_dim, in_dim):
    """Algorithmic bytes of the Q4_K GEMM kernel alone: weights once, packed fp16 x in, fp32 out."""
    return out_dim * (in_dim // 256) * 144 + 2 * tokens * in_dim + 4 * tokens * out_dim


def cpu_baseline(oracle, case, budget_s=10.0, threads=1):
    """The CPU oracle (C restatement of QuantMatmul.matmul_add, f64 accumulation) on the same matrix: one thread, or
    the output rows divided among `threads` host threads."""
    zero = np.zeros(case.out_dim, dtype=np.float32)
    reps, t0 = 0, time.perf_counter()
    while True:
        ref = oracle.matmul_add(case.host_x, case.tokens, case.in_dim, case.host_w, case.w_type, case.out_dim, zero,
                                threads=threads)
        reps += 1
        el = time.perf_counter() - t0
        if el >= budget_s and reps >= 3 or reps >= 200:
            break
    return ref, reps, el


def kernel_source_hash():
    """sha256 (first 16 hex digits) over the kernel sources of the code object: a traffic record counted on other sources
    is reported as stale."""
    import glob
    import hashlib
    h = hashlib.sha256()
    base = os.path.join(ROOT, "cogni-ml_amd", "csrc")
    for path in sorted(glob.glob(os.path.join(base, "kernels", "*.h*")) + [os.path.join(base, "cogni_quant_kernels.hip")]):
        h.update(open(path, "rb").read())
    return h.hexdigest()[:16]


def recorded_traffic(kernel):
    """HBM bytes per launch of `kernel` as the profiler counted them: the record of that kernel in profiles/traffic.json
    (written from two rocprofv3 --pmc runs of `bench.py --mode pmc`; the file names the commit and the commands). Returns
    (bytes or None, record or None); the record carries "stale": true when the kernel sources have changed since."""
    try:
        doc = json.load(open(TRAFFIC_JSON))
        rec = dict(doc["kernels"][kernel])
        rec["commit"] = doc.get("commit")
        rec["stale"] = doc.get("kernel_source_hash") != kernel_source_hash()
        return int(rec["bytes_per_launch"]), rec
    except Exception as e:
        log("no recorded traffic for %s (%s)" % (kernel, e))
        return None, None


def traffic_field(kernel, algorithmic_bytes):
    """The "traffic" entry of a case record."""
    nbytes, rec = recorded_traffic(kernel)
    if rec is None:
        return None
    return {"kernel": kernel, "bytes_per_launch": nbytes, "x_algorithmic": round(nbytes / max(1, algorithmic_bytes), 3),
            "workload": rec.get("workload"), "commit": rec.get("commit"), "stale": rec["stale"]}


def gemv_kernel_of(quant, w_type, tokens, in_dim, out_dim):
    """The kernel that dominates a gemv_dev call of this shape."""
    frm = quant.gemv_one_pass_from(w_type, in_dim, out_dim)
    if frm and tokens >= frm:
        return {Q4_K: "q4_k", Q5_K: "q5_k", Q6_K: "q6_k", Q8_0: "q8_0"}[w_type] + "_gemv_mt_f32"
    return quant.gemv_plan(w_type, min(tokens, 4) if tokens > 1 else 1, in_dim, out_dim)[0]


def steps_for(args, bytes_per_step, cap_bytes=6e9):
    return int(max(4, min(args.steps, cap_bytes // max(1, bytes_per_step))))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--mode", choices=["headline", "cases", "pmc", "pmc-gemm", "ceiling"], default="headline")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--launch", choices=["graph", "direct"], default="graph",
                    help="direct: no HIP graphs, for runs under rocprofv3 (it crashes in hipGraphLaunch when a graph is "
                         "replayed back to back); per-step times then include the host's launch cost, kernel durations do not")
    ap.add_argument("--seed", type=int, default=1234)
    args = ap.parse_args()
    global USE_GRAPHS
    USE_GRAPHS = args.launch == "graph"
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the path has no multi-GPU part (run with --gpus 1)")
    if args.steps <= 0 or args.warmup < 0:
        sys.exit("--steps must be positive and --warmup non-negative")

    from cogni_ml_amd import hip, quant, synth
    from oracle import oracle

    t_start = time.perf_counter()
    ctx = hip.Context.create(0)
    quant.init(0)
    log("device=%s arch=%s compute_units=%d clock_mhz=%d host_cores=%d" % (
        ctx.device_name, ctx.arch, ctx.compute_units, ctx.clock_khz // 1000, os.cpu_count()))
    rng = np.random.default_rng(args.seed)
    stream = hip.HIPStream()

    if args.mode == "pmc-gemm":
        # plain launches of the prefill GEMM (M = 512) for profiler runs
        rec = bench_gemm(hip, quant, synth, rng, stream, Q4_K, 512, 12288, 4096, args.steps, args.warmup, graph=False)
        log("pmc-gemm mode: M=512 us=%.2f tflops=%.1f" % (rec["us"], rec["tflops"]))
        return

    head = GemvCase(hip, quant, synth, rng, Q4_K, 12288, 4096, 1)

    if args.mode == "pmc":
        # plain (uncaptured) launches so a profiler attributes counters per dispatch: the dominant kernel of the headline,
        # of the Q6_K down projection, of the one-pass decode at 8 tokens and of the prefill GEMM at M = 512 and 2048, each
        # over rotating weight copies, then a copy kernel that moves a known number of bytes and calibrates the counters' units
        mk = MeasureKernels(hip)
        copy_fn = mk.fn("copy_bytes_16")
        nbytes = 512 << 20
        src, dst = hip.DeviceBuffer(nbytes), hip.DeviceBuffer(nbytes)
        params = hip.KernelParams(ctypes.c_uint64(src.ptr), ctypes.c_uint64(dst.ptr), ctypes.c_uint64(nbytes))
        n = args.warmup + args.steps
        for i in range(n):
            head.launch(i % head.copies, stream)
        stream.synchronize()
        for w_type, out_dim, in_dim, tokens in ((Q6_K, 4096, 12288, 1), (Q4_K, 12288, 4096, 8), (Q6_K, 4096, 12288, 8), (Q8_0, 4096, 4096, 8)):
            c = GemvCase(hip, quant, synth, rng, w_type, out_dim, in_dim, tokens, min_total_bytes=LLC_BYTES + (64 << 20))
            for i in range(n):
                c.launch(i % c.copies, stream)
            stream.synchronize()
            log("pmc mode: %d x %s %dx%d M=%d -> %s over %d weight copies" % (
                n, TYPE_NAME[w_type], in_dim, out_dim, tokens, gemv_kernel_of(quant, w_type, tokens, in_dim, out_dim), c.copies))
            c.close()
        for tokens in (512, 2048):
            rec = bench_gemm(hip, quant, synth, rng, stream, Q4_K, tokens, 12288, 4096, max(4, n // 4), 2, graph=False)
            log("pmc mode: prefill GEMM M=%d -> %s (pack_x_f16_q4k in front), %d weight copies" % (tokens, rec["kernel"], rec["weight_copies_rotated"]))
        # the bulk dequantize of a 12288x4096 matrix, Q4_K and Q6_K (the copy kernel's 512 MiB destination takes the output)
        for w_type in (Q4_K, Q6_K):
            draw = synth.make_weights(rng, w_type, 12288, 4096)
            dbufs = []
            for c in range(3):
                b = hip.DeviceBuffer(draw.nbytes)
                hip.copy_htod(b.ptr, draw, draw.nbytes, "w")
                dbufs.append(b)
            for i in range(max(6, n // 4)):
                quant.dequantize_dev(dbufs[i % 3].ptr, w_type, 12288 * 4096, dst.ptr + (i % 2) * (256 << 20), stream.handle)
            stream.synchronize()
            log("pmc mode: %d x %s of a 12288x4096 matrix" % (max(6, n // 4), quant.dequantize_kernel_name(w_type)))
            for b in dbufs:
                b.close()
        with hip.with_stream(stream):
            for i in range(8):
                hip.launch(copy_fn, 8192, 1, 1, 256, 1, 1, params, "copy_bytes_16")
        stream.synchronize()
        log("pmc mode: %d x %s over %d weight copies, 8 x copy_bytes_16 of %d bytes" % (
            n, quant.gemv_kernel_name(Q4_K, 1), head.copies, nbytes))
        return

    if args.mode == "ceiling":
        # what the machine gives a trivial kernel under the same timing method: an empty launch, and a
        # read-only stream over the same rotating weight buffers
        mk = MeasureKernels(hip)
        copy_fn, read_fn = mk.fn("copy_bytes_16"), mk.fn("read_bytes_16")
        nul = hip.KernelParams(ctypes.c_uint64(head.w[0].ptr), ctypes.c_uint64(mk.sink.ptr), ctypes.c_uint64(0))

        def empty(copy, st):
            with hip.with_stream(st):
                hip.launch(copy_fn, 768, 1, 1, 256, 1, 1, nul, "empty")
        r = measure(hip, stream, Rotating(empty, 1, 1 << 30), args.steps, args.warmup)
        log("empty_kernel_us=%.3f" % r["us"])
        for grid in (256, 512, 1024, 2048, 4096, 8192):
            boxes = [hip.KernelParams(ctypes.c_uint64(b.ptr), ctypes.c_uint64(mk.sink.ptr), ctypes.c_uint64(head.w_bytes))
                     for b in head.w]

            def rd(copy, st, grid=grid, boxes=boxes):
                with hip.with_stream(st):
                    hip.launch(read_fn, grid, 1, 1, 256, 1, 1, boxes[copy], "read")
            r = measure(hip, stream, Rotating(rd, head.copies, head.w_bytes), args.steps, args.warmup)
            log("read_only grid=%d us=%.3f gbps=%.1f" % (grid, r["us"], head.w_bytes / r["us"] / 1e3))
        # a loop of nothing but fp16 MFMAs on every SIMD of the chip, one and two wavefronts per SIMD, short and long
        # (the clock the chip sustains under that load is part of the answer)
        ops = hip.DeviceBuffer(7 * 64 * 16)
        vals = (rng.standard_normal(7 * 64 * 8) * 0.5).astype(np.float16)
        hip.copy_htod(ops.ptr, vals, vals.nbytes, "mfma operands")
        res = hip.DeviceBuffer(4 * 512 * 1024)
        for name, block in (("mfma_f16_ceiling_w4", 256), ("mfma_f16_ceiling_w8", 512)):
            fn = mk.fn(name)
            for wgs in (256, 1024):
                for iters in (128, 1024):
                    box = hip.KernelParams(ctypes.c_uint64(ops.ptr), ctypes.c_uint64(res.ptr), ctypes.c_uint32(iters))

                    def mm(copy, st, fn=fn, wgs=wgs, block=block, box=box):
                        with hip.with_stream(st):
                            hip.launch(fn, wgs, 1, 1, block, 1, 1, box, "mfma")
                    r = measure(hip, stream, Rotating(mm, 1, 1 << 30), 20, 3)
                    flops = 2.0 * 32 * 32 * 16 * 12 * iters * (block // 64) * wgs
                    log("%s workgroups=%d iters=%d us=%.2f tflops=%.1f frac_of_published_peak=%.3f" % (
                        name, wgs, iters, r["us"], flops / r["us"] / 1e6, flops / r["us"] / 1e6 / MFMA_F16_PEAK_TFLOPS))
        # the same twelve MFMAs per k-step with the prefill GEMM's other work added piece by piece: token-tile reads
        # from LDS (all variants), global -> LDS copies of 1 KiB per wavefront, the 4-bit decode's vector instructions
        region = hip.DeviceBuffer((1 << 20) + (1 << 17))
        fill = (rng.standard_normal(region.bytesize // 2) * 0.25).astype(np.float16)
        hip.copy_htod(region.ptr, fill, fill.nbytes, "probe operands")
        iters, wgs = 256, 256
        base = None
        for name in ("bare", "decode", "copy1", "copy2", "copy3", "copy2_decode", "copy3_decode"):
            fn = mk.fn("mfma_step_probe_" + name)
            box = hip.KernelParams(ctypes.c_uint64(region.ptr), ctypes.c_uint64(res.ptr), ctypes.c_uint32(iters))

            def pr(copy, st, fn=fn, box=box):
                with hip.with_stream(st):
                    hip.launch(fn, wgs, 1, 1, 256, 1, 1, box, "probe")
            r = measure(hip, stream, Rotating(pr, 1, 1 << 30), 20, 3)
            step_ns = r["us"] * 1e3 / (iters * 8)
            base = step_ns if base is None else base
            flops = 2.0 * 32 * 32 * 16 * 12 * 8 * iters * 4 * wgs
            log("mfma_step_probe_%s k_step_ns=%.1f (+%.1f over bare) tflops=%.1f frac_of_published_peak=%.3f" % (
                name, step_ns, step_ns - base, flops / r["us"] / 1e6, flops / r["us"] / 1e6 / MFMA_F16_PEAK_TFLOPS))
        return

    mk = MeasureKernels(hip)
    cases = {}

    # ---- the headline: timed first, checked against the oracle afterwards -------------------------------------
    head.launch(0, stream)
    stream.synchronize()
    got = head.read_out()
    hr = measure(hip, stream, head.rotating(), args.steps, args.warmup)
    ms_per_step = hr["us"] * 1e-3
    gbps = head.bytes_per_step / hr["us"] / 1e3
    # cache-resident figure (one copy only), reported beside the HBM one
    hot = measure(hip, stream, Rotating(lambda c, s: head.launch(0, s), 1, head.w_bytes), args.steps, args.warmup)
    # (for reading a kernel trace of this run: the first dispatches of the headline kernel, in order)
    log("headline_dispatch_order=1 parity launch, %d over rotating copies, %d over one copy" % (hr["launches"], hot["launches"]))
    hot_gbps = head.bytes_per_step / hot["us"] / 1e3
    floor_us, floor_grid = mk.read_floor(stream, head, args.steps, args.warmup)
    log("case=q4_k_gemv ffn_up\ntype=Q4_K\nshape=%dx%d\ntokens=1\nraw_bytes=%d\ncopies=%d\nreps=%d\nwarmup=%d\n"
        "hip_us=%.3f\nhip_us_min=%.3f\nhip_us_max=%.3f\nsamples=%d\ngbps_hbm=%.1f\ngbps_cache_hot=%.1f\nread_only_us=%.3f\ngraph=%s" % (
            head.in_dim, head.out_dim, head.w_bytes, hr["buffers_rotated"], args.steps, args.warmup, hr["us"], hr["us_min"],
            hr["us_max"], hr["samples"], gbps, hot_gbps, floor_us, hr["graphed"]))

    def gemv_case(name, w_type, out_dim, in_dim, tokens, floor=None):
        c = GemvCase(hip, quant, synth, rng, w_type, out_dim, in_dim, tokens)
        steps = steps_for(args, c.bytes_per_step)
        r = measure(hip, stream, c.rotating(), steps, min(args.warmup, steps))
        rec = gemv_record(r, c.bytes_per_step)
        rec["steps"] = steps
        rec["kernel"] = gemv_kernel_of(quant, w_type, tokens, in_dim, out_dim)
        rec["passes_over_weights"] = quant.gemv_passes(w_type, tokens, in_dim, out_dim)
        rec["traffic"] = traffic_field(rec["kernel"], c.bytes_per_step)
        if floor if floor is not None else c.w_bytes < (16 << 20):
            fu, fg = mk.read_floor(stream, c, steps, min(args.warmup, steps))
            rec["read_only_us"] = round(fu, 3)
            rec["x_read_only"] = round(r["us"] / fu, 3)
        cases[name] = rec
        log("case=%s\ntype=%s\nshape=%dx%d\ntokens=%d\nraw_bytes=%d\ncopies=%d\nreps=%d\nhip_us=%.3f\ngbps_hbm=%.1f\nfrac_hbm=%.4f\n%s" % (
            name, TYPE_NAME[w_type], in_dim, out_dim, tokens, c.w_bytes, r["buffers_rotated"], steps, r["us"], rec["gbps"],
            rec["frac_hbm"], "read_only_us=%.3f\n" % rec["read_only_us"] if "read_only_us" in rec else ""))
        c.close()

    # config 1, the rest of config 2, config 3
    gemv_case("cfg1 q8_0 gemv 3584x1024 M=1", Q8_0, 3584, 1024, 1)
    gemv_case("cfg2 q4_k gemv down 4096x12288 M=1", Q4_K, 4096, 12288, 1)
    gemv_case("cfg3 q6_k gemv output head 151936x4096 M=1", Q6_K, 151936, 4096, 1)
    gemv_case("cfg3 q6_k gemv down 4096x12288 M=1", Q6_K, 4096, 12288, 1)
    gemv_case("cfg3 q5_k gemv 4096x4096 M=1", Q5_K, 4096, 4096, 1)
    # several tokens against one pass over the weights (what config 5's row batches are made of)
    gemv_case("q4_k gemv 12288x4096 M=4", Q4_K, 12288, 4096, 4)
    gemv_case("q4_k gemv 12288x4096 M=8", Q4_K, 12288, 4096, 8)
    # the same GEMV against an activation image that is already there (the norm in front wrote it, or an earlier matrix of the
    # same input paid for the pack): what a projection costs inside a runner
    img_case = GemvCase(hip, quant, synth, rng, Q4_K, 12288, 4096, 8)
    image = hip.DeviceBuffer(quant.gemv_image_bytes(Q4_K, 4096, 8))
    quant.gemv_pack_dev(img_case.x.ptr, Q4_K, 4096, 8, image.ptr, stream.handle)

    def packed_only(copy, st):
        quant.gemv_packed_dev([img_case.w[copy].ptr], Q4_K, image.ptr, [img_case.out.ptr], [12288], 4096, 8, 0, st.handle)
    steps = steps_for(args, img_case.bytes_per_step)
    r = measure(hip, stream, Rotating(packed_only, img_case.copies, img_case.w_bytes), steps, min(args.warmup, steps))
    rec = gemv_record(r, img_case.bytes_per_step)
    rec.update({"steps": steps, "kernel": "q4_k_gemv_mt_f32", "passes_over_weights": 1,
                "traffic": traffic_field("q4_k_gemv_mt_f32", img_case.bytes_per_step)})
    cases["q4_k gemv 12288x4096 M=8, image kept by the caller (no pack launch)"] = rec
    log("case=q4_k gemv M=8 against a kept image\nhip_us=%.3f\ngbps_hbm=%.1f\n" % (r["us"], rec["gbps"]))
    image.close()
    img_case.close()
    # Q8_0 at eight tokens: the draft model's ffn_up and ffn_down shapes, one pass on the matrix cores
    gemv_case("q8_0 gemv 3584x1024 M=8", Q8_0, 3584, 1024, 8)
    gemv_case("q8_0 gemv 1024x3584 M=8", Q8_0, 1024, 3584, 8)
    if args.mode == "cases":
        gemv_case("q4_k gemv 4096x12288 M=4", Q4_K, 4096, 12288, 4)
        gemv_case("q4_k gemv 4096x12288 M=8", Q4_K, 4096, 12288, 8)
        gemv_case("q6_k gemv 4096x12288 M=4", Q6_K, 4096, 12288, 4)
        gemv_case("q6_k gemv 4096x12288 M=8", Q6_K, 4096, 12288, 8)
        gemv_case("q5_k gemv 4096x4096 M=4", Q5_K, 4096, 4096, 4)
        gemv_case("q5_k gemv attn_qkv 8192x4096 M=8", Q5_K, 8192, 4096, 8)
        gemv_case("q6_k gemv output head 151936x4096 M=2", Q6_K, 151936, 4096, 2)
        gemv_case("q6_k gemv output head 151936x4096 M=8", Q6_K, 151936, 4096, 8)

    # bulk dequantize (Dequant.dequantize_* on device pointers): a 12288x4096 matrix of each block format to float32, three
    # rotating sets of input and output (690 MB per rotation: nothing comes out of or stays in the last-level cache)
    dq_n = 12288 * 4096
    dq_out = [hip.DeviceBuffer(4 * dq_n) for _ in range(3)]
    for w_type in (Q8_0, Q4_K, Q5_K, Q6_K):
        draw = synth.make_weights(rng, w_type, 12288, 4096)
        dws = []
        for c in range(3):
            b = hip.DeviceBuffer(draw.nbytes)
            hip.copy_htod(b.ptr, draw if c == 0 else np.roll(draw, 4096 * c + 34), draw.nbytes, "w")
            dws.append(b)

        def deq(copy, st, dws=dws, w_type=w_type):
            quant.dequantize_dev(dws[copy].ptr, w_type, dq_n, dq_out[copy].ptr, st.handle)
        r = measure(hip, stream, Rotating(deq, 3, draw.nbytes + 4 * dq_n), max(5, min(30, args.steps)), 3)
        rec = gemv_record(r, draw.nbytes + 4 * dq_n)
        rec["kernel"] = quant.dequantize_kernel_name(w_type)
        rec["traffic"] = traffic_field(rec["kernel"], draw.nbytes + 4 * dq_n)
        cases["%s dequantize 12288x4096 (50.3 M values to float32)" % TYPE_NAME[w_type].lower()] = rec
        log("case=dequantize\ntype=%s\nelements=%d\nhip_us=%.2f\ngbps_hbm=%.1f\nfrac_hbm=%.4f\n" % (
            TYPE_NAME[w_type], dq_n, r["us"], rec["gbps"], rec["frac_hbm"]))
        for b in dws:
            b.close()
    for b in dq_out:
        b.close()

    # config 4: prefill GEMM
    gemm = {}
    for tokens in (64, 512, 2048):
        gsteps = max(5, min(100, args.steps, int(4e12 // (2.0 * tokens * 12288 * 4096))))
        rec = bench_gemm(hip, quant, synth, rng, stream, Q4_K, tokens, 12288, 4096, gsteps, min(5, args.warmup))
        rec["steps"] = gsteps
        rec["traffic"] = traffic_field(rec["kernel"], raw_gemm_bytes(tokens, 12288, 4096))
        gemm["M=%d" % tokens] = rec
        cases["cfg4 q4_k gemm 12288x4096 M=%d" % tokens] = rec
        log("case=q4_k_gemm prefill\ntype=Q4_K\nshape=4096x12288\ntokens=%d\nreps=%d\nhip_us=%.2f\ntflops=%.1f\nfrac_mfma_f16_peak=%.4f\n" % (
            tokens, gsteps, rec["us"], rec["tflops"], rec["frac_mfma_f16"]))
    # the same GEMM behind a producer that hands it packed activations (the norm, the SwiGLU GEMM): no pack launch in the step
    rec = bench_gemm(hip, quant, synth, rng, stream, Q4_K, 512, 12288, 4096, max(5, min(100, args.steps)), min(5, args.warmup), packed=True)
    rec["traffic"] = traffic_field(rec["kernel"], raw_gemm_bytes(512, 12288, 4096))
    cases["cfg4 q4_k gemm 12288x4096 M=512, activations packed by the producer (no pack launch)"] = rec
    log("case=q4_k_gemm prefill, packed activations\ntokens=512\nhip_us=%.2f\ntflops=%.1f\nfrac_mfma_f16_peak=%.4f\n" % (
        rec["us"], rec["tflops"], rec["frac_mfma_f16"]))
    # the feed-forward block of a layer at M = 512 in its prefill form: add + RMSNorm, pack, gate | up GEMM with SwiGLU inside
    # (its epilogue writes the down GEMM's packed input), Q6_K down GEMM with the residual inside (three rotating sets of
    # weights: 290 MB)
    from cogni_ml_amd.ffn_sequence import FFNSequenceRunner as _FFN
    ffn_tokens = 512
    fx = rng.uniform(-0.1, 0.1, ffn_tokens * 4096).astype(np.float32)
    fnorm = np.full(4096, 0.1, dtype=np.float32)
    ffns = []
    for _ in range(3):
        fr = _FFN(synth.make_weights(rng, Q4_K, 12288, 4096), synth.make_weights(rng, Q4_K, 12288, 4096),
                  synth.make_weights(rng, Q6_K, 4096, 12288), 4096, 12288, ffn_tokens, fx, norm=fnorm, add=fx.copy(), keep_combined=False)
        fr.upload_weights()
        fr.reset_sequence()
        ffns.append(fr)

    def ffn_seq(copy, st, ffns=ffns):
        with hip.with_stream(st):
            ffns[copy].run_sequence()
    r = measure(hip, stream, Rotating(ffn_seq, 3, 97 << 20), max(5, min(30, args.steps)), 3)
    fflops = ffns[0].flops_per_sequence()
    cases["cfg4 ffn block prefill M=512 (add+rmsnorm, gate|up|swiglu gemm, q6_k down gemm + residual)"] = {
        "us": round(r["us"], 2), "tflops": round(fflops / r["us"] / 1e6, 1),
        "frac_mfma_f16": round(fflops / r["us"] / 1e6 / MFMA_F16_PEAK_TFLOPS, 4), "flops": fflops,
        "launches": "add_rmsnorm, pack, q4_k_gemm_swiglu_pack_q6k_f16, q6_k_gemm_n128_f16 (k split) + plane sum with the residual"}
    log("case=ffn block prefill M=512\nhip_us=%.2f\ntflops=%.1f\nfrac_mfma_f16_peak=%.4f\n" % (
        r["us"], fflops / r["us"] / 1e6, fflops / r["us"] / 1e6 / MFMA_F16_PEAK_TFLOPS))
    for fr in ffns:
        fr.close()

    if args.mode == "cases":
        for name, t, o, i in (("q6_k gemm down 4096x12288 M=512", Q6_K, 4096, 12288), ("q5_k gemm 12288x4096 M=512", Q5_K, 12288, 4096)):
            rec = bench_gemm(hip, quant, synth, rng, stream, t, 512, o, i, 50, 5)
            cases[name] = rec
            log("case=%s\nhip_us=%.2f\ntflops=%.1f\nfrac_mfma_f16_peak=%.4f\n" % (name, rec["us"], rec["tflops"], rec["frac_mfma_f16"]))

        # gate and up of one layer at M = 512 against activations packed once (cogni_gemm_pack_dev + 2 x cogni_gemm_packed_dev)
        tokens = 512
        graws = [synth.make_weights(rng, Q4_K, 12288, 4096) for _ in range(2)]
        gx = synth.make_activations(rng, tokens, 4096)
        gwsb = quant.gemm_workspace_bytes(Q4_K, 4096, tokens, 12288)
        gbufs = [hip.DeviceBuffer(n) for n in (graws[0].nbytes, graws[1].nbytes, gx.nbytes, 4 * tokens * 12288, 4 * tokens * 12288, gwsb)]
        for b_, h_ in zip(gbufs[:3], graws + [gx]):
            hip.copy_htod(b_.ptr, h_, h_.nbytes, "gemm pair input")

        def gpair(copy, st):
            quant.gemm_pack_dev(gbufs[2].ptr, Q4_K, 4096, tokens, gbufs[5].ptr, gwsb, st.handle)
            quant.gemm_packed_dev(gbufs[0].ptr, Q4_K, gbufs[5].ptr, gwsb, gbufs[3].ptr, 4096, 12288, tokens, 0, st.handle)
            quant.gemm_packed_dev(gbufs[1].ptr, Q4_K, gbufs[5].ptr, gwsb, gbufs[4].ptr, 4096, 12288, tokens, 0, st.handle)
        r = measure(hip, stream, Rotating(gpair, 1, 2 * graws[0].nbytes), 50, 5)
        gflops = 2 * 2.0 * tokens * 12288 * 4096
        cases["q4_k gemm gate and up 12288x4096 M=512, x packed once"] = {
            "us": round(r["us"], 2), "tflops": round(gflops / r["us"] / 1e6, 1),
            "frac_mfma_f16": round(gflops / r["us"] / 1e6 / MFMA_F16_PEAK_TFLOPS, 4), "flops": gflops,
            "includes": "one activation repack + two GEMMs"}
        log("case=q4_k gemm gate and up, x packed once M=512\nhip_us=%.2f\ntflops=%.1f\nfrac_mfma_f16_peak=%.4f\n" % (
            r["us"], gflops / r["us"] / 1e6, gflops / r["us"] / 1e6 / MFMA_F16_PEAK_TFLOPS))
        for b_ in gbufs:
            b_.close()

    # config 5: the mixed-quant projection stack, back to back in one stream. Three resident layers are walked in turn
    # (364 MB of weights), so that a layer's weights come from HBM as they do in a model of many layers; the figure
    # with one layer alone (121.5 MB, which the last-level cache keeps between repetitions) is reported beside it.
    from cogni_ml_amd.projection_stack import QwenProjectionStackRunner, Weights
    layers = [Weights.synthetic(rng) for _ in range(3)]
    for tokens in (1, 4, 8):
        xs = synth.make_activations(rng, tokens, layers[0].hidden)
        runners = [QwenProjectionStackRunner.from_weights(w, tokens, xs) for w in layers]
        for r_ in runners:
            r_.upload_weights()
            r_.reset_sequence()

        def seq(copy, st, runners=runners):
            with hip.with_stream(st):
                runners[copy].run_sequence()
        nbytes = runners[0].bytes_per_sequence()
        steps = max(6, min(args.steps, 300))
        r = measure(hip, stream, Rotating(seq, 3, layers[0].raw_bytes), steps, min(args.warmup, 10))
        rec = gemv_record(r, nbytes)
        rec["steps"] = steps
        r1 = measure(hip, stream, Rotating(seq, 1, layers[0].raw_bytes), steps, min(args.warmup, 10))
        rec["us_cache_resident"] = round(r1["us"], 3)
        rec["gbps_cache_resident"] = round(nbytes / r1["us"] / 1e3, 1)
        rec["launches_per_sequence"] = "q|k|v, o, gate|up, down per group of tokens"
        cases["cfg5 projection stack M=%d" % tokens] = rec
        log("case=projection stack (q,k,v,o,gate,up Q4_K + down Q6_K)\ntokens=%d\nraw_bytes=%d\nreps=%d\nhip_us=%.3f\n"
            "gbps_hbm=%.1f\nfrac_hbm=%.4f\nhip_us_cache_resident=%.3f\n" % (
                tokens, layers[0].raw_bytes, steps, r["us"], rec["gbps"], rec["frac_hbm"], r1["us"]))
        for r_ in runners:
            r_.close()
    # sixteen tokens through the router: between the GEMM threshold and sixteen tokens cogni_matmul_dev takes the one-pass decode
    # kernels with sixteen single-term tokens (image + kernel), the GEMM's precision class
    mraw = synth.make_weights(rng, Q4_K, 12288, 4096)
    mcopies = int(max(2, min(24, -(-int(1.2 * LLC_BYTES) // mraw.nbytes))))
    mbufs = []
    for c in range(mcopies):
        b = hip.DeviceBuffer(mraw.nbytes)
        hip.copy_htod(b.ptr, mraw if c == 0 else np.roll(mraw, 4096 * c + 17), mraw.nbytes, "w")
        mbufs.append(b)
    mx = synth.make_activations(rng, 16, 4096)
    mwsb = quant.gemm_workspace_bytes(Q4_K, 4096, 16, 12288)
    mdev = [hip.DeviceBuffer(n) for n in (mx.nbytes, 4 * 16 * 12288, mwsb)]
    hip.copy_htod(mdev[0].ptr, mx, mx.nbytes, "x")

    def m16(copy, st):
        quant.matmul_dev(mbufs[copy].ptr, Q4_K, mdev[0].ptr, mdev[1].ptr, 4096, 12288, 16, mdev[2].ptr, mwsb, 0, st.handle)
    r = measure(hip, stream, Rotating(m16, mcopies, mraw.nbytes), max(5, min(100, args.steps)), min(5, args.warmup))
    m16_bytes = mraw.nbytes + 4 * 16 * (4096 + 12288)
    rec = gemv_record(r, m16_bytes)
    rec["launches"] = "pack_x_mt16_q4k_f16, q4_k_gemv_mt16_f32"
    cases["q4_k matmul 12288x4096 M=16 (router: sixteen tokens in one pass)"] = rec
    log("case=q4_k matmul M=16\nhip_us=%.3f\ngbps_hbm=%.1f\nfrac_hbm=%.4f\n" % (r["us"], rec["gbps"], rec["frac_hbm"]))
    for b in mbufs + mdev:
        b.close()
    # the same stack beyond the GEMM threshold (its prefill route): x packed once, q | k | v | gate | up as one list GEMM, o and
    # the Q6_K down projection behind their own packs
    for tokens in (16, 64, 512):
        xs = rng.uniform(-1.0, 1.0, tokens * layers[0].hidden).astype(np.float32)
        runners = [QwenProjectionStackRunner.from_weights(w, tokens, xs) for w in layers]
        for r_ in runners:
            r_.upload_weights()
            r_.reset_sequence()

        def pseq(copy, st, runners=runners):
            with hip.with_stream(st):
                runners[copy].run_sequence()
        steps = max(5, min(args.steps, 30))
        r = measure(hip, stream, Rotating(pseq, 3, layers[0].raw_bytes), steps, 3)
        pflops = 2.0 * tokens * sum(e[3] * e[4] for e in layers[0].entries)
        cases["cfg5 projection stack prefill M=%d" % tokens] = {
            "us": round(r["us"], 2), "tflops": round(pflops / r["us"] / 1e6, 1),
            "frac_mfma_f16": round(pflops / r["us"] / 1e6 / MFMA_F16_PEAK_TFLOPS, 4), "flops": pflops, "steps": steps,
            "launches": ("images of x, q and gate for sixteen single-term tokens; q|k|v, gate|up, o, down on the one-pass decode kernels" if tokens <= 16 else
                         "pack x, list GEMM q|k|v|gate|up, pack q, o GEMM, pack gate, Q6_K down GEMM (+ plane sums where the k range is split)")}
        log("case=projection stack prefill\ntokens=%d\nhip_us=%.2f\ntflops=%.1f\nfrac_mfma_f16_peak=%.4f\n" % (
            tokens, r["us"], pflops / r["us"] / 1e6, pflops / r["us"] / 1e6 / MFMA_F16_PEAK_TFLOPS))
        for r_ in runners:
            r_.close()

    if args.mode == "cases":
        # output head without the logits: RMSNorm -> Q6_K vocabulary projection with arg-max -> top-1 reduce (510 MB)
        from cogni_ml_amd.output_head import QwenOutputHeadRunner, Weights as HeadWeights
        hw = HeadWeights(np.ones(4096, dtype=np.float32), synth.make_weights(rng, Q6_K, 151936, 4096), Q6_K, 4096, 151936)
        for tokens in (1, 3, 8):
            ohead = QwenOutputHeadRunner.from_weights(hw, tokens, synth.make_activations(rng, tokens, 4096).reshape(-1), 1e-6)
            ohead.upload_weights()
            ohead.reset_sequence()

            def hseq(copy, st, ohead=ohead):
                with hip.with_stream(st):
                    ohead.run_sequence()
            r = measure(hip, stream, Rotating(hseq, 1, hw.output_raw.size), 10, 3)
            cases["q6_k output head top-1 M=%d" % tokens] = gemv_record(r, ohead.bytes_per_sequence())
            log("case=output head top-1 (rmsnorm -> q6_k gemv top1 partial -> reduce)\ntokens=%d\nhip_us=%.3f\n" % (tokens, r["us"]))
            ohead.close()

        # the gate | up pair of one layer against the same x in one launch (q4_k_dual_gemv_f32)
        a = GemvCase(hip, quant, synth, rng, Q4_K, 12288, 4096, 1, min_total_bytes=LLC_BYTES + (32 << 20))
        b = GemvCase(hip, quant, synth, rng, Q4_K, 12288, 4096, 1, min_total_bytes=LLC_BYTES + (32 << 20))
        out_b = hip.DeviceBuffer(4 * 12288)

        def dual(copy, st):
            quant.gemv_dual_dev(a.w[copy].ptr, b.w[copy].ptr, Q4_K, a.x.ptr, a.out.ptr, out_b.ptr, 4096, 12288, 1, st.handle)
        dsteps = max(20, min(args.steps, 1000))
        r = measure(hip, stream, Rotating(dual, min(a.copies, b.copies), 2 * a.w_bytes), dsteps, min(args.warmup, dsteps))
        cases["q4_k gate|up pair, one launch"] = gemv_record(r, 2 * a.w_bytes + 4 * 4096 + 2 * 4 * 12288)
        log("case=q4_k gate|up pair in one launch\nhip_us=%.3f\n" % r["us"])
        for o in (a, b, out_b):
            o.close()

        # FFN sequence of one layer: gate | up | SwiGLU in one launch, then Q6_K down with the residual add
        from cogni_ml_amd.ffn_sequence import FFNSequenceRunner
        graw = [synth.make_weights(rng, Q4_K, 12288, 4096) for _ in range(2)] + [synth.make_weights(rng, Q6_K, 4096, 12288)]
        for tokens, block in ((1, False), (4, False), (1, True), (4, True)):
            fx = rng.uniform(-1.0, 1.0, tokens * 4096).astype(np.float32)
            if block:   # the FFN half of a decoder layer: add + RMSNorm ahead of the projections
                ffn = FFNSequenceRunner(graw[0], graw[1], graw[2], 4096, 12288, tokens, fx, norm=np.ones(4096, dtype=np.float32), add=fx.copy())
            else:
                ffn = FFNSequenceRunner(graw[0], graw[1], graw[2], 4096, 12288, tokens, fx, fx.copy())
            ffn.upload_weights()
            ffn.reset_sequence()

            def fseq(copy, st, ffn=ffn):
                with hip.with_stream(st):
                    ffn.run_sequence()
            r = measure(hip, stream, Rotating(fseq, 1, sum(x_.size for x_ in graw)), max(20, min(args.steps // 4, 300)), 10)
            rec = gemv_record(r, ffn.bytes_per_sequence())
            rec["note"] = "weights (%.0f MB) stay in the last-level cache between repetitions" % (sum(x_.size for x_ in graw) / 1e6)
            cases["%s M=%d" % ("add+rmsnorm+ffn" if block else "ffn sequence", tokens)] = rec
            log("case=ffn sequence (gate|up Q4_K -> SwiGLU -> down Q6_K + residual)%s\ntokens=%d\nhip_us=%.3f\n" % (
                " with add+rmsnorm" if block else "", tokens, r["us"]))
            ffn.close()

    gpu_seconds = time.perf_counter() - t_start

    # ---- the oracle: parity of the measured kernel's output, and the CPU baseline (after the GPU work) ---------
    ref, cpu_reps, cpu_s = cpu_baseline(oracle, head, args.cpu_seconds)
    dense_max = float(np.max(np.abs(oracle.dequantize(head.host_w[:16 * 144 * 256], Q4_K, 256 * 4096))))
    max_diff = float(np.max(np.abs(got - ref)))
    cos = float(got.astype(np.float64) @ ref.astype(np.float64) /
                np.sqrt((got.astype(np.float64) @ got.astype(np.float64)) * (ref.astype(np.float64) @ ref.astype(np.float64))))
    tol = 1e-4 * float(np.linalg.norm(head.host_x)) * dense_max
    ok = cos >= 0.99999 and max_diff <= 1e-3 and max_diff <= tol
    cpu_gbps = head.bytes_per_step * cpu_reps / cpu_s / 1e9
    # the same restatement with the rows divided among the host cores this job may use (16 on a one-GPU box)
    mt_cores = max(1, min(16, os.cpu_count() or 1))
    _, mt_reps, mt_s = cpu_baseline(oracle, head, min(3.0, args.cpu_seconds), threads=mt_cores)
    mt_gbps = head.bytes_per_step * mt_reps / mt_s / 1e9
    log("cpu_baseline: 1 thread %.4f GB/s (%d reps, %.1f s); %d threads %.4f GB/s (%d reps, %.1f s); gcc -O2 -ffp-contract=off, "
        "stands in for the reference's Crystal QuantMatmul\ncpu_ms=%.3f\ncos=%.8f\nmax_diff=%g\nok=%s" % (
            cpu_gbps, cpu_reps, cpu_s, mt_cores, mt_gbps, mt_reps, mt_s, cpu_s / cpu_reps * 1e3, cos, max_diff, str(ok).lower()))

    traffic, traffic_rec = recorded_traffic("q4_k_gemv_f32")
    result = {
        "metric": "Q4_K GEMV GB/s 4096x12288 M=1",
        "value": round(gbps, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "Q4_K decode GEMV, W 12288x4096 (in 4096 -> out 12288), M=1, fp32 x, fp32 accumulate",
            "weight_bytes": head.w_bytes, "bytes_per_step": head.bytes_per_step,
            "weight_copies_rotated": hr["buffers_rotated"],
            "timed_region": ("median of %d samples, each %d replay(s) of a hip graph of K launches" if hr["graphed"] else
                             "median of %d samples, each %d x K direct launches") % (hr["samples"], hr["replays_per_sample"]),
        },
        "us_per_step": {"median": round(hr["us"], 3), "min": round(hr["us_min"], 3), "max": round(hr["us_max"], 3)},
        "timed_region_ms": round(hr["timed_region_ms"], 2),
        "pct_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "cache_hot_gbps": round(hot_gbps, 1),
        "read_only_kernel_same_bytes": {"us": round(floor_us, 3), "grid": floor_grid, "gbps": round(head.w_bytes / floor_us / 1e3, 1)},
        "prefill_gemm_q4k_12288x4096": gemm,
        "parity": {"cos": round(cos, 8), "max_diff": max_diff, "ok": ok, "tol_1e-4_x_wmax": tol},
        "roofline": {
            "bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": traffic,
            "traffic_source": None if traffic_rec is None else "profiles/traffic.json: rocprofv3 --pmc record for q4_k_gemv_f32 at commit %s%s, not counted in this run" % (
                traffic_rec.get("commit"), " (stale: the kernel sources have changed since)" if traffic_rec["stale"] else ""),
        },
        "cpu_baseline": {
            "value": round(cpu_gbps, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "%d x the same 12288x4096 Q4_K GEMV (M=1) through the C restatement of QuantMatmul.matmul_add, "
                      "1 thread, %.1f s" % (cpu_reps, cpu_s),
        },
        "cpu_baseline_all_cores": {"value": round(mt_gbps, 4), "unit": "GB/s", "cores": mt_cores, "kind": "port",
                                   "sample": "%d x the same GEMV, rows divided among %d threads, %.1f s" % (mt_reps, mt_cores, mt_s)},
        "cases": cases,
        "gpu_phase_seconds": round(gpu_seconds, 1),
    }
    head.close()
    stream.close()
    ctx.close()
    print(json.dumps(result), flush=True)
    if not ok:
        sys.exit(1)


if __name__ == "__main__":
    main()
