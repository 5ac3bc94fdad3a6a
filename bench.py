#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

Headline (the JSON line on stdout): Q4_K decode GEMV, W = 12288 x 4096 (in_dim 4096 -> out_dim 12288,
the ffn_gate/ffn_up shape), M = 1, fp32 activations and accumulation. One "step" is one GEMV launch.
Weights are seeded synthetic super-blocks, already resident in HBM; consecutive steps read different
copies of the matrix (more bytes in total than the 256 MB last-level cache) so every step streams
its 28 MB from HBM. The K timed steps are captured into one HIP graph and bracketed by HIP events
on the launch stream.

  python bench.py [--gpus 1] [--steps K] [--warmup W]
  python bench.py --mode cases      per-shape table (key=value blocks, stderr) + the JSON line
  python bench.py --mode pmc        plain launches of the dominant kernel and of a copy kernel of
                                    known size, for rocprofv3 --pmc / --kernel-trace runs
"""
import argparse
import json
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
# HBM bytes one q4_k_gemv_f32 launch moves at 12288x4096, M=1: rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE
# (13974.0 and 48.0 per dispatch), scaled by what a 512 MiB copy kernel reads on the same counters (2.0, 1.0)
MEASURED_TRAFFIC_BYTES = int((13967.0 * 2.0 + 48.0 * 1.0) * 1024)
LLC_BYTES = 256 << 20           # last-level (Infinity) cache
Q4_K, Q5_K, Q6_K, Q8_0 = 12, 13, 14, 8
TYPE_NAME = {Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K", Q8_0: "Q8_0"}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def gemv_bytes(w_bytes, in_dim, out_dim, tokens):
    """Algorithmic bytes of one GEMV: weights once + activations in + results out."""
    return w_bytes + 4 * tokens * in_dim + 4 * tokens * out_dim


class GemvCase:
    """Rotating weight copies + activations + output for one (type, shape, tokens)."""

    def __init__(self, hip, quant, synth, rng, w_type, out_dim, in_dim, tokens, min_total_bytes=2 * LLC_BYTES,
                 max_copies=24):
        from cogni_ml_amd.types import TensorType
        self.hip, self.quant = hip, quant
        self.w_type, self.out_dim, self.in_dim, self.tokens = w_type, out_dim, in_dim, tokens
        self.w_bytes = TensorType(w_type).data_bytes(in_dim) * out_dim
        self.copies = int(max(1, min(max_copies, -(-min_total_bytes // self.w_bytes))))
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

    def launch(self, step, stream):
        self.quant.gemv_dev(self.w[step % self.copies].ptr, self.w_type, self.x.ptr, self.out.ptr, self.in_dim,
                            self.out_dim, self.tokens, 0, stream.handle)

    def read_out(self):
        out = np.empty(self.tokens * self.out_dim, dtype=np.float32)
        self.hip.synchronize()
        self.hip.copy_dtoh(out, self.out.ptr, out.nbytes, "out")
        return out

    def close(self):
        for b in self.w + [self.x, self.out]:
            b.close()


def time_steps(hip, stream, launch, steps, warmup, graph=True):
    """Run `warmup` untimed and exactly `steps` timed launches on `stream`; returns ms for the timed region.
    The timed launches are captured into one HIP graph so host launch latency does not gate the GPU."""
    graph_wanted = bool(graph)
    graph, exe = None, None
    try:
        if not graph_wanted:
            raise RuntimeError("direct launches requested")
        stream.begin_capture(1)
        for i in range(steps):
            launch(warmup + i, stream)
        graph = stream.end_capture()
        exe = graph.instantiate()
        exe.upload(stream)
        stream.synchronize()
    except Exception as e:  # stream capture unavailable or not wanted: direct launches
        if graph_wanted:
            log("graph capture failed (%s); timing direct launches" % e)
        graph, exe = None, None
    # the warm-up runs once the graph is built, directly ahead of the timed region: capture and instantiation are
    # host work during which the GPU would otherwise sit idle and drop its clocks
    for i in range(warmup):
        launch(i, stream)
    e0, e1 = hip.Event(), hip.Event()
    hip.synchronize()
    e0.record(stream)
    if exe is not None:
        exe.launch(stream)
    else:
        for i in range(steps):
            launch(warmup + i, stream)
    e1.record(stream)
    e1.synchronize()
    hip.synchronize()
    ms = e0.elapsed_ms(e1)
    for o in (exe, graph):
        if o is not None:
            o.close()
    e0.close()
    e1.close()
    return ms, exe is not None


def bench_gemm(hip, quant, synth, rng, stream, tokens, out_dim, in_dim, steps, warmup, graph=True, Q4_K=Q4_K):
    """Prefill GEMM (x repack + MFMA kernel) at `tokens`, Q4_K unless another type is given; returns (ms per call, TFLOP/s)."""
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    wsb = quant.gemm_workspace_bytes(Q4_K, in_dim, tokens, out_dim)
    bufs = [hip.DeviceBuffer(n) for n in (raw.nbytes, x.nbytes, 4 * tokens * out_dim, wsb)]
    hip.copy_htod(bufs[0].ptr, raw, raw.nbytes, "w")
    hip.copy_htod(bufs[1].ptr, x, x.nbytes, "x")

    def launch(i, st):
        quant.gemm_dev(bufs[0].ptr, Q4_K, bufs[1].ptr, bufs[2].ptr, in_dim, out_dim, tokens, bufs[3].ptr, wsb, 0,
                       st.handle)
    ms, _ = time_steps(hip, stream, launch, steps, warmup, graph)
    for b in bufs:
        b.close()
    per = ms / steps
    return per, 2.0 * tokens * out_dim * in_dim / (per * 1e-3) / 1e12


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--mode", choices=["headline", "cases", "pmc", "pmc-gemm", "ceiling"], default="headline")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--seed", type=int, default=1234)
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the path has no multi-GPU part (run with --gpus 1)")
    if args.steps <= 0 or args.warmup < 0:
        sys.exit("--steps must be positive and --warmup non-negative")

    from cogni_ml_amd import hip, quant, synth
    from oracle import oracle

    ctx = hip.Context.create(0)
    quant.init(0)
    log("device=%s arch=%s compute_units=%d clock_mhz=%d host_cores=%d" % (
        ctx.device_name, ctx.arch, ctx.compute_units, ctx.clock_khz // 1000, os.cpu_count()))
    rng = np.random.default_rng(args.seed)
    stream = hip.HIPStream()

    if args.mode == "pmc-gemm":
        # plain launches of the prefill GEMM (M = 512) for profiler runs
        per, tf = bench_gemm(hip, quant, synth, rng, stream, 512, 12288, 4096, args.steps, args.warmup, graph=False)
        log("pmc-gemm mode: M=512 ms=%.5f tflops=%.1f" % (per, tf))
        return

    head = GemvCase(hip, quant, synth, rng, Q4_K, 12288, 4096, 1)

    if args.mode == "pmc":
        # plain (uncaptured) launches so a profiler attributes counters per dispatch; the copy kernel moves a
        # known number of bytes and calibrates the counters' units
        mod = hip.HIPModule.load_builtin()
        copy_fn = mod.function("copy_bytes_16")
        import ctypes
        nbytes = 512 << 20
        src, dst = hip.DeviceBuffer(nbytes), hip.DeviceBuffer(nbytes)
        params = hip.KernelParams(ctypes.c_uint64(src.ptr), ctypes.c_uint64(dst.ptr), ctypes.c_uint64(nbytes))
        with hip.with_stream(stream):
            for i in range(args.warmup + args.steps):
                head.launch(i, stream)
            for i in range(8):
                hip.launch(copy_fn, 8192, 1, 1, 256, 1, 1, params, "copy_bytes_16")
        stream.synchronize()
        log("pmc mode: %d x %s over %d weight copies, 8 x copy_bytes_16 of %d bytes" % (
            args.warmup + args.steps, quant.gemv_kernel_name(Q4_K, 1), head.copies, nbytes))
        return

    if args.mode == "ceiling":
        # what the machine gives a trivial kernel under the same timing method: an empty launch, and a
        # read-only stream over the same rotating weight buffers
        import ctypes
        mod = hip.HIPModule.load_builtin()
        copy_fn, read_fn = mod.function("copy_bytes_16"), mod.function("read_bytes_16")
        sink = hip.DeviceBuffer(4 * 65536)
        nul = hip.KernelParams(ctypes.c_uint64(head.w[0].ptr), ctypes.c_uint64(sink.ptr), ctypes.c_uint64(0))

        def empty(i, st):
            with hip.with_stream(st):
                hip.launch(copy_fn, 768, 1, 1, 256, 1, 1, nul, "empty")
        ms, _ = time_steps(hip, stream, empty, args.steps, args.warmup)
        log("empty_kernel_us=%.3f" % (ms / args.steps * 1e3))
        for grid in (256, 512, 1024, 2048, 4096, 8192):
            boxes = [hip.KernelParams(ctypes.c_uint64(b.ptr), ctypes.c_uint64(sink.ptr), ctypes.c_uint64(head.w_bytes))
                     for b in head.w]

            def rd(i, st, grid=grid, boxes=boxes):
                with hip.with_stream(st):
                    hip.launch(read_fn, grid, 1, 1, 256, 1, 1, boxes[i % len(boxes)], "read")
            ms, _ = time_steps(hip, stream, rd, args.steps, args.warmup)
            us = ms / args.steps * 1e3
            log("read_only grid=%d us=%.3f gbps=%.1f" % (grid, us, head.w_bytes / us / 1e3))
        # a loop of nothing but fp16 MFMAs on every SIMD of the chip, one and two wavefronts per SIMD, short and long
        # (the clock the chip sustains under that load is part of the answer)
        ops = hip.DeviceBuffer(7 * 64 * 16)
        vals = (rng.standard_normal(7 * 64 * 8) * 0.5).astype(np.float16)
        hip.copy_htod(ops.ptr, vals, vals.nbytes, "mfma operands")
        res = hip.DeviceBuffer(4 * 512 * 1024)
        for name, block in (("mfma_f16_ceiling_w4", 256), ("mfma_f16_ceiling_w8", 512)):
            fn = mod.function(name)
            for wgs in (256, 1024):
                for iters in (128, 1024):
                    box = hip.KernelParams(ctypes.c_uint64(ops.ptr), ctypes.c_uint64(res.ptr), ctypes.c_uint32(iters))

                    def mm(i, st, fn=fn, wgs=wgs, block=block, box=box):
                        with hip.with_stream(st):
                            hip.launch(fn, wgs, 1, 1, block, 1, 1, box, "mfma")
                    reps = 20
                    ms, _ = time_steps(hip, stream, mm, reps, 3)
                    us = ms / reps * 1e3
                    flops = 2.0 * 32 * 32 * 16 * 12 * iters * (block // 64) * wgs
                    log("%s workgroups=%d iters=%d us=%.2f tflops=%.1f frac_of_published_peak=%.3f" % (
                        name, wgs, iters, us, flops / us / 1e6, flops / us / 1e6 / MFMA_F16_PEAK_TFLOPS))
        return

    # ---- parity spot check of the measured kernel against the oracle, and the CPU baseline ------------
    head.launch(0, stream)
    stream.synchronize()
    got = head.read_out()
    ref, cpu_reps, cpu_s = cpu_baseline(oracle, head, args.cpu_seconds)
    dense_max = float(np.max(np.abs(oracle.dequantize(head.host_w[:16 * 144 * 256], Q4_K, 256 * 4096))))
    max_diff = float(np.max(np.abs(got - ref)))
    cos = float(got.astype(np.float64) @ ref.astype(np.float64) /
                np.sqrt((got.astype(np.float64) @ got.astype(np.float64)) * (ref.astype(np.float64) @ ref.astype(np.float64))))
    ok = cos >= 0.99999 and max_diff <= 1e-3
    cpu_gbps = head.bytes_per_step * cpu_reps / cpu_s / 1e9
    # the same restatement with the rows divided among the host cores this job may use (16 on a one-GPU box)
    mt_cores = max(1, min(16, os.cpu_count() or 1))
    _, mt_reps, mt_s = cpu_baseline(oracle, head, min(3.0, args.cpu_seconds), threads=mt_cores)
    mt_gbps = head.bytes_per_step * mt_reps / mt_s / 1e9
    log("cpu_baseline: 1 thread %.4f GB/s (%d reps, %.1f s); %d threads %.4f GB/s (%d reps, %.1f s); gcc -O2 -ffp-contract=off, "
        "stands in for the reference's Crystal QuantMatmul" % (cpu_gbps, cpu_reps, cpu_s, mt_cores, mt_gbps, mt_reps, mt_s))

    # ---- timed region ------------------------------------------------------------------------------------
    ms, graphed = time_steps(hip, stream, head.launch, args.steps, args.warmup)
    ms_per_step = ms / args.steps
    gbps = head.bytes_per_step / (ms_per_step * 1e-3) / 1e9

    # cache-resident figure (one copy only), reported beside the HBM one
    hot_ms, _ = time_steps(hip, stream, lambda i, s: head.launch(0, s), args.steps, args.warmup)
    hot_gbps = head.bytes_per_step / (hot_ms / args.steps * 1e-3) / 1e9

    log("case=q4_k_gemv ffn_up\ntype=Q4_K\nshape=%dx%d\ntokens=1\nraw_bytes=%d\ncopies=%d\nreps=%d\nwarmup=%d\n"
        "hip_ms=%.5f\ncpu_ms=%.3f\ncos=%.8f\nmax_diff=%g\nok=%s\ngbps_hbm=%.1f\ngbps_cache_hot=%.1f\ngraph=%s" % (
            head.in_dim, head.out_dim, head.w_bytes, head.copies, args.steps, args.warmup, ms_per_step,
            cpu_s / cpu_reps * 1e3, cos, max_diff, str(ok).lower(), gbps, hot_gbps, graphed))

    gemm = {}
    for tokens in ((64, 512, 2048) if args.mode == "cases" else (512,)):
        gsteps = max(10, min(200, args.steps // 10))
        per, tf = bench_gemm(hip, quant, synth, rng, stream, tokens, 12288, 4096, gsteps, 5)
        gemm["M=%d" % tokens] = {"ms": round(per, 5), "tflops": round(tf, 1), "frac_mfma_f16": round(tf / MFMA_F16_PEAK_TFLOPS, 4)}
        log("case=q4_k_gemm prefill\ntype=Q4_K\nshape=4096x12288\ntokens=%d\nreps=%d\nhip_ms=%.5f\ntflops=%.1f\nfrac_mfma_f16_peak=%.4f\n" % (
            tokens, gsteps, per, tf, tf / MFMA_F16_PEAK_TFLOPS))

    if args.mode == "cases":
        gsteps = max(10, min(200, args.steps // 10))
        per, tf = bench_gemm(hip, quant, synth, rng, stream, 512, 4096, 12288, gsteps, 5, Q4_K=Q6_K)
        gemm["q6_k down 4096x12288 M=512"] = {"ms": round(per, 5), "tflops": round(tf, 1), "frac_mfma_f16": round(tf / MFMA_F16_PEAK_TFLOPS, 4)}
        log("case=q6_k_gemm prefill\ntype=Q6_K\nshape=12288x4096\ntokens=512\nreps=%d\nhip_ms=%.5f\ntflops=%.1f\nfrac_mfma_f16_peak=%.4f\n" % (
            gsteps, per, tf, tf / MFMA_F16_PEAK_TFLOPS))
        per, tf = bench_gemm(hip, quant, synth, rng, stream, 512, 12288, 4096, gsteps, 5, Q4_K=Q5_K)
        gemm["q5_k 12288x4096 M=512"] = {"ms": round(per, 5), "tflops": round(tf, 1), "frac_mfma_f16": round(tf / MFMA_F16_PEAK_TFLOPS, 4)}
        log("case=q5_k_gemm prefill\ntype=Q5_K\nshape=4096x12288\ntokens=512\nreps=%d\nhip_ms=%.5f\ntflops=%.1f\nfrac_mfma_f16_peak=%.4f\n" % (
            gsteps, per, tf, tf / MFMA_F16_PEAK_TFLOPS))

    extra = {}
    if args.mode == "cases":
        table = [
            ("q8_0 ffn_up 0.8B", Q8_0, 3584, 1024, 1), ("q4_k ffn_down", Q4_K, 4096, 12288, 1),
            ("q6_k ffn_down", Q6_K, 4096, 12288, 1), ("q5_k attn_qkv-like", Q5_K, 4096, 4096, 1),
            ("q6_k output head", Q6_K, 151936, 4096, 1),
            ("q4_k ffn_up M=4", Q4_K, 12288, 4096, 4), ("q4_k ffn_up M=8", Q4_K, 12288, 4096, 8),
        ]
        for name, t, out_dim, in_dim, tokens in table:
            c = GemvCase(hip, quant, synth, rng, t, out_dim, in_dim, tokens)
            steps = max(20, min(args.steps, int(2e9 // c.bytes_per_step)))
            cms, _ = time_steps(hip, stream, c.launch, steps, min(args.warmup, steps))
            cg = c.bytes_per_step / (cms / steps * 1e-3) / 1e9
            extra[name] = {"gbps": round(cg, 1), "ms": round(cms / steps, 5), "frac_hbm": round(cg / HBM_PEAK_GBPS, 4)}
            log("case=%s\ntype=%s\nshape=%dx%d\ntokens=%d\nraw_bytes=%d\ncopies=%d\nreps=%d\nhip_ms=%.5f\ngbps_hbm=%.1f\n" % (
                name, TYPE_NAME[t], in_dim, out_dim, tokens, c.w_bytes, c.copies, steps, cms / steps, cg))
            c.close()

    if args.mode == "cases":
        # output head without the logits: RMSNorm -> Q6_K vocabulary projection with arg-max -> top-1 reduce (510 MB)
        from cogni_ml_amd.output_head import QwenOutputHeadRunner, Weights as HeadWeights
        hw = HeadWeights(np.ones(4096, dtype=np.float32), synth.make_weights(rng, Q6_K, 151936, 4096), Q6_K, 4096, 151936)
        for tokens in (1, 3):
            ohead = QwenOutputHeadRunner.from_weights(hw, tokens, synth.make_activations(rng, tokens, 4096).reshape(-1), 1e-6)
            ohead.upload_weights()
            ohead.reset_sequence()

            def hseq(i, st, ohead=ohead):
                with hip.with_stream(st):
                    ohead.run_sequence()
            reps = 20
            hms, _ = time_steps(hip, stream, hseq, reps, 3)
            hg = ohead.bytes_per_sequence() / (hms / reps * 1e-3) / 1e9
            extra["q6_k output head top-1 M=%d" % tokens] = {"gbps": round(hg, 1), "ms": round(hms / reps, 5), "frac_hbm": round(hg / HBM_PEAK_GBPS, 4)}
            log("case=output head top-1 (rmsnorm -> q6_k gemv top1 partial -> reduce)\ntokens=%d\nraw_bytes=%d\nreps=%d\nhip_ms=%.5f\ngbps_hbm=%.1f\n" % (
                tokens, hw.output_raw.size, reps, hms / reps, hg))
            ohead.close()

    if args.mode == "cases":
        # the gate | up pair of one layer against the same x in one launch (q4_k_dual_gemv_f32)
        a = GemvCase(hip, quant, synth, rng, Q4_K, 12288, 4096, 1, min_total_bytes=LLC_BYTES)
        b = GemvCase(hip, quant, synth, rng, Q4_K, 12288, 4096, 1, min_total_bytes=LLC_BYTES)
        out_b = hip.DeviceBuffer(4 * 12288)

        def dual(i, st):
            quant.gemv_dual_dev(a.w[i % a.copies].ptr, b.w[i % b.copies].ptr, Q4_K, a.x.ptr, a.out.ptr, out_b.ptr, 4096, 12288,
                                1, st.handle)
        dsteps = max(20, min(args.steps, 1000))
        dms, _ = time_steps(hip, stream, dual, dsteps, min(args.warmup, dsteps))
        dbytes = 2 * a.w_bytes + 4 * 4096 + 2 * 4 * 12288
        dg = dbytes / (dms / dsteps * 1e-3) / 1e9
        extra["q4_k gate|up pair, one launch"] = {"gbps": round(dg, 1), "ms": round(dms / dsteps, 5), "frac_hbm": round(dg / HBM_PEAK_GBPS, 4)}
        log("case=q4_k gate|up pair in one launch\ntype=Q4_K\nshape=2 x 4096x12288\ntokens=1\nraw_bytes=%d\nreps=%d\nhip_ms=%.5f\ngbps_hbm=%.1f\n" % (
            2 * a.w_bytes, dsteps, dms / dsteps, dg))
        a.close()
        b.close()
        out_b.close()

    if args.mode == "cases":
        # FFN sequence of one layer: gate | up | SwiGLU in one launch, then Q6_K down with the residual add
        from cogni_ml_amd.ffn_sequence import FFNSequenceRunner
        graw = [synth.make_weights(rng, Q4_K, 12288, 4096) for _ in range(2)] + [synth.make_weights(rng, Q6_K, 4096, 12288)]
        for tokens, block in ((1, False), (4, False), (1, True)):
            fx = rng.uniform(-1.0, 1.0, tokens * 4096).astype(np.float32)
            if block:   # the FFN half of a decoder layer: add + RMSNorm ahead of the projections
                ffn = FFNSequenceRunner(graw[0], graw[1], graw[2], 4096, 12288, tokens, fx, norm=np.ones(4096, dtype=np.float32), add=fx.copy())
            else:
                ffn = FFNSequenceRunner(graw[0], graw[1], graw[2], 4096, 12288, tokens, fx, fx.copy())
            ffn.upload_weights()
            ffn.reset_sequence()

            def fseq(i, st, ffn=ffn):
                with hip.with_stream(st):
                    ffn.run_sequence()
            reps = max(20, min(args.steps // 4, 300))
            fms, _ = time_steps(hip, stream, fseq, reps, 10)
            fg = ffn.bytes_per_sequence() / (fms / reps * 1e-3) / 1e9
            extra["%s M=%d" % ("add+rmsnorm+ffn" if block else "ffn sequence", tokens)] = {"gbps": round(fg, 1), "ms": round(fms / reps, 5), "frac_hbm": round(fg / HBM_PEAK_GBPS, 4)}
            log("case=ffn sequence (gate|up Q4_K -> SwiGLU -> down Q6_K + residual)\ntokens=%d\nraw_bytes=%d\nreps=%d\nhip_ms=%.5f\n"
                "gbps=%.1f\nnote=weights %.0f MB stay in the 256 MB last-level cache between repetitions\n" % (
                    tokens, sum(r.size for r in graw), reps, fms / reps, fg, sum(r.size for r in graw) / 1e6))
            ffn.close()

    if args.mode == "cases":
        # config 5: the mixed-quant projection stack, resident, back to back in one stream
        from cogni_ml_amd.projection_stack import QwenProjectionStackRunner, Weights
        wts = Weights.synthetic(rng)
        for tokens in (1, 4, 8):
            runner = QwenProjectionStackRunner.from_weights(wts, tokens, synth.make_activations(rng, tokens, wts.hidden))
            runner.upload_weights()
            runner.reset_sequence()

            def seq(i, st, runner=runner):
                with hip.with_stream(st):
                    runner.run_sequence()
            reps = max(20, min(args.steps // 4, 300))
            sms, _ = time_steps(hip, stream, seq, reps, 10)
            sg = runner.bytes_per_sequence() / (sms / reps * 1e-3) / 1e9
            extra["projection stack M=%d" % tokens] = {"gbps": round(sg, 1), "ms": round(sms / reps, 5),
                                                        "frac_hbm": round(sg / HBM_PEAK_GBPS, 4)}
            log("case=projection stack (q,k,v,o,gate,up Q4_K + down Q6_K)\ntokens=%d\nraw_bytes=%d\nreps=%d\nhip_ms=%.5f\n"
                "gbps=%.1f\nnote=weights %.0f MB stay in the 256 MB last-level cache between repetitions\n" % (
                    tokens, wts.raw_bytes, reps, sms / reps, sg, wts.raw_bytes / 1e6))
            runner.close()

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
            "weight_copies_rotated": head.copies, "timed_region": "hip graph of K launches" if graphed else "K direct launches",
        },
        "pct_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "cache_hot_gbps": round(hot_gbps, 1),
        "prefill_gemm_q4k_12288x4096": gemm,
        "parity": {"cos": round(cos, 8), "max_diff": max_diff, "ok": ok, "tol_1e-4_x_wmax": 1e-4 * float(np.linalg.norm(head.host_x)) * dense_max},
        "roofline": {
            "bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(gbps / HBM_PEAK_GBPS, 4), "traffic": MEASURED_TRAFFIC_BYTES,
        },
        "cpu_baseline": {
            "value": round(cpu_gbps, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "%d x the same 12288x4096 Q4_K GEMV (M=1) through the C restatement of QuantMatmul.matmul_add, "
                      "1 thread, %.1f s" % (cpu_reps, cpu_s),
        },
        "cpu_baseline_all_cores": {"value": round(mt_gbps, 4), "unit": "GB/s", "cores": mt_cores, "kind": "port",
                                   "sample": "%d x the same GEMV, rows divided among %d threads, %.1f s" % (mt_reps, mt_cores, mt_s)},
    }
    if extra:
        result["cases"] = extra
    head.close()
    stream.close()
    ctx.close()
    print(json.dumps(result), flush=True)
    if not ok:
        sys.exit(1)


if __name__ == "__main__":
    main()
