#!/usr/bin/env python3
"""GEMV probe harness: the HIP counterpart of the reference's per-type CUDA probes
(bin/cuda_q4k_gemv_probe.cr:118-289 and the type-generic bin/gemma4_cuda_primitive_probe.cr:49-211).

Same sequence (weights -> CPU reference per token -> upload -> warm-up -> timed reps -> read back ->
cos / max_diff / ok), same printed keys per case, a summary line and the process exit code. Weights are
seeded synthetic blocks instead of a GGUF tensor; the CPU reference is the oracle.

  python tests/probe_quant_gemv.py [--seed N] [--reps N] [--warmup N] [--tokens N] [--include-head]
"""
import argparse
import ctypes
import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "cogni-ml_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

import numpy as np  # noqa: E402

CASES = [
    ("blk.0.ffn_up.weight (0.8B)", 8, 1024, 3584), ("blk.0.ffn_gate.weight", 12, 4096, 12288),
    ("blk.0.ffn_down.weight", 12, 12288, 4096), ("blk.0.ffn_down.weight (Q6_K)", 14, 12288, 4096),
    ("blk.0.attn_qkv.weight", 13, 4096, 4096), ("blk.0.attn_k.weight", 12, 4096, 1024),
]
HEAD = ("output.weight", 14, 4096, 151936)
TYPE_NAME = {8: "Q8_0", 12: "Q4_K", 13: "Q5_K", 14: "Q6_K"}


def run_case(hip, quant, synth, oracle, mod, name, t, in_dim, out_dim, tokens, reps, warmup, seed):
    rng = np.random.default_rng(seed)
    w_raw = synth.make_weights(rng, t, out_dim, in_dim)
    x = rng.uniform(-1.0, 1.0, tokens * in_dim).astype(np.float32)      # U(-1,1), as the reference's probes
    zero_bias = np.zeros(out_dim, dtype=np.float32)
    t0 = time.perf_counter()
    cpu = np.concatenate([oracle.matmul_add(x[k * in_dim:(k + 1) * in_dim], 1, in_dim, w_raw, t, out_dim, zero_bias)
                          for k in range(tokens)])
    cpu_ms = (time.perf_counter() - t0) * 1e3
    w_buf, x_buf, out_buf = hip.DeviceBuffer(w_raw.size), hip.DeviceBuffer(x.nbytes), hip.DeviceBuffer(4 * tokens * out_dim)
    try:
        hip.copy_htod(w_buf.ptr, w_raw, w_raw.size, "%s weights" % name)
        hip.copy_htod(x_buf.ptr, x, x.nbytes, "%s input" % name)
        groups = [(k, min(8, tokens - k)) for k in range(0, tokens, 8)]

        def launch_all():
            for k, m in groups:
                fn = mod.function(quant.gemv_kernel_name(t, m))
                grid, block, lds = quant.gemv_launch_dims(t, m, in_dim, out_dim)
                params = hip.KernelParams(ctypes.c_uint64(w_buf.ptr), ctypes.c_uint64(x_buf.ptr + 4 * k * in_dim),
                                          ctypes.c_uint64(out_buf.ptr + 4 * k * out_dim), ctypes.c_uint32(in_dim),
                                          ctypes.c_uint32(out_dim))
                hip.launch(fn, grid, 1, 1, block, 1, 1, params, fn.name, lds)
        for _ in range(warmup):
            launch_all()
        if warmup:
            hip.synchronize("warmup %s" % name)
        t0 = time.perf_counter()
        for _ in range(reps):
            launch_all()
        hip.synchronize("timed %s" % name)
        hip_ms = (time.perf_counter() - t0) * 1e3 / reps
        gpu = np.empty(tokens * out_dim, dtype=np.float32)
        hip.copy_dtoh(gpu, out_buf.ptr, gpu.nbytes, "%s output" % name)
        max_diff = float(np.max(np.abs(gpu - cpu)))
        a, b = gpu.astype(np.float64), cpu.astype(np.float64)
        cos = float(a @ b / np.sqrt((a @ a) * (b @ b)))
        ok = cos >= 0.99999 and max_diff <= 1e-3
        print("case=%s\ntype=%s\nshape=%dx%d\ntokens=%d\nraw_bytes=%d\nreps=%d\nwarmup=%d\nhip_ms=%.3f\ncpu_ms=%.3f\n"
              "cos=%.8f\nmax_diff=%s\nok=%s\n" % (name, TYPE_NAME[t], in_dim, out_dim, tokens, w_raw.size, reps, warmup,
                                                   hip_ms, cpu_ms, cos, max_diff, str(ok).lower()), flush=True)
        return ok
    finally:
        for b in (out_buf, x_buf, w_buf):
            b.close()


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--seed", type=int, default=23)
    ap.add_argument("--reps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--tokens", type=int, default=1)
    ap.add_argument("--include-head", action="store_true", help="also run the 4096 -> 151936 Q6_K head (510 MB)")
    args = ap.parse_args(argv)
    if args.reps <= 0:
        raise SystemExit("reps must be positive")
    if args.warmup < 0:
        raise SystemExit("warmup must be non-negative")
    if args.tokens <= 0:
        raise SystemExit("tokens must be positive")
    from cogni_ml_amd import hip, quant, synth
    from oracle import oracle
    ctx = hip.Context.create()
    mod = hip.HIPModule.load_builtin()
    try:
        print("device=%s\ncompute_capability=%d.%d\narch=%s\ncpu_impl=c_restatement_of_quant_matmul.cr\n" % (
            ctx.device_name, ctx.compute_capability_major, ctx.compute_capability_minor, ctx.arch), flush=True)
        cases = list(CASES)
        if args.include_head:
            cases.append(HEAD)
        ok_all = True
        for i, (name, t, in_dim, out_dim) in enumerate(cases):
            reps, warmup = (min(args.reps, 5), min(args.warmup, 1)) if name == HEAD[0] else (args.reps, args.warmup)
            ok_all &= run_case(hip, quant, synth, oracle, mod, name, t, in_dim, out_dim, args.tokens, reps, warmup, args.seed + i)
        print("summary_ok=%s" % str(ok_all).lower(), flush=True)
        return 0 if ok_all else 1
    finally:
        mod.close()
        ctx.close()


if __name__ == "__main__":
    sys.exit(main())
