"""Seeded sweep over random valid shapes: every decode entry point and the prefill GEMM against the CPU oracle.

The shapes are drawn, not chosen: odd out_dim (partial row groups), in_dim of any whole number of blocks (partial column
sets), every token count and weight type. Same tolerances as the per-kernel tests.
"""
import numpy as np
import pytest

from cogni_ml_amd import quant, synth
from gpu_common import DevArray, gpu  # noqa: F401
from helpers import BLOCK, Q4_K, Q5_K, Q6_K, Q8_0
from test_gpu_gemm import check as check_gemm
from test_gpu_gemv import check as check_gemv
from test_gpu_output_head import run_top1

pytestmark = pytest.mark.gpu


def draw_shape(rng, type_id, max_out, max_blocks):
    be = BLOCK[type_id][1]
    out_dim = int(rng.integers(1, max_out + 1))
    in_dim = be * int(rng.integers(1, max_blocks * (256 // be) + 1))
    return out_dim, in_dim


@pytest.mark.parametrize("seed", range(6))
def test_random_gemv_shapes(gpu, oracle, seed):
    rng = np.random.default_rng(7000 + seed)
    for case in range(10):
        type_id = [Q8_0, Q4_K, Q5_K, Q6_K][int(rng.integers(0, 4))]
        tokens = int(rng.integers(1, 9))
        out_dim, in_dim = draw_shape(rng, type_id, 600, 20)
        raw = synth.make_weights(rng, type_id, out_dim, in_dim)
        x = synth.make_activations(rng, tokens, in_dim)
        res = rng.standard_normal(tokens * out_dim).astype(np.float32) if rng.integers(0, 2) else None
        what = "seed %d case %d: type %d M=%d out=%d in=%d add=%s" % (seed, case, type_id, tokens, out_dim, in_dim, res is not None)
        print(what, flush=True)
        check_gemv(oracle, raw, type_id, x, in_dim, out_dim, tokens, res, what)


@pytest.mark.parametrize("seed", range(3))
def test_random_top1_shapes(gpu, oracle, seed):
    rng = np.random.default_rng(8000 + seed)
    for case in range(6):
        type_id = [Q8_0, Q4_K, Q5_K, Q6_K][int(rng.integers(0, 4))]
        tokens = int(rng.integers(1, 8))
        out_dim, in_dim = draw_shape(rng, type_id, 3000, 8)
        raw = synth.make_weights(rng, type_id, out_dim, in_dim)
        x = synth.make_activations(rng, tokens, in_dim)
        print("seed %d case %d: type %d M=%d out=%d in=%d" % (seed, case, type_id, tokens, out_dim, in_dim), flush=True)
        ids, vals, logits = run_top1(raw, type_id, x, in_dim, out_dim, tokens)
        want = oracle.matmul_add(x, tokens, in_dim, raw, type_id, out_dim, np.zeros(out_dim, dtype=np.float32),
                                 threads=8).reshape(tokens, out_dim)
        for tok in range(tokens):
            # the winner is the first maximum of the device's own logits, up to the different summation order of the
            # kernels that produce the two; against the oracle it is within the GEMV tolerance of the best row
            assert ids[tok] == int(np.argmax(logits[tok])) or np.isclose(vals[tok], logits[tok].max(), rtol=2e-5, atol=0)
            top, scale = float(want[tok].max()), float(np.abs(want[tok]).max())
            assert abs(float(vals[tok]) - top) <= 1e-4 * scale
            assert want[tok][ids[tok]] >= top - 1e-4 * scale


@pytest.mark.parametrize("seed", range(4))
def test_random_gemm_shapes(gpu, oracle, seed):
    rng = np.random.default_rng(9000 + seed)
    for case in range(5):
        t = [Q4_K, Q5_K, Q6_K][int(rng.integers(0, 3))]
        tokens = int(rng.integers(9, 400))
        out_dim, in_dim = draw_shape(rng, t, 700, 12)
        raw = synth.make_weights(rng, t, out_dim, in_dim)
        x = synth.make_activations(rng, tokens, in_dim)
        bias = rng.standard_normal(out_dim).astype(np.float32) if rng.integers(0, 2) else None
        what = "seed %d case %d: type %d M=%d out=%d in=%d bias=%s" % (seed, case, t, tokens, out_dim, in_dim, bias is not None)
        print(what, flush=True)
        check_gemm(oracle, raw, x, in_dim, out_dim, tokens, bias, what, t=t)


@pytest.mark.parametrize("seed", range(4))
def test_random_one_pass_shapes(gpu, oracle, seed):
    """Shapes the one-pass kernels take (in_dim a multiple of 256 up to 12288, half of the draws a multiple of 2048; Q4_K,
    Q5_K, Q6_K, Q8_0), drawn: 2..17 tokens (a
    group of eight and what is left), single matrices with and without residual, lists of two to five matrices with row
    counts that are and are not multiples of 16, top-1, activations scaled far out of the binary16 range."""
    from test_gpu_gemv_one_pass import assert_bars, oracle_rows
    rng = np.random.default_rng(9100 + seed)
    for case in range(12):
        t = [Q4_K, Q5_K, Q6_K, Q8_0][int(rng.integers(0, 4))]
        in_dim = 2048 * int(rng.integers(1, 7)) if rng.integers(0, 2) else 256 * int(rng.integers(1, 49))
        tokens = int(rng.integers(2, 18))
        kind = ["single", "residual", "list", "top1"][int(rng.integers(0, 4))]
        if kind == "top1" and t in (Q5_K, Q8_0):
            kind = "single"
        count = int(rng.integers(2, 6)) if kind == "list" else 1
        dims = [int(rng.integers(1, 1500)) if rng.integers(0, 3) else 16 * int(rng.integers(1, 90)) for _ in range(count)]
        what = "seed %d case %d: type %d in=%d M=%d %s dims=%s" % (seed, case, t, in_dim, tokens, kind, dims)
        print(what, flush=True)
        raws = [synth.make_weights(rng, t, d, in_dim) for d in dims]
        x = synth.make_activations(rng, tokens, in_dim)
        if rng.integers(0, 4) == 0 and kind != "residual":
            x *= np.float32(10.0 ** float(rng.integers(-20, 20)))
        if kind == "residual":
            res = rng.standard_normal(tokens * dims[0]).astype(np.float32)
            check_gemv(oracle, raws[0], t, x, in_dim, dims[0], tokens, res, what)
            continue
        if kind == "top1":
            ids, vals, logits = run_top1(raws[0], t, x, in_dim, dims[0], tokens)
            for tok in range(tokens):
                assert ids[tok] == int(np.argmax(logits[tok])) or np.isclose(vals[tok], logits[tok].max(), rtol=3e-5, atol=0), what
            continue
        ws, xd = [DevArray(r) for r in raws], DevArray(x)
        outs = [DevArray(nbytes=4 * tokens * d) for d in dims]
        if kind == "list":
            quant.gemv_many_dev([w.ptr for w in ws], t, xd.ptr, [o.ptr for o in outs], dims, in_dim, tokens)
        else:
            quant.gemv_dev(ws[0].ptr, t, xd.ptr, outs[0].ptr, in_dim, dims[0], tokens)
        for raw, o, d in zip(raws, outs, dims):
            want, tol = oracle_rows(oracle, raw, x, in_dim, d, tokens, t)
            assert_bars(o.read(np.float32, tokens * d), want, tol, tokens, d, what + " member %d" % d)
        for a in ws + outs + [xd]:
            a.close()


@pytest.mark.parametrize("seed", range(4))
def test_random_prefill_ffn_blocks(gpu, oracle, seed):
    """The feed-forward block of a prefill layer at drawn sizes (hidden and FFN width multiples of 256, 9..300 tokens, the down
    matrix of any GEMM type), once with its producers packing - the norm writes the packed input of gate | up, the SwiGLU GEMM
    that of the down GEMM - and once as five launches with the two pack launches: the same bits. Two tokens of it against the
    CPU form."""
    rng = np.random.default_rng(9500 + seed)
    for case in range(4):
        hidden, ffn = 256 * int(rng.integers(1, 9)), 256 * int(rng.integers(1, 13))
        tokens = int(rng.integers(9, 301))
        dt = [Q4_K, Q5_K, Q6_K][int(rng.integers(0, 3))]
        what = "seed %d case %d: hidden=%d ffn=%d M=%d down type %d" % (seed, case, hidden, ffn, tokens, dt)
        print(what, flush=True)
        gate_raw, up_raw = synth.make_weights(rng, Q4_K, ffn, hidden), synth.make_weights(rng, Q4_K, ffn, hidden)
        down_raw = synth.make_weights(rng, dt, hidden, ffn)
        x = rng.uniform(-0.1, 0.1, tokens * hidden).astype(np.float32)
        add = rng.uniform(-1.0, 1.0, tokens * hidden).astype(np.float32)
        norm = (0.1 + 0.01 * rng.standard_normal(hidden)).astype(np.float32)
        wsx, wsa = quant.gemm_workspace_bytes(Q4_K, hidden, tokens), quant.gemm_workspace_bytes(dt, ffn, tokens, hidden)
        wg, wu, wd, xd, ad, nd = (DevArray(a) for a in (gate_raw, up_raw, down_raw, x, add, norm))
        outs = []
        for fused in (False, True):
            res, normed, out = (DevArray(nbytes=x.nbytes) for _ in range(3))
            act, ws_x, ws_a = DevArray(nbytes=4 * tokens * ffn), DevArray(nbytes=wsx), DevArray(nbytes=wsa)
            if fused:
                quant.add_rmsnorm_gemm_pack_dev(xd.ptr, ad.ptr, nd.ptr, res.ptr, 0, Q4_K, ws_x.ptr, wsx, hidden, tokens, 1e-6)
                quant.gemm_packed_swiglu_pack_dev(wg.ptr, wu.ptr, Q4_K, ws_x.ptr, wsx, 0, dt, ws_a.ptr, wsa, hidden, ffn, tokens)
            else:
                quant.add_rmsnorm_dev(xd.ptr, ad.ptr, nd.ptr, res.ptr, normed.ptr, hidden, tokens, 1e-6)
                quant.gemm_pack_dev(normed.ptr, Q4_K, hidden, tokens, ws_x.ptr, wsx)
                quant.gemm_packed_swiglu_dev(wg.ptr, wu.ptr, Q4_K, ws_x.ptr, wsx, act.ptr, hidden, ffn, tokens)
                quant.gemm_pack_dev(act.ptr, dt, ffn, tokens, ws_a.ptr, wsa)
            quant.gemm_packed_add_dev(wd.ptr, dt, ws_a.ptr, wsa, res.ptr, out.ptr, ffn, hidden, tokens)
            outs.append(out.read(np.float32, tokens * hidden))
            for a in (res, normed, out, act, ws_x, ws_a):
                a.close()
        assert np.array_equal(outs[0], outs[1]), what
        zero_f = np.zeros(ffn, dtype=np.float32)
        for tok in (0, tokens - 1):
            r = x[tok * hidden:(tok + 1) * hidden] + add[tok * hidden:(tok + 1) * hidden]
            h = oracle.rms_norm(r, norm, 1e-6)
            g = oracle.matmul_add(h, 1, hidden, gate_raw, Q4_K, ffn, zero_f, threads=8)
            u = oracle.matmul_add(h, 1, hidden, up_raw, Q4_K, ffn, zero_f, threads=8)
            want = oracle.matmul_add(oracle.swiglu(g, u), 1, ffn, down_raw, dt, hidden, r, threads=8)
            got = outs[1][tok * hidden:(tok + 1) * hidden]
            assert np.max(np.abs(got - want)) <= 4e-3 * np.max(np.abs(want)), what + " token %d" % tok
        for a in (wg, wu, wd, xd, ad, nd):
            a.close()


@pytest.mark.parametrize("seed", range(4))
def test_random_gemm_lists(gpu, seed):
    """cogni_gemm_packed_many_dev at drawn sizes: one to six Q4_K or Q5_K matrices of 1..1500 rows, rows of 256..3072 values,
    9..300 tokens; every output bit for bit the single launch's (no k split: the workspace holds the packed activations only)."""
    rng = np.random.default_rng(9700 + seed)
    for case in range(5):
        t = [Q4_K, Q5_K][int(rng.integers(0, 2))]
        count, in_dim, tokens = int(rng.integers(1, 7)), 256 * int(rng.integers(1, 13)), int(rng.integers(9, 301))
        dims = [int(rng.integers(1, 1501)) if rng.integers(0, 2) else 64 * int(rng.integers(1, 24)) for _ in range(count)]
        what = "seed %d case %d: type %d in=%d M=%d dims=%s" % (seed, case, t, in_dim, tokens, dims)
        print(what, flush=True)
        raws = [synth.make_weights(rng, t, d, in_dim) for d in dims]
        x = synth.make_activations(rng, tokens, in_dim)
        wsb = quant.gemm_workspace_bytes(t, in_dim, tokens)
        ws, xd, wd = DevArray(nbytes=wsb), DevArray(x), [DevArray(r) for r in raws]
        singles = [DevArray(nbytes=4 * tokens * d) for d in dims]
        lists = [DevArray(np.full(tokens * d, np.float32(7.0))) for d in dims]
        quant.gemm_pack_dev(xd.ptr, t, in_dim, tokens, ws.ptr, wsb)
        for w, o, d in zip(wd, singles, dims):
            quant.gemm_packed_dev(w.ptr, t, ws.ptr, wsb, o.ptr, in_dim, d, tokens)
        quant.gemm_packed_many_dev([w.ptr for w in wd], t, ws.ptr, wsb, [o.ptr for o in lists], dims, in_dim, tokens)
        for o1, o2, d in zip(singles, lists, dims):
            assert np.array_equal(o2.read(np.float32, tokens * d), o1.read(np.float32, tokens * d)), what + " member %d" % d
        for a in [ws, xd] + wd + singles + lists:
            a.close()


@pytest.mark.parametrize("seed", range(4))
def test_random_sixteen_token_shapes(gpu, oracle, seed):
    """The one-pass kernels with sixteen single-term tokens at drawn sizes: any of the four block types, rows of 256..12288
    values, 1..16 tokens, one to four matrices of 1..1500 rows, with a residual on single matrices; against the CPU form of
    the activations rounded to binary16, to the one-pass bars."""
    from test_gpu_gemv_one_pass import assert_bars, oracle_rows
    rng = np.random.default_rng(9900 + seed)
    for case in range(8):
        t = [Q4_K, Q5_K, Q6_K, Q8_0][int(rng.integers(0, 4))]
        in_dim = 2048 * int(rng.integers(1, 7)) if rng.integers(0, 2) else 256 * int(rng.integers(1, 49))
        tokens = int(rng.integers(1, 17))
        count = int(rng.integers(1, 5))
        dims = [int(rng.integers(1, 1500)) if rng.integers(0, 3) else 16 * int(rng.integers(1, 90)) for _ in range(count)]
        what = "seed %d case %d: type %d in=%d M=%d dims=%s" % (seed, case, t, in_dim, tokens, dims)
        print(what, flush=True)
        raws = [synth.make_weights(rng, t, d, in_dim) for d in dims]
        x = synth.make_activations(rng, tokens, in_dim)
        x16 = x.astype(np.float16).astype(np.float32)
        res = rng.standard_normal(tokens * dims[0]).astype(np.float32) if count == 1 and rng.integers(0, 2) else None
        image = DevArray(np.full(quant.gemv_image_bytes(t, in_dim, 8), 0xFF, dtype=np.uint8))
        xd, wd = DevArray(x), [DevArray(r) for r in raws]
        rd = DevArray(res) if res is not None else None
        outs = [DevArray(np.full(tokens * d, np.float32(-9.0))) for d in dims]
        quant.gemv_pack16_dev(xd.ptr, t, in_dim, tokens, image.ptr)
        quant.gemv_packed16_dev([w.ptr for w in wd], t, image.ptr, [o.ptr for o in outs], dims, in_dim, tokens, rd.ptr if rd else 0)
        for raw, o, d in zip(raws, outs, dims):
            want, tol = oracle_rows(oracle, raw, x16, in_dim, d, tokens, t)
            got = o.read(np.float32, tokens * d)
            if res is not None:
                got = got - res   # (the residual is added last, in fp32: taking it off again costs one rounding of the sum)
                tol = tol + 1e-6 * (np.abs(res) + np.abs(want))
                err = np.abs(got.astype(np.float64) - want)
                assert np.all(err <= tol + 2e-5 * np.max(np.abs(want))), what
            else:
                assert_bars(got, want, tol, tokens, d, what + " member %d" % d)
        for a in [image, xd] + wd + outs + ([rd] if rd else []):
            a.close()
