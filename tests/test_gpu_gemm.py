"""GPU prefill GEMM (Q4_K, Q5_K and Q6_K, fp16 MFMA path) vs the CPU oracle.

Tolerance (fp16-MFMA path): max|err| <= 2e-3 * max|ref| over the output, plus cos >= 0.9999 -- the
reference's own convention for its Metal GEMM (spec/qwen35_metal_spec.cr:78,104 uses 0.05 * max|cpu|).
The figure normalised the fp32 way, max|err| / (||x||_2 * max|w_row|), is printed beside it.
"""
import numpy as np
import pytest

from cogni_ml_amd import quant, synth
from gpu_common import DevArray, gpu  # noqa: F401
from helpers import Q4_K, Q5_K, Q6_K, Q8_0, cosine

pytestmark = pytest.mark.gpu


def run_gemm(raw, x, in_dim, out_dim, tokens, bias=None, router=False, t=Q4_K, split=True):
    w, xd, od = DevArray(raw), DevArray(x), DevArray(nbytes=4 * tokens * out_dim)
    wsb = quant.gemm_workspace_bytes(t, in_dim, tokens, out_dim if split else None)
    ws = DevArray(nbytes=wsb)
    bd = DevArray(bias) if bias is not None else None
    fn = quant.matmul_dev if router else quant.gemm_dev
    fn(w.ptr, t, xd.ptr, od.ptr, in_dim, out_dim, tokens, ws.ptr, wsb, bd.ptr if bd else 0)
    out = od.read(np.float32, tokens * out_dim)
    for a in (w, xd, od, ws, bd):
        if a:
            a.close()
    return out


def check(oracle, raw, x, in_dim, out_dim, tokens, bias=None, what="", router=False, sample_tokens=None, t=Q4_K):
    got = run_gemm(raw, x, in_dim, out_dim, tokens, bias, router, t).reshape(tokens, out_dim)
    b = bias if bias is not None else np.zeros(out_dim, dtype=np.float32)
    rows = np.arange(tokens) if sample_tokens is None else np.asarray(sample_tokens)
    xs = x.reshape(tokens, in_dim)[rows]
    want = oracle.matmul_add(xs.reshape(-1), len(rows), in_dim, raw, t, out_dim, b, threads=16).reshape(len(rows), out_dim)
    err = np.max(np.abs(got[rows].astype(np.float64) - want))
    ref_max = np.max(np.abs(want))
    dense_max = np.max(np.abs(oracle.dequantize(raw, t, out_dim * in_dim)))
    fp32_style = err / (np.max(np.linalg.norm(xs, axis=1)) * dense_max)
    print("%s: max|err|/max|ref| = %.3e, max|err|/(||x|| max|w|) = %.3e" % (what, err / ref_max, fp32_style))
    assert cosine(got[rows].reshape(-1), want.reshape(-1)) >= 0.9999, what
    assert err <= 2e-3 * ref_max, "%s: err %.3e > 2e-3 * %.3e" % (what, err, ref_max)
    return got


@pytest.mark.parametrize("t", [Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("tokens,out_dim,in_dim", [(9, 192, 256), (16, 48, 512), (64, 200, 1024), (128, 192, 256),
                                                     (130, 400, 768), (257, 31, 256)])
def test_small_shapes_and_tails(gpu, oracle, tokens, out_dim, in_dim, t):
    rng = np.random.default_rng(tokens * 1000 + out_dim)
    raw = synth.make_weights(rng, t, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    check(oracle, raw, x, in_dim, out_dim, tokens, None, "type %d M=%d N=%d K=%d" % (t, tokens, out_dim, in_dim), t=t)


def test_q6_k_codes_and_scales_one_at_a_time(gpu, oracle):
    """Q6_K blocks with a single non-zero scale and codes that count up: every (quadrant, 16-run, byte) of the operand
    assembly lands on its own activation, so a swapped piece, a wrong shift or a wrong scale byte shows as a wrong value."""
    in_dim, out_dim, tokens = 256, 32, 16
    rng = np.random.default_rng(66)
    x = synth.make_activations(rng, tokens, in_dim)
    for which in range(16):
        raw = np.zeros((out_dim, 210), dtype=np.uint8)
        codes = (np.arange(256)[None, :] * 7 + np.arange(out_dim)[:, None] * 3) % 64          # 6-bit codes per element
        for nn in range(2):
            for l in range(32):
                e = 128 * nn + l
                raw[:, 64 * nn + l] = (codes[:, e] & 15) | ((codes[:, e + 64] & 15) << 4)
                raw[:, 64 * nn + 32 + l] = (codes[:, e + 32] & 15) | ((codes[:, e + 96] & 15) << 4)
                raw[:, 128 + 32 * nn + l] = ((codes[:, e] >> 4) | ((codes[:, e + 32] >> 4) << 2) |
                                             ((codes[:, e + 64] >> 4) << 4) | ((codes[:, e + 96] >> 4) << 6))
        raw[:, 192 + which] = np.uint8(5 + which)                                            # one live sub-block scale
        raw[:, 208:210] = np.frombuffer(np.float16(0.01).tobytes(), dtype=np.uint8)
        check(oracle, raw.reshape(-1), x, in_dim, out_dim, tokens, None, "Q6_K scale %d" % which, t=Q6_K)


@pytest.mark.parametrize("t", [Q4_K, Q5_K, Q6_K])
def test_bias_and_router(gpu, oracle, t):
    Q4_K = t        # (the body below is written for one type; it runs for both)
    rng = np.random.default_rng(4)
    out_dim, in_dim = 384, 512
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    bias = rng.standard_normal(out_dim).astype(np.float32)
    x = synth.make_activations(rng, 40, in_dim)
    check(oracle, raw, x, in_dim, out_dim, 40, bias, "bias M=40", router=True, t=t)
    # at or below the threshold the router takes the fp32 GEMV path: agreement with the oracle is ~1e-6
    assert quant.get_gemm_threshold() == 8
    got = run_gemm(raw, x[:8 * in_dim], in_dim, out_dim, 8, None, router=True, t=t)
    want = oracle.matmul_add(x[:8 * in_dim], 8, in_dim, raw, Q4_K, out_dim, np.zeros(out_dim, dtype=np.float32))
    assert np.max(np.abs(got - want)) <= 1e-5 * np.max(np.abs(want))
    # host-level matmul_add with rows > 8 goes through the GEMM as well
    mine = quant.matmul_add(x, 40, in_dim, raw, Q4_K, out_dim, bias)
    ref = oracle.matmul_add(x, 40, in_dim, raw, Q4_K, out_dim, bias)
    assert np.max(np.abs(mine - ref)) <= 2e-3 * np.max(np.abs(ref))
    quant.set_gemm_threshold(64)
    try:
        mine32 = quant.matmul_add(x, 40, in_dim, raw, Q4_K, out_dim, bias)
        assert np.max(np.abs(mine32 - ref)) <= 1e-5 * np.max(np.abs(ref))
    finally:
        quant.set_gemm_threshold(8)


@pytest.mark.parametrize("t", [Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("tokens,out_dim,in_dim", [(64, 384, 4096), (20, 100, 1280), (200, 4096, 2048), (128, 1000, 1536)])
def test_k_split_matches_unsplit(gpu, oracle, tokens, out_dim, in_dim, t):
    """Few tiles: the k range is divided among workgroups (the workspace has room for the planes). Against the oracle,
    against the unsplit launch, with a bias, and the same bits on a second run."""
    rng = np.random.default_rng(tokens + out_dim + in_dim + t)
    raw = synth.make_weights(rng, t, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    bias = rng.standard_normal(out_dim).astype(np.float32)
    assert quant.gemm_workspace_bytes(t, in_dim, tokens, out_dim) > quant.gemm_workspace_bytes(t, in_dim, tokens)
    got = check(oracle, raw, x, in_dim, out_dim, tokens, bias, "split M=%d N=%d K=%d" % (tokens, out_dim, in_dim), t=t)
    one = run_gemm(raw, x, in_dim, out_dim, tokens, bias, t=t, split=False).reshape(tokens, out_dim)
    assert np.max(np.abs(one - got)) <= 2e-5 * np.max(np.abs(got))
    assert np.array_equal(run_gemm(raw, x, in_dim, out_dim, tokens, bias, t=t).reshape(tokens, out_dim), got)


@pytest.mark.parametrize("tokens,out_dim,in_dim,with_bias", [(128, 65536, 256, False), (130, 65301, 768, True), (100, 65536, 512, False)])
def test_wide_tiles(gpu, oracle, tokens, out_dim, in_dim, with_bias):
    """Launches of whole rounds of 128 x 256 tiles go to the eight-wavefront kernel: a clipped last tile with an out_dim that
    is no multiple of 4, an odd number of super-blocks, a partial token tile and a bias, against the oracle on a sample of
    tokens; and every output against a four-wavefront kernel's, which adds in the same order (bit for bit)."""
    rng = np.random.default_rng(out_dim + tokens)
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    bias = rng.standard_normal(out_dim).astype(np.float32) if with_bias else None
    wsb = quant.gemm_workspace_bytes(Q4_K, in_dim, tokens, out_dim)
    kernel, grid_x, splits, block = quant.gemm_plan(Q4_K, in_dim, out_dim, tokens, wsb)
    assert (kernel, splits, block) == ("q4_k_gemm_wide_f16", 1, 512) and grid_x >= ((tokens + 127) // 128) * ((out_dim + 255) // 256)
    got = check(oracle, raw, x, in_dim, out_dim, tokens, bias, "wide M=%d N=%d K=%d" % (tokens, out_dim, in_dim),
                sample_tokens=[0, 1, 31, 32, 63, 64, 97, tokens - 1])
    # the same rows through the narrow kernel: 8192 rows at a time are fewer than a round of wide tiles
    for r0 in (0, 8192 * 3, out_dim - 8192):
        rows = slice(r0, r0 + 8192)
        assert quant.gemm_plan(Q4_K, in_dim, 8192, tokens, 0)[0] in ("q4_k_gemm_f16", "q4_k_gemm_n128_f16")
        part = run_gemm(raw[r0 * (in_dim // 256) * 144:(r0 + 8192) * (in_dim // 256) * 144], x, in_dim, 8192, tokens,
                        None if bias is None else bias[rows], split=False).reshape(tokens, 8192)
        assert np.array_equal(part, got[:, rows]), r0


@pytest.mark.parametrize("t", [Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("tokens,out_dim,in_dim", [(512, 4096, 2048), (130, 4096 + 37, 768), (64, 250, 4096), (300, 1024, 256)])
def test_tile_heights_agree(gpu, oracle, t, tokens, out_dim, in_dim, monkeypatch):
    """Every type has a 128-row and a 192-row workgroup tile and the library picks by launch shape; forced either way
    (COGNI_GEMM_N128, read per call) the results are the same bits - clipped tiles, k splits, a bias - and within the bar."""
    rng = np.random.default_rng(t * 31 + tokens + out_dim)
    raw = synth.make_weights(rng, t, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    bias = rng.standard_normal(out_dim).astype(np.float32)
    outs, splits = {}, {}
    for mode in ("0", "1"):
        monkeypatch.setenv("COGNI_GEMM_N128", mode)
        wsb = quant.gemm_workspace_bytes(t, in_dim, tokens, out_dim)
        name, _, splits[mode], _ = quant.gemm_plan(t, in_dim, out_dim, tokens, wsb)
        assert name.endswith("_n128_f16") == (mode == "1") or name == "q4_k_gemm_wide_f16", name
        outs[mode] = run_gemm(raw, x, in_dim, out_dim, tokens, bias, t=t)
    monkeypatch.delenv("COGNI_GEMM_N128")
    assert splits["0"] == splits["1"]       # (the k split, which these shapes share, is what fixes the order of the sums)
    assert np.array_equal(outs["0"], outs["1"])
    check(oracle, raw, x, in_dim, out_dim, tokens, bias, "type %d M=%d N=%d K=%d" % (t, tokens, out_dim, in_dim), t=t,
          sample_tokens=[i for i in (0, 1, 63, 64, 127, 128, tokens - 1) if i < tokens])


@pytest.mark.parametrize("t", [Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("tokens,out_dim,in_dim", [(64, 12288, 1024), (9, 4096 + 37, 768), (33, 250, 4096), (64, 1024, 256)])
def test_launches_of_up_to_64_tokens(gpu, oracle, t, tokens, out_dim, in_dim, monkeypatch):
    """Up to 64 tokens run the kernels that work on the first 64 tokens of the token tile (<type>_gemm_m64[_n128]_f16): the
    bits of the 128-token kernels (COGNI_GEMM_M64=0), whole and clipped tiles, k splits, a bias; and the bar."""
    rng = np.random.default_rng(t * 37 + tokens + out_dim)
    raw = synth.make_weights(rng, t, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    bias = rng.standard_normal(out_dim).astype(np.float32)
    wsb = quant.gemm_workspace_bytes(t, in_dim, tokens, out_dim)
    assert "_m64" in quant.gemm_plan(t, in_dim, out_dim, tokens, wsb)[0]
    half = run_gemm(raw, x, in_dim, out_dim, tokens, bias, t=t)
    monkeypatch.setenv("COGNI_GEMM_M64", "0")
    assert "_m64" not in quant.gemm_plan(t, in_dim, out_dim, tokens, wsb)[0]
    full = run_gemm(raw, x, in_dim, out_dim, tokens, bias, t=t)
    monkeypatch.delenv("COGNI_GEMM_M64")
    assert np.array_equal(half, full)
    check(oracle, raw, x, in_dim, out_dim, tokens, bias, "type %d M=%d N=%d K=%d" % (t, tokens, out_dim, in_dim), t=t)


@pytest.mark.parametrize("t,tokens,out_dim,in_dim", [(Q4_K, 130, 400, 768), (Q6_K, 64, 384, 4096), (Q5_K, 40, 100, 512),
                                                     (Q4_K, 128, 65536, 256), (Q6_K, 512, 4096, 2048)])
def test_residual_add_in_the_epilogue(gpu, oracle, t, tokens, out_dim, in_dim):
    """cogni_gemm_packed_add_dev: the GEMM's sums plus a [tokens][out_dim] residual, unsplit, k-split (the plane sum adds it)
    and on the wide tiles; the bits of the plain GEMM followed by an fp32 add, also when the residual is the output buffer."""
    rng = np.random.default_rng(tokens + out_dim)
    raw = synth.make_weights(rng, t, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    res = (rng.standard_normal(tokens * out_dim) * 30).astype(np.float32)
    plain = run_gemm(raw, x, in_dim, out_dim, tokens, t=t)
    wsb = quant.gemm_workspace_bytes(t, in_dim, tokens, out_dim)
    w, xd, ws = DevArray(raw), DevArray(x), DevArray(nbytes=wsb)
    rd, od = DevArray(res), DevArray(nbytes=4 * tokens * out_dim)
    quant.gemm_pack_dev(xd.ptr, t, in_dim, tokens, ws.ptr, wsb)
    quant.gemm_packed_add_dev(w.ptr, t, ws.ptr, wsb, rd.ptr, od.ptr, in_dim, out_dim, tokens)
    got = od.read(np.float32, tokens * out_dim)
    assert np.array_equal(got, plain + res)
    quant.gemm_packed_add_dev(w.ptr, t, ws.ptr, wsb, rd.ptr, rd.ptr, in_dim, out_dim, tokens)      # in place
    assert np.array_equal(rd.read(np.float32, tokens * out_dim), got)
    sample = [0, 1, tokens // 2, tokens - 1]
    xs = np.ascontiguousarray(x.reshape(tokens, in_dim)[sample].reshape(-1))
    want = oracle.matmul_add(xs, len(sample), in_dim, raw, t, out_dim, np.zeros(out_dim, dtype=np.float32), threads=16).reshape(len(sample), out_dim)
    want = want + res.reshape(tokens, out_dim)[sample]
    assert np.max(np.abs(got.reshape(tokens, out_dim)[sample] - want)) <= 2e-3 * np.max(np.abs(want))
    with pytest.raises(quant.QuantError, match="null device pointer"):
        quant.gemm_packed_add_dev(w.ptr, t, ws.ptr, wsb, 0, od.ptr, in_dim, out_dim, tokens)
    for a in (w, xd, ws, rd, od):
        a.close()


@pytest.mark.parametrize("tokens,out_dim,in_dim", [(130, 200, 512), (9, 96, 256), (64, 12288, 4096), (512, 12288, 4096), (257, 1000, 768)])
def test_gate_up_swiglu_in_one_gemm(gpu, oracle, tokens, out_dim, in_dim):
    """cogni_gemm_packed_swiglu_dev: silu(x W_gate^T) * (x W_up^T) without the two matrices in memory. The bits of the two
    GEMMs followed by swiglu_f32 (same sums in the same order, the same device function), clipped tiles in both directions
    and an odd number of super-blocks; against the oracle's CPU form on a sample of tokens."""
    rng = np.random.default_rng(tokens * 7 + out_dim)
    raw_g = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    raw_u = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    n = tokens * out_dim
    wsb = quant.gemm_workspace_bytes(Q4_K, in_dim, tokens)          # packed activations only: the two plain GEMMs run unsplit
    wg, wu, xd, ws = DevArray(raw_g), DevArray(raw_u), DevArray(x), DevArray(nbytes=wsb)
    og, ou, o2, of = (DevArray(nbytes=4 * n) for _ in range(4))
    quant.gemm_pack_dev(xd.ptr, Q4_K, in_dim, tokens, ws.ptr, wsb)
    quant.gemm_packed_dev(wg.ptr, Q4_K, ws.ptr, wsb, og.ptr, in_dim, out_dim, tokens)
    quant.gemm_packed_dev(wu.ptr, Q4_K, ws.ptr, wsb, ou.ptr, in_dim, out_dim, tokens)
    quant.swiglu_dev(og.ptr, ou.ptr, o2.ptr, n)
    quant.gemm_packed_swiglu_dev(wg.ptr, wu.ptr, Q4_K, ws.ptr, wsb, of.ptr, in_dim, out_dim, tokens)
    fused, two_step = of.read(np.float32, n), o2.read(np.float32, n)
    assert np.array_equal(fused, two_step)
    sample = sorted({t_ for t_ in (0, 1, 31, 32, tokens // 2, tokens - 1) if t_ < tokens})
    xs = np.ascontiguousarray(x.reshape(tokens, in_dim)[sample].reshape(-1))
    zero = np.zeros(out_dim, dtype=np.float32)
    ref = oracle.swiglu(oracle.matmul_add(xs, len(sample), in_dim, raw_g, Q4_K, out_dim, zero, threads=16),
                        oracle.matmul_add(xs, len(sample), in_dim, raw_u, Q4_K, out_dim, zero, threads=16))
    got = fused.reshape(tokens, out_dim)[sample].reshape(-1)
    assert cosine(got, ref) >= 0.9999
    assert np.max(np.abs(got - ref)) <= 4e-3 * np.max(np.abs(ref))      # a product of two sums that each carry 2e-3
    with pytest.raises(quant.QuantError, match="Unsupported quant type for the fused gate/up SwiGLU GEMM: Q6_K"):
        quant.gemm_packed_swiglu_dev(wg.ptr, wu.ptr, Q6_K, ws.ptr, wsb, of.ptr, in_dim, out_dim, tokens)
    for a in (wg, wu, xd, ws, og, ou, o2, of):
        a.close()


@pytest.mark.parametrize("next_type", [Q4_K, Q5_K, Q6_K])
@pytest.mark.parametrize("tokens,out_dim,in_dim", [(130, 256, 512), (9, 768, 256), (64, 1024, 768), (300, 2560, 512), (512, 12288, 4096)])
def test_gate_up_swiglu_hands_on_packed_activations(gpu, tokens, out_dim, in_dim, next_type):
    """cogni_gemm_packed_swiglu_pack_dev: the products of the gate | up GEMM written by its epilogue as the packed fp16
    activations of the next GEMM - every byte of what cogni_gemm_pack_dev writes from the fp32 products, for the three weight
    types' layouts, last token tiles that are not full (zeros for the absent tokens), a row count that is not a multiple of
    the 96-row tile (1024, 2560: the last tile is clipped), with and without the fp32 products stored as well."""
    rng = np.random.default_rng(tokens * 11 + out_dim + int(next_type))
    raw_g = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    raw_u = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    n = tokens * out_dim
    wsb = quant.gemm_workspace_bytes(Q4_K, in_dim, tokens)
    nxb = quant.gemm_workspace_bytes(next_type, out_dim, tokens)
    wg, wu, xd, ws = DevArray(raw_g), DevArray(raw_u), DevArray(x), DevArray(nbytes=wsb)
    # the buffers the fused launch writes start as 0xFF bytes: every byte of the packed block has to be written by it
    ff = np.full(nxb, 0xFF, dtype=np.uint8)
    of, o2 = DevArray(nbytes=4 * n), DevArray(np.full(n, np.float32(-7.0)))
    p_ref, p_a, p_b = DevArray(nbytes=nxb), DevArray(ff), DevArray(ff)
    quant.gemm_pack_dev(xd.ptr, Q4_K, in_dim, tokens, ws.ptr, wsb)
    quant.gemm_packed_swiglu_dev(wg.ptr, wu.ptr, Q4_K, ws.ptr, wsb, of.ptr, in_dim, out_dim, tokens)
    quant.gemm_pack_dev(of.ptr, next_type, out_dim, tokens, p_ref.ptr, nxb)
    quant.gemm_packed_swiglu_pack_dev(wg.ptr, wu.ptr, Q4_K, ws.ptr, wsb, o2.ptr, next_type, p_a.ptr, nxb, in_dim, out_dim, tokens)
    quant.gemm_packed_swiglu_pack_dev(wg.ptr, wu.ptr, Q4_K, ws.ptr, wsb, 0, next_type, p_b.ptr, nxb, in_dim, out_dim, tokens)
    want = p_ref.read(np.uint8, nxb)
    assert np.array_equal(p_a.read(np.uint8, nxb), want)
    assert np.array_equal(p_b.read(np.uint8, nxb), want)
    assert np.array_equal(o2.read(np.float32, n), of.read(np.float32, n))
    with pytest.raises(quant.QuantError, match="out_dim must be a multiple of 256"):
        quant.gemm_packed_swiglu_pack_dev(wg.ptr, wu.ptr, Q4_K, ws.ptr, wsb, 0, next_type, p_b.ptr, nxb, in_dim, out_dim - 64, tokens)
    with pytest.raises(quant.QuantError, match="next_workspace too small"):
        quant.gemm_packed_swiglu_pack_dev(wg.ptr, wu.ptr, Q4_K, ws.ptr, wsb, 0, next_type, p_b.ptr, nxb - 1, in_dim, out_dim, tokens)
    with pytest.raises(quant.QuantError, match="Unsupported quant type for the prefill GEMM"):
        quant.gemm_packed_swiglu_pack_dev(wg.ptr, wu.ptr, Q4_K, ws.ptr, wsb, 0, Q8_0, p_b.ptr, nxb, in_dim, out_dim, tokens)
    for a in (wg, wu, xd, ws, of, o2, p_ref, p_a, p_b):
        a.close()


@pytest.mark.parametrize("t,tokens,in_dim,dims", [
    (Q4_K, 130, 512, [200, 96, 1000]), (Q4_K, 64, 4096, [4096, 1024, 1024, 12288, 12288]), (Q5_K, 9, 256, [7]),
    (Q5_K, 300, 768, [129, 128, 192, 193, 5, 640]), (Q4_K, 512, 4096, [4096, 1024, 1024]), (Q4_K, 33, 1024, [191, 385]),
    (Q4_K, 2048, 512, [1024, 12288, 1024])])          # (the 12288-row member gets the eight-wavefront kernel, by itself)
def test_lists_of_matrices_in_one_gemm(gpu, t, tokens, in_dim, dims):
    """cogni_gemm_packed_many_dev: up to six matrices of one type and row length against one packed activation block in one
    launch; every output bit for bit what cogni_gemm_packed_dev gives for that matrix alone without a k split (row counts that
    are and are not multiples of either tile height, a single matrix, up to 64 tokens and more, the shapes of a layer)."""
    rng = np.random.default_rng(tokens + in_dim + len(dims))
    raws = [synth.make_weights(rng, t, d, in_dim) for d in dims]
    x = synth.make_activations(rng, tokens, in_dim)
    wsb = quant.gemm_workspace_bytes(t, in_dim, tokens)              # packed activations only: the single launches run unsplit
    ws, xd, wd = DevArray(nbytes=wsb), DevArray(x), [DevArray(r) for r in raws]
    singles = [DevArray(nbytes=4 * tokens * d) for d in dims]
    lists = [DevArray(np.full(tokens * d, np.float32(-3.0))) for d in dims]
    quant.gemm_pack_dev(xd.ptr, t, in_dim, tokens, ws.ptr, wsb)
    for w, o, d in zip(wd, singles, dims):
        quant.gemm_packed_dev(w.ptr, t, ws.ptr, wsb, o.ptr, in_dim, d, tokens)
    quant.gemm_packed_many_dev([w.ptr for w in wd], t, ws.ptr, wsb, [o.ptr for o in lists], dims, in_dim, tokens)
    for o1, o2, d in zip(singles, lists, dims):
        assert np.array_equal(o2.read(np.float32, tokens * d), o1.read(np.float32, tokens * d)), d
    with pytest.raises(quant.QuantError, match="Unsupported quant type for the list GEMM: Q6_K"):
        quant.gemm_packed_many_dev([w.ptr for w in wd], Q6_K, ws.ptr, wsb, [o.ptr for o in lists], dims, in_dim, tokens)
    with pytest.raises(quant.QuantError, match="one to six matrices"):
        quant.gemm_packed_many_dev([wd[0].ptr] * 7, t, ws.ptr, wsb, [lists[0].ptr] * 7, [dims[0]] * 7, in_dim, tokens)
    with pytest.raises(quant.QuantError, match="null device pointer"):
        quant.gemm_packed_many_dev([0], t, ws.ptr, wsb, [lists[0].ptr], [dims[0]], in_dim, tokens)
    for a in [ws, xd] + wd + singles + lists:
        a.close()


def test_projections_share_one_packed_activation_block(gpu, oracle):
    """gemm_pack_dev once, then gemm_packed_dev for several matrices of one type family (Q4_K and Q5_K read the same packed
    layout; a k-split and an unsplit shape, with and without bias): the bits of gemm_dev on each matrix alone."""
    tokens, in_dim = 96, 2048
    rng = np.random.default_rng(321)
    x = synth.make_activations(rng, tokens, in_dim)
    members = [(Q4_K, 1000, None), (Q5_K, 384, rng.standard_normal(384).astype(np.float32)), (Q4_K, 4096, None)]
    raws = [synth.make_weights(rng, t, d, in_dim) for t, d, _ in members]
    nbytes = max(quant.gemm_workspace_bytes(t, in_dim, tokens, d) for t, d, _ in members)
    ws, xd = DevArray(nbytes=nbytes), DevArray(x)
    quant.gemm_pack_dev(xd.ptr, Q4_K, in_dim, tokens, ws.ptr, nbytes)
    for (t, d, bias), raw in zip(members, raws):
        wd, od = DevArray(raw), DevArray(nbytes=4 * tokens * d)
        bd = DevArray(bias) if bias is not None else None
        quant.gemm_packed_dev(wd.ptr, t, ws.ptr, nbytes, od.ptr, in_dim, d, tokens, bd.ptr if bd else 0)
        got = od.read(np.float32, tokens * d)
        assert np.array_equal(got, run_gemm(raw, x, in_dim, d, tokens, bias, t=t)), (t, d)
        for a_ in (wd, od) + ((bd,) if bd else ()):
            a_.close()
    with pytest.raises(quant.QuantError, match="workspace has 16 bytes"):
        quant.gemm_pack_dev(xd.ptr, Q4_K, in_dim, tokens, ws.ptr, 16)
    with pytest.raises(quant.QuantError, match="null device pointer"):
        quant.gemm_packed_dev(0, Q4_K, ws.ptr, nbytes, xd.ptr, in_dim, 16, tokens)
    for a_ in (ws, xd):
        a_.close()


def test_argument_checks(gpu):
    w, x, o = DevArray(nbytes=4096), DevArray(nbytes=4096), DevArray(nbytes=4096)
    with pytest.raises(quant.QuantError, match="Unsupported quant type for the prefill GEMM") as e:
        quant.gemm_dev(w.ptr, Q8_0, x.ptr, o.ptr, 256, 1, 16, w.ptr, 4096)
    assert e.value.code == -2
    with pytest.raises(quant.QuantError, match="workspace has 16 bytes, needs 65536"):
        quant.gemm_dev(w.ptr, Q4_K, x.ptr, o.ptr, 256, 1, 16, w.ptr, 16)
    with pytest.raises(quant.QuantError, match="in_dim multiple of 256"):
        quant.gemm_dev(w.ptr, Q4_K, x.ptr, o.ptr, 100, 1, 16, w.ptr, 1 << 20)
    with pytest.raises(quant.QuantError, match="bias is only accepted"):
        quant.matmul_dev(w.ptr, Q4_K, x.ptr, o.ptr, 256, 1, 4, 0, 0, bias_ptr=o.ptr)
    for a in (w, x, o):
        a.close()


@pytest.mark.parametrize("tokens", [64, 512])
def test_configured_prefill_shapes(gpu, oracle, tokens):
    """Config 4: X tokens x 4096, W Q4_K 12288 x 4096."""
    rng = np.random.default_rng(4096 + tokens)
    out_dim, in_dim = 12288, 4096
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    sample = None if tokens <= 64 else np.concatenate([np.arange(0, 24), np.arange(250, 262), np.arange(tokens - 12, tokens)])
    check(oracle, raw, x, in_dim, out_dim, tokens, None, "cfg4 M=%d" % tokens, sample_tokens=sample)


def test_q5_k_fifth_bits_one_position_at_a_time(gpu, oracle):
    """Q5_K blocks whose nibbles are zero and whose fifth bits are set for one sub-block at a time, with distinct scales:
    a bit taken from the wrong position of qh, or put beside the wrong nibble, moves weight to other activations."""
    in_dim, out_dim, tokens = 256, 32, 16
    rng = np.random.default_rng(55)
    x = synth.make_activations(rng, tokens, in_dim)
    for sub in range(8):
        raw = np.zeros((out_dim, 176), dtype=np.uint8)
        raw[:, 0:2] = np.frombuffer(np.float16(0.03).tobytes(), dtype=np.uint8)      # d; dmin = 0
        raw[:, 4:8] = np.array([3, 5, 7, 9], dtype=np.uint8)                         # scales of sub-blocks 0..3
        raw[:, 12:16] = np.array([11, 13, 15, 2], dtype=np.uint8)                    # low 4 bits: scales of sub-blocks 4..7
        pattern = ((np.arange(32)[None, :] + np.arange(out_dim)[:, None]) % 3 != 0)  # which l carry the bit
        raw[:, 16:48] = (pattern.astype(np.uint8) << sub)
        raw[:, 48:176] = ((np.arange(128)[None, :] * 5 + np.arange(out_dim)[:, None]) % 16 * 17).astype(np.uint8)
        check(oracle, raw.reshape(-1), x, in_dim, out_dim, tokens, None, "Q5_K fifth bits of sub-block %d" % sub, t=Q5_K)


def test_q6_k_down_projection_prefill(gpu, oracle):
    """The Q6_K down projection of the mixed-quant layer (12288 -> 4096) at M = 512: a sample of tokens against the
    oracle and every token against the same token in a smaller GEMM."""
    rng = np.random.default_rng(6)
    out_dim, in_dim, tokens = 4096, 12288, 512
    raw = synth.make_weights(rng, Q6_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    got = check(oracle, raw, x, in_dim, out_dim, tokens, None, "Q6_K down M=512", sample_tokens=[0, 1, 127, 128, 300, 511], t=Q6_K)
    # the same tokens in a launch of their own, without the k split: equal up to the order of the fp32 sums
    part = run_gemm(raw, x[400 * in_dim:], in_dim, out_dim, tokens - 400, t=Q6_K, split=False).reshape(-1, out_dim)
    assert np.max(np.abs(part - got[400:])) <= 2e-5 * np.max(np.abs(got))
    again = run_gemm(raw, x, in_dim, out_dim, tokens, t=Q6_K).reshape(tokens, out_dim)
    assert np.array_equal(again, got)                      # the split sums its planes in a fixed order


def test_m2048_row_identity(gpu, oracle):
    """M = 2048: a sample of tokens against the oracle, and every token against the same token run through a
    smaller unsplit GEMM (the result for a token does not depend on which tile it sits in)."""
    rng = np.random.default_rng(2048)
    out_dim, in_dim, tokens = 12288, 4096, 2048
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    got = check(oracle, raw, x, in_dim, out_dim, tokens, None, "cfg4 M=2048",
                sample_tokens=[0, 1, 127, 128, 1000, 1023, 1024, 2046, 2047])
    part = run_gemm(raw, x[1900 * in_dim:], in_dim, out_dim, tokens - 1900, split=False).reshape(-1, out_dim)
    assert np.array_equal(part, got[1900:])


def test_activation_magnitude_on_both_sides_of_the_router_threshold(gpu, oracle):
    """QuantWeight.matmul changes kernels between 8 and 9 rows. Activations up to 3e4 (inside binary16) must pass both bars on
    both sides; an activation of 1e5 stays exact on the GEMV side (per-super-block scaling) and, as documented for the
    GEMM (x is converted with a plain float -> half cast, like the reference's Metal kernel), turns that token's outputs
    non-finite on the GEMM side while every other token stays within the bar."""
    rng = np.random.default_rng(65504)
    in_dim, out_dim = 1024, 192
    raw = synth.make_weights(rng, Q4_K, out_dim, in_dim)
    zero = np.zeros(out_dim, dtype=np.float32)
    for rows in (8, 9):
        x = (synth.make_activations(rng, rows, in_dim) * np.float32(1e4)).astype(np.float32)      # |x| up to about 4e4
        x = np.clip(x, -3e4, 3e4).astype(np.float32)
        qw = quant.QuantWeight(raw, Q4_K, out_dim, in_dim, "range")
        got = qw.matmul(x, rows)
        want = oracle.matmul_add(x, rows, in_dim, raw, Q4_K, out_dim, zero, threads=8)
        assert np.max(np.abs(got - want)) <= (2e-3 if rows > 8 else 1e-5) * np.max(np.abs(want)), rows
        x2 = x.copy().reshape(rows, in_dim)
        x2[3, 100] = np.float32(1e5)
        x2 = np.ascontiguousarray(x2.reshape(-1))
        got2 = qw.matmul(x2, rows).reshape(rows, out_dim)
        want2 = oracle.matmul_add(x2, rows, in_dim, raw, Q4_K, out_dim, zero, threads=8).reshape(rows, out_dim)
        others = [r for r in range(rows) if r != 3]
        assert np.max(np.abs(got2[others] - want2[others])) <= (2e-3 if rows > 8 else 1e-5) * np.max(np.abs(want2)), rows
        if rows <= 8:
            assert np.max(np.abs(got2[3] - want2[3])) <= 1e-5 * np.max(np.abs(want2[3]))
        else:
            assert not np.isfinite(got2[3]).any()
        qw.close()
