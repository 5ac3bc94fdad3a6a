"""cogni_gemv_top1_noalloc_dev (the output-head arg-max with its partial results in the library's static device array)
against cogni_gemv_top1_dev (the same launches with caller-owned partial buffers): ids and values must agree bit for bit,
on two calls in a row, the second with a smaller input, so that what the first call left in the array is shown not to
matter. Collected last: a failure here must not hide the other GPU tests."""
import ctypes

import numpy as np
import pytest

from cogni_ml_amd import hip, quant, synth
from gpu_common import DevArray, gpu  # noqa: F401

pytestmark = pytest.mark.gpu
Q8_0, Q4_K, Q5_K, Q6_K = 8, 12, 13, 14


def top1_both(raw, t, x, in_dim, out_dim, tokens):
    """(ids, values) from the existing entry point and from the one that allocates nothing, on the same device inputs."""
    stride = quant.gemv_top1_partials(t, out_dim)
    wd, xd = DevArray(raw), DevArray(x)
    pi, pv = DevArray(nbytes=4 * tokens * stride), DevArray(nbytes=4 * tokens * stride)
    oi, ov = DevArray(nbytes=4 * tokens), DevArray(nbytes=4 * tokens)
    ni, nv = DevArray(np.full(tokens, 0xFFFFFFFF, dtype=np.uint32)), DevArray(np.full(tokens, np.nan, dtype=np.float32))
    try:
        quant.gemv_top1_dev(wd.ptr, t, xd.ptr, pi.ptr, pv.ptr, oi.ptr, ov.ptr, in_dim, out_dim, tokens)
        quant.gemv_top1_noalloc_dev(wd.ptr, t, xd.ptr, ni.ptr, nv.ptr, in_dim, out_dim, tokens)
        return (oi.read(np.uint32, tokens), ov.read(np.float32, tokens)), (ni.read(np.uint32, tokens), nv.read(np.float32, tokens))
    finally:
        for d in (wd, xd, pi, pv, oi, ov, ni, nv):
            d.close()


# (first call, second call): the second is smaller in rows, row length or tokens, and of another type in two of the pairs
PAIRS = [
    ((Q6_K, 1024, 40003, 4), (Q6_K, 512, 3001, 1)),     # matrix-core kernel walking row groups, then one token
    ((Q4_K, 2048, 20011, 7), (Q4_K, 256, 530, 2)),      # 4 + 3 tokens, then a pair on the vector ALU
    ((Q8_0, 1024, 3584, 3), (Q5_K, 512, 1001, 2)),      # one launch pair per token
]


@pytest.mark.parametrize("first,second", PAIRS)
def test_noalloc_top1_equals_top1_with_caller_buffers_twice_in_a_row(gpu, oracle, first, second):
    for call, (t, in_dim, out_dim, tokens) in enumerate((first, second)):
        print("case type=%d in_dim=%d out_dim=%d tokens=%d call=%d" % (t, in_dim, out_dim, tokens, call), flush=True)
        rng = np.random.default_rng(out_dim * 7 + tokens)
        raw = synth.make_weights(rng, t, out_dim, in_dim)
        x = synth.make_activations(rng, tokens, in_dim)
        (ids, vals), (nids, nvals) = top1_both(raw, t, x, in_dim, out_dim, tokens)
        assert np.array_equal(ids, nids), (call, ids, nids)
        assert np.array_equal(vals.view(np.uint32), nvals.view(np.uint32)), (call, vals, nvals)
        # and both are the oracle's winner within the GEMV tolerance (bit equality alone would also hold for two wrong answers)
        want = oracle.matmul_add(x, tokens, in_dim, raw, t, out_dim, np.zeros(out_dim, dtype=np.float32), threads=8).reshape(tokens, out_dim)
        for tok in range(tokens):
            top = float(want[tok].max())
            scale = float(np.abs(want[tok]).max())
            assert abs(float(nvals[tok]) - top) <= 1e-4 * scale
            assert want[tok][nids[tok]] >= top - 1e-4 * scale


def device_memory_free():
    """Free device memory as the HIP runtime reports it (test-only: the driver ABI of the library has no such call)."""
    rt = ctypes.CDLL("/opt/rocm/lib/libamdhip64.so")
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert rt.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


@pytest.mark.parametrize("t,in_dim,out_dim,tokens", [(Q6_K, 2048, 20011, 8), (Q4_K, 1024, 5003, 3), (Q6_K, 512, 3001, 1)])
def test_noalloc_top1_recorded_into_a_graph(gpu, t, in_dim, out_dim, tokens):
    """What the entry point is for: recorded under stream capture (eight tokens: the one-pass kernel with the library's
    image of the capture stream; three: the matrix-core kernel; one: the vector ALU), the device's free memory the same
    before and after the recording, and every replay - with eager calls of the same entry point in between, which use the
    same static array - equal to cogni_gemv_top1_dev bit for bit."""
    rng = np.random.default_rng(out_dim + tokens)
    raw = synth.make_weights(rng, t, out_dim, in_dim)
    x = synth.make_activations(rng, tokens, in_dim)
    x2 = synth.make_activations(rng, tokens, in_dim)
    (ids, vals), _ = top1_both(raw, t, x, in_dim, out_dim, tokens)
    (ids2, vals2), _ = top1_both(raw, t, x2, in_dim, out_dim, tokens)
    wd, xd = DevArray(raw), DevArray(x)
    gi, gv = DevArray(nbytes=4 * tokens), DevArray(nbytes=4 * tokens)
    ei, ev, x2d = DevArray(nbytes=4 * tokens), DevArray(nbytes=4 * tokens), DevArray(x2)
    st = hip.HIPStream()
    quant.gemv_top1_noalloc_dev(wd.ptr, t, xd.ptr, gi.ptr, gv.ptr, in_dim, out_dim, tokens, st.handle)   # (kernels resolved, image slot taken)
    st.synchronize()
    free0 = device_memory_free()
    st.begin_capture(1)
    quant.gemv_top1_noalloc_dev(wd.ptr, t, xd.ptr, gi.ptr, gv.ptr, in_dim, out_dim, tokens, st.handle)
    graph = st.end_capture()
    assert device_memory_free() == free0
    ex = graph.instantiate()
    try:
        for rep in range(3):
            hip.copy_htod(gi.ptr, np.full(tokens, 0xFFFFFFFF, dtype=np.uint32), 4 * tokens, "poison")
            ex.launch(st)
            st.synchronize()
            assert np.array_equal(gi.read(np.uint32, tokens), ids), rep
            assert np.array_equal(gv.read(np.float32, tokens).view(np.uint32), vals.view(np.uint32)), rep
            # an eager call on the same stream with other activations between the replays: it shares the static array
            quant.gemv_top1_noalloc_dev(wd.ptr, t, x2d.ptr, ei.ptr, ev.ptr, in_dim, out_dim, tokens, st.handle)
            st.synchronize()
            assert np.array_equal(ei.read(np.uint32, tokens), ids2) and np.array_equal(ev.read(np.float32, tokens).view(np.uint32), vals2.view(np.uint32))
    finally:
        ex.close()
        graph.close()
        st.close()
        for d in (wd, xd, gi, gv, ei, ev, x2d):
            d.close()


def test_noalloc_top1_rejects_what_does_not_fit_the_static_array(gpu):
    """Q8_0 has one workgroup per 16 rows: 8 tokens x 9496 partial results exceed the 65536 the array holds. The call must
    fail before it launches anything (the pointers are never dereferenced)."""
    out_dim = 151936
    assert 8 * quant.gemv_top1_partials(Q8_0, out_dim) > quant.TOP1_NOALLOC_MAX_PARTIALS
    # (real device memory behind every pointer, as large as the matrix named: a call accepted by mistake would stay inside it)
    big = DevArray(nbytes=out_dim * (1024 // 32) * 34)
    p = big.ptr
    with pytest.raises(quant.QuantError, match="exceed the static scratch of 65536") as e:
        quant.gemv_top1_noalloc_dev(p, Q8_0, p, p, p, 1024, out_dim, 8)
    assert e.value.code == -1
    # the operator's own argument checks still apply
    with pytest.raises(quant.QuantError, match="Unsupported quant type"):
        quant.gemv_top1_noalloc_dev(p, 20, p, p, p, 1024, 64, 1)
    big.close()
