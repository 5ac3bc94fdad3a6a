"""CPU-side checks of the C-ABI boundary: the library loads, exports every declared symbol, embeds a
gfx950 code object with the documented kernel symbols, and fails loudly when there is no GPU."""
import ctypes
import os
import re
import struct

import numpy as np
import pytest

from cogni_ml_amd import hip, quant
from cogni_ml_amd.types import TensorType

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:mlhip|cogni)_[a-z0-9_]+)\s*\(", text)))


@pytest.mark.parametrize("header", ["ml_hip_driver.h", "cogni_quant.h"])
def test_every_declared_symbol_is_exported(header):
    L = hip.lib()
    names = declared_functions(header)
    assert len(names) >= 10
    for n in names:
        assert hasattr(L, n), "%s declared in %s but not exported" % (n, header)


def test_the_crystal_binding_names_every_operator():
    """The `lib` block a cogni-ml maintainer would use (crystal/src/ml/hip/driver.cr) declares every function of cogni_quant.h."""
    src = open(os.path.join(ROOT, "cogni-ml_amd", "crystal", "src", "ml", "hip", "driver.cr")).read()
    bound = set(re.findall(r"^\s*fun (\w+)", src, re.M))
    missing = [n for n in declared_functions("cogni_quant.h") if n not in bound]
    assert not missing, missing


def test_geometry_matches_reference_table():
    L = hip.lib()
    for t in TensorType:
        assert L.cogni_block_bytes(int(t)) == t.block_bytes
        assert L.cogni_block_elements(int(t)) == t.block_elements
    assert L.cogni_data_bytes(12, 12288 * 4096) == 28311552
    assert L.cogni_data_bytes(14, 151936 * 4096) == 510504960
    assert L.cogni_data_bytes(8, 3584 * 1024) == 3899392
    assert L.cogni_block_bytes(99) == -1 and L.cogni_data_bytes(99, 10) == -1


def code_object():
    img, size = ctypes.c_void_p(), ctypes.c_size_t()
    assert hip.lib().cogni_quant_code_object(ctypes.byref(img), ctypes.byref(size)) == 0
    return ctypes.string_at(img, size.value)


def test_code_object_is_amdgpu_elf_with_kernel_symbols():
    blob = code_object()
    assert blob[:4] == b"\x7fELF" and blob[4] == 2                      # ELF64
    assert struct.unpack_from("<H", blob, 18)[0] == 224                  # EM_AMDGPU
    assert struct.unpack_from("<I", blob, 48)[0] & 0xFF == 0x4F          # EF_AMDGPU_MACH_AMDGCN_GFX950
    for t in (8, 12, 13, 14):
        for m in range(1, 9):
            for add in (0, 1):
                name = quant.gemv_kernel_name(t, m, add)
                assert name and (name.encode() + b"\x00") in blob, name
    for t in (0, 1, 8, 12, 13, 14, 20):
        assert (quant.dequantize_kernel_name(t).encode() + b"\x00") in blob
    assert quant.gemv_kernel_name(12, 1) == "q4_k_gemv_f32"               # the reference's naming scheme
    assert quant.gemv_kernel_name(14, 4, True) == "q6_k_gemv_add_f32_tbatch4"
    assert quant.gemv_kernel_name(20, 1) is None and quant.gemv_kernel_name(12, 9) is None
    assert quant.dequantize_kernel_name(10) is None


def test_gemv_launch_dims():
    for t in (8, 12, 13, 14):
        for m in range(1, 9):
            grid, block, lds = quant.gemv_launch_dims(t, m, 4096, 12288)
            assert block == 256 and 12288 % grid == 0 and 4 <= 12288 // grid <= 32
            assert 0 < lds <= 49152 and lds % 256 == 0
    # K-quants, M = 1: a row of one 4096-value column set is staged as that; a longer one in chunks of three sets
    assert quant.gemv_launch_dims(12, 1, 4096, 12288)[2] == 4096 * 4
    assert quant.gemv_launch_dims(12, 1, 8192, 4096)[2] == 12288 * 4
    assert quant.gemv_launch_dims(14, 1, 12288, 4096)[2] == 12288 * 4
    assert quant.gemv_launch_dims(12, 1, 65536, 4096)[2] <= 49152
    # Q8_0 keeps per-lane sums beside the staged activations: one per 1024-value column set and lane
    assert quant.gemv_launch_dims(8, 1, 1024, 3584)[2] == 1024 * 4 + 256
    # one token of a long K-quant matrix: the workgroups resident together share the row groups (Q6_K 1280, Q5_K 768 evenly)
    g_head = quant.gemv_launch_dims(14, 1, 4096, 151936)[0]
    groups = -(-151936 // 8)
    assert g_head == 1280 and groups > g_head          # five workgroups per compute unit walk 14 or 15 groups each
    # two tokens (one token group) walk the row groups too, 512 workgroups at most; three tokens and Q8_0 do not
    g2 = quant.gemv_launch_dims(14, 2, 4096, 151936)[0]
    assert g2 <= 512 and -(-groups // g2) * (g2 - 1) < groups
    assert quant.gemv_launch_dims(14, 3, 4096, 151936)[0] == groups and quant.gemv_launch_dims(8, 1, 4096, 151936)[0] == 151936 // 16
    # the top-1 scratch holds one entry per workgroup of the widest launch it is used with (one or two tokens)
    assert quant.gemv_top1_partials(14, 151936) == max(g_head, g2)
    # one token of Q4_K: 8 rows per workgroup, at most 1024 workgroups (four per compute unit), which walk the rest
    assert quant.gemv_launch_dims(12, 1, 256, 17)[0] == 3 and quant.gemv_launch_dims(12, 1, 4096, 4096)[0] == 512
    assert quant.gemv_launch_dims(12, 1, 4096, 12288)[0] == 1024 and quant.gemv_launch_dims(12, 1, 4096, 151936)[0] == 1024
    assert quant.gemv_launch_dims(12, 2, 4096, 12288)[0] == 384                    # two tokens: 768 groups of 16 rows, two per workgroup
    with pytest.raises(quant.QuantError):
        quant.gemv_launch_dims(20, 1, 256, 16)
    with pytest.raises(quant.QuantError):
        quant.gemv_launch_dims(12, 9, 256, 16)


def test_one_token_of_a_short_matrix_gets_fewer_rows_per_wavefront():
    """Matrices whose rows would fill fewer than 256 workgroups of the plain one-token kernel: the plan names the variant with
    one row per wavefront (Q8_0, whose kernel has four: two from 2048 rows), and its grid still covers every row."""
    assert quant.gemv_plan(12, 1, 4096, 1024) == ("q4_k_gemv_f32_r1", 256, 256, quant.gemv_launch_dims(12, 1, 4096, 1024)[2])
    assert quant.gemv_plan(12, 1, 4096, 1024, add=True)[0] == "q4_k_gemv_add_f32_r1"
    assert quant.gemv_plan(13, 1, 4096, 2040)[:2] == ("q5_k_gemv_f32_r1", 510) and quant.gemv_plan(13, 1, 4096, 2041)[0] == "q5_k_gemv_f32"
    assert quant.gemv_plan(14, 1, 4096, 37)[:2] == ("q6_k_gemv_f32_r1", 10)
    assert quant.gemv_plan(8, 1, 1024, 3584)[:2] == ("q8_0_gemv_f32_r2", 448)          # config 1's shape
    assert quant.gemv_plan(8, 1, 3584, 1024)[:2] == ("q8_0_gemv_f32_r1", 256)
    assert quant.gemv_plan(8, 1, 1024, 2040)[:2] == ("q8_0_gemv_f32_r1", 510) and quant.gemv_plan(8, 1, 1024, 2041)[:2] == ("q8_0_gemv_f32_r2", 256)
    assert quant.gemv_plan(8, 1, 1024, 4080)[0] == "q8_0_gemv_f32_r2" and quant.gemv_plan(8, 1, 1024, 4081)[0] == "q8_0_gemv_f32"
    for t, rows_default in ((12, 2), (13, 2), (14, 2), (8, 4)):
        for out_dim in (1, 3, 4, 5, 255, 1023, 1024, 1025, 2047, 2048, 4095, 4096, 12288):
            name, grid, block, lds = quant.gemv_plan(t, 1, 1024, out_dim)
            r = int(name.rsplit("_r", 1)[1]) if "_r" in name.rsplit("f32", 1)[1] else rows_default
            assert block == 256 and grid * 4 * r >= out_dim > (grid - 1) * 4 * r or grid < -(-out_dim // (4 * r)), (t, out_dim, name, grid)
            assert r == rows_default or -(-out_dim // (8 * r)) < 256      # halved only while the larger size gave fewer than 256 groups
    # the names by token count and their launch geometry stay those of the plain kernels (hosts that launch by name)
    assert quant.gemv_kernel_name(12, 1) == "q4_k_gemv_f32" and quant.gemv_launch_dims(12, 1, 4096, 1024)[0] == 128


def test_gemv_plan_picks_the_kernel_for_the_shape():
    # one token: the vector-ALU kernel and its geometry
    assert quant.gemv_plan(12, 1, 4096, 12288) == ("q4_k_gemv_f32",) + quant.gemv_launch_dims(12, 1, 4096, 12288)
    # 2..4 tokens of a Q4_K matrix: the matrix-core kernel, 8 wavefronts, one workgroup per 48 rows at 12288 rows
    name, grid, block, lds = quant.gemv_plan(12, 4, 4096, 12288)
    assert (name, grid, block) == ("q4_k_gemv_mfma_f32_tbatch4", 256, 512)
    assert lds == 64 + 8 * 3 * 1024 + 8 * 3 * 4 * 64 + 4 * 16 * (4 + 32 + 1024)
    assert quant.gemv_plan(12, 2, 4096, 12288, add=True)[0] == "q4_k_gemv_mfma_add_f32_tbatch2"
    assert quant.gemv_plan(12, 2, 4096, 4096)[1] == 256 and quant.gemv_plan(12, 2, 1024, 3584)[1] == 112
    # more groups of 48 rows than compute units: 256 workgroups walk them (9496 tiles of the 151936-row head)
    assert quant.gemv_plan(14, 4, 4096, 151936)[1] == 256 and quant.gemv_plan(12, 4, 4096, 12288 + 48)[1] == 256
    # rows of a multiple of 2048 values whose activations do not fit the staging buffer: staged a chunk at a time,
    # 8 wavefronts x 2 super-blocks x 4 tokens of LDS image
    name, grid, block, lds = quant.gemv_plan(12, 4, 12288, 4096)
    assert (name, grid, block) == ("q4_k_gemv_mfma_f32_tbatch4", 256, 512)
    assert lds == 64 + 8 * 3 * 1024 + 8 * 3 * 4 * 64 + 64 * (4 + 32 + 1024)
    assert quant.gemv_plan(12, 3, 12288, 4096)[3] == 64 + 8 * 3 * 1024 + 8 * 3 * 4 * 64 + 48 * (4 + 32 + 1024)
    # other row lengths that do not fit, other types, more tokens: the vector-ALU kernels
    assert quant.gemv_plan(12, 4, 8448, 4096)[0] == "q4_k_gemv_f32_tbatch4"
    assert quant.gemv_plan(12, 2, 12288, 4096)[0] == "q4_k_gemv_mfma_f32_tbatch2"
    # Q6_K: three and four tokens on the matrix cores (16 sub-block sums per staged super-block), two on the vector ALU
    name, grid, block, lds = quant.gemv_plan(14, 4, 4096, 4096)
    assert (name, grid, block) == ("q6_k_gemv_mfma_f32_tbatch4", 256, 512)
    assert lds == 64 + 8 * 3 * 1024 + 8 * 3 * 4 * 64 + 64 * (4 + 64 + 1024)
    assert quant.gemv_plan(14, 3, 12288, 4096, add=True)[0] == "q6_k_gemv_mfma_add_f32_tbatch3"
    assert quant.gemv_plan(14, 2, 4096, 4096)[0] == "q6_k_gemv_f32_tbatch2"
    assert quant.gemv_plan(14, 4, 8448, 4096)[0] == "q6_k_gemv_f32_tbatch4"
    assert quant.gemv_plan(13, 4, 4096, 4096)[0] == "q5_k_gemv_mfma_f32_tbatch4"     # Q5_K: as Q6_K, from three tokens
    assert quant.gemv_plan(13, 3, 12288, 4096, add=True)[0] == "q5_k_gemv_mfma_add_f32_tbatch3"
    assert quant.gemv_plan(13, 2, 4096, 4096)[0] == "q5_k_gemv_f32_tbatch2"          # two tokens: the vector-ALU pair is as fast
    assert quant.gemv_plan(13, 4, 8448, 4096)[0] == "q5_k_gemv_f32_tbatch4"
    assert quant.gemv_plan(12, 8, 4096, 4096)[0] == "q4_k_gemv_f32_tbatch8"
    with pytest.raises(quant.QuantError):
        quant.gemv_plan(12, 9, 4096, 4096)
    with pytest.raises(quant.QuantError):
        quant.gemv_plan(20, 1, 4096, 4096)


def test_gemm_plan_picks_tile_and_split_for_the_shape():
    blob = code_object()
    for k in ("q4_k_gemm_f16", "q4_k_gemm_wide_f16", "q5_k_gemm_f16", "q6_k_gemm_f16", "q4_k_gemm_n128_f16", "q5_k_gemm_n128_f16",
              "q6_k_gemm_n128_f16", "q4_k_gemm_m64_f16", "q5_k_gemm_m64_n128_f16", "q6_k_gemm_m64_f16", "q6_k_gemm_m64_n128_f16", "gemm_sum_splits_f32", "pack_x_f16_q4k", "pack_x_f16_q6k"):
        assert (k.encode() + b"\x00") in blob, k
    big = 1 << 40
    # 512 x 12288: 256 tiles of 128 x 192, one per compute unit; 192 wide tiles would leave a quarter of them idle
    assert quant.gemm_plan(12, 4096, 12288, 512, big) == ("q4_k_gemm_f16", 256, 1, 256)
    # 2048 x 12288: 768 wide tiles are three rounds of 256 where the narrow ones need four
    assert quant.gemm_plan(12, 4096, 12288, 2048, big) == ("q4_k_gemm_wide_f16", 768, 1, 512)
    assert quant.gemm_plan(12, 4096, 12288, 1024, big) == ("q4_k_gemm_f16", 512, 1, 256)       # two rounds either way
    assert quant.gemm_plan(12, 4096, 12288, 4096, big) == ("q4_k_gemm_wide_f16", 1536, 1, 512)  # 6 rounds instead of 8
    # the grid is whole blocks of 32 tiles (8 weight tiles x 4 token tiles), 8 blocks at a time: a clipped shape rounds up
    assert quant.gemm_plan(12, 4096, 12288 + 192, 512, big)[1] == 8 * 32 * 2 and quant.gemm_plan(12, 256, 400, 130, big)[1:3] == (16, 1)
    # the 12288 -> 4096 down projection at M = 512: 88 tiles of 192 rows with the k range split in two are 176 workgroups,
    # 128 tiles of 128 rows are 256 (blocks of 4 x 4 tiles, one per XCD) - every type has the smaller tile for such shapes
    for t, pfx in ((12, "q4_k"), (13, "q5_k"), (14, "q6_k")):
        assert quant.gemm_plan(t, 12288, 4096, 512, big) == (pfx + "_gemm_n128_f16", 128, 2, 256)
        assert quant.gemm_plan(t, 4096, 4096, 512, big) == (pfx + "_gemm_n128_f16", 128, 2, 256)
        assert quant.gemm_plan(t, 12288, 4096, 64, big) == (pfx + "_gemm_m64_n128_f16", 32, 8, 256)   # up to 64 tokens: half a token tile
        assert quant.gemm_plan(t, 12288, 4096, 65, big)[0] == pfx + "_gemm_n128_f16" and quant.gemm_plan(t, 4096, 12288, 9, big)[0] == pfx + "_gemm_m64_f16"
        assert quant.gemm_plan(t, 4096, 12288, 512, big)[0] == pfx + "_gemm_f16"            # 256 tiles of 192 rows fill the chip exactly
        assert quant.gemm_plan(t, 4096, 12288, 1024, big)[0] == pfx + "_gemm_f16"           # two rounds of 192 rows against three of 128
        # the planes of a split launch are sized by the same plan
        assert quant.gemm_workspace_bytes(t, 12288, 512, 4096) == quant.gemm_workspace_bytes(t, 12288, 512) + 2 * 512 * 4096 * 4
    assert quant.gemm_plan(13, 12288, 4096, 2048, big) == ("q5_k_gemm_n128_f16", 512, 1, 256)   # two rounds either way, of less work each
    assert quant.gemm_plan(12, 12288, 4096, 2048, big)[0] == "q4_k_gemm_wide_f16"              # one round of the 256-row tiles
    # few tiles: the k range is split when the workspace has room for the planes, else not
    name, gx, gy, block = quant.gemm_plan(12, 4096, 12288, 64, big)
    assert (name, gx, block) == ("q4_k_gemm_m64_f16", 64, 256) and gy == 4
    # (unsplit, 96 tiles of 128 rows spread over more compute units than 64 of 192)
    assert quant.gemm_plan(12, 4096, 12288, 64, quant.gemm_workspace_bytes(12, 4096, 64)) == ("q4_k_gemm_m64_n128_f16", 96, 1, 256)
    # the eight-wavefront kernel is Q4_K's alone
    assert quant.gemm_plan(13, 4096, 12288, 2048, big)[0] == "q5_k_gemm_f16" and quant.gemm_plan(14, 4096, 12288, 2048, big)[0] == "q6_k_gemm_f16"
    with pytest.raises(quant.QuantError, match="Unsupported quant type"):
        quant.gemm_plan(8, 4096, 12288, 512, big)
    with pytest.raises(quant.QuantError, match="multiple of 256"):
        quant.gemm_plan(12, 100, 12288, 512, big)


def test_argument_errors_do_not_need_a_gpu():
    import numpy as np
    x = np.zeros(256, dtype=np.float32)
    w = np.zeros(144, dtype=np.uint8)
    with pytest.raises(quant.QuantError, match="Unsupported quant type for fused matmul: Q4_0") as e:
        quant.matmul_add(x, 1, 256, w, 2, 1, None)
    assert e.value.code == -2
    with pytest.raises(quant.QuantError, match="requires in_dim multiple of 256") as e:
        quant.matmul_add(x, 1, 100, w, 12, 1, None)
    assert e.value.code == -1
    with pytest.raises(quant.QuantError, match="shape needs 288") as e:
        quant.matmul_add(x, 1, 256, w, 12, 2, None)
    assert e.value.code == -1
    with pytest.raises(quant.QuantError, match="Unsupported dequantization type") as e:
        quant.dequantize(w, 10, 256)
    assert e.value.code == -2


def test_quant_weight_matmul_checks_buffer_sizes_before_the_library_reads_them():
    # cogni_weight_matmul copies rows*in_dim floats from x and out_dim from bias: a short buffer must never reach it.
    # (The checks sit in front of the library call, so a weight without a device copy is enough to exercise them.)
    qw = quant.QuantWeight.__new__(quant.QuantWeight)
    qw.out_dim, qw.in_dim, qw._handle = 8, 256, None
    with pytest.raises(ValueError, match="x has 255 elements, rows\\*in_dim is 256"):
        qw.matmul(np.zeros(255, dtype=np.float32))
    with pytest.raises(ValueError, match="x has 256 elements, rows\\*in_dim is 512"):
        qw.matmul(np.zeros(256, dtype=np.float32), rows=2)
    with pytest.raises(ValueError, match="bias has 7 elements, out_dim is 8"):
        qw.matmul(np.zeros(256, dtype=np.float32), bias=np.zeros(7, dtype=np.float32))
    with pytest.raises(ValueError, match="rows must be positive"):
        qw.matmul(np.zeros(256, dtype=np.float32), rows=0)


def gpu_present():
    return os.path.exists("/dev/kfd")


@pytest.mark.skipif(gpu_present(), reason="checks the no-GPU failure mode")
def test_no_gpu_means_error_not_fallback():
    import numpy as np
    with pytest.raises(quant.QuantError, match="no CPU fallback") as e:
        quant.init(0)
    assert e.value.code == -4
    with pytest.raises(quant.QuantError, match="cogni_quant_init has not been called") as e:
        quant.dequantize(np.zeros(144, dtype=np.uint8), 12, 256)
    assert e.value.code == -3


# ---- ResidentSequenceRunner: the reference's three examples (spec/cuda_resident_sequence_runner_spec.cr:5-50)

def test_runner_runs_only_the_active_token_prefix():
    seen = []
    r = hip.ResidentSequenceRunner(4, lambda: None, lambda: None, seen.append)
    r.active_tokens = 2
    r.run_sequence()
    assert seen == [0, 1]
    assert r.run_repeated(3) == 6


def test_runner_passes_active_count_to_override():
    seen = []
    r = hip.ResidentSequenceRunner(8, lambda: None, lambda: None, lambda tok: None, None, seen.append)
    r.active_tokens = 4
    r.run_sequence()
    assert seen == [4]


def test_runner_rejects_invalid_active_counts():
    r = hip.ResidentSequenceRunner(4, lambda: None, lambda: None, lambda tok: None)
    with pytest.raises(ValueError, match="active_tokens must be positive"):
        r.active_tokens = 0
    with pytest.raises(ValueError, match="active_tokens must be <= tokens"):
        r.active_tokens = 5
    with pytest.raises(ValueError, match="tokens must be positive"):
        hip.ResidentSequenceRunner(0, lambda: None, lambda: None, lambda tok: None)
    with pytest.raises(ValueError, match="reps must be positive"):
        r.run_repeated(0)
    r.reset_active_tokens()
    assert r.active_tokens == 4


def test_one_pass_geometry_and_thresholds():
    """Pack + one pass over the weights: which shapes have a kernel, the size of the activation image (8 KiB of operands
    per super-block, then the scales and the sub-block sums), where gemv_dev switches to it,
    and that the planned grid reaches every 16-row tile: a workgroup's eight wavefronts split the row, a row group is t
    tiles and the workgroups walk the groups with stride grid."""
    assert quant.gemv_image_bytes(12, 4096, 8) == 16 * (8192 + 1024)
    assert quant.gemv_image_bytes(14, 12288, 2) == 48 * (8192 + 1024)
    assert quant.gemv_image_bytes(13, 4096, 4) == quant.gemv_image_bytes(12, 4096, 4)      # Q5_K reads the Q4_K image
    # rows that are not a multiple of 2048 values: the image is filled up to a multiple of 8 super-blocks
    assert quant.gemv_image_bytes(12, 1024, 4) == 8 * (8192 + 1024)
    assert quant.gemv_image_bytes(14, 5120, 8) == 24 * (8192 + 1024)
    assert quant.gemv_image_bytes(13, 256, 2) == 8 * (8192 + 1024)
    assert quant.gemv_image_bytes(8, 4096, 4) == quant.gemv_image_bytes(12, 4096, 4)       # so does Q8_0, eight blocks at a time
    for t, in_dim, tokens in ((12, 4096, 1), (12, 4096, 9), (12, 1000, 4), (12, 14336, 4), (13, 12544, 4), (8, 4128, 4), (2, 4096, 4), (12, 0, 4)):
        assert quant.gemv_image_bytes(t, in_dim, tokens) == 0, (t, in_dim, tokens)
    assert [quant.gemv_one_pass_from(12, d, 4096) for d in (2048, 4096, 6144, 12288, 14336, 1024)] == [5, 4, 4, 4, 0, 5]
    assert [quant.gemv_one_pass_from(13, d, 8192) for d in (2048, 4096, 6144, 12288, 14336, 1024)] == [5, 4, 4, 4, 0, 5]
    # rows that fill less than three quarters of their k-slices wait for five tokens, whatever the type and the height
    assert [quant.gemv_one_pass_from(14, d, 4096) for d in (1024, 2560, 3584, 5120)] == [5, 5, 3, 3]
    assert [quant.gemv_one_pass_from(12, d, 151936) for d in (1024, 2560, 3584)] == [5, 5, 2]
    assert [quant.gemv_one_pass_multi_from(12, d) for d in (256, 1024, 1536, 2048, 2560, 3072, 4096, 5120, 12288, 12544, 1000)] == \
        [5, 5, 2, 2, 5, 2, 2, 2, 2, 0, 0]
    assert quant.gemv_one_pass_multi_from(8, 4096) == 2 and quant.gemv_one_pass_multi_from(14, 1024) == 5 and quant.gemv_one_pass_multi_from(2, 4096) == 0
    # Q8_0: from two tokens on long rows and on tall matrices, from three on shorter rows, from five on half-filled ones
    assert [quant.gemv_one_pass_from(8, d, 4096) for d in (1024, 2048, 3584, 4096, 12288, 12320)] == [5, 3, 2, 2, 2, 0]
    assert quant.gemv_one_pass_from(8, 1024, 248320) == 2
    assert [quant.gemv_one_pass_from(t, 4096, 12288) for t in (14, 8, 2)] == [3, 2, 0]
    # tall matrices of up to 4096 columns (an output head) take the path earlier
    assert [quant.gemv_one_pass_from(14, 4096, r) for r in (40959, 40960, 151936)] == [3, 2, 2]
    assert [quant.gemv_one_pass_from(12, 4096, r) for r in (40959, 40960, 98303, 98304, 151936)] == [4, 3, 3, 2, 2]
    assert [quant.gemv_one_pass_from(13, 2048, r) for r in (40960, 98304)] == [3, 2]
    assert [quant.gemv_one_pass_from(t, 12288, 151936) for t in (12, 14)] == [4, 3] and quant.gemv_one_pass_from(12, 14336, 151936) == 0
    rng = np.random.default_rng(11)
    for t, tmax, lds in ((12, 3, 8 * 3 * 8 * 16 * 4 + 8 * 6 * 16 * 144), (13, 3, 8 * 3 * 8 * 16 * 4 + 8 * 6 * 16 * 176),
                         (14, 2, 8 * 3 * 8 * 16 * 4 + 8 * 4 * 16 * 240)):
        for in_dim in (256, 1024, 2048, 3584, 4096, 5120, 6144, 8192, 10240, 11008, 12288):
            for rows in [1, 15, 16, 17, 4096, 4097, 12288, 8 * 4096 - 16, 151936] + [int(r) for r in rng.integers(1, 400000, 40)]:
                grid, block, shmem = quant.gemv_packed_launch_dims(t, in_dim, rows)
                ntiles = -(-rows // 16)
                tiles = 1 if in_dim > 4096 else max(1, min(tmax, ntiles // 256))     # the kernel's own rule
                groups = -(-ntiles // tiles)
                assert (block, shmem) == (512, lds) and shmem <= 160 * 1024
                assert grid == min(256, groups) and grid >= 1
    for bad in ((12, 1000, 16), (12, 12544, 16), (8, 4128, 16), (2, 4096, 16), (12, 4096, 0)):
        with pytest.raises(quant.QuantError):
            quant.gemv_packed_launch_dims(*bad)


def test_one_pass_argument_errors_do_not_need_a_gpu():
    assert hip.lib().cogni_gemv_release_stream(None) == 0          # a stream without an image: nothing to do
    with pytest.raises(quant.QuantError, match="no one-pass kernel") as e:
        quant.gemv_pack_dev(0x1000, 12, 1000, 4, 0x2000)
    assert e.value.code == -1
    with pytest.raises(quant.QuantError, match="null device pointer"):
        quant.gemv_pack_dev(0, 12, 4096, 4, 0x2000)
    with pytest.raises(quant.QuantError, match="count must be 1..8"):
        quant.gemv_packed_dev([], 12, 0x2000, [], [], 4096, 4)
    with pytest.raises(quant.QuantError, match="no one-pass kernel"):
        quant.gemv_packed_dev([0x1000], 2, 0x2000, [0x3000], [16], 4096, 4)
    with pytest.raises(quant.QuantError, match="a residual goes with a single matrix"):
        quant.gemv_packed_dev([0x1000, 0x1100], 12, 0x2000, [0x3000, 0x3100], [16, 16], 4096, 4, residual_ptr=0x4000)
    with pytest.raises(quant.QuantError, match="null pointer or zero rows"):
        quant.gemv_packed_dev([0x1000, 0x1100], 12, 0x2000, [0x3000, 0x3100], [16, 0], 4096, 4)
    with pytest.raises(quant.QuantError, match="no one-pass kernel"):
        quant.gemv_packed_swiglu_dev(0x1000, 0x1100, 14, 0x2000, 0x3000, 4096, 16, 4)
    with pytest.raises(quant.QuantError, match="no one-pass top-1 kernel"):
        quant.gemv_packed_top1_dev(0x1000, 13, 0x2000, 0x3000, 0x4000, 0x5000, 0x6000, 4096, 1000, 4)    # Q5_K: no top-1 form
    with pytest.raises(quant.QuantError, match="no one-pass top-1 kernel"):
        quant.gemv_packed_top1_dev(0x1000, 14, 0x2000, 0x3000, 0x4000, 0x5000, 0x6000, 4096, 1000, 9)
    with pytest.raises(quant.QuantError, match="null device pointer"):
        quant.gemv_packed_top1_dev(0x1000, 14, 0, 0x3000, 0x4000, 0x5000, 0x6000, 4096, 1000, 4)
    with pytest.raises(quant.QuantError, match="one-pass GEMV takes"):
        quant.rmsnorm_pack_dev(0x1000, 0x2000, 0, 12, 0x3000, 1000, 4)
    with pytest.raises(quant.QuantError, match="bad out_dim"):
        quant.gemv_packed_swiglu_dev(0x1000, 0x1100, 12, 0x2000, 0x3000, 4096, 0, 4)


def test_matrix_core_gemv_grid_covers_every_row():
    """The matrix-core kernels derive the tiles per wavefront from the grid they are launched with and cover rows
    beyond one group per workgroup only by walking (not where the activations are staged in chunks): for a sweep of
    shapes the planned grid must reach every 16-row tile under exactly those rules, and its LDS must fit a compute unit."""
    def log2_kslices(nsb):
        lg = 0
        while lg < 3 and (2 << lg) <= nsb:
            lg += 1
        return lg
    rng = np.random.default_rng(5)
    shapes = [(4096, 12288), (12288, 4096), (4096, 151936), (256, 1), (256, 17), (512, 70003), (2048, 20011), (26624, 33),
              (4096, 12288 + 48), (4096, 24576), (6144, 40), (8192, 300000)]
    shapes += [(256 * int(rng.integers(1, 120)), int(rng.integers(1, 200000))) for _ in range(300)]
    checked = 0
    for t in (12, 13, 14):
        for tokens in (2, 3, 4):
            for in_dim, out_dim in shapes:
                name, grid, block, lds = quant.gemv_plan(t, tokens, in_dim, out_dim)
                if "mfma" not in name:
                    continue
                checked += 1
                nsb = in_dim // 256
                units = tokens * nsb
                chunked = units > (64 if tokens >= 3 else 96)
                assert not chunked or in_dim % 2048 == 0
                nwr = 8 >> log2_kslices(nsb)
                ntiles = (out_dim + 15) // 16
                tk = -(-ntiles // (grid * nwr))                      # what the kernel computes from gridDim.x
                T = 1 if tk <= 1 else (2 if tk == 2 else 3)
                groups = -(-ntiles // (nwr * T))
                assert block == 512 and 0 < grid <= groups and lds <= 160 * 1024, (name, in_dim, out_dim, grid)
                assert grid == groups or (grid == 256 and not chunked), (name, in_dim, out_dim, grid, groups)
    assert checked > 500


def test_gemm_tile_numbering_covers_every_tile_once():
    """gemm_tile_of / gemm_grid_x (gemv_config.h) through a small C++ program: every tile of a launch is taken by exactly
    one workgroup, and the workgroups that share an XCD side by side hold a compact block of tiles."""
    import subprocess
    import tempfile
    src = r'''
#include <cstdio>
#include <set>
#include <utility>
#include "gemv_config.h"
int main() {
  int bad = 0;
  for (unsigned mt = 1; mt <= 40; mt++)
    for (unsigned nt = 1; nt <= 130; nt += (nt < 70 ? 1 : 7)) {
      const unsigned grid = gemm_grid_x(mt, nt);
      std::set<std::pair<unsigned, unsigned>> seen;
      for (unsigned id = 0; id < grid; id++) {
        unsigned a, b;
        if (!gemm_tile_of(id, mt, nt, &a, &b)) continue;
        if (a >= mt || b >= nt || !seen.insert({a, b}).second) bad++;
      }
      if (seen.size() != (size_t)mt * nt || grid % 8 != 0 || grid > 8 * (mt * nt + 32 * 8)) bad++;
    }
  // 512 x 12288 in 128 x 192 tiles: the first 32 workgroups of XCD 0 hold 8 weight tiles x 4 token tiles
  std::set<unsigned> ms, ns;
  for (unsigned l = 0; l < 32; l++) { unsigned a, b; gemm_tile_of(8 * l, 4, 64, &a, &b); ms.insert(a); ns.insert(b); }
  if (ms.size() != 4 || ns.size() != 8) bad++;
  std::printf("bad=%d\n", bad);
  return bad != 0;
}
'''
    with tempfile.TemporaryDirectory() as d:
        open(os.path.join(d, "t.cpp"), "w").write(src)
        subprocess.run(["g++", "-O1", "-std=c++17", "-I", os.path.join(ROOT, "cogni-ml_amd", "csrc", "kernels"), "-o", os.path.join(d, "t"),
                        os.path.join(d, "t.cpp")], check=True)
        r = subprocess.run([os.path.join(d, "t")], capture_output=True, text=True)
        assert r.returncode == 0 and "bad=0" in r.stdout, r.stdout + r.stderr
