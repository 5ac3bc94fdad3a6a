"""GGUFFile against files written by tests/gguf_writer.py: header, every metadata value type, tensor table, data
alignment, zero-copy raw bytes, and the reference's error behaviour (src/ml/gguf/reader.cr:278-314)."""
import numpy as np
import pytest

import gguf_writer as gw
from cogni_ml_amd import gguf, synth
from cogni_ml_amd.types import TensorType


def sample(tmp_path, **kw):
    rng = np.random.default_rng(3)
    q4 = synth.make_weights(rng, 12, 8, 512)                 # [in 512, out 8]
    q6 = synth.make_weights(rng, 14, 4, 256)
    f32 = rng.standard_normal(7).astype(np.float32)
    kv = [("general.architecture", gw.STRING, "qwen35"), ("qwen35.block_count", gw.UINT32, 32),
          ("qwen35.context_length", gw.INT64, -5), ("big", gw.UINT64, 2 ** 40), ("i32", gw.INT32, -7),
          ("qwen35.rope.freq_base", gw.FLOAT32, 1e6), ("f64", gw.FLOAT64, 0.125), ("flag", gw.BOOL, True),
          ("u8", gw.UINT8, 200), ("i8", gw.INT8, -3), ("u16", gw.UINT16, 65535), ("i16", gw.INT16, -300),
          ("tokens", gw.ARRAY, ["<s>", "", "héllo"], gw.STRING), ("head_kv", gw.ARRAY, [8, 8, 0, 2], gw.INT32),
          ("mask", gw.ARRAY, [True, False, True], gw.BOOL), ("empty", gw.ARRAY, [], gw.UINT32),
          ("scores", gw.ARRAY, [0.5, -1.0], gw.FLOAT32)]
    tensors = [("blk.0.ffn_gate.weight", [512, 8], 12, q4.tobytes()), ("output_norm.weight", [7], 0, f32.tobytes()),
               ("blk.0.ffn_down.weight", [256, 4], 14, q6.tobytes())]
    path = str(tmp_path / "m.gguf")
    data_offset = gw.write_gguf(path, kv, tensors, **kw)
    return path, data_offset, q4, q6, f32


@pytest.mark.parametrize("version,alignment", [(3, None), (2, None), (3, 64), (3, 4096)])
def test_header_metadata_and_tensor_table(tmp_path, version, alignment):
    path, data_offset, q4, q6, f32 = sample(tmp_path, version=version, alignment=alignment)
    with gguf.GGUFFile(path) as g:
        assert g.version == version and g.data_offset == data_offset and data_offset % (alignment or 32) == 0
        assert g.get_string("general.architecture") == "qwen35" and g.get_string("qwen35.block_count") is None
        assert g.get_int("qwen35.block_count") == 32 and g.get_int("qwen35.context_length") == -5
        assert g.get_int("big") == 2 ** 40 and g.get_int("i32") == -7
        assert g.get_int("u8") is None and g.get_int("i16") is None          # only 32- and 64-bit integers (reader.cr:229-237)
        assert g.get_float("qwen35.rope.freq_base") == 1e6 and g.get_float("f64") == 0.125 and g.get_float("i32") is None
        assert g.metadata["flag"].value is True and g.metadata["u16"].value == 65535 and g.metadata["i8"].value == -3
        assert g.metadata["tokens"].value == ["<s>", "", "héllo"]
        assert g.get_int_array("head_kv") == [8, 8, 0, 2] and g.get_int_array("tokens") is None and g.get_int_array("nope") is None
        assert g.get_bool_array("mask") == [True, False, True] and g.get_bool_array("head_kv") is None
        assert g.get_int_array("empty") == [] and g.get_float("scores") is None
        assert [t.name for t in g.tensors] == ["blk.0.ffn_gate.weight", "output_norm.weight", "blk.0.ffn_down.weight"]
        t = g.tensor("blk.0.ffn_gate.weight")
        assert t.dims == [512, 8] and t.type == TensorType.Q4_K and t.n_elements == 4096 and t.data_bytes == 16 * 144
        assert g.tensor("missing") is None
        raw = g.read_tensor_raw(t)
        assert raw.base is not None and not raw.flags.writeable and np.array_equal(raw, q4)      # a view of the mmap
        d = g.tensor("blk.0.ffn_down.weight")
        assert d.offset % (alignment or 32) == 0 and np.array_equal(g.read_tensor_raw(d), q6)
        n = g.tensor("output_norm.weight")
        assert n.data_bytes == 28 and np.array_equal(g.read_tensor_raw(n).view(np.float32), f32)
        whole, size = g.mmap_region()
        assert size == whole.size and np.array_equal(whole[g.data_offset + d.offset:][:q6.size], q6)
        del raw, whole


def test_errors(tmp_path):
    p = str(tmp_path / "bad.gguf")
    gw.write_gguf(p, [], [], magic=b"GGML")
    with pytest.raises(gguf.GGUFError, match="Not a GGUF file: magic='GGML'"):
        gguf.GGUFFile(p)
    for v in (1, 4):
        gw.write_gguf(p, [], [], version=v)
        with pytest.raises(gguf.GGUFError, match="Unsupported GGUF version: %d" % v):
            gguf.GGUFFile(p)
    open(p, "wb").write(b"GG")
    with pytest.raises(gguf.GGUFError, match="Not a GGUF file"):
        gguf.GGUFFile(p)
    open(p, "wb").close()
    with pytest.raises(gguf.GGUFError, match="Not a GGUF file"):
        gguf.GGUFFile(p)
    # truncated data blob: the table parses, reading the tensor does not
    path, data_offset, q4, _, _ = sample(tmp_path)
    blob = open(path, "rb").read()
    open(p, "wb").write(blob[:data_offset + 100])
    with gguf.GGUFFile(p) as g:
        with pytest.raises(gguf.GGUFError, match="ends at byte"):
            g.read_tensor_raw(g.tensor("blk.0.ffn_gate.weight"))
    # truncated header
    open(p, "wb").write(blob[:40])
    with pytest.raises(gguf.GGUFError, match="unexpected end of file"):
        gguf.GGUFFile(p)
    # unknown ggml type in the tensor table
    gw.write_gguf(p, [], [("t", [32], 99, b"\0" * 32)])
    with pytest.raises(gguf.GGUFError, match="unknown ggml type 99"):
        gguf.GGUFFile(p)
    with pytest.raises(gguf.GGUFError, match="missing tensor 'nope'"):
        with gguf.GGUFFile(path) as g:
            gguf.load_f32(g, "nope")


def test_duplicate_names_resolve_to_the_first(tmp_path):
    p = str(tmp_path / "dup.gguf")
    gw.write_gguf(p, [], [("w", [4], 0, np.arange(4, dtype=np.float32).tobytes()),
                          ("w", [4], 0, np.ones(4, dtype=np.float32).tobytes())])
    with gguf.GGUFFile(p) as g:
        assert np.array_equal(g.read_tensor_raw(g.tensor("w")).view(np.float32), np.arange(4, dtype=np.float32))
