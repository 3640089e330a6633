"""The GGUF reader of the upload path against files written by the test (all
metadata value types, several tensors, a non-default alignment) and, where the
compiled reference reader is available (oracle/_ref), byte-for-byte against
what the reference's own GGUFReader returns for the same file."""
import ctypes as C
import os

import numpy as np
import pytest

import oracle
from cut_amd import gguf
from helpers import write_gguf


def _model_file(tmp_path, alignment=32):
    rng = np.random.default_rng(0)
    w_q4k = oracle.quantize(oracle.Q4_K, rng.standard_normal(8 * 512).astype(np.float32))
    w_q6k = oracle.quantize(oracle.Q6_K, rng.standard_normal(4 * 256).astype(np.float32))
    w_q80 = oracle.quantize(oracle.Q8_0, rng.standard_normal(3 * 64).astype(np.float32))
    norm = rng.standard_normal(512).astype(np.float32)
    meta = {
        "general.architecture": (8, "llama"), "general.alignment": (4, alignment), "general.name": (8, "tiny"),
        "llama.embedding_length": (4, 512), "llama.block_count": (4, 2), "llama.attention.head_count": (4, 8),
        "llama.attention.head_count_kv": (4, 2), "llama.feed_forward_length": (4, 1024),
        "llama.rope.freq_base": (6, 500000.0), "llama.attention.layer_norm_rms_epsilon": (6, 1e-5),
        "llama.context_length": (4, 4096), "some.u8": (0, 7), "some.i8": (1, -7), "some.u16": (2, 65535), "some.i16": (3, -3),
        "some.i32": (5, -100000), "some.bool": (7, True), "some.u64": (10, 1 << 40), "some.i64": (11, -(1 << 40)),
        "some.f64": (12, 2.5), "tokenizer.tokens": (9, (8, ["a", "bc", ""])), "some.scores": (9, (6, [0.5, -1.0, 2.0])),
        "some.ids": (9, (5, [1, -2, 3])),
    }
    tensors = [("blk.0.attn_q.weight", (512, 8), 12, w_q4k), ("blk.0.attn_v.weight", (256, 4), 14, w_q6k),
               ("output.weight", (64, 3), 8, w_q80), ("blk.0.attn_norm.weight", (512,), 0, norm.tobytes())]
    path = str(tmp_path / "tiny.gguf")
    write_gguf(path, meta, tensors, alignment=alignment)
    return path, {"blk.0.attn_q.weight": w_q4k, "blk.0.attn_v.weight": w_q6k, "output.weight": w_q80,
                  "blk.0.attn_norm.weight": np.frombuffer(norm.tobytes(), np.uint8)}


@pytest.mark.parametrize("alignment", [32, 64])
def test_reads_back_what_was_written(tmp_path, alignment):
    path, want = _model_file(tmp_path, alignment)
    f = gguf.GGUFFile(path)
    assert f.version == 3 and f.data_offset % alignment == 0
    for name, data in want.items():
        assert np.array_equal(np.asarray(f.raw(name)), data), name
    t = f.tensors["blk.0.attn_q.weight"]
    assert t.dimensions == (512, 8) and t.type_name == "Q4_K" and t.nbytes == 8 * 2 * 144
    m = f.metadata
    assert m["some.u8"] == 7 and m["some.i8"] == -7 and m["some.u16"] == 65535 and m["some.i16"] == -3
    assert m["some.i32"] == -100000 and m["some.bool"] is True and m["some.u64"] == 1 << 40 and m["some.i64"] == -(1 << 40)
    assert m["some.f64"] == 2.5 and m["tokenizer.tokens"] == ["a", "bc", ""]
    assert np.array_equal(m["some.scores"], np.array([0.5, -1.0, 2.0], np.float32)) and list(m["some.ids"]) == [1, -2, 3]
    cfg = f.model_config()
    assert cfg == {"arch": "llama", "hidden": 512, "n_layers": 2, "n_heads": 8, "n_kv_heads": 2, "head_dim": 64, "ffn": 1024,
                   "rope_theta": 500000.0, "eps": pytest.approx(1e-5), "context_length": 4096}
    # the bytes are usable as they are: dequantizing them gives the same values as the source blocks
    assert np.array_equal(oracle.dequant(oracle.Q4_K, np.asarray(f.raw("blk.0.attn_q.weight")), 8 * 512),
                          oracle.dequant(oracle.Q4_K, want["blk.0.attn_q.weight"], 8 * 512))


def test_errors(tmp_path):
    bad = tmp_path / "bad.gguf"
    bad.write_bytes(b"NOPE" + b"\0" * 60)
    with pytest.raises(gguf.GGUFError, match="magic"):
        gguf.GGUFFile(str(bad))
    path, _ = _model_file(tmp_path)
    f = gguf.GGUFFile(path)
    with pytest.raises(gguf.GGUFError, match="not found"):
        f.raw("nope")
    data = open(path, "rb").read()
    trunc = tmp_path / "trunc.gguf"
    trunc.write_bytes(data[:-100])
    with pytest.raises(gguf.GGUFError, match="past the end"):
        gguf.GGUFFile(str(trunc))
    v9 = tmp_path / "v9.gguf"
    v9.write_bytes(data[:4] + (9).to_bytes(4, "little") + data[8:])
    with pytest.raises(gguf.GGUFError, match="version"):
        gguf.GGUFFile(str(v9))
    # general.alignment = 0 and an array that claims more elements than the file has bytes: errors, not crashes
    import struct

    def kv_file(name, key, type_code, payload):
        k = key.encode()
        blob = struct.pack("<IIQQ", 0x46554747, 3, 0, 1) + struct.pack("<Q", len(k)) + k + struct.pack("<I", type_code) + payload
        f = tmp_path / name
        f.write_bytes(blob + b"\0" * 64)
        return str(f)
    with pytest.raises(gguf.GGUFError, match="alignment"):
        gguf.GGUFFile(kv_file("align0.gguf", "general.alignment", 4, struct.pack("<I", 0)))
    with pytest.raises(gguf.GGUFError, match="array"):    # array of strings (type 8), count 2^40
        gguf.GGUFFile(kv_file("count.gguf", "tokenizer.tokens", 9, struct.pack("<IQ", 8, 1 << 40)))


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref (compiled reference reader) is not built")
def test_agrees_with_the_reference_reader(tmp_path):
    path, want = _model_file(tmp_path, alignment=64)
    ref = C.CDLL(os.path.join(os.path.dirname(oracle.__file__), "_ref", "libcut_ref.so"))
    ref.ref_read_raw.restype = C.c_long
    ref.ref_read_raw.argtypes = [C.c_char_p, C.c_char_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p]
    ref.ref_meta_u32.restype = C.c_uint32
    ref.ref_meta_u32.argtypes = [C.c_char_p, C.c_char_p]
    f = gguf.GGUFFile(path)
    for name in want:
        buf = np.zeros(1 << 16, np.uint8)
        dims = np.zeros(4, np.uint64)
        typ = C.c_uint32(0)
        n = ref.ref_read_raw(path.encode(), name.encode(), buf.ctypes.data, buf.size, dims.ctypes.data, C.byref(typ))
        info = f.tensors[name]
        assert n == info.nbytes and typ.value == info.ggml_type
        assert tuple(int(d) for d in dims[:len(info.dimensions)]) == info.dimensions
        assert np.array_equal(buf[:n], np.asarray(f.raw(name)))
    assert ref.ref_meta_u32(path.encode(), b"llama.embedding_length") == 512
    assert ref.ref_meta_u32(path.encode(), b"general.alignment") == 64
