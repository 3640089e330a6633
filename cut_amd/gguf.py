"""GGUF file reader for the weight-upload path: parses the header, metadata and
tensor table the way the reference reader does
(interface/loader/gguf/gguf_reader.cpp:15-58 header, :281-311 tensor infos,
value types gguf_types.hpp:56-70) and hands out the tensor bytes unchanged
(``read_tensor_raw``, gguf_reader.cpp:313-324), memory-mapped so that a model is
streamed to the device without a host copy of the whole file.  The block
formats this backend computes on (Q8_0, Q4_0, Q4_K, Q6_K) stay exactly as
stored: row n of a [K, N] tensor is K/blk consecutive blocks."""
from __future__ import annotations

import dataclasses
import struct

import numpy as np

GGUF_MAGIC = 0x46554747   # "GGUF" little-endian
DEFAULT_ALIGNMENT = 32

# GGML type -> (elements per block, bytes per block)   (gguf_types.hpp:109-142)
GGML_BLOCK = {0: (1, 4), 1: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 9: (32, 36),
              10: (256, 84), 11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 15: (256, 292),
              30: (1, 2)}
GGML_NAME = {0: "F32", 1: "F16", 2: "Q4_0", 3: "Q4_1", 6: "Q5_0", 7: "Q5_1", 8: "Q8_0", 9: "Q8_1", 10: "Q2_K", 11: "Q3_K",
             12: "Q4_K", 13: "Q5_K", 14: "Q6_K", 15: "Q8_K", 30: "BF16"}

_SCALAR = {0: "B", 1: "b", 2: "H", 3: "h", 4: "I", 5: "i", 6: "f", 7: "?", 10: "Q", 11: "q", 12: "d"}
T_STRING, T_ARRAY = 8, 9


class GGUFError(RuntimeError):
    pass


@dataclasses.dataclass
class TensorInfo:
    name: str
    dimensions: tuple[int, ...]   # innermost first: (K, N) for a weight matrix with N rows
    ggml_type: int
    offset: int                   # into the data section

    @property
    def n_elements(self) -> int:
        n = 1
        for d in self.dimensions:
            n *= d
        return n

    @property
    def nbytes(self) -> int:
        if self.ggml_type not in GGML_BLOCK:
            raise GGUFError(f"tensor {self.name}: GGML type {self.ggml_type} has no known size")
        elems, size = GGML_BLOCK[self.ggml_type]
        if self.n_elements % elems:
            raise GGUFError(f"tensor {self.name}: {self.n_elements} elements are not a multiple of the block size {elems}")
        return self.n_elements // elems * size

    @property
    def type_name(self) -> str:
        return GGML_NAME.get(self.ggml_type, f"type{self.ggml_type}")


class GGUFFile:
    def __init__(self, path: str):
        self.path = path
        self._buf = np.memmap(path, dtype=np.uint8, mode="r")
        self._pos = 0
        self._e = "<"
        magic = self._read("I")
        if magic != GGUF_MAGIC:
            if struct.unpack(">I", struct.pack("<I", magic))[0] != GGUF_MAGIC:
                raise GGUFError("Invalid GGUF magic number")
            self._e = ">"
        self.version = self._read("I")
        if self.version > 3:
            raise GGUFError(f"Unsupported GGUF version: {self.version}")
        n_tensors, n_kv = self._read("Q"), self._read("Q")
        self.metadata: dict[str, object] = {}
        for _ in range(n_kv):
            key = self._string()
            self.metadata[key] = self._value(self._read("I"))
        self.tensors: dict[str, TensorInfo] = {}
        for _ in range(n_tensors):
            name = self._string()
            nd = self._read("I")
            dims = tuple(self._read("Q") for _ in range(nd))
            t = self._read("I")
            self.tensors[name] = TensorInfo(name, dims, t, self._read("Q"))
        align = int(self.metadata.get("general.alignment", DEFAULT_ALIGNMENT))
        if align <= 0:
            raise GGUFError(f"general.alignment must be positive, got {align}")
        self.data_offset = (self._pos + align - 1) // align * align
        for info in self.tensors.values():
            if self.data_offset + info.offset + info.nbytes > self._buf.size:
                raise GGUFError(f"tensor {info.name} reaches past the end of the file")

    # -- low-level readers --
    def _read(self, fmt: str):
        size = struct.calcsize(fmt)
        if self._pos + size > self._buf.size:
            raise GGUFError("unexpected end of file")
        (v,) = struct.unpack_from(self._e + fmt, self._buf, self._pos)
        self._pos += size
        return v

    def _string(self) -> str:
        n = self._read("Q")
        if self._pos + n > self._buf.size:
            raise GGUFError("unexpected end of file in a string")
        s = bytes(self._buf[self._pos:self._pos + n]).decode("utf-8", errors="replace")
        self._pos += n
        return s

    def _value(self, t: int):
        if t in _SCALAR:
            return self._read(_SCALAR[t])
        if t == T_STRING:
            return self._string()
        if t == T_ARRAY:
            et, n = self._read("I"), self._read("Q")
            if et in _SCALAR and et != 7:
                dt = np.dtype(self._e + {"B": "u1", "b": "i1", "H": "u2", "h": "i2", "I": "u4", "i": "i4", "f": "f4",
                                         "Q": "u8", "q": "i8", "d": "f8"}[_SCALAR[et]])
                nbytes = n * dt.itemsize
                if self._pos + nbytes > self._buf.size:
                    raise GGUFError("unexpected end of file in an array")
                arr = np.frombuffer(self._buf[self._pos:self._pos + nbytes].tobytes(), dtype=dt)
                self._pos += nbytes
                return arr
            if n > self._buf.size - self._pos:   # every element takes at least one byte
                raise GGUFError("unexpected end of file in an array")
            return [self._value(et) for _ in range(n)]
        raise GGUFError(f"Unsupported metadata value type {t}")

    # -- tensors --
    def raw(self, name: str) -> np.ndarray:
        """The tensor's bytes as stored (a view into the memory map)."""
        if name not in self.tensors:
            raise GGUFError(f"Tensor not found: {name}")
        info = self.tensors[name]
        start = self.data_offset + info.offset
        return self._buf[start:start + info.nbytes]

    def upload(self, name: str, device="cuda:0"):
        """The tensor's blocks as a 1-byte device tensor (what cut_amd.ops.matmul_gguf / dequantize take)."""
        import torch
        return torch.from_numpy(np.ascontiguousarray(self.raw(name))).to(device)

    # -- hyper-parameters (llama.cpp:1082-1115 of the reference runner) --
    def model_config(self) -> dict:
        m = self.metadata
        arch = m.get("general.architecture", "llama")
        p = arch + "."
        dim, n_heads = int(m.get(p + "embedding_length", 0)), int(m.get(p + "attention.head_count", 0))
        n_layers = int(m.get(p + "block_count", 0))
        if dim == 0 or n_layers == 0 or n_heads == 0:
            raise GGUFError("Failed to read model config from GGUF metadata")
        n_kv = int(m.get(p + "attention.head_count_kv", n_heads))
        head_dim = int(m.get(p + "attention.key_length", dim // n_heads))
        return {"arch": arch, "hidden": dim, "n_layers": n_layers, "n_heads": n_heads, "n_kv_heads": n_kv,
                "head_dim": head_dim, "ffn": int(m.get(p + "feed_forward_length", 0)),
                "rope_theta": float(m.get(p + "rope.freq_base", 10000.0)),
                "eps": float(m.get(p + "attention.layer_norm_rms_epsilon", 1e-5)),
                "context_length": int(m.get(p + "context_length", 2048))}
