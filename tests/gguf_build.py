"""Writes small GGUF v3 files for the ingest tests: a byte-level writer that follows the published layout
(magic, version, counts, key-value pairs, tensor records, aligned data section), independent of the parser
under test.  Tensor payloads are whatever bytes the caller passes."""
from __future__ import annotations

import struct
from typing import List, Optional, Sequence, Tuple

F32, F16, Q4_0, Q8_0, Q4K, Q5K, Q6K, BF16 = 0, 1, 2, 8, 12, 13, 14, 30
BLOCK = {F32: (1, 4), F16: (1, 2), Q4_0: (32, 18), Q8_0: (32, 34), Q4K: (256, 144), Q5K: (256, 176), Q6K: (256, 210),
         BF16: (1, 2)}
T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STRING, T_ARRAY, T_U64, T_I64, T_F64 = range(13)
_FMT = {T_U8: "<B", T_I8: "<b", T_U16: "<H", T_I16: "<h", T_U32: "<I", T_I32: "<i", T_F32: "<f", T_BOOL: "<B",
        T_U64: "<Q", T_I64: "<q", T_F64: "<d"}


def gstring(s) -> bytes:
    b = s if isinstance(s, bytes) else s.encode()
    return struct.pack("<Q", len(b)) + b


class GgufWriter:
    def __init__(self, version: int = 3, magic: bytes = b"GGUF"):
        self.version, self.magic = version, magic
        self.kvs: List[bytes] = []
        self.tensors: List[Tuple[str, Sequence[int], int, Optional[bytes], Optional[int]]] = []
        self.alignment = 32

    def kv(self, key: str, tag: int, value) -> "GgufWriter":
        body = gstring(value) if tag == T_STRING else struct.pack(_FMT[tag], value)
        self.kvs.append(gstring(key) + struct.pack("<i", tag) + body)
        if key == "general.alignment" and tag == T_U32:
            self.alignment = value
        return self

    def kv_array(self, key: str, elem_tag: int, values) -> "GgufWriter":
        body = b"".join(gstring(v) if elem_tag == T_STRING else struct.pack(_FMT[elem_tag], v) for v in values)
        self.kvs.append(gstring(key) + struct.pack("<iiQ", T_ARRAY, elem_tag, len(values)) + body)
        return self

    def kv_raw(self, raw: bytes) -> "GgufWriter":
        self.kvs.append(raw)
        return self

    def tensor(self, name: str, dims: Sequence[int], ggml_type: int, data: Optional[bytes] = None,
               offset: Optional[int] = None) -> "GgufWriter":
        """data=None writes zeros of the right size; offset overrides the computed position."""
        self.tensors.append((name, tuple(dims), ggml_type, data, offset))
        return self

    def build(self, n_tensors: Optional[int] = None, n_kv: Optional[int] = None, pad_data: bool = True) -> bytes:
        head = self.magic + struct.pack("<Iqq", self.version, len(self.tensors) if n_tensors is None else n_tensors,
                                        len(self.kvs) if n_kv is None else n_kv)
        head += b"".join(self.kvs)
        records, blobs, pos = b"", [], 0
        a = max(self.alignment, 1)
        for name, dims, ty, data, offset in self.tensors:
            n = 1
            for d in dims:
                n *= d
            be, bb = BLOCK.get(ty, (1, 1))
            size = len(data) if data is not None else (n // be) * bb
            off = pos if offset is None else offset
            records += gstring(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<q", d) for d in dims)
            records += struct.pack("<iQ", ty, off)
            blobs.append((off, data if data is not None else bytes(size)))
            pos = (off + size + a - 1) // a * a
        meta = head + records
        out = bytearray(meta)
        if pad_data and blobs:
            start = (len(meta) + a - 1) // a * a
            end = max(off + len(b) for off, b in blobs)
            out += bytes(start - len(meta)) + bytes(end)
            for off, b in blobs:
                out[start + off:start + off + len(b)] = b
        return bytes(out)
