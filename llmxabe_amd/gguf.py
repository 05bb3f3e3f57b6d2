"""Mirror of `xabe_gguf::{GgufFile, TensorInfo, GgmlType, GgufError}` (crates/xabe-gguf/src/{file,tensor,types,
error}.rs) and of the layer uploads `MoeLayerWeights::upload` (crates/xabe-engine/src/block/moe.rs:660-756) and
`DenseFfnLayerWeights::upload` (crates/xabe-engine/src/block/dense_ffn.rs:663-760).  Parsing, bounds checks and
the uploads live in the library (csrc/gguf.hip); these classes hold the handles."""
from __future__ import annotations

import ctypes as C
import enum
import os
from dataclasses import dataclass
from typing import List, Optional, Tuple

from . import _ffi
from ._ffi import TensorInfoC
from .moe import ExpertQuant, MoeError, MoeGeometry, _ERRORS, _stream, check


# ---------------------------------------------------------------- errors (error.rs:11-108, block/moe.rs:494-547)
class MissingTensor(MoeError): status = 13
class UnsupportedDenseType(MoeError): status = 14
class ShapeMismatch(MoeError): status = 15


class GgufError(MoeError):
    pass


class BadMagic(GgufError): status = 20
class UnsupportedVersion(GgufError): status = 21
class UnexpectedEof(GgufError): status = 22
class InvalidUtf8(GgufError): status = 23
class NegativeCount(GgufError): status = 24
class DuplicateKey(GgufError): status = 25
class UnknownValueType(GgufError): status = 26
class NestedArray(GgufError): status = 27
class BadAlignmentType(GgufError): status = 28
class BadAlignment(GgufError): status = 29
class TooManyDimensions(GgufError): status = 30
class ZeroDimension(GgufError): status = 31
class DuplicateTensor(GgufError): status = 32
class UnsupportedGgmlType(GgufError): status = 33
class UnalignedElementCount(GgufError): status = 34
class OffsetOverflow(GgufError): status = 35
class TensorOutOfBounds(GgufError): status = 36
class Io(GgufError): status = 37


for _c in (MissingTensor, UnsupportedDenseType, ShapeMismatch, BadMagic, UnsupportedVersion, UnexpectedEof, InvalidUtf8,
           NegativeCount, DuplicateKey, UnknownValueType, NestedArray, BadAlignmentType, BadAlignment, TooManyDimensions,
           ZeroDimension, DuplicateTensor, UnsupportedGgmlType, UnalignedElementCount, OffsetOverflow, TensorOutOfBounds,
           Io):
    _ERRORS[_c.status] = _c


class GgmlType(enum.IntEnum):
    """`enum ggml_type` ids (types.rs:38-60)."""
    F32 = 0
    F16 = 1
    Q4_0 = 2
    Q8_0 = 8
    Q4K = 12
    Q5K = 13
    Q6K = 14
    Bf16 = 30

    def block_size(self) -> int: return _ffi.lib().xabe_ggml_type_block_size(int(self))
    def type_size(self) -> int: return _ffi.lib().xabe_ggml_type_size(int(self))
    def type_name(self) -> str: return _ffi.lib().xabe_ggml_type_name(int(self)).decode()

    def bytes_for_elements(self, n: int) -> int:
        out = C.c_uint64(0)
        check(_ffi.lib().xabe_ggml_type_bytes_for_elements(int(self), n, C.byref(out)))
        return out.value

    @staticmethod
    def try_from(raw: int) -> "GgmlType":
        if _ffi.lib().xabe_ggml_type_block_size(raw) == 0:
            raise UnsupportedGgmlType(f"unsupported ggml tensor type id {raw}")
        return GgmlType(raw)


@dataclass(frozen=True)
class TensorInfo:
    """tensor.rs:11-28.  `dims[0]` is the innermost dimension; `offset` is relative to the data section."""
    name: str
    dims: Tuple[int, ...]
    ggml_type: GgmlType
    offset: int
    n_elements: int
    n_bytes: int


def _info(c: TensorInfoC) -> TensorInfo:
    return TensorInfo(c.name.decode(), tuple(c.dims[i] for i in range(c.n_dims)), GgmlType(c.ggml_type), c.offset,
                      c.n_elements, c.n_bytes)


_ARRAY_CTYPES = {0: C.c_uint8, 1: C.c_int8, 2: C.c_uint16, 3: C.c_int16, 4: C.c_uint32, 5: C.c_int32, 6: C.c_float,
                 7: C.c_uint8, 10: C.c_uint64, 11: C.c_int64, 12: C.c_double}


class GgufFile:
    """A parsed GGUF v3 file (file.rs:66-270).  `open` memory-maps; tensor bytes are never copied on the host."""

    def __init__(self, handle: int):
        self._h = handle

    @staticmethod
    def open(path) -> "GgufFile":
        h = C.c_void_p()
        check(_ffi.lib().xabe_gguf_open(os.fsencode(path), C.byref(h)))
        return GgufFile(h.value)

    @staticmethod
    def from_bytes(data: bytes) -> "GgufFile":
        h = C.c_void_p()
        buf = (C.c_char * len(data)).from_buffer_copy(data) if data else None
        check(_ffi.lib().xabe_gguf_from_bytes(C.cast(buf, C.c_void_p) if buf is not None else None, len(data), C.byref(h)))
        return GgufFile(h.value)

    def close(self):
        if getattr(self, "_h", None):
            _ffi.lib().xabe_gguf_close(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:  # interpreter shutdown
            pass

    def version(self) -> int: return _ffi.lib().xabe_gguf_version(self._h)
    def alignment(self) -> int: return _ffi.lib().xabe_gguf_alignment(self._h)
    def n_kv(self) -> int: return _ffi.lib().xabe_gguf_n_kv(self._h)
    def n_tensors(self) -> int: return _ffi.lib().xabe_gguf_n_tensors(self._h)
    def data_offset(self) -> int: return _ffi.lib().xabe_gguf_data_offset(self._h)

    def tensors(self) -> List[TensorInfo]:
        out = []
        for i in range(self.n_tensors()):
            c = TensorInfoC()
            check(_ffi.lib().xabe_gguf_tensor_at(self._h, i, C.byref(c)))
            out.append(_info(c))
        return out

    def tensor(self, name: str) -> Optional[TensorInfo]:
        c = TensorInfoC()
        if _ffi.lib().xabe_gguf_tensor(self._h, name.encode(), C.byref(c)) != 0:
            return None
        return _info(c)

    def tensor_bytes(self, name: str) -> Optional[memoryview]:
        """Read-only view of the tensor's bytes inside the mapping (valid while the file is open)."""
        n = C.c_size_t(0)
        p = _ffi.lib().xabe_gguf_tensor_bytes(self._h, name.encode(), C.byref(n))
        if not p:
            return None
        return memoryview((C.c_uint8 * n.value).from_address(p)).toreadonly()

    def metadata_keys(self) -> List[str]:
        return [_ffi.lib().xabe_gguf_key_at(self._h, i).decode() for i in range(self.n_kv())]

    def get_u32(self, key: str) -> Optional[int]:
        v = C.c_uint32(0)
        return v.value if _ffi.lib().xabe_gguf_get_u32(self._h, key.encode(), C.byref(v)) else None

    def get_u64(self, key: str) -> Optional[int]:
        v = C.c_uint64(0)
        return v.value if _ffi.lib().xabe_gguf_get_u64(self._h, key.encode(), C.byref(v)) else None

    def get_f32(self, key: str) -> Optional[float]:
        v = C.c_float(0)
        return v.value if _ffi.lib().xabe_gguf_get_f32(self._h, key.encode(), C.byref(v)) else None

    def get_str(self, key: str) -> Optional[str]:
        n = C.c_size_t(0)
        p = _ffi.lib().xabe_gguf_get_str(self._h, key.encode(), C.byref(n))
        return C.string_at(p, n.value).decode() if p else None

    def value_type(self, key: str) -> Optional[Tuple[int, int, int]]:
        """(type tag, element tag, count) of a key's value; None when absent."""
        t, e, n = C.c_int(0), C.c_int(0), C.c_uint64(0)
        if not _ffi.lib().xabe_gguf_value_type_of(self._h, key.encode(), C.byref(t), C.byref(e), C.byref(n)):
            return None
        return t.value, e.value, n.value

    def _array(self, key: str, elem_type: int):
        n = C.c_uint64(0)
        p = _ffi.lib().xabe_gguf_get_array(self._h, key.encode(), elem_type, C.byref(n))
        if not p:
            return None
        return list((_ARRAY_CTYPES[elem_type] * n.value).from_address(p))

    def get_i32_array(self, key: str): return self._array(key, 5)
    def get_u32_array(self, key: str): return self._array(key, 4)
    def get_f32_array(self, key: str): return self._array(key, 6)

    def get_bool_array(self, key: str):
        v = self._array(key, 7)
        return None if v is None else [bool(b) for b in v]

    def get_string_array(self, key: str) -> Optional[List[str]]:
        t = self.value_type(key)
        if t is None or t[0] != 9 or t[1] != 8:
            return None
        out = []
        for i in range(t[2]):
            n = C.c_size_t(0)
            p = _ffi.lib().xabe_gguf_get_string_array_item(self._h, key.encode(), i, C.byref(n))
            out.append(C.string_at(p, n.value).decode())
        return out


class UploadedMoeLayer:
    """One layer's MoE tensors on the device, in the formats the file holds (block/moe.rs:634-800).
    Passed to `MoeBlock.forward` in place of a `MoeLayerWeights`."""

    def __init__(self, handle: int):
        self._h = handle

    @staticmethod
    def upload(file: GgufFile, layer: int, geometry: MoeGeometry) -> "UploadedMoeLayer":
        h = C.c_void_p()
        check(_ffi.lib().xabe_moe_layer_upload(_stream(), file._h, layer, C.byref(geometry._c()), C.byref(h)))
        return UploadedMoeLayer(h.value)

    def __del__(self):
        if getattr(self, "_h", None):
            try:
                _ffi.lib().xabe_moe_layer_free(self._h)
            except Exception:  # interpreter shutdown
                pass
            self._h = None

    def _c(self):
        return _ffi.lib().xabe_moe_layer_weights_of(self._h).contents

    def layer(self) -> int: return _ffi.lib().xabe_moe_layer_index(self._h)
    def bytes(self) -> int: return _ffi.lib().xabe_moe_layer_bytes(self._h)

    def _triple(self, fn, n=3):
        out = (C.c_int * n)()
        check(getattr(_ffi.lib(), fn)(self._h, C.byref(out)))
        return list(out)

    def expert_quants(self): return [ExpertQuant(q) for q in self._triple("xabe_moe_layer_expert_quants")]
    def shared_quants(self): return [ExpertQuant(q) for q in self._triple("xabe_moe_layer_shared_quants")]
    def router_types(self): return tuple(GgmlType(t) for t in self._triple("xabe_moe_layer_router_types", 2))


class UploadedDenseFfnLayer:
    """One layer's dense feed-forward tensors on the device (dense_ffn.rs:628-760, quantized residency)."""

    def __init__(self, handle: int):
        self._h = handle

    @staticmethod
    def upload(file: GgufFile, layer: int, hidden: int, intermediate: int) -> "UploadedDenseFfnLayer":
        h = C.c_void_p()
        check(_ffi.lib().xabe_dense_ffn_layer_upload(_stream(), file._h, layer, hidden, intermediate, C.byref(h)))
        return UploadedDenseFfnLayer(h.value)

    def __del__(self):
        if getattr(self, "_h", None):
            try:
                _ffi.lib().xabe_dense_ffn_layer_free(self._h)
            except Exception:  # interpreter shutdown
                pass
            self._h = None

    def _c(self):
        return _ffi.lib().xabe_dense_ffn_layer_weights_of(self._h).contents

    def bytes(self) -> int: return _ffi.lib().xabe_dense_ffn_layer_bytes(self._h)

    def quants(self):
        out = (C.c_int * 3)()
        check(_ffi.lib().xabe_dense_ffn_layer_quants(self._h, C.byref(out)))
        return [ExpertQuant(q) for q in out]
