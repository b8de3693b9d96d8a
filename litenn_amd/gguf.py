"""Front end of the library's GGUF container reader (the counterpart of ImportGGUFArchive and
ParseLLaMAHyperparameters, tools/gguf/GGUFImporter.cpp:505-678).  Parsing happens in the library;
this module only wraps the C ABI."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import _lib
from ._lib import GgufTensor, LlamaParams, check


@dataclass
class TensorInfo:
    name: str
    ggml_type: int
    fmt: int        # QuantizedBlockFormat the backend executes, or -1
    dtype: int      # DataType of a plain tensor, or -1
    quantized: bool
    shape: tuple    # slowest dimension first ([N, K] for a weight)
    file_offset: int
    bytes: int


class GGUFFile:
    def __init__(self, path: str):
        self._h = C.c_void_p()
        check(_lib.load().litenn_gguf_open(str(path).encode(), C.byref(self._h)))

    def close(self) -> None:
        if self._h:
            _lib.load().litenn_gguf_close(self._h)
            self._h = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def version(self) -> int:
        return _lib.load().litenn_gguf_version(self._h)

    @property
    def tensor_count(self) -> int:
        return _lib.load().litenn_gguf_tensor_count(self._h)

    @property
    def metadata_count(self) -> int:
        return _lib.load().litenn_gguf_metadata_count(self._h)

    @staticmethod
    def _info(t: GgufTensor) -> TensorInfo:
        return TensorInfo(t.name.decode(), t.ggml_type, t.fmt, t.dtype, bool(t.quantized),
                          tuple(t.shape[i] for i in range(t.rank)), t.file_offset, t.bytes)

    def tensor(self, key) -> TensorInfo:
        t = GgufTensor()
        if isinstance(key, int):
            check(_lib.load().litenn_gguf_tensor_info(self._h, key, C.byref(t)))
        else:
            check(_lib.load().litenn_gguf_find_tensor(self._h, str(key).encode(), C.byref(t)))
        return self._info(t)

    def payload(self, key) -> np.ndarray:
        """The raw bytes of a tensor (a copy)."""
        t = GgufTensor()
        if isinstance(key, int):
            check(_lib.load().litenn_gguf_tensor_info(self._h, key, C.byref(t)))
        else:
            check(_lib.load().litenn_gguf_find_tensor(self._h, str(key).encode(), C.byref(t)))
        return np.ctypeslib.as_array(C.cast(t.data, C.POINTER(C.c_uint8)), shape=(t.bytes,)).copy()

    def tensors(self):
        return [self.tensor(i) for i in range(self.tensor_count)]

    def keys(self):
        return [_lib.load().litenn_gguf_metadata_key(self._h, i).decode() for i in range(self.metadata_count)]

    def get_size(self, key: str) -> int:
        v = C.c_uint64()
        check(_lib.load().litenn_gguf_metadata_u64(self._h, key.encode(), C.byref(v)))
        return v.value

    def get_double(self, key: str) -> float:
        v = C.c_double()
        check(_lib.load().litenn_gguf_metadata_f64(self._h, key.encode(), C.byref(v)))
        return v.value

    def get_string(self, key: str) -> str:
        v = C.c_char_p()
        check(_lib.load().litenn_gguf_metadata_str(self._h, key.encode(), C.byref(v)))
        return v.value.decode()

    def get_bool(self, key: str) -> bool:
        v = C.c_int()
        check(_lib.load().litenn_gguf_metadata_bool(self._h, key.encode(), C.byref(v)))
        return bool(v.value)

    def get_array_info(self, key: str):
        """(element type id of the container format, element count)."""
        et, n = C.c_uint(), C.c_size_t()
        check(_lib.load().litenn_gguf_metadata_array(self._h, key.encode(), C.byref(et), C.byref(n)))
        return et.value, n.value

    def llama_params(self) -> LlamaParams:
        p = LlamaParams()
        check(_lib.load().litenn_gguf_llama_params(self._h, C.byref(p)))
        return p
