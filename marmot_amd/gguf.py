"""GGUF files through libmarmot_hip's reader (marmot_hip_gguf_*): the host-side counterpart of marmot_gguf_load /
marmot_gguf_find_tensor (src/graph/gguf/loader.cpp:577-770, 808-818). Tensors are views into the read-only mapping;
``GgufFile.array`` exposes one as a numpy array without copying, ``GgufFile.upload`` copies one to the device."""
import ctypes as C
from typing import Dict, List, NamedTuple, Tuple

import numpy as np

from . import capi


class GgufTensorInfo(NamedTuple):
    index: int
    name: str
    ggml_type: int
    kind: int          # capi.KIND_*, 0 for a dense tensor
    dtype: int         # capi.DT_* (6 = uint8 storage of quantized tensors)
    shape: Tuple[int, ...]
    address: int
    nbytes: int


class GgufFile:
    def __init__(self, path: str):
        self.lib = capi.load_library()
        h = C.c_void_p()
        capi.check(self.lib.marmot_hip_gguf_open(path.encode(), C.byref(h)))
        self.handle = h
        self.alignment = int(self.lib.marmot_hip_gguf_alignment(h))
        self.tensors: List[GgufTensorInfo] = []
        for i in range(self.lib.marmot_hip_gguf_tensor_count(h)):
            t = capi.GgufTensor()
            capi.check(self.lib.marmot_hip_gguf_tensor(h, i, C.byref(t)))
            self.tensors.append(self._info(i, t))
        self.by_name: Dict[str, GgufTensorInfo] = {t.name: t for t in self.tensors}

    @staticmethod
    def _info(i, t) -> GgufTensorInfo:
        return GgufTensorInfo(i, t.name.decode(), t.ggml_type, t.kind, t.dtype, tuple(t.shape[:t.ndim]), t.data, t.nbytes)

    def find(self, name: str) -> GgufTensorInfo:
        t = capi.GgufTensor()
        capi.check(self.lib.marmot_hip_gguf_find(self.handle, name.encode(), C.byref(t)))
        return self.by_name[t.name.decode()]

    # ---- key/value metadata (marmot_gguf_find_kv)
    def _value(self, kv):
        """Python value of one entry: int / float / bool / str, or a list of them for arrays."""
        def one(t, i):
            if t == 8:
                p, n = C.c_char_p(), C.c_size_t()
                capi.check(self.lib.marmot_hip_gguf_kv_string(C.byref(kv), i, C.byref(p), C.byref(n)))
                return C.string_at(p, n.value).decode()
            if t in (6, 12):
                v = C.c_double()
                capi.check(self.lib.marmot_hip_gguf_kv_float(C.byref(kv), i, C.byref(v)))
                return v.value
            v = C.c_int64()
            capi.check(self.lib.marmot_hip_gguf_kv_int(C.byref(kv), i, C.byref(v)))
            return bool(v.value) if t == 7 else v.value
        if kv.type == 9:
            return [one(kv.elem_type, i) for i in range(kv.count)]
        return one(kv.type, 0)

    def metadata(self) -> Dict[str, object]:
        """Every key of the file with its value, in file order."""
        out = {}
        for i in range(self.lib.marmot_hip_gguf_kv_count(self.handle)):
            kv = capi.GgufKv()
            capi.check(self.lib.marmot_hip_gguf_kv(self.handle, i, C.byref(kv)))
            out[kv.key.decode()] = self._value(kv)
        return out

    def get(self, key: str):
        kv = capi.GgufKv()
        capi.check(self.lib.marmot_hip_gguf_find_kv(self.handle, key.encode(), C.byref(kv)))
        return self._value(kv)

    def array(self, info: GgufTensorInfo) -> np.ndarray:
        """The tensor's bytes inside the mapping (no copy; valid until close): uint8 block bytes for quantized
        tensors, else the dense values in the file's dimension order."""
        buf = (C.c_uint8 * info.nbytes).from_address(info.address)
        raw = np.frombuffer(buf, dtype=np.uint8)
        if info.kind != 0:
            return raw
        np_dt = {capi.DT_F32: np.float32, capi.DT_F16: np.float16, capi.DT_I32: np.int32}[info.dtype]
        shape = info.shape if len(info.shape) == 2 else tuple(reversed(info.shape))
        return raw.view(np_dt).reshape(shape)

    def upload(self, backend, info: GgufTensorInfo):
        """Device copy of one tensor (a DeviceBuffer owned by the caller)."""
        from .backend import DeviceBuffer

        p = C.c_void_p()
        capi.check(self.lib.marmot_hip_gguf_upload(backend.dev, self.handle, info.index, C.byref(p)))
        buf = DeviceBuffer.__new__(DeviceBuffer)
        buf.backend, buf.nbytes, buf.ptr = backend, info.nbytes, p.value
        return buf

    def close(self):
        if self.handle:
            self.lib.marmot_hip_gguf_close(self.handle)
            self.handle = C.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
