"""GGUF v3 container: host-side mirror of the reference's src/gguf (GgufFile, TensorInfo,
MetaValue) over the C ABI.  The file stays a read-only mapping inside librein.so; what this
module hands out are views into it, valid until close()."""
import ctypes as C
import struct

import numpy as np

from . import _lib
from ._lib import GgufDims, GgufTensor, ReinError, check

# gguf_metadata_value_type (src/gguf/types.rs:108-113)
U8, I8, U16, I16, U32, I32, F32, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)
_FIXED = {U8: "<u1", I8: "<i1", U16: "<u2", I16: "<i2", U32: "<u4", I32: "<i4", F32: "<f4", BOOL: "<u1",
          U64: "<u8", I64: "<i8", F64: "<f8"}


def align_up(v, align):
    """align_up (src/gguf/mod.rs:208-210)"""
    return _lib.load().rein_gguf_align_up(v, align)


class TensorInfo:
    """TensorInfo (src/gguf/tensor_info.rs:7-32)"""

    def __init__(self, t):
        self.name = t.name.decode()
        self.ggml_type = t.ggml_type
        self.shape = tuple(int(t.dims[d]) for d in range(t.n_dims))
        self.offset = int(t.offset)
        self.byte_size = int(t.byte_size)
        self._data = t.data

    @property
    def n_elements(self):
        n = 1
        for d in self.shape:
            n *= d
        return n

    def __repr__(self):
        return f"TensorInfo({self.name!r}, type={self.ggml_type}, shape={self.shape}, offset={self.offset})"


class GgufFile:
    """GgufFile (src/gguf/mod.rs:53-205).  `GgufFile.open(path)` maps a file, `GgufFile.from_bytes(b)`
    parses a buffer this object keeps alive."""

    def __init__(self, handle, keep=None):
        self._lib = _lib.load()
        self._h = handle
        self._keep = keep
        ver, nt, nkv, al, off = C.c_uint32(), C.c_uint64(), C.c_uint64(), C.c_uint64(), C.c_uint64()
        check(self._lib.rein_gguf_header(handle, C.byref(ver), C.byref(nt), C.byref(nkv), C.byref(al), C.byref(off)))
        self.header = {"version": ver.value, "tensor_count": nt.value, "metadata_kv_count": nkv.value}
        self.alignment, self.data_section_offset = al.value, off.value
        self.tensors = []
        t = GgufTensor()
        for i in range(nt.value):
            check(self._lib.rein_gguf_tensor_at(handle, i, C.byref(t)))
            self.tensors.append(TensorInfo(t))

    @classmethod
    def open(cls, path):
        h = C.c_void_p()
        check(_lib.load().rein_gguf_open(str(path).encode(), C.byref(h)))
        return cls(h)

    @classmethod
    def from_bytes(cls, data):
        buf = np.frombuffer(bytes(data), np.uint8)
        h = C.c_void_p()
        check(_lib.load().rein_gguf_from_bytes(buf.ctypes.data, buf.size, C.byref(h)))
        return cls(h, keep=buf)

    def close(self):
        if self._h:
            self._lib.rein_gguf_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ---- tensors
    def tensor(self, name):
        """GgufFile::tensor (mod.rs:186-188): None when absent"""
        t = GgufTensor()
        rc = self._lib.rein_gguf_tensor_by_name(self._h, name.encode(), C.byref(t))
        if rc == -8:
            return None
        check(rc)
        return TensorInfo(t)

    def tensor_data(self, name):
        """GgufFile::tensor_data (mod.rs:196-201): a uint8 view into the mapping, None when absent"""
        info = self.tensor(name)
        if info is None:
            return None
        if info.byte_size == 0:
            return np.empty(0, np.uint8)
        return np.ctypeslib.as_array(C.cast(info._data, C.POINTER(C.c_uint8)), shape=(info.byte_size,))

    def load_for_matvec(self, name):
        """GpuMatvecTensor::from_gguf_matvec / GpuExpertTensor::from_gguf (src/runtime/qwen35.rs:235-245,
        397-431): (repacked bytes, kernel format id, dims dict)"""
        fmt, dims = C.c_int(0), GgufDims()
        check(self._lib.rein_gguf_load_for_matvec(self._h, name.encode(), None, 0, C.byref(fmt), C.byref(dims)))
        out = np.empty(dims.bytes_per_expert * dims.n_expert, np.uint8)
        check(self._lib.rein_gguf_load_for_matvec(self._h, name.encode(), out.ctypes.data, out.size, C.byref(fmt),
                                                  C.byref(dims)))
        return out, fmt.value, {"in_dim": dims.in_dim, "out_dim": dims.out_dim, "n_expert": dims.n_expert,
                                "bytes_per_expert": dims.bytes_per_expert}

    # ---- metadata
    def metadata_keys(self):
        key, vt = C.c_char_p(), C.c_int()
        out = []
        for i in range(self.header["metadata_kv_count"]):
            check(self._lib.rein_gguf_meta_at(self._h, i, C.byref(key), C.byref(vt)))
            out.append((key.value.decode(), vt.value))
        return out

    def metadata_type(self, key):
        vt = C.c_int()
        rc = self._lib.rein_gguf_meta_type(self._h, key.encode(), C.byref(vt))
        if rc == -8:
            return None
        check(rc)
        return vt.value

    def metadata_get(self, key):
        """GgufFile::metadata_get (mod.rs:181-183) decoded to a Python value: int, float, bool, str,
        numpy array (fixed-width arrays) or list of str; None when absent"""
        vt = self.metadata_type(key)
        if vt is None:
            return None
        k = key.encode()
        if vt == ARRAY:
            return self._decode_array(k)
        p = C.c_void_p()
        check(self._lib.rein_gguf_meta_raw(self._h, k, None, C.byref(p)))
        if vt == STRING:
            (ln,) = struct.unpack("<Q", C.string_at(p, 8))
            return C.string_at(p.value + 8, ln).decode()
        dt = np.dtype(_FIXED[vt])
        v = np.frombuffer(C.string_at(p, dt.itemsize), dt)[0]
        return bool(v) if vt == BOOL else v.item()

    def as_u64(self, key):
        """MetaValue::as_u64 (src/gguf/value.rs:69-81): None when absent, negative or not an integer"""
        v = C.c_uint64()
        return v.value if self._lib.rein_gguf_meta_u64(self._h, key.encode(), C.byref(v)) == 0 else None

    def as_f32(self, key):
        """MetaValue::as_f32 (value.rs:88-94)"""
        v = C.c_float()
        return v.value if self._lib.rein_gguf_meta_f32(self._h, key.encode(), C.byref(v)) == 0 else None

    def _decode_array(self, k):
        et, n, first = C.c_int(), C.c_uint64(), C.c_void_p()
        check(self._lib.rein_gguf_meta_array(self._h, k, C.byref(et), C.byref(n), C.byref(first)))
        if et.value in _FIXED:
            dt = np.dtype(_FIXED[et.value])
            arr = np.frombuffer(C.string_at(first, n.value * dt.itemsize), dt)
            return arr.astype(bool) if et.value == BOOL else arr
        if et.value == STRING:
            out, at = [], first.value
            for _ in range(n.value):
                (ln,) = struct.unpack("<Q", C.string_at(at, 8))
                out.append(C.string_at(at + 8, ln).decode())
                at += 8 + ln
            return out
        raise ReinError(-2, "nested metadata arrays are validated and skipped, not decoded")
