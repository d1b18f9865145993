"""Host-side mirror of the reference's GGUF reader (ms::Gguf, src/gguf/gguf.hpp:38-96) and expert layout
(ms::ExpertLayout::from_gguf, src/store/experts.hpp:35-42) over the C ABI, plus resident placement of a layer's experts
in HBM. Parsing is host code inside libmsq.so; there is no Python fallback parser.
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import MsqExpertLayout, MsqExpertSlot, MsqGgufTensor
from .quant import Buffer, _bp, _check

KV_TYPES = ("u8", "i8", "u16", "i16", "u32", "i32", "f32", "bool", "str", "arr", "u64", "i64", "f64")  # gguf.hpp:24


def type_bytes(ggml_type, n_elems):  # reference: ms::type_bytes
    return _lib.load().msq_gguf_type_bytes(int(ggml_type), int(n_elems))


def type_name(ggml_type):  # reference: ms::type_name
    return _lib.load().msq_gguf_type_name(int(ggml_type)).decode()


def expand_splits_count(path):  # reference: Gguf::expand_splits(path).size()
    return _lib.load().msq_gguf_split_count_of_path(path.encode())


class TensorInfo:  # reference: ms::TensorInfo
    def __init__(self, index, t):
        self.index, self.name, self.type, self.n_dims = index, t.name.decode(), t.type, t.n_dims
        self.ne = list(t.ne)
        self.nbytes, self.split, self.offset = t.nbytes, t.split, t.offset

    def row_bytes(self):
        return type_bytes(self.type, self.ne[0])


class Gguf:
    def __init__(self, path):
        self._h = None
        self._L = _lib.load()
        h = C.c_void_p()
        _check(self._L.msq_gguf_open(path.encode(), C.byref(h)))
        self._h = h

    def close(self):
        if self._h:
            self._L.msq_gguf_close(self._h)
            self._h = None

    def __del__(self):
        self.close()

    # ---- file facts
    def n_splits(self):
        return self._L.msq_gguf_n_splits(self._h)

    def alignment(self):
        return self._L.msq_gguf_alignment(self._h)

    def version(self):
        return self._L.msq_gguf_version(self._h)

    def path(self, split):
        return self._L.msq_gguf_split_path(self._h, split).decode()

    def data_offset(self, split):
        return self._L.msq_gguf_data_offset(self._h, split)

    # ---- metadata
    def keys(self):
        return [self._L.msq_gguf_key(self._h, i).decode() for i in range(self._L.msq_gguf_n_kv(self._h))]

    def kv_type(self, key):
        """(type name, element type name or None), or None when the key is missing."""
        at = C.c_int(-1)
        t = self._L.msq_gguf_kv_type(self._h, key.encode(), C.byref(at))
        return None if t < 0 else (KV_TYPES[t], KV_TYPES[at.value] if at.value >= 0 else None)

    def get_i64(self, key, dflt=0):
        return self._L.msq_gguf_get_i64(self._h, key.encode(), dflt)

    def get_f64(self, key, dflt=0.0):
        return self._L.msq_gguf_get_f64(self._h, key.encode(), dflt)

    def get_str(self, key, dflt=""):
        r = self._L.msq_gguf_get_str(self._h, key.encode(), None)
        return dflt if r is None else r.decode()

    def arr_len(self, key):
        return self._L.msq_gguf_arr_len(self._h, key.encode())

    def get_arr_i64(self, key):
        n = max(0, self.arr_len(key))
        out = np.zeros(n, dtype=np.int64)
        got = self._L.msq_gguf_arr_i64(self._h, key.encode(), out.ctypes.data, n) if n else 0
        return out[:max(0, got)]

    def get_arr_f32(self, key):
        n = max(0, self.arr_len(key))
        out = np.zeros(n, dtype=np.float64)
        got = self._L.msq_gguf_arr_f64(self._h, key.encode(), out.ctypes.data, n) if n else 0
        return out[:max(0, got)].astype(np.float32)

    def get_arr_str(self, key):
        n = max(0, self.arr_len(key))
        out = []
        for i in range(n):
            s = self._L.msq_gguf_arr_str(self._h, key.encode(), i)
            if s is None:
                break
            out.append(s.decode())
        return out

    def get_arr_nested_i64(self, key):
        out = []
        for i in range(max(0, self.arr_len(key))):
            n = self._L.msq_gguf_arr_nested_i64(self._h, key.encode(), i, None, 0)
            v = np.zeros(max(0, n), dtype=np.int64)
            if n > 0:
                self._L.msq_gguf_arr_nested_i64(self._h, key.encode(), i, v.ctypes.data, n)
            out.append(v)
        return out

    # ---- tensors
    def tensors(self):
        return [self.tensor(i) for i in range(self._L.msq_gguf_n_tensors(self._h))]

    def tensor(self, index):
        t = MsqGgufTensor()
        _check(self._L.msq_gguf_tensor(self._h, index, C.byref(t)))
        return TensorInfo(index, t)

    def find(self, name):
        i = self._L.msq_gguf_find(self._h, name.encode())
        return None if i < 0 else self.tensor(i)

    def read(self, tensor, byte_off=0, length=None):
        """Bytes of a tensor's data as a numpy uint8 array (host)."""
        t = tensor if isinstance(tensor, TensorInfo) else self.tensor(tensor)
        n = t.nbytes - byte_off if length is None else length
        out = np.empty(n, dtype=np.uint8)
        got = self._L.msq_gguf_read(self._h, t.index, byte_off, out.ctypes.data, n)
        if got != n:
            raise IOError("gguf: short read of %s" % t.name)
        return out

    def load_tensor(self, e, tensor, dst, byte_off=0, length=None):
        t = tensor if isinstance(tensor, TensorInfo) else self.tensor(tensor)
        _check(self._L.msq_gguf_load_tensor(e.handle, self._h, t.index, byte_off, t.nbytes - byte_off if length is None else length, _bp(dst)))

    # ---- experts
    def expert_layout(self, layer):
        L = MsqExpertLayout()
        _check(self._L.msq_gguf_expert_layout(self._h, layer, C.byref(L)))
        return L

    def place_experts(self, e, layer, arena):
        """Copies the layer's experts into `arena` (a Buffer of at least expert_layout(layer).arena_bytes, 256-byte
        aligned) and returns (layout, ctypes array of MsqExpertSlot views)."""
        L = self.expert_layout(layer)
        slots = (MsqExpertSlot * L.n_experts)()
        _check(self._L.msq_gguf_place_experts(e.handle, self._h, layer, _bp(arena), slots, L.n_experts))
        return L, slots


def slot_buffers(slot, owner=None):
    """(gate, up, down) Buffers of an MsqExpertSlot."""
    return tuple(Buffer(b.dev, b.off, b.size, owner) for b in (slot.gate, slot.up, slot.down))
