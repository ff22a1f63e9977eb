"""GGUF files through the library's reader (``ogm_gguf_*``): header, metadata, tensor table and the
2-D matrix view (src/gguf.rs:149-280 and engine/loader.rs:1552-1580 of orangu)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import capi
from .capi import OgmError


class GgufFile:
    def __init__(self, path: str | None = None, *, data: bytes | None = None, offset: int = 0):
        self._lib = capi.load_library()
        self._h = C.c_void_p()
        err = C.create_string_buffer(512)
        if data is not None:
            self._keep = (C.c_char * len(data)).from_buffer_copy(data)
            rc = self._lib.ogm_gguf_parse(self._keep, len(data), C.byref(self._h), err, len(err))
        else:
            rc = self._lib.ogm_gguf_open(str(path).encode(), offset, C.byref(self._h), err, len(err))
        if rc != 0:
            raise OgmError(rc, "ogm_gguf_open", err.value.decode(errors="replace"))
        v, a, d, nt, nm = C.c_uint32(), C.c_uint64(), C.c_uint64(), C.c_uint64(), C.c_uint64()
        self._lib.ogm_gguf_info(self._h, C.byref(v), C.byref(a), C.byref(d), C.byref(nt), C.byref(nm))
        self.version, self.alignment, self.data_offset = v.value, a.value, d.value
        self.n_tensors, self.n_metadata = nt.value, nm.value

    def _fail(self, rc, where):
        raise OgmError(rc, where, self._lib.ogm_gguf_last_error(self._h).decode(errors="replace"))

    def meta_u64(self, key: str):
        out = C.c_uint64()
        return out.value if self._lib.ogm_gguf_meta_u64(self._h, key.encode(), C.byref(out)) == 0 else None

    def meta_f64(self, key: str):
        out = C.c_double()
        return out.value if self._lib.ogm_gguf_meta_f64(self._h, key.encode(), C.byref(out)) == 0 else None

    def meta_string(self, key: str):
        out, n = C.c_char_p(), C.c_size_t()
        if self._lib.ogm_gguf_meta_string(self._h, key.encode(), C.byref(out), C.byref(n)) != 0:
            return None
        return C.string_at(out, n.value).decode(errors="replace")

    def meta_array(self, key: str):
        t, n = C.c_uint32(), C.c_uint64()
        if self._lib.ogm_gguf_meta_array(self._h, key.encode(), C.byref(t), C.byref(n)) != 0:
            return None
        return t.value, n.value

    def tensor(self, index: int):
        name, nd, dims, t, off = C.c_char_p(), C.c_uint32(), (C.c_uint64 * 8)(), C.c_uint32(), C.c_uint64()
        rc = self._lib.ogm_gguf_tensor(self._h, index, C.byref(name), C.byref(nd), dims, C.byref(t), C.byref(off))
        if rc != 0:
            self._fail(rc, "ogm_gguf_tensor")
        return name.value.decode(errors="replace"), list(dims[:nd.value]), t.value, off.value   # (from_utf8_lossy, gguf.rs:384)

    def find_tensor(self, name: str) -> int:
        return self._lib.ogm_gguf_find_tensor(self._h, name.encode())

    def tensor_data(self, index: int) -> np.ndarray:
        p, n = C.c_void_p(), C.c_uint64()
        rc = self._lib.ogm_gguf_tensor_data(self._h, index, C.byref(p), C.byref(n))
        if rc != 0:
            self._fail(rc, "ogm_gguf_tensor_data")
        return np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), shape=(n.value,)).copy()

    def matrix(self, name: str):
        """(ggml_type, in_dim, out_dim, row_bytes, raw bytes) of a 2-D tensor."""
        t, i, o, rb, p = C.c_uint32(), C.c_uint32(), C.c_uint32(), C.c_size_t(), C.c_void_p()
        rc = self._lib.ogm_gguf_matrix(self._h, name.encode(), C.byref(t), C.byref(i), C.byref(o), C.byref(rb), C.byref(p))
        if rc != 0:
            self._fail(rc, "ogm_gguf_matrix")
        raw = np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_uint8)), shape=(rb.value * o.value,)).copy()
        return t.value, i.value, o.value, rb.value, raw

    def upload_matrix(self, be, name: str) -> int:
        h = C.c_void_p()
        rc = self._lib.ogm_gguf_upload_matrix(be._ctx, self._h, name.encode(), C.byref(h))
        if rc != 0:
            self._fail(rc, "ogm_gguf_upload_matrix")
        return h.value

    def close(self):
        if self._h:
            self._lib.ogm_gguf_close(self._h)
            self._h = None
