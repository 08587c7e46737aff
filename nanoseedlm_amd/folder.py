"""ctypes mirror of csrc/model_folder.h: NanoSeedLM model folders (safetensors shards + index) and expert bank files.
Reading needs no GPU; the load_* calls copy into the HBM layout of a MoeStack."""
import ctypes as C

import numpy as np

from . import backend

BF16, SEED4, Q8, Q4, SEED4P4, SEED6P8, TCQ = 0, 1, 2, 3, 4, 5, 8
PAGE = 16384


class Stream(C.Structure):
    _fields_ = [("p", C.c_void_p), ("len", C.c_uint64), ("off", C.c_uint64), ("shard", C.c_int)]


class Tensor(C.Structure):
    _fields_ = [("name", C.c_char * 96), ("enc", C.c_int), ("slices", C.c_int), ("rows", C.c_int), ("cols", C.c_int), ("group", C.c_int),
                ("s", Stream * 4)]

    def stream(self, i):
        """A copy of stream i's bytes."""
        s = self.s[i]
        if not s.len:
            return np.zeros(0, dtype=np.uint8)
        return np.ctypeslib.as_array(C.cast(s.p, C.POINTER(C.c_uint8)), shape=(s.len,)).copy()


def _lib():
    L = backend.host()
    L.nsf_open.restype = C.c_void_p
    L.nsf_at.restype = C.POINTER(Tensor)
    L.nsf_find.restype = C.POINTER(Tensor)
    L.nsf_stream_len.restype = C.c_uint64
    L.nsf_open.argtypes = [C.c_char_p, C.c_char_p, C.c_int]
    L.nsf_at.argtypes = [C.c_void_p, C.c_int]
    L.nsf_find.argtypes = [C.c_void_p, C.c_char_p]
    L.nsf_close.argtypes = [C.c_void_p]
    L.nsf_count.argtypes = [C.c_void_p]
    L.nsf_shards.argtypes = [C.c_void_p]
    L.nsf_mappable.argtypes = [C.c_void_p, C.POINTER(Stream)]
    return L


def stream_len(enc, slices, rows, cols, s):
    return int(_lib().nsf_stream_len(enc, slices, rows, cols, s))


def blk_stream(blk, p, E, rows, cols, s, out_bytes):
    """Stream s of a .blk (p = 3) / .blk4 (p = 4) bank image; None when the image is not that bank."""
    blk = np.ascontiguousarray(blk, dtype=np.uint8)
    dst = np.zeros(out_bytes, dtype=np.uint8)
    rc = _lib().nsf_blk_stream(blk.ctypes.data_as(C.c_void_p), C.c_size_t(blk.size), p, E, rows, cols, s, dst.ctypes.data_as(C.c_void_p))
    return None if rc else dst


class ModelFolder:
    def __init__(self, path):
        self.L = _lib()
        err = C.create_string_buffer(512)
        self.h = self.L.nsf_open(str(path).encode(), err, 512)
        if not self.h:
            raise ValueError(err.value.decode() or "nsf_open failed")

    def close(self):
        if self.h:
            self.L.nsf_close(self.h)
            self.h = None

    def __len__(self):
        return self.L.nsf_count(self.h)

    @property
    def shards(self):
        return self.L.nsf_shards(self.h)

    def at(self, i):
        return self.L.nsf_at(self.h, i).contents

    def find(self, name):
        t = self.L.nsf_find(self.h, name.encode())
        return t.contents if t else None

    def mappable(self, stream):
        return bool(self.L.nsf_mappable(self.h, C.byref(stream)))

    def load_experts(self, stack, layer, which, name):
        """Tensor `name` as the experts' matrix `which` (0 gate, 1 up, 2 down) of a moe.MoeStack's layer."""
        t = self.L.nsf_find(self.h, name.encode())
        if not t or self.L.nslm_moe_load_experts(stack.h, layer, which, t):
            raise RuntimeError(f"nslm_moe_load_experts({name}) failed")

    def load_router(self, stack, layer, name, bias=None):
        t = self.L.nsf_find(self.h, name.encode())
        b = self.L.nsf_find(self.h, bias.encode()) if bias else None
        if not t or (bias and not b) or self.L.nslm_moe_load_router(stack.h, layer, t, b):
            raise RuntimeError(f"nslm_moe_load_router({name}) failed")
