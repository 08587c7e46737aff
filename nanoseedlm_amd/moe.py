"""Python view of the C99 MoE layer host (nanoseedlm_amd/csrc/moe_layer.c) and small device-memory helpers over the
nh_* runtime layer.  Everything here drives the HIP library through its C ABI; nothing computes on the CPU."""
import ctypes as C

import numpy as np

from . import backend, packs

ROUTE_SOFTMAX, ROUTE_SIGMOID = 0, 1


class NslmMoeCfg(C.Structure):
    _fields_ = [("n_layer", C.c_int), ("n_exp", C.c_int), ("top_k", C.c_int), ("d", C.c_int), ("ff", C.c_int), ("fmt", C.c_int),
                ("router", C.c_int), ("max_rows", C.c_int), ("slots", C.c_int), ("route_scale", C.c_float), ("host_units", C.c_int),
                ("prefetch", C.c_int)]


def _lib():
    L = backend.host()
    L.nslm_moe_open.restype = C.c_void_p
    L.nslm_graph_end.restype = C.c_void_p
    L.nslm_moe_tab.restype = C.c_void_p
    L.nslm_moe_unit_bytes.restype = C.c_uint64
    L.nslm_moe_expert_bytes.restype = C.c_uint64
    return L


class DevBuf:
    """A device allocation (nh_malloc) with numpy upload / download."""

    def __init__(self, nbytes):
        self.ptr = C.c_void_p()
        self.nbytes = int(nbytes)
        backend.check(backend.hip().nh_malloc(C.byref(self.ptr), C.c_size_t(self.nbytes)), "nh_malloc")

    @classmethod
    def from_array(cls, a):
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        backend.check(backend.hip().nh_memcpy_h2d(b.ptr, a.ctypes.data_as(C.c_void_p), C.c_size_t(a.nbytes)), "nh_memcpy_h2d")
        return b

    def to_array(self, dtype, shape):
        out = np.zeros(shape, dtype=dtype)
        backend.check(backend.hip().nh_memcpy_d2h(out.ctypes.data_as(C.c_void_p), self.ptr, C.c_size_t(out.nbytes)), "nh_memcpy_d2h")
        return out

    def at(self, byte_offset):
        return C.c_void_p(self.ptr.value + int(byte_offset))

    def free(self):
        if self.ptr:
            backend.hip().nh_free(self.ptr)
            self.ptr = C.c_void_p()


class Event:
    def __init__(self):
        self.e = C.c_void_p()
        backend.check(backend.hip().nh_event_create(C.byref(self.e)), "nh_event_create")

    def record(self, stream=None):
        backend.check(backend.hip().nh_event_record(self.e, stream), "nh_event_record")

    def sync(self):
        backend.check(backend.hip().nh_event_sync(self.e), "nh_event_sync")

    def ms_since(self, start):
        ms = C.c_float(0)
        backend.check(backend.hip().nh_event_elapsed_ms(C.byref(ms), start.e, self.e), "nh_event_elapsed_ms")
        return ms.value


def new_stream():
    s = C.c_void_p()
    backend.check(backend.hip().nh_stream_create(C.byref(s)), "nh_stream_create")
    return s


def device_sync():
    backend.check(backend.hip().nh_device_sync(), "nh_device_sync")


class MoeStack:
    """n_layer routed-expert layers resident in HBM: experts from seeded packs, one BF16 router per layer."""

    def __init__(self, n_layer, n_exp, top_k, d, ff, fmt=packs.MF_SEED4P4, router=ROUTE_SOFTMAX, max_rows=8, slots=0,
                 route_scale=1.0, host_units=0, prefetch=0):
        backend.require_gpu()
        self.L = _lib()
        self.cfg = NslmMoeCfg(n_layer, n_exp, top_k, d, ff, fmt, router, max_rows, slots, route_scale, host_units, prefetch)
        err = C.create_string_buffer(256)
        self.h = C.c_void_p(self.L.nslm_moe_open(C.byref(self.cfg), err, 256))
        if not self.h:
            raise RuntimeError(err.value.decode())

    def set_layer(self, layer, gate, up, down, router_w, router_b=None):
        """gate / up [E][ff][d] and down [E][d][ff] packs (S = n_exp slices); router_w BF16 bits [E][d]."""
        for ti, p in enumerate((gate, up, down)):
            words = p["coefs"] if p["fmt"] == packs.MF_SEED4P4 else p["nibs"]
            for x in range(self.cfg.n_exp):
                codes = p["codes"][x].ctypes.data_as(C.c_void_p) if p["fmt"] == packs.MF_SEED4P4 else None
                rc = self.L.nslm_moe_set_expert(self.h, layer, x, ti, np.ascontiguousarray(p["seeds"][x]).ctypes.data_as(C.c_void_p),
                                                np.ascontiguousarray(words[x]).ctypes.data_as(C.c_void_p), codes, int(p["eb"][x]))
                if rc:
                    raise RuntimeError("nslm_moe_set_expert failed")
        rw = np.ascontiguousarray(router_w, dtype=np.uint16)
        rb = None if router_b is None else np.ascontiguousarray(router_b, dtype=np.uint16).ctypes.data_as(C.c_void_p)
        if self.L.nslm_moe_set_router(self.h, layer, rw.ctypes.data_as(C.c_void_p), rb):
            raise RuntimeError("nslm_moe_set_router failed")

    def finalize(self):
        if self.L.nslm_moe_finalize(self.h):
            raise RuntimeError("nslm_moe_finalize failed")

    def step(self, stream, layer, xn_ptr, T, io_ptr):
        if self.L.nslm_moe_step(self.h, stream, layer, xn_ptr, T, io_ptr):
            raise RuntimeError("nslm_moe_step failed")

    def step_seq(self, stream, layers, xn_ptrs, T, io_ptr, before=None, after=None):
        """The steps (layers[i], xn_ptrs[i]) issued one after the other by one call into the C host (no interpreter between the
        launches); before / after: Events recorded on the stream directly around them."""
        n = len(layers)
        la = (C.c_int * n)(*layers)
        xa = (C.c_void_p * n)(*[p.value if isinstance(p, C.c_void_p) else p for p in xn_ptrs])
        if self.L.nslm_moe_step_seq(self.h, stream, n, la, xa, T, io_ptr, before.e if before else None, after.e if after else None):
            raise RuntimeError("nslm_moe_step_seq failed")

    def last_routing(self, T):
        ind = np.zeros((T, self.cfg.top_k), dtype=np.int32)
        wt = np.zeros((T, self.cfg.top_k), dtype=np.float32)
        if self.L.nslm_moe_last_routing(self.h, T, ind.ctypes.data_as(C.c_void_p), wt.ctypes.data_as(C.c_void_p)):
            raise RuntimeError("nslm_moe_last_routing failed")
        return ind, wt

    def last_logits(self, T):
        """The last step's router logits [T][n_exp] as the GPU formed them (what its selection was made on)."""
        lg = np.zeros((T, self.cfg.n_exp), dtype=np.float32)
        if self.L.nslm_moe_last_logits(self.h, T, lg.ctypes.data_as(C.c_void_p)):
            raise RuntimeError("nslm_moe_last_logits failed")
        return lg

    def last_pairs(self, pairs):
        """The last step's per-pair intermediates: A [pairs][ff] (SwiGLU outputs; uint16 BF16 bits in the batched path's packed
        layout are returned as the raw f32 buffer - see moe_layer.h) and D [pairs][d] (expert outputs)."""
        A = np.zeros((pairs, self.cfg.ff), dtype=np.float32)
        D = np.zeros((pairs, self.cfg.d), dtype=np.float32)
        if self.L.nslm_moe_last_pairs(self.h, pairs, A.ctypes.data_as(C.c_void_p), D.ctypes.data_as(C.c_void_p)):
            raise RuntimeError("nslm_moe_last_pairs failed")
        return A, D

    def cache_stats(self):
        h, m = C.c_uint32(0), C.c_uint32(0)
        if self.L.nslm_moe_cache_stats(self.h, C.byref(h), C.byref(m)):
            raise RuntimeError("nslm_moe_cache_stats failed")
        return h.value, m.value

    def prefetch_stats(self):
        h, m = C.c_uint32(0), C.c_uint32(0)
        if self.L.nslm_moe_prefetch_stats(self.h, C.byref(h), C.byref(m)):
            raise RuntimeError("nslm_moe_prefetch_stats failed")
        return h.value, m.value

    def set_fused(self, on):
        self.L.nslm_moe_set_fused(self.h, int(on))

    def fused_mode(self):
        return self.L.nslm_moe_fused_mode(self.h)

    def fallbacks(self):
        return self.L.nslm_moe_fallbacks(self.h)

    def fused_steps(self):
        """Steps that the persistent kernel took since the stack was made."""
        self.L.nslm_moe_fused_steps.restype = C.c_long
        return int(self.L.nslm_moe_fused_steps(self.h))

    def fused_error(self):
        return self.L.nslm_moe_fused_error(self.h)

    def expert_bytes(self):
        return int(self.L.nslm_moe_expert_bytes(self.h))

    def graph_of_step(self, stream, layer, xn_ptr, T, io_ptr):
        """The step's launches captured once and instantiated (the reference captures forwards of <= 8 rows the same way)."""
        backend.check(self.L.nslm_graph_begin(stream), "nslm_graph_begin")
        self.step(stream, layer, xn_ptr, T, io_ptr)
        g = C.c_void_p(self.L.nslm_graph_end(stream))
        if not g:
            raise RuntimeError("graph capture failed")
        return g

    def launch(self, g, stream):
        backend.check(self.L.nslm_graph_launch(g, stream), "nslm_graph_launch")

    def close(self):
        if self.h:
            self.L.nslm_moe_close(self.h)
            self.h = C.c_void_p()
