"""Host mirror of csrc/decode_model.h: a whole synthetic seeded-MoE model's greedy decode on the gfx950 kernels
(the benchmark's full-model configuration).  ctypes only; every launch goes through libnslm_host.so / libnslm_hip.so."""
import ctypes as C

import numpy as np

from . import backend, moe, packs

W_Q, W_KVA, W_KR, W_O, W_SG, W_SU, W_SD = range(7)
H_QRMIX, H_QLAT, H_VUP = range(3)


class ModelCfg(C.Structure):
    _fields_ = [("n_layer", C.c_int), ("d", C.c_int), ("n_head", C.c_int), ("head_dim", C.c_int), ("r", C.c_int), ("rope", C.c_int),
                ("n_exp", C.c_int), ("top_k", C.c_int), ("ff", C.c_int), ("ff_shared", C.c_int), ("vocab", C.c_int), ("max_ctx", C.c_int),
                ("max_rows", C.c_int), ("kv_fmt", C.c_int), ("n_splits", C.c_int), ("eps", C.c_float), ("rope_theta", C.c_float)]


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


class DecodeModel:
    def __init__(self, **kw):
        self.L = backend.host()
        self.cfg = ModelCfg(**kw)
        err = C.create_string_buffer(256)
        self.L.nslm_model_open.restype = C.c_void_p
        self.L.nslm_model_moe.restype = C.c_void_p
        self.L.nslm_model_step_bytes.restype = C.c_uint64
        self.L.nslm_graph_end.restype = C.c_void_p
        self.h = C.c_void_p(self.L.nslm_model_open(C.byref(self.cfg), err, 256))
        if not self.h:
            raise RuntimeError(err.value.decode())

    def close(self):
        if self.h:
            self.L.nslm_model_close(self.h)
            self.h = C.c_void_p()

    def fill_random(self, seed=1, eb=-24):
        backend.check(self.L.nslm_model_fill_random(self.h, C.c_uint64(seed), eb), "nslm_model_fill_random")

    def set_dense(self, layer, which, pack):
        """pack: packs.seed4p4(rng, 1, R, K)."""
        backend.check(self.L.nslm_model_set_dense(self.h, layer, which, _p(pack["seeds"][0]), _p(pack["coefs"][0]), _p(pack["codes"][0]),
                                                  int(pack["eb"][0])), "nslm_model_set_dense")

    def set_heads(self, layer, which, w_bits):
        w = np.ascontiguousarray(w_bits, dtype=np.uint16)
        backend.check(self.L.nslm_model_set_heads(self.h, layer, which, _p(w)), "nslm_model_set_heads")

    def set_norm(self, layer, which, w):
        w = np.ascontiguousarray(w, dtype=np.float32)
        backend.check(self.L.nslm_model_set_norm(self.h, layer, which, _p(w)), "nslm_model_set_norm")

    def set_embed(self, w_bits):
        w = np.ascontiguousarray(w_bits, dtype=np.uint16)
        backend.check(self.L.nslm_model_set_embed(self.h, _p(w)), "nslm_model_set_embed")

    def set_experts(self, layer, gate, up, down, router_bits):
        m = C.c_void_p(self.L.nslm_model_moe(self.h))
        for t, p in enumerate((gate, up, down)):
            for e in range(p["S"]):
                backend.check(self.L.nslm_moe_set_expert(m, layer, e, t, _p(p["seeds"][e]), _p(p["coefs"][e]), _p(p["codes"][e]), int(p["eb"][e])),
                              "nslm_moe_set_expert")
        rw = np.ascontiguousarray(router_bits, dtype=np.uint16)
        backend.check(self.L.nslm_moe_set_router(m, layer, _p(rw), None), "nslm_moe_set_router")

    def finalize(self):
        backend.check(self.L.nslm_model_finalize(self.h), "nslm_model_finalize")

    def start(self, ids, pos):
        ids, pos = np.ascontiguousarray(ids, dtype=np.int32), np.ascontiguousarray(pos, dtype=np.int32)
        backend.check(self.L.nslm_model_start(self.h, ids.size, _p(ids), _p(pos)), "nslm_model_start")

    def fill_cache(self, T, upto, seed=3):
        backend.check(self.L.nslm_model_fill_cache(self.h, T, upto, C.c_uint64(seed)), "nslm_model_fill_cache")

    def set_branches(self, on=True):
        backend.check(self.L.nslm_model_set_branches(self.h, int(on)), "nslm_model_set_branches")

    def step(self, stream, T):
        backend.check(self.L.nslm_model_step(self.h, stream, T), "nslm_model_step")

    def graph_of_step(self, stream, T):
        backend.check(self.L.nslm_graph_begin(stream), "nslm_graph_begin")
        self.step(stream, T)
        g = C.c_void_p(self.L.nslm_graph_end(stream))
        if not g:
            raise RuntimeError("graph capture failed")
        return g

    def launch(self, g, stream):
        """One replay of a captured step; refused (RuntimeError) when a sequence slot is full."""
        backend.check(self.L.nslm_model_launch(self.h, g, stream), "nslm_model_launch: the cache slot is full, or the launch failed")

    def steps_left(self):
        return int(self.L.nslm_model_steps_left(self.h))

    def ids(self, T):
        out = np.zeros(T, dtype=np.int32)
        backend.check(self.L.nslm_model_ids(self.h, T, _p(out)), "nslm_model_ids")
        return out

    def logits(self, T):
        out = np.zeros((T, self.cfg.vocab), dtype=np.float32)
        backend.check(self.L.nslm_model_logits(self.h, T, _p(out)), "nslm_model_logits")
        return out

    def hidden(self, T):
        out = np.zeros((T, self.cfg.d), dtype=np.float32)
        backend.check(self.L.nslm_model_hidden(self.h, T, _p(out)), "nslm_model_hidden")
        return out

    def embed_rows(self, first, rows):
        out = np.zeros((rows, self.cfg.d), dtype=np.uint16)
        backend.check(self.L.nslm_model_get_embed(self.h, first, rows, _p(out)), "nslm_model_get_embed")
        return out

    def step_bytes(self):
        return int(self.L.nslm_model_step_bytes(self.h))
