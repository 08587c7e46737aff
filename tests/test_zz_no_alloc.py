"""kc_moe_decode_static (the decode step whose scratch lives in an array inside the library, so the call allocates nothing)
against kc_moe_decode with caller-owned scratch: routing, weights and outputs bit for bit, on calls in a row that share the
array - a larger step, then smaller ones, per-pair kernel (T <= 8) and the expert-sharing kernel (T > 8) - and the limits."""
import ctypes as C

import numpy as np
import pytest

from nanoseedlm_amd import packs

pytestmark = pytest.mark.gpu


def test_static_scratch_step_equals_workspace_step():
    from nanoseedlm_amd import backend, moe
    backend.require_gpu()
    L, K = backend.hip(), backend.host()
    rng = np.random.default_rng(321)
    E, k, d, ff = 16, 4, 256, 128
    st = moe.MoeStack(1, E, k, d, ff, fmt=packs.MF_SEED4P4, router=moe.ROUTE_SOFTMAX, max_rows=32)
    gate, up, down = packs.seed4p4(rng, E, ff, d, eb=-12), packs.seed4p4(rng, E, ff, d, eb=-12), packs.seed4p4(rng, E, d, ff, eb=-12)
    st.set_layer(0, gate, up, down, packs.f32_to_bf16_bits((rng.standard_normal((E, d)) * 0.3).astype(np.float32)))
    st.finalize()
    K.nslm_moe_router_w.restype = C.c_void_p
    K.nslm_moe_tab.restype = C.c_void_p
    rw = C.c_void_p(K.nslm_moe_router_w(st.h, 0))
    tabs = [C.c_void_p(K.nslm_moe_tab(st.h, 0, i)) for i in range(3)]
    L.kc_moe_decode_sync_words.restype = C.c_size_t
    vp, ci = C.c_void_p, C.c_int
    L.kc_moe_decode.argtypes = [vp, ci, vp, vp, vp, vp, ci, ci, ci, ci, vp, ci, ci, vp, ci, vp, vp, vp, vp, vp, vp]
    L.kc_moe_decode_static.argtypes = [vp, ci, vp, vp, vp, vp, ci, ci, ci, ci, vp, ci, ci, vp, ci, vp, vp, vp, ci]
    TM = 24
    nsync = L.kc_moe_decode_sync_words(TM, d)
    sync = moe.DevBuf.from_array(np.zeros(nsync, dtype=np.uint32))
    lg, A, D = moe.DevBuf(4 * TM * E), moe.DevBuf(4 * TM * k * ff), moe.DevBuf(4 * TM * k * d)
    status = moe.DevBuf.from_array(np.full(1, 77, dtype=np.uint32))
    for T in (8, 3, 16, 9, 1):   # every call shares the library's array with the one before it
        x = packs.round_bf16(rng.standard_normal((T, d)).astype(np.float32))
        dx = moe.DevBuf.from_array(x)
        res = []
        for static in (0, 1):
            out, ind, wt = (moe.DevBuf.from_array(np.full((T, d), 9.0, dtype=np.float32)), moe.DevBuf.from_array(np.full((T, k), -1, dtype=np.int32)),
                            moe.DevBuf.from_array(np.zeros((T, k), dtype=np.float32)))
            if static:
                rc = L.kc_moe_decode_static(None, packs.MF_SEED4P4, rw, tabs[0], tabs[1], tabs[2], E, k, d, ff, dx.ptr, d, T, out.ptr, d, ind.ptr, wt.ptr,
                                            status.ptr, 0)
            else:
                rc = L.kc_moe_decode(None, packs.MF_SEED4P4, rw, tabs[0], tabs[1], tabs[2], E, k, d, ff, dx.ptr, d, T, out.ptr, d, lg.ptr, ind.ptr, wt.ptr,
                                     A.ptr, D.ptr, sync.ptr)
            assert rc == 0, (T, static, rc)
            moe.device_sync()
            assert L.kc_last_error() == 0
            res.append((out.to_array(np.float32, (T, d)), ind.to_array(np.int32, (T, k)), wt.to_array(np.float32, (T, k))))
            for b in (out, ind, wt):
                b.free()
        dx.free()
        (o0, i0, w0), (o1, i1, w1) = res
        assert status.to_array(np.uint32, (1,))[0] == 0
        assert np.abs(o0).max() > 0 and not np.any(o0 == 9.0) and (i0 >= 0).all()
        assert np.array_equal(i0, i1) and np.array_equal(w0.view(np.uint32), w1.view(np.uint32)), T
        assert np.array_equal(o0.view(np.uint32), o1.view(np.uint32)), T
    # beyond the array: refused with -2, nothing launched, the error is on record
    dummy = moe.DevBuf(64)
    assert L.kc_moe_decode_static(None, packs.MF_SEED4P4, rw, tabs[0], tabs[1], tabs[2], 1024, 32, 8192, 8192, dummy.ptr, 8192, 24, dummy.ptr, 8192,
                                  dummy.ptr, dummy.ptr, None, 0) == -2
    assert L.kc_last_error() != 0 and L.kc_last_error() == 0
    # a clear first (the call after a reported error), then the same step again: the same bits
    T = 5
    x = packs.round_bf16(rng.standard_normal((T, d)).astype(np.float32))
    dx = moe.DevBuf.from_array(x)
    outs = []
    for clear in (1, 0):
        out, ind, wt = moe.DevBuf(4 * T * d), moe.DevBuf(4 * T * k), moe.DevBuf(4 * T * k)
        assert L.kc_moe_decode_static(None, packs.MF_SEED4P4, rw, tabs[0], tabs[1], tabs[2], E, k, d, ff, dx.ptr, d, T, out.ptr, d, ind.ptr, wt.ptr, status.ptr,
                                      clear) == 0
        moe.device_sync()
        outs.append(out.to_array(np.float32, (T, d)))
    assert status.to_array(np.uint32, (1,))[0] == 0 and np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32)) and np.abs(outs[0]).max() > 0
    st.close()
