"""The MoE layer step (router -> slot table -> gate+up+SwiGLU -> down -> combine) on the GPU against the oracle's
composition of the same rounding points, for both compositions the reference defines, the decode path (T <= 8, gathers)
and the batched path (T > 8, grouping + grouped MFMA GEMMs), with every expert resident and with a pool smaller than the
expert set (LRU slot table)."""
import numpy as np
import pytest

from nanoseedlm_amd import packs

pytestmark = pytest.mark.gpu


def slice_of(orc, p, s):
    if p["fmt"] == packs.MF_SEED4P4:
        return orc.make_slice(p["fmt"], p["seeds"][s], p["coefs"][s], None, p["codes"][s], eb=p["eb"][s])
    return orc.make_slice(p["fmt"], p["seeds"][s], p["nibs"][s], eb=p["eb"][s])


def expert_ref(orc, gate, up, down, e, x, gemm):
    """One (token, expert) pair with the GPU path's rounding points: G, U, A, D rounded to BF16
    (engine/kernels_moe.cu:338-348 decode; :2365-2383 + k_swiglu batched, whose GEMM rounds seed weights to BF16)."""
    r = packs.round_bf16
    d, ff = gate["K"], gate["R"]
    wg = orc.rows_f32(gate["fmt"], slice_of(orc, gate, e), ff, d).astype(np.float64)
    wu = orc.rows_f32(up["fmt"], slice_of(orc, up, e), ff, d).astype(np.float64)
    wd = orc.rows_f32(down["fmt"], slice_of(orc, down, e), d, ff).astype(np.float64)
    if gemm:
        wg, wu, wd = (r(w.astype(np.float32)).astype(np.float64) for w in (wg, wu, wd))
    xd = x.astype(np.float64)
    g = r((wg @ xd).astype(np.float32)).astype(np.float64)
    u = r((wu @ xd).astype(np.float32)).astype(np.float64)
    sg = r((1 / (1 + np.exp(-g))).astype(np.float32)).astype(np.float64)
    a = r((r((g * sg).astype(np.float32)).astype(np.float64) * u).astype(np.float32)).astype(np.float64)
    return r((wd @ a).astype(np.float32)).astype(np.float64)


def check_routing_on_gpu_logits(oracle, st, T, k, xn, rw, ind, wt):
    """The selection must be exactly the oracle's on the logits the GPU itself formed (ties included), the weights within 1e-5,
    and those logits within one BF16 ulp of the float64 x . W."""
    lg = st.last_logits(T)
    oi, ow = oracle.route_softmax(lg, k)
    assert np.array_equal(ind, oi), (ind, oi)
    assert np.max(np.abs(wt - ow)) <= 1e-5
    ref = xn.astype(np.float64) @ packs.bf16_bits_to_f32(rw).astype(np.float64).T
    mag = np.abs(xn).astype(np.float64) @ np.abs(packs.bf16_bits_to_f32(rw)).astype(np.float64).T
    assert np.all(np.abs(lg - ref) <= np.abs(ref) / 128 + 2e-6 * mag + 1e-30)
    assert np.array_equal(lg, packs.round_bf16(lg))          # BF16 values


@pytest.mark.parametrize("router", [0, 1])
@pytest.mark.parametrize("T", [1, 5, 8, 20, 27])
@pytest.mark.parametrize("slots", [0, 20])
def test_moe_step(oracle, router, T, slots):
    from nanoseedlm_amd import moe
    rng = np.random.default_rng(1000 + 10 * T + router)
    nl, E, k, d, ff = 2, 16, 4, 256, 128
    fmt = packs.MF_SEED4P4 if router == 0 else packs.MF_SEED4
    mk = packs.seed4p4 if fmt == packs.MF_SEED4P4 else packs.seed4
    st = moe.MoeStack(nl, E, k, d, ff, fmt=fmt, router=router, max_rows=32, slots=slots, route_scale=2.5)
    layers = []
    for l in range(nl):
        gate, up, down = mk(rng, E, ff, d, eb=-21), mk(rng, E, ff, d, eb=-21), mk(rng, E, d, ff, eb=-20)
        rw = packs.f32_to_bf16_bits((rng.standard_normal((E, d)) * 0.05).astype(np.float32))
        rb = packs.f32_to_bf16_bits((rng.standard_normal(E) * 0.01).astype(np.float32)) if router else None
        st.set_layer(l, gate, up, down, rw, rb)
        layers.append((gate, up, down, rw, rb))
    st.finalize()
    r = packs.round_bf16
    total_pairs = 0
    for rep in range(3):          # several steps so a small pool has to evict
        for l in range(nl):
            gate, up, down, rw, rb = layers[l]
            xn = r(rng.standard_normal((T, d)).astype(np.float32))
            x0 = r(rng.standard_normal((T, d)).astype(np.float32))
            dx, dio = moe.DevBuf.from_array(xn), moe.DevBuf.from_array(x0)
            st.step(None, l, dx.ptr, T, dio.ptr)
            ind, wt = st.last_routing(T)
            out = dio.to_array(np.float32, (T, d))
            if router == 0 and slots == 0 and T <= 8:
                # this step ran as the one persistent kernel: the separate launchers must give the same bits
                assert st.fused_error() == 0
                st.set_fused(0)
                dio2 = moe.DevBuf.from_array(x0)
                st.step(None, l, dx.ptr, T, dio2.ptr)
                ind2, wt2 = st.last_routing(T)
                out2 = dio2.to_array(np.float32, (T, d))
                dio2.free()
                st.set_fused(1)
                assert np.array_equal(ind, ind2) and np.array_equal(wt.view(np.uint32), wt2.view(np.uint32))
                assert np.array_equal(out.view(np.uint32), out2.view(np.uint32))
            dx.free(); dio.free()
            total_pairs += T * k
            # routing: exact given the scores the GPU saw is covered by the kernel tests; here the selection must agree
            # with the oracle's on its own logits except for near-ties moved by a BF16 flip of a logit
            W = packs.bf16_bits_to_f32(rw).astype(np.float64)
            if router == 0:
                lg = r((xn.astype(np.float64) @ W.T).astype(np.float32))
                oi, ow = oracle.route_softmax(lg, k)
                check_routing_on_gpu_logits(oracle, st, T, k, xn, rw, ind, wt)
            else:
                _, _, oi, ow = oracle.route_sigmoid(rw, rb, xn, k, d // 2, 2.5)
            agree = np.mean([len(set(ind[t]) & set(oi[t])) / k for t in range(T)])
            assert agree >= 0.9, agree
            assert all(len(set(ind[t])) == k for t in range(T))
            # the layer output from the GPU's own routing
            for t in range(T):
                # above 8 rows the separate launches take the grouped GEMM (BF16-rounded weights); the persistent kernel
                # (softmax routing, every expert resident) keeps the exact weights of the decode path up to 24 rows
                gemm = T > 8 and not (router == 0 and slots == 0 and T <= 24)
                ys = np.stack([expert_ref(oracle, gate, up, down, int(ind[t, j]), xn[t], gemm=gemm) for j in range(k)])
                if router == 0:
                    want = (wt[t].astype(np.float64)[:, None] * ys).sum(0)
                    tol = 2e-2 * np.abs(wt[t].astype(np.float64)[:, None] * ys).sum(0) + 1e-6
                else:
                    s = np.zeros(d, dtype=np.float32)
                    for j in range(k):
                        s = (s + r((ys[j] * float(r(wt[t, j]))).astype(np.float32))).astype(np.float32)
                    want = r(x0[t] + r(r(s) + 0.0)).astype(np.float64)
                    tol = 2e-2 * (np.abs(x0[t]) + np.abs(ys).sum(0) * np.abs(wt[t]).max()) + 1e-6
                # Elementwise the bound is 2e-2 of the summed magnitudes: G, U, A, D are rounded to BF16 at the reference's rounding
                # points, and a sum next to a rounding boundary may round the other way on the GPU (one BF16 ulp = 2^-8 of the
                # value).  As a max-rel-err (the form of the stated 2e-3 bar) such flips average out over the down projection.
                assert np.all(np.abs(out[t] - want) <= tol), (rep, l, t, np.max(np.abs(out[t] - want) / tol))
                # (this small layer sums 128 products a down row, so one flipped A weighs eight times what it does at 768 or 2880: the
                # stated bars - 1e-2 MFMA, 2e-3 fp32 - are asserted at the full sizes in test_gpu_full_size.py, here 1e-2 / 5e-3)
                assert np.max(np.abs(out[t] - want)) / np.max(np.abs(want)) < (1e-2 if gemm else 5e-3), (rep, l, t)
    hits, misses = st.cache_stats()
    if slots == 0:
        assert (hits, misses) == (0, 0)          # all resident: the table is never consulted
    else:
        assert hits + misses > 0 and misses > 0  # a pool of 20 slots over 32 experts must evict
    st.close()


@pytest.mark.parametrize("T", [1, 3, 4, 5, 6, 7, 8, 12, 16, 19, 24])
def test_whole_expert_block_in_one_launch(T):
    """nslm_moe_step_layer (input RMSNorm + routed experts + shared expert + residual inside the persistent kernel) writes the
    same bits as kq4_norm1p + nslm_moe_step + kc_mv_gu / kc_mv (shared expert, up to 8 rows a call) + kc_residual_add.  With the shared expert
    the grouped kernel takes over at 5 rows (below: one decode a pair), the separate launches group above 8 only."""
    import ctypes as C
    from nanoseedlm_amd import backend, moe
    backend.require_gpu()
    L, K = backend.hip(), backend.host()
    rng = np.random.default_rng(77 + T)
    E, k, d, ff = 16, 4, 256, 128
    st = moe.MoeStack(1, E, k, d, ff, fmt=packs.MF_SEED4P4, router=moe.ROUTE_SOFTMAX, max_rows=32)
    gate, up, down = packs.seed4p4(rng, E, ff, d, eb=-12), packs.seed4p4(rng, E, ff, d, eb=-12), packs.seed4p4(rng, E, d, ff, eb=-12)
    st.set_layer(0, gate, up, down, packs.f32_to_bf16_bits((rng.standard_normal((E, d)) * 0.3).astype(np.float32)))
    st.finalize()
    keep, sh = [], (backend.WSlice * 3)()
    for i, (R, Kk) in enumerate(((ff, d), (ff, d), (d, ff))):
        p = packs.seed4p4(rng, 1, R, Kk, eb=-12)
        bufs = [moe.DevBuf.from_array(p["seeds"][0]), moe.DevBuf.from_array(p["coefs"][0]), moe.DevBuf.from_array(p["codes"][0])]
        sh[i].p[0], sh[i].p[1], sh[i].p[3], sh[i].eb = bufs[0].ptr.value, bufs[1].ptr.value, bufs[2].ptr.value, int(p["eb"][0])
        keep += bufs
    shd = moe.DevBuf(C.sizeof(sh))
    backend.check(L.nh_memcpy_h2d(shd.ptr, sh, C.c_size_t(C.sizeof(sh))), "h2d")
    x0 = packs.round_bf16(rng.standard_normal((T, d)).astype(np.float32))
    nw = moe.DevBuf.from_array((0.2 * rng.standard_normal(d)).astype(np.float32))
    # separate launches
    xa, xn, mo, a_, shv = moe.DevBuf.from_array(x0), moe.DevBuf(4 * T * d), moe.DevBuf(4 * T * d), moe.DevBuf(4 * T * ff), moe.DevBuf(4 * T * d)
    sel0 = moe.DevBuf.from_array(np.zeros(T, dtype=np.int32))
    L.kq4_norm1p.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_float, C.c_void_p, C.c_int]
    L.kq4_norm1p(None, xa.ptr, d, d, nw.ptr, 1e-6, xn.ptr, T)
    st.step(None, 0, xn.ptr, T, mo.ptr)
    ws = backend.WSlice
    L.kc_mv_gu(None, packs.MF_SEED4P4, shd.ptr, shd.at(C.sizeof(ws)), d, ff, xn.ptr, d, a_.ptr, ff, sel0.ptr, T, 1, None)
    for t0 in range(0, T, 8):   # in runs of up to 8 rows: kc_mv gives those the bits of one-row calls, which the one launch forms
        L.kc_mv(None, packs.MF_SEED4P4, sh[2], ff, d, a_.at(4 * t0 * ff), ff, shv.at(4 * t0 * d), d, min(8, T - t0), 0, None)
    L.kc_residual_add(None, xa.ptr, mo.ptr, shv.ptr, C.c_size_t(T * d))
    # the one launch
    xb = moe.DevBuf.from_array(x0)
    K.nslm_moe_step_layer.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.POINTER(ws), C.c_void_p, C.c_void_p, C.c_void_p, C.c_float]
    assert K.nslm_moe_step_layer(st.h, None, 0, xb.ptr, T, sh, xb.ptr, xb.ptr, nw.ptr, 1e-6) == 0
    moe.device_sync()
    A, B = xa.to_array(np.float32, (T, d)), xb.to_array(np.float32, (T, d))
    bad = np.argwhere(A.view(np.uint32) != B.view(np.uint32))
    assert not np.array_equal(A, x0) and len(bad) == 0, (len(bad), bad[:8].tolist(), A[tuple(bad[0])], B[tuple(bad[0])], x0[tuple(bad[0])])
    st.close()


@pytest.mark.parametrize("E", [16, 200, 320])
@pytest.mark.parametrize("case", ["pairs", "all_equal"])
def test_fused_step_equal_logits(oracle, case, E):
    """Equal router logits (BF16 logits tie often): the persistent kernel orders them as the separate router does,
    ties to the higher expert id (k_q4_route, engine/kernels_qwen4.cu:385-422).  16 and 200 experts take the register
    path of the kernel's ranking, 320 the path for more than 256 experts."""
    from nanoseedlm_amd import moe
    rng = np.random.default_rng(5 + E)
    k, d, ff, T = 4, 256, 128, 3
    st = moe.MoeStack(1, E, k, d, ff, fmt=packs.MF_SEED4P4, router=moe.ROUTE_SOFTMAX, max_rows=8)
    gate, up, down = packs.seed4p4(rng, E, ff, d, eb=-21), packs.seed4p4(rng, E, ff, d, eb=-21), packs.seed4p4(rng, E, d, ff, eb=-20)
    W = (rng.standard_normal((E, d)) * 0.05).astype(np.float32)
    groups = ((3, 7, 12), (0, E - 1), (5, 6), (E // 2, E // 2 + 1, E - 2))
    for grp in groups:      # identical router rows -> identical logits for every input
        W[list(grp)] = 3.0 * W[grp[0]]      # large, so that the groups reach the top k for some inputs
    rw = packs.f32_to_bf16_bits(W)
    st.set_layer(0, gate, up, down, rw)
    st.finalize()
    xn = packs.round_bf16(rng.standard_normal((T, d)).astype(np.float32))
    if case == "all_equal":
        xn[:] = 0.0
    outs = []
    for fused in (1, 0):
        st.set_fused(fused)
        dx, dio = moe.DevBuf.from_array(xn), moe.DevBuf.from_array(np.zeros((T, d), dtype=np.float32))
        st.step(None, 0, dx.ptr, T, dio.ptr)
        ind, wt = st.last_routing(T)
        outs.append((ind.copy(), wt.copy(), dio.to_array(np.float32, (T, d)).copy()))
        dx.free(); dio.free()
    assert st.fused_error() == 0
    assert np.array_equal(outs[0][0], outs[1][0]), (outs[0][0], outs[1][0])
    assert np.array_equal(outs[0][1].view(np.uint32), outs[1][1].view(np.uint32))
    assert np.array_equal(outs[0][2].view(np.uint32), outs[1][2].view(np.uint32))
    Wd = packs.bf16_bits_to_f32(rw).astype(np.float64)
    lg = packs.round_bf16((xn.astype(np.float64) @ Wd.T).astype(np.float32))
    oi, _ = oracle.route_softmax(lg, k)
    if case == "all_equal":
        assert np.array_equal(outs[0][0], np.tile(np.arange(E - 1, E - 1 - k, -1, dtype=np.int32), (T, 1)))
    # the groups really tie on the GPU: members of a group that are both chosen appear in descending id order
    for t in range(T):
        sel = outs[0][0][t].tolist()
        for grp in groups:
            pos = [sel.index(g) for g in grp if g in sel]
            ids = [g for g in grp if g in sel]
            assert pos == sorted(pos, reverse=True) or len(ids) < 2, (sel, grp)
    assert np.mean([len(set(outs[0][0][t]) & set(oi[t])) / k for t in range(T)]) >= 0.75
    st.close()


@pytest.mark.parametrize("fmt", [packs.MF_SEED4P4, packs.MF_SEED4])
@pytest.mark.parametrize("d,ff,k", [(2880, 2880, 2), (2880, 2880, 4), (2816, 2880, 2), (4480, 5760, 2)])
def test_fused_step_rows_that_do_not_fill_a_workgroup(d, ff, k, fmt):
    """Rows of 44, 45, 70 or 90 chunks (hidden 2880 = the mixed-format configuration): whole rows do not fill a workgroup's
    256 threads, the row sums go through LDS in both passes, and 2816 rows are 563.2 iterations of 5, so the last item
    ends inside an iteration.  Same bits as the separate launches, at 1, 3 and 8 rows.  With a workgroup a CU (1 and 2 rows) a
    pass's last iteration holds 2, 3, 4 or 6 rows, whose chunks 8, 4 or 2 lanes share (top-4 of 2880 x 2880: 4 lanes in the down pass)."""
    from nanoseedlm_amd import moe
    rng = np.random.default_rng(d + ff + fmt + k)
    E = 6
    mk = packs.seed4p4 if fmt == packs.MF_SEED4P4 else packs.seed4
    st = moe.MoeStack(1, E, k, d, ff, fmt=fmt, router=moe.ROUTE_SOFTMAX, max_rows=8)
    gate, up, down = mk(rng, E, ff, d, eb=-23), mk(rng, E, ff, d, eb=-23), mk(rng, E, d, ff, eb=-22)
    st.set_layer(0, gate, up, down, packs.f32_to_bf16_bits((rng.standard_normal((E, d)) * 0.05).astype(np.float32)))
    st.finalize()
    for T in (1, 2, 3, 8):
        xn = packs.round_bf16(rng.standard_normal((T, d)).astype(np.float32))
        dx = moe.DevBuf.from_array(xn)
        outs = []
        for fused in (1, 0):
            st.set_fused(fused)
            dio = moe.DevBuf.from_array(np.zeros((T, d), dtype=np.float32))
            st.step(None, 0, dx.ptr, T, dio.ptr)
            outs.append((st.last_routing(T), dio.to_array(np.float32, (T, d))))
            dio.free()
            assert st.fused_error() == 0
        dx.free()
        (i1, w1), o1 = outs[0]
        (i0, w0), o0 = outs[1]
        assert np.abs(o0).max() > 0
        assert np.array_equal(i1, i0) and np.array_equal(w1.view(np.uint32), w0.view(np.uint32))
        bad = np.argwhere(o1.view(np.uint32) != o0.view(np.uint32))
        assert len(bad) == 0, (T, len(bad), bad[:6].tolist())
    st.close()


@pytest.mark.parametrize("fmt", [packs.MF_SEED4P4, packs.MF_SEED4])
@pytest.mark.parametrize("E,k", [(16, 4), (64, 4), (200, 8), (300, 6)])
@pytest.mark.parametrize("T", [9, 13, 16, 21, 24])
def test_grouped_step_equals_per_pair_steps(T, E, k, fmt):
    """More than 8 rows: the persistent kernel groups the pairs of an expert, and every row comes out as the per-pair kernel
    computes it in steps of at most 8 rows - routing, weights and outputs bit for bit (16 experts: many pairs an expert,
    several groups; 64 experts: mostly one or two)."""
    from nanoseedlm_amd import moe
    rng = np.random.default_rng(900 + T + E)
    d, ff = 256, 192
    mk = packs.seed4p4 if fmt == packs.MF_SEED4P4 else packs.seed4
    st = moe.MoeStack(1, E, k, d, ff, fmt=fmt, router=moe.ROUTE_SOFTMAX, max_rows=24)
    gate, up, down = mk(rng, E, ff, d, eb=-21), mk(rng, E, ff, d, eb=-21), mk(rng, E, d, ff, eb=-20)
    st.set_layer(0, gate, up, down, packs.f32_to_bf16_bits((rng.standard_normal((E, d)) * 0.05).astype(np.float32)))
    st.finalize()
    xn = packs.round_bf16(rng.standard_normal((T, d)).astype(np.float32))
    dx, dio = moe.DevBuf.from_array(xn), moe.DevBuf.from_array(np.zeros((T, d), dtype=np.float32))
    for rep in range(2):      # twice: the second launch finds the counters as the first left them
        st.step(None, 0, dx.ptr, T, dio.ptr)
        assert st.fused_error() == 0
    ind, wt = st.last_routing(T)
    out = dio.to_array(np.float32, (T, d))
    dx.free(); dio.free()
    assert np.abs(out).max() > 0
    for r0 in range(0, T, 8):
        n = min(8, T - r0)
        dx, dio = moe.DevBuf.from_array(xn[r0:r0 + n]), moe.DevBuf.from_array(np.zeros((n, d), dtype=np.float32))
        st.step(None, 0, dx.ptr, n, dio.ptr)
        i2, w2 = st.last_routing(n)
        o2 = dio.to_array(np.float32, (n, d))
        dx.free(); dio.free()
        assert np.array_equal(ind[r0:r0 + n], i2)
        assert np.array_equal(wt[r0:r0 + n].view(np.uint32), w2.view(np.uint32))
        bad = np.argwhere(out[r0:r0 + n].view(np.uint32) != o2.view(np.uint32))
        assert len(bad) == 0, (r0, len(bad), bad[:6].tolist())
    assert st.fused_error() == 0
    st.close()


def test_steps_of_changing_size_share_the_barrier_words():
    """Launches of the per-pair kernel (up to 8 rows) and of the grouped kernel (9 to 24 rows), of different grid sizes, follow
    each other on one set of sync words: no wait gives up, and every step returns what the same step returned the first time."""
    from nanoseedlm_amd import moe
    rng = np.random.default_rng(4242)
    E, k, d, ff = 32, 4, 256, 192
    st = moe.MoeStack(1, E, k, d, ff, fmt=packs.MF_SEED4P4, router=moe.ROUTE_SOFTMAX, max_rows=24)
    gate, up, down = packs.seed4p4(rng, E, ff, d, eb=-21), packs.seed4p4(rng, E, ff, d, eb=-21), packs.seed4p4(rng, E, d, ff, eb=-20)
    st.set_layer(0, gate, up, down, packs.f32_to_bf16_bits((rng.standard_normal((E, d)) * 0.05).astype(np.float32)))
    st.finalize()
    xn = packs.round_bf16(rng.standard_normal((24, d)).astype(np.float32))
    dx, dio = moe.DevBuf.from_array(xn), moe.DevBuf(4 * 24 * d)
    first = {}
    for rep in range(6):
        for T in (1, 12, 3, 24, 16, 8, 9, 19, 9, 2, 13, 1, 24, 1, 16):
            st.step(None, 0, dx.ptr, T, dio.ptr)
            out = dio.to_array(np.float32, (24, d))[:T].copy()
            assert st.fused_error() == 0, (rep, T)
            if T not in first:
                first[T] = out
                assert np.abs(out).max() > 0
            assert np.array_equal(out.view(np.uint32), first[T].view(np.uint32)), (rep, T)
    # rows are the same whatever the step size they came in
    assert np.array_equal(first[16][:8].view(np.uint32), first[8].view(np.uint32))
    assert np.array_equal(first[24][:16].view(np.uint32), first[16].view(np.uint32))
    assert np.array_equal(first[19][:9].view(np.uint32), first[9].view(np.uint32))
    assert np.array_equal(first[13][:1].view(np.uint32), first[1].view(np.uint32))
    dx.free(); dio.free()
    st.close()


@pytest.mark.parametrize("fmt", [packs.MF_SEED4P4, packs.MF_SEED4])
@pytest.mark.parametrize("E,k,d,ff", [(32, 4, 512, 256), (6, 2, 2880, 2816), (5, 3, 1088, 704)])
def test_both_step_kernels_give_the_separate_launches_bits(fmt, E, k, d, ff):
    """The library's two persistent step kernels (a workgroup per CU; a workgroup per (pair, row tile)), each forced in turn at 1
    to 6 rows, against the separate launches: the same bits three ways, and no wait gives up.  Rows of 8 chunks (row sums by
    shuffles in the CU kernel's gate + up pass) and of 45 and 17 chunks (that pass by iterations of the workgroup, sums through LDS;
    2816 = 44 chunks and 704 = 11 chunks in the down pass)."""
    from nanoseedlm_amd import backend, moe
    L = backend.hip()
    rng = np.random.default_rng(600 + fmt + d)
    mk = packs.seed4p4 if fmt == packs.MF_SEED4P4 else packs.seed4
    st = moe.MoeStack(1, E, k, d, ff, fmt=fmt, router=moe.ROUTE_SOFTMAX, max_rows=8)
    st.set_layer(0, mk(rng, E, ff, d, eb=-21), mk(rng, E, ff, d, eb=-21), mk(rng, E, d, ff, eb=-20),
                 packs.f32_to_bf16_bits((rng.standard_normal((E, d)) * 0.05).astype(np.float32)))
    st.finalize()
    try:
        for T in range(1, 7):
            dx = moe.DevBuf.from_array(packs.round_bf16(rng.standard_normal((T, d)).astype(np.float32)))
            outs = {}
            for which in (0, 1, 2):   # 0: the separate launches
                st.set_fused(1 if which else 0)
                L.kc_moe_decode_kernel(which)
                before = st.fused_steps()
                dio = moe.DevBuf.from_array(np.zeros((T, d), dtype=np.float32))
                st.step(None, 0, dx.ptr, T, dio.ptr)
                outs[which] = dio.to_array(np.float32, (T, d))
                dio.free()
                assert st.fused_error() == 0 and st.fused_steps() == before + (1 if which else 0), (T, which)
            dx.free()
            assert np.abs(outs[0]).max() > 0
            for which in (1, 2):
                assert np.array_equal(outs[which].view(np.uint32), outs[0].view(np.uint32)), (T, which)
    finally:
        L.kc_moe_decode_kernel(0)
        st.close()


def test_steps_issued_by_one_call_equal_single_steps():
    """nslm_moe_step_seq (n steps and the two timing events from one call into the C host) leaves what the same steps leave when
    issued one by one, and its events bracket them; nslm_mv_seq does the same for the dense matvec."""
    import ctypes as C
    from nanoseedlm_amd import backend, moe
    rng = np.random.default_rng(99)
    st = _small_stack(rng)
    d, T = 512, 2
    xs = [moe.DevBuf.from_array(packs.round_bf16(rng.standard_normal((T, d)).astype(np.float32))) for _ in range(3)]
    out = moe.DevBuf(4 * T * d)
    stream = moe.new_stream()
    layers, xi = [0, 1, 1, 0, 1], [0, 1, 2, 2, 0]
    for l, x in zip(layers, xi):
        st.step(stream, l, xs[x].ptr, T, out.ptr)
    moe.device_sync()
    want = out.to_array(np.float32, (T, d)).copy()
    backend.check(backend.hip().nh_memset(out.ptr, 0, C.c_size_t(out.nbytes)), "nh_memset")
    e0, e1 = moe.Event(), moe.Event()
    st.step_seq(stream, layers, [xs[x].ptr for x in xi], T, out.ptr, e0, e1)
    e1.sync()
    got = out.to_array(np.float32, (T, d))
    assert st.fused_error() == 0 and np.abs(want).max() > 0
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert 0.0 < e1.ms_since(e0) < 50.0
    # the dense matvec over two slices, the last launch's result
    R = K = 256
    p = packs.seed4p4(rng, 2, R, K, eb=-20)
    ds, dc, de = moe.DevBuf.from_array(p["seeds"]), moe.DevBuf.from_array(p["coefs"]), moe.DevBuf.from_array(p["codes"])
    sl = (backend.WSlice * 2)()
    for i in range(2):
        sl[i].p[0], sl[i].p[1], sl[i].p[3] = ds.ptr.value + i * R * K // 4, dc.ptr.value + i * R * K // 4, de.ptr.value + i * R * K // 16
        sl[i].eb = -20
    x = moe.DevBuf.from_array(rng.standard_normal(K).astype(np.float32))
    y0, y1 = moe.DevBuf(4 * R), moe.DevBuf(4 * R)
    backend.hip().kc_mv(stream, packs.MF_SEED4P4, sl[1], K, R, x.ptr, K, y0.ptr, R, 1, 0, None)
    backend.check(backend.host().nslm_mv_seq(stream, packs.MF_SEED4P4, sl, 2, 0, 4, K, R, x.ptr, y1.ptr, None, None), "nslm_mv_seq")
    moe.device_sync()
    a, b = y0.to_array(np.float32, (R,)), y1.to_array(np.float32, (R,))
    assert np.abs(a).max() > 0 and np.array_equal(a.view(np.uint32), b.view(np.uint32))
    for buf in xs + [out, ds, dc, de, x, y0, y1]:
        buf.free()
    st.close()


def test_small_shape_then_long_rows_in_one_process():
    """The per-item step kernel's launcher keeps the number of workgroups a CU holds per kernel variant; the LDS a workgroup
    asks for grows with the longer of hidden and expert width (8192: 51,200 bytes, above the 48 KB a kernel may have without
    asking).  A small shape first, then the long rows, in one process, through that kernel: no wait gives up, and the bits
    are those of the separate launches."""
    from nanoseedlm_amd import backend, moe
    L = backend.hip()
    rng = np.random.default_rng(8192)
    L.kc_moe_decode_kernel(1)   # the per-item kernel at every size
    try:
        for d, ff in ((256, 192), (8192, 512), (256, 192)):
            E, k = 4, 2
            st = moe.MoeStack(1, E, k, d, ff, fmt=packs.MF_SEED4P4, router=moe.ROUTE_SOFTMAX, max_rows=8)
            gate, up, down = packs.seed4p4(rng, E, ff, d, eb=-23), packs.seed4p4(rng, E, ff, d, eb=-23), packs.seed4p4(rng, E, d, ff, eb=-22)
            st.set_layer(0, gate, up, down, packs.f32_to_bf16_bits((rng.standard_normal((E, d)) * 0.05).astype(np.float32)))
            st.finalize()
            for T in (1, 8):
                dx = moe.DevBuf.from_array(packs.round_bf16(rng.standard_normal((T, d)).astype(np.float32)))
                outs = []
                for fused in (1, 0):
                    st.set_fused(fused)
                    dio = moe.DevBuf.from_array(np.zeros((T, d), dtype=np.float32))
                    st.step(None, 0, dx.ptr, T, dio.ptr)
                    outs.append(dio.to_array(np.float32, (T, d)))
                    dio.free()
                    assert st.fused_error() == 0, (d, T, fused)
                dx.free()
                assert np.abs(outs[1]).max() > 0
                assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32)), (d, T)
            assert st.fused_steps() == 2   # both sizes went through the kernel, none was refused to the separate launches
            st.close()
    finally:
        L.kc_moe_decode_kernel(0)


def _small_stack(rng, E=32, k=4, d=512, ff=256, nl=2):
    from nanoseedlm_amd import moe
    st = moe.MoeStack(nl, E, k, d, ff, fmt=packs.MF_SEED4P4, router=moe.ROUTE_SOFTMAX, max_rows=24)
    for l in range(nl):
        gate, up, down = packs.seed4p4(rng, E, ff, d, eb=-21), packs.seed4p4(rng, E, ff, d, eb=-21), packs.seed4p4(rng, E, d, ff, eb=-20)
        st.set_layer(l, gate, up, down, packs.f32_to_bf16_bits((rng.standard_normal((E, d)) * 0.05).astype(np.float32)))
    st.finalize()
    return st


def _quiet_results(st, dx, dio, d, cases, fused):
    """the steps with nothing else on the GPU: through the separate launchers (fused = 0) or the persistent kernel (1).  Up to
    8 rows the two give the same bits; above, the launchers take the grouped GEMMs on BF16-rounded weights."""
    st.set_fused(fused)
    want = {}
    for l, T in cases:
        st.step(None, l, dx.ptr, T, dio.ptr)
        want[(l, T)] = dio.to_array(np.float32, (24, d))[:T].copy()
        assert np.abs(want[(l, T)]).max() > 0 and st.fused_error() == 0
    return want


def _same(a, b):
    return np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_checked_step_beside_another_streams_kernels():
    """The persistent kernel's workgroups wait for each other, so its grid must be resident at once - which another stream's
    kernels can prevent for a while (the reference engine runs a copy stream beside compute, engine/mova_cuda.c:136-146).
    Here a queue of large GEMMs occupies the GPU on a second stream while checked steps (nslm_moe_set_fused(2)) run: every
    step must return the separate launchers' bits, whether the kernel got through or the step was redone; the other stream's
    queue is finite, so every wait ends and every kernel exits by itself."""
    import ctypes as C
    from nanoseedlm_amd import backend, moe
    backend.require_gpu()
    L = backend.hip()
    rng = np.random.default_rng(777)
    d = 512
    st = _small_stack(rng, d=d)
    xn = packs.round_bf16(rng.standard_normal((24, d)).astype(np.float32))
    dx, dio = moe.DevBuf.from_array(xn), moe.DevBuf(4 * 24 * d)
    cases = [(l, T) for T in (1, 4, 8, 16) for l in (0, 1)]
    want, wantf = _quiet_results(st, dx, dio, d, cases, 0), _quiet_results(st, dx, dio, d, cases, 1)
    assert all(_same(want[c], wantf[c]) == (c[1] <= 8) for c in cases)
    # the other stream's work: a dense seed GEMM 4096 x 4096 x 512 on device-filled records, a hundred times over
    R = K = 4096
    seeds, coefs, codes = moe.DevBuf(R * K // 8 * 2), moe.DevBuf(R * K // 8 * 2), moe.DevBuf(R * K // 16 // 2 * 2)
    for i, b in enumerate((seeds, coefs, codes)):
        L.kc_fill_random(None, b.ptr, C.c_size_t(b.nbytes), C.c_uint64(5 + i))
    w = backend.WSlice()
    w.p[0], w.p[1], w.p[3], w.eb = seeds.ptr.value, coefs.ptr.value, codes.ptr.value, -30
    gx = moe.DevBuf.from_array(packs.round_bf16(rng.standard_normal((512, K)).astype(np.float32)))
    gy = moe.DevBuf(4 * 512 * R)
    sa, sb = moe.new_stream(), moe.new_stream()
    moe.device_sync()
    st.set_fused(2)
    for rep in range(3):
        for i in range(100):
            L.kc_mm(sb, packs.MF_SEED4P4, w, K, R, gx.ptr, K, gy.ptr, R, 512, 0, None)
        for l, T in cases:
            if st.fused_mode() == 0:      # a step was redone: the stack went back to the launchers; turn the kernel on again
                st.set_fused(2)
            st.step(sa, l, dx.ptr, T, dio.ptr)
            backend.check(L.nh_stream_sync(sa), "nh_stream_sync")
            got = dio.to_array(np.float32, (24, d))[:T]
            assert _same(got, wantf[(l, T)]) or (st.fused_mode() == 0 and _same(got, want[(l, T)])), (rep, l, T, st.fallbacks())
        moe.device_sync()
        assert L.kc_last_error() == 0
    print("steps redone by the launchers:", st.fallbacks())
    st.set_fused(1)
    assert st.fused_error() == 0          # whatever happened, the sync words are in order again
    for b in (dx, dio, seeds, coefs, codes, gx, gy):
        b.free()
    st.close()


def test_checked_step_is_redone_when_a_wait_gives_up():
    """The error path, driven from the host: with a spin limit of one poll the first workgroup that finds a logit not yet
    there gives up (every kernel still runs to its end).  A plain step then reports the error word; a checked step notices
    it, zeroes the sync words, redoes the step through the launchers - the same bits - and leaves the stack on the
    launchers.  With the limit back at its default the kernel can be turned on again and works on the zeroed words."""
    from nanoseedlm_amd import backend, moe
    backend.require_gpu()
    L = backend.hip()
    rng = np.random.default_rng(778)
    d = 512
    st = _small_stack(rng, d=d)
    xn = packs.round_bf16(rng.standard_normal((24, d)).astype(np.float32))
    dx, dio = moe.DevBuf.from_array(xn), moe.DevBuf(4 * 24 * d)
    cases = [(0, 1), (1, 8), (0, 16)]     # the per-pair kernel and the grouped one
    want, wantf = _quiet_results(st, dx, dio, d, cases, 0), _quiet_results(st, dx, dio, d, cases, 1)
    try:
        for n, (l, T) in enumerate(cases):
            L.kc_moe_decode_spin_limit(1)
            st.set_fused(2)
            st.step(None, l, dx.ptr, T, dio.ptr)
            moe.device_sync()
            assert st.fallbacks() == n + 1 and st.fused_mode() == 0, (l, T)
            got = dio.to_array(np.float32, (24, d))[:T]
            assert _same(got, want[(l, T)]), (l, T)
            L.kc_moe_decode_spin_limit(0)
            st.set_fused(1)                # on again, on the zeroed words: no error, the kernel's bits
            for l2, T2 in cases:
                st.step(None, l2, dx.ptr, T2, dio.ptr)
                assert st.fused_error() == 0
                got = dio.to_array(np.float32, (24, d))[:T2]
                assert _same(got, wantf[(l2, T2)]), (l, T, l2, T2)
        # unchecked, the same failure is reported by the error word (and the caller zeroes the words)
        L.kc_moe_decode_spin_limit(1)
        st.step(None, 0, dx.ptr, 1, dio.ptr)
        assert st.fused_error() != 0
    finally:
        L.kc_moe_decode_spin_limit(0)
    dx.free(); dio.free()
    st.close()


def test_engine_order_host_units_and_next_layer_prefetch():
    """The reference engine's expert block in its own order on the runtime layer (engine/mova_cuda.c:1279-1325): sigmoid router ->
    wait for the predicted experts' copies -> admit -> copy -> next layer's router on this layer's input, admit with
    CACHE_PROTECT_PREV, copies on a second stream behind an event -> gathers -> combine; the experts' units in pinned host
    memory that the copy kernel reads through its device address (:340-360), a pool of 24 slots for 48 experts.
    Residency must never change a result: the same steps on a stack with every expert resident in HBM, on the host-unit pool
    without prefetch and on it with prefetch give the same bits, and the prefetch turns demand misses into hits."""
    from nanoseedlm_amd import moe
    rng = np.random.default_rng(909)
    nl, E, k, d, ff = 3, 16, 4, 256, 128
    layers = []
    for l in range(nl):
        gate, up, down = packs.seed4(rng, E, ff, d, eb=-21), packs.seed4(rng, E, ff, d, eb=-21), packs.seed4(rng, E, d, ff, eb=-20)
        rw = packs.f32_to_bf16_bits((rng.standard_normal((E, d)) * 0.05).astype(np.float32))
        rb = packs.f32_to_bf16_bits((rng.standard_normal(E) * 0.01).astype(np.float32))
        layers.append((gate, up, down, rw, rb))
    stacks = []
    for slots, host_units, prefetch in ((0, 0, 0), (24, 1, 0), (24, 1, 1)):
        st = moe.MoeStack(nl, E, k, d, ff, fmt=packs.MF_SEED4, router=moe.ROUTE_SIGMOID, max_rows=8, slots=slots, route_scale=2.5,
                          host_units=host_units, prefetch=prefetch)
        for l, lay in enumerate(layers):
            st.set_layer(l, *lay)
        st.finalize()
        stacks.append(st)
    s = moe.new_stream()
    r = packs.round_bf16
    for rep in range(6):
        T = (1, 3, 8, 2, 5, 1)[rep]
        x = r(rng.standard_normal((T, d)).astype(np.float32))          # the residual stream, through the three layers
        xs = [moe.DevBuf.from_array(x) for _ in stacks]
        for l in range(nl):
            xn = r(rng.standard_normal((T, d)).astype(np.float32))     # (stands for the layer's norm output)
            dxn = moe.DevBuf.from_array(xn)
            outs = []
            for st, dio in zip(stacks, xs):
                st.step(s, l, dxn.ptr, T, dio.ptr)
                moe.device_sync()
                outs.append(dio.to_array(np.float32, (T, d)))
            assert not np.array_equal(outs[0], x)
            for o in outs[1:]:
                assert np.array_equal(o.view(np.uint32), outs[0].view(np.uint32)), (rep, l)
            dxn.free()
        for b in xs:
            b.free()
    h0, m0 = stacks[1].cache_stats()
    h1, m1 = stacks[2].cache_stats()
    ph, pm = stacks[2].prefetch_stats()
    print(f"demand hits/misses without prefetch {h0}/{m0}, with {h1}/{m1}; predicted: resident already {ph}, copied ahead {pm}")
    assert h0 + m0 == h1 + m1 and m0 > 0          # the same requests; 24 slots for 48 experts must evict
    assert pm > 0 and m1 < m0                      # experts copied ahead of their layer are hits when it comes
    for st in stacks:
        st.close()
