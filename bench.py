#!/usr/bin/env python3
"""bench.py - the SeedLM decode-in-matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2b1|c2b8|c2b32|c0|c1|c3b1|c3b16|c4b1|c4b16] [--matrices N] [--no-cpu]

A step is one pass of the workload over one batch of seeded synthetic input already resident in HBM:
  c2b1 (default; the configuration the metric is quoted on): one MoE decode layer step at batch 1 - 128 experts seeded
        P=4, top-8 softmax routing, hidden 2048, expert intermediate 768 (router GEMV, top-k, fused gate+up+SwiGLU
        gather, down gather, combine).  Steps rotate over `layers` resident layers and 16 inputs so the selected experts
        change from step to step and the traffic comes from HBM, not from the 256 MB Infinity Cache.
  c2b8 / c2b32: the same at 8 and 32 tokens (32: grouping + grouped MFMA GEMMs).
  c0:   dense GEMV, W 4096x4096 P=4, batch 1, rotating over --matrices 64 matrices (604 MB); the line also carries the same
        launches on one matrix, resident in the Infinity Cache (roofline.cache_resident).
  c1:   prefill GEMM, W 14336x4096 P=4, X bf16 [512 x 4096].
  c3b1 / c3b16: the mixed-format layer - 64 experts P=3 top-4, hidden 2880, intermediate 2880, plus seven 2880 x 2880
        Q4-g64 projections (q, k, v, o and the shared expert's gate / up / down) - at batch 1 and 16.
Prints ONE JSON line: value = effective GB/s of compressed weight bytes (whole job), with the dominant kernel's roofline
(timed live with HIP events on the launch stream) and the CPU baseline (the reference's own lib_cpu_seed4 when the
compiled reference is present, else this repository's restatement) on a bounded sample of the same workload."""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "seeded GEMV effective GB/s (%HBM peak); MoE decode tokens/s at batch 1"
HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0


COUNTERS = "profiles/traffic.json"
# Untimed steps before the W warmup steps: a fresh GPU reaches its steady clocks only after a few hundred milliseconds of work
# (the same 400 timed steps: 23.8 us a step after 50 warmup steps, 22.9 after 4000; a box that had just been handed out once
# read 22.5 us behind 0.3 s of it where the next runs read 19.9), and a short run would measure the ramp.
PREWARM_S = 1.0


def counters_of(workload):
    """What the committed rocprofv3 --pmc summaries hold for the workload's dominant kernel: HBM bytes per launch and the share
    of the kernel's time its vector ALUs were busy.  Constants of an earlier profiled run of the same command, not measurements
    of this run: the JSON line says so (traffic_source)."""
    try:
        with open(os.path.join(ROOT, COUNTERS)) as f:
            e = json.load(f).get(workload, {})
    except OSError:
        e = {}
    return dict(traffic=e.get("hbm_bytes_per_launch"), traffic_source=COUNTERS if e.get("hbm_bytes_per_launch") else None,
                valu_busy=e.get("valu_busy_pct") / 100.0 if e.get("valu_busy_pct") is not None else None,
                valu_busy_source=COUNTERS if e.get("valu_busy_pct") is not None else None,
                valu_insts_per_block=e.get("valu_insts_per_block"))


def fail_on_kernel_error(st=None):
    """A launch error, or a wait inside the persistent MoE kernel that gave up (its results are void): no throughput is printed."""
    from nanoseedlm_amd import backend
    err = backend.hip().kc_last_error()
    if err:
        sys.exit(f"bench.py: a kernel launch failed ({err}); no result")
    if st is not None and st.fused_error():
        sys.exit("bench.py: a wait between workgroups of the persistent MoE kernel gave up (error word set); no result")


class Q4Projections:
    """Config 3's affine-int4 side of the layer: q / k / v / o and the shared expert's gate / up / down, each d x d, Q4
    group 64 (BF16 scale ~U(0.005, 0.02), zero point uniform [0, 15] stored as bias = -z * scale).  The benchmark definition gives no
    shapes for them; these are fixed here.  run() is the launch sequence of one step: matvecs for few tokens, the packed
    MFMA GEMMs above (the reference's enc_dense / enc_dense_packed change over at 8, engine/mova_cuda.c:1020-1028).  From
    gemm_from to 32 tokens the matrices that share an input go through the grouped GEMM's entry points as "experts" that every
    token chose - q, k and v as one launch of three tiles, the shared expert's gate and up with SwiGLU as one launch - so that a
    launch has 135 and 90 workgroups where a 2880-row matrix alone has 45."""

    def __init__(self, rng, n_layers, d, T, gemm_from=9):
        from nanoseedlm_amd import backend, moe, packs
        self.L, self.d, self.T, self.keep = backend.hip(), d, T, []
        self.layers = []
        for _ in range(n_layers):
            pk = packs.affine(rng, 7, d, d, bits=4, group=64)
            bufs = [moe.DevBuf.from_array(pk[k]) for k in ("words", "scales", "biases")]
            self.keep += bufs
            arr = (backend.WSlice * 7)()
            for i in range(7):
                arr[i].p[0] = bufs[0].ptr.value + i * d * d // 2
                arr[i].p[1] = bufs[1].ptr.value + i * d * (d // 64) * 2
                arr[i].p[2] = bufs[2].ptr.value + i * d * (d // 64) * 2
                arr[i].gs = 6
            tab = moe.DevBuf(C.sizeof(arr))
            backend.check(self.L.nh_memcpy_h2d(tab.ptr, arr, C.c_size_t(C.sizeof(arr))), "nh_memcpy_h2d")
            self.keep.append(tab)
            self.layers.append((arr, tab))
        self.bytes_per_layer = 7 * (d * d // 2 + 2 * d * (d // 64) * 2)
        f = lambda n: moe.DevBuf(4 * n)
        self.q, self.kk, self.v, self.o, self.a, self.g, self.u, self.sh = (f(T * d) for _ in range(8))
        self.px, self.pa = moe.DevBuf(2 * T * d), moe.DevBuf(2 * T * d)
        self.sel0 = moe.DevBuf.from_array(np.zeros(max(T, 1), dtype=np.int32))
        self.gemm_from = gemm_from
        # grouped launches: pair (matrix e, token t) reads row perm / n = t of the input and writes row perm = t n + e of the output
        self.y3g, self.p3g = moe.DevBuf(4 * T * 3 * d), moe.DevBuf(2 * T * 3 * d)
        self.perm3 = moe.DevBuf.from_array(np.array([t * 3 + e for e in range(3) for t in range(T)], dtype=np.int32))
        self.tiles3 = moe.DevBuf.from_array(np.array([[e, e * T, T, 0] for e in range(3)], dtype=np.int32))
        self.perm1 = moe.DevBuf.from_array(np.arange(T, dtype=np.int32))
        self.tiles1 = moe.DevBuf.from_array(np.array([[0, 0, T, 0]], dtype=np.int32))
        self.nt3, self.nt1 = moe.DevBuf.from_array(np.array([3], dtype=np.int32)), moe.DevBuf.from_array(np.array([1], dtype=np.int32))
        self.R3, self.add3 = (C.c_int * 3)(d, d, d), (C.c_int * 3)(0, 0, 0)
        self.y3 = (C.c_void_p * 3)(self.q.ptr.value, self.kk.ptr.value, self.v.ptr.value)
        self.L.kc_mv_multi.argtypes = [C.c_void_p, C.c_int, C.c_int, C.POINTER(backend.WSlice), C.POINTER(C.c_int), C.POINTER(C.c_void_p),
                                       C.POINTER(C.c_int), C.POINTER(C.c_int), C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_float]

    def run(self, stream, layer, x_ptr):
        from nanoseedlm_amd import packs
        L, d, T, Q4 = self.L, self.d, self.T, packs.MF_Q4
        arr, tab = self.layers[layer]
        if self.gemm_from <= T <= 32:
            ws = C.sizeof(arr[0])
            L.kc_pack_input_bf16(stream, x_ptr, self.px.ptr, C.c_size_t(T * d))
            L.kc_mm_grouped_packed_rows(stream, Q4, tab.ptr, d, d, self.px.ptr, d, self.y3g.ptr, d, 3, self.perm3.ptr, self.tiles3.ptr,
                                        self.nt3.ptr, 3, T)                                  # [T][q | k | v]
            L.kc_pack_input_bf16(stream, self.y3g.ptr, self.p3g.ptr, C.c_size_t(T * 3 * d))
            L.kc_mm_packed(stream, Q4, arr[3], d, d, self.p3g.ptr, 3 * d, self.o.ptr, d, T, 0, None)   # o over the q columns
            if L.kc_mm_grouped_swiglu(stream, Q4, tab.at(4 * ws), tab.at(5 * ws), d, d, self.px.ptr, d, self.pa.ptr, d, 1, self.perm1.ptr,
                                      self.tiles1.ptr, self.nt1.ptr, 1, T):
                raise RuntimeError("kc_mm_grouped_swiglu refused the shared expert's shape")
            L.kc_mm_packed(stream, Q4, arr[6], d, d, self.pa.ptr, d, self.sh.ptr, d, T, 0, None)
        elif T <= 16:   # (matvecs: ahead of the one-matrix GEMMs on these 2880 x 2880 matrices, 19 against 23 us a projection at 16 rows)
            # q, k, v over the same input: one launch (kc_mv_multi; the same bits as one kc_mv each), else the three launches
            if L.kc_mv_multi(stream, Q4, 3, arr, self.R3, self.y3, self.R3, self.add3, d, x_ptr, d, T, None, C.c_float(0.0)):
                for i, y in enumerate((self.q, self.kk, self.v)):
                    L.kc_mv(stream, Q4, arr[i], d, d, x_ptr, d, y.ptr, d, T, 0, None)
            L.kc_mv(stream, Q4, arr[3], d, d, self.q.ptr, d, self.o.ptr, d, T, 0, None)
            # shared expert: the gather entry points with every pair on slice 0 (as engine/qwen4_cuda.c:1029 does)
            L.kc_mv_gu(stream, Q4, tab.at(4 * C.sizeof(arr[0])), tab.at(5 * C.sizeof(arr[0])), d, d, x_ptr, d, self.a.ptr, d,
                       self.sel0.ptr, T, 1, None)
            L.kc_mv(stream, Q4, arr[6], d, d, self.a.ptr, d, self.sh.ptr, d, T, 0, None)
        else:
            L.kc_pack_input_bf16(stream, x_ptr, self.px.ptr, C.c_size_t(T * d))
            for i, y in enumerate((self.q, self.kk, self.v)):
                L.kc_mm_packed(stream, Q4, arr[i], d, d, self.px.ptr, d, y.ptr, d, T, 0, None)
            L.kc_pack_input_bf16(stream, self.q.ptr, self.pa.ptr, C.c_size_t(T * d))
            L.kc_mm_packed(stream, Q4, arr[3], d, d, self.pa.ptr, d, self.o.ptr, d, T, 0, None)
            L.kc_mm_packed(stream, Q4, arr[4], d, d, self.px.ptr, d, self.g.ptr, d, T, 0, None)
            L.kc_mm_packed(stream, Q4, arr[5], d, d, self.px.ptr, d, self.u.ptr, d, T, 0, None)
            L.kc_swiglu(stream, self.g.ptr, self.u.ptr, self.a.ptr, T * d)
            L.kc_pack_input_bf16(stream, self.a.ptr, self.pa.ptr, C.c_size_t(T * d))
            L.kc_mm_packed(stream, Q4, arr[6], d, d, self.pa.ptr, d, self.sh.ptr, d, T, 0, None)


def moe_workload(name, steps, warmup, n_layers, no_graph, q4_gemm_from=9):
    from nanoseedlm_amd import backend, moe, packs
    cfgs = {"c2": dict(E=128, k=8, d=2048, ff=768, fmt=packs.MF_SEED4P4), "c3": dict(E=64, k=4, d=2880, ff=2880, fmt=packs.MF_SEED4)}
    c = cfgs[name[:2]]
    T = int(name[3:])
    E, k, d, ff, fmt = c["E"], c["k"], c["d"], c["ff"], c["fmt"]
    rng = np.random.default_rng(20261125)
    mk = packs.seed4p4 if fmt == packs.MF_SEED4P4 else packs.seed4
    st = moe.MoeStack(n_layers, E, k, d, ff, fmt=fmt, router=moe.ROUTE_SOFTMAX, max_rows=max(T, 8))
    for l in range(n_layers):
        gate, up, down = mk(rng, E, ff, d, eb=-22), mk(rng, E, ff, d, eb=-22), mk(rng, E, d, ff, eb=-22)
        rw = packs.f32_to_bf16_bits((rng.standard_normal((E, d)) * 0.02).astype(np.float32))
        st.set_layer(l, gate, up, down, rw)
        del gate, up, down
    st.finalize()
    q4 = Q4Projections(rng, n_layers, d, T, q4_gemm_from) if name[:2] == "c3" else None
    NX = 16
    xs = [moe.DevBuf.from_array(packs.round_bf16(rng.standard_normal((T, d)).astype(np.float32))) for _ in range(NX)]
    out = moe.DevBuf(4 * T * d)
    stream = moe.new_stream()
    combos = [(l, xi) for xi in range(NX) for l in range(n_layers)]
    graphs = None
    if not no_graph:
        for l, xi in combos[:2]:
            st.step(stream, l, xs[xi].ptr, T, out.ptr)          # warm every kernel before capture
            if q4:
                q4.run(stream, l, xs[xi].ptr)
        moe.device_sync()

        def capture(l, xi):
            if not q4:
                return st.graph_of_step(stream, l, xs[xi].ptr, T, out.ptr)
            backend.check(st.L.nslm_graph_begin(stream), "nslm_graph_begin")
            st.step(stream, l, xs[xi].ptr, T, out.ptr)
            q4.run(stream, l, xs[xi].ptr)
            g = C.c_void_p(st.L.nslm_graph_end(stream))
            if not g:
                raise RuntimeError("graph capture failed")
            return g
        graphs = [capture(l, xi) for l, xi in combos]

    def run(i):
        l, xi = combos[i % len(combos)]
        if graphs:
            st.launch(graphs[i % len(combos)], stream)
        else:
            st.step(stream, l, xs[xi].ptr, T, out.ptr)
            if q4:
                q4.run(stream, l, xs[xi].ptr)

    # A step that is one launch is issued from the C host's own loop (nslm_moe_step_seq): with an interpreter between launches of
    # ~23 us the timed region measured the interpreter, not the kernel.
    seq = graphs is None and q4 is None

    def run_many(first, n, before=None, after=None):
        if seq:   # (the events recorded by the same call, directly around the steps)
            idx = [combos[(first + i) % len(combos)] for i in range(n)]
            st.step_seq(stream, [l for l, _ in idx], [xs[xi].ptr for _, xi in idx], T, out.ptr, before, after)
        else:
            if before:
                before.record(stream)
            for i in range(n):
                run(first + i)
            if after:
                after.record(stream)

    t_pre = time.perf_counter()
    while time.perf_counter() - t_pre < PREWARM_S:
        run_many(0, 256)
        moe.device_sync()
    run_many(0, warmup)
    moe.device_sync()
    e0, e1 = moe.Event(), moe.Event()
    t0 = time.perf_counter()
    run_many(warmup, steps, e0, e1)
    e1.sync()
    moe.device_sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms = e1.ms_since(e0) / steps
    fail_on_kernel_error(st)

    # bytes: unique selected experts x expert bytes + the BF16 router weight; at batch 1 every pair is unique
    uniq = []
    for i in range(min(steps, len(combos))):
        l, xi = combos[(warmup + i) % len(combos)]
        st.step(stream, l, xs[xi].ptr, T, out.ptr)
        ind, _ = st.last_routing(T)
        uniq.append(len(set(ind.reshape(-1).tolist())))
    fail_on_kernel_error(st)
    eb = st.expert_bytes()
    bytes_step = float(np.mean(uniq)) * eb + E * d * 2 + (q4.bytes_per_layer if q4 else 0)
    res = dict(ms_per_step=ms, wall_ms_per_step=wall_ms / steps, bytes_per_step=bytes_step, tokens=T,
               flops_per_step=2.0 * T * k * 3 * d * ff + (2.0 * T * 7 * d * d if q4 else 0.0))

    # dominant kernel alone, timed with events on its stream
    P = T * k
    L = backend.hip()
    if T <= 8:
        ind = moe.DevBuf.from_array(np.stack([rng.permutation(E)[:k] for _ in range(T * NX)]).astype(np.int32))
        A = moe.DevBuf(4 * P * ff)
        reps = max(50, steps)
        st.L.nslm_moe_tab.restype = C.c_void_p

        def gu(i):
            l, xi = combos[i % len(combos)]
            g = C.c_void_p(st.L.nslm_moe_tab(st.h, l, 0))
            u = C.c_void_p(st.L.nslm_moe_tab(st.h, l, 1))
            L.kc_mv_gu(stream, fmt, g, u, d, ff, xs[xi].ptr, d, A.ptr, ff, ind.at(4 * P * xi), P, k, None)
        for i in range(10):
            gu(i)
        moe.device_sync()
        e0.record(stream)
        for i in range(reps):
            gu(i)
        e1.record(stream)
        e1.sync()
        kms = e1.ms_since(e0) / reps
        kbytes = P * 2 * eb / 3.0        # P pairs x (gate + up) records
        part = dict(kernel="k_mv_seed<gate+up+SwiGLU> launched alone", launch_us=kms * 1e3, algorithmic_bytes=kbytes,
                    achieved=kbytes / kms / 1e6, frac=kbytes / kms / 1e6 / HBM_PEAK_GBS)
        # The timed step is ONE launch of the persistent decode kernel (router, top-k, gate + up + SwiGLU, down, combine),
        # so that kernel is the dominant one: its algorithmic bytes are the step's, its duration the step's event time.
        # Its launch duration is the step's event time: HIP events over the timed region on the launch stream (launches are
        # queued back to back, so there is no gap between them unless the step is wrapped in a graph).
        res["roofline"] = dict(bound="hbm", achieved=bytes_step / ms / 1e6, peak=HBM_PEAK_GBS, unit="GB/s",
                               frac=bytes_step / ms / 1e6 / HBM_PEAK_GBS,
                               kernel=("k_moe_decode_cu" if T == 1 else "k_moe_decode") + " (one launch per step)",
                               launch_us=ms * 1e3, algorithmic_bytes=bytes_step, gate_up_alone=part, **counters_of(name))
        ind.free(); A.free()
    else:
        # Batched steps: 9 to 24 rows of C2 are one launch of the grouped persistent kernel; beyond that (and for C3) three
        # grouped GEMM launches over tiles of a few pairs each dominate, and what they spend is the records' expansion, not
        # matrix flops: priced against HBM on the records the step has to read.
        res["roofline"] = dict(bound="hbm", achieved=bytes_step / ms / 1e6, peak=HBM_PEAK_GBS, unit="GB/s",
                               frac=bytes_step / ms / 1e6 / HBM_PEAK_GBS,
                               kernel=("k_moe_decode_grouped (one launch per step)" if T <= 24 and name[:2] == "c2" else
                                       "k_mm_stream<1, %d, %d> grouped (two launches of the step: gate + up + SwiGLU, down; with its glue kernels)" % (1 if T <= 32 else 4, 2 if T <= 32 and name[:2] == "c2" else 3)),
                               launch_us=ms * 1e3, algorithmic_bytes=bytes_step, **counters_of(name))
    desc = {"c2": "C2 MoE decode layer step: 128 experts seeded P=4, top-8 softmax, hidden 2048, intermediate 768",
            "c3": "C3 mixed-format layer step: 64 experts seeded P=3, top-4, hidden 2880, intermediate 2880, plus seven 2880 x 2880 Q4-g64 projections (q, k, v, o, shared gate / up / down)"}[name[:2]]
    res["config"] = {"workload": f"{desc}, batch {T}", "layers_rotated": n_layers, "inputs_rotated": NX,
                     "launch": "stream" if no_graph else "hipGraph per step",
                     "router_weight": "bf16 (cast of the fp32 ~N(0, 0.02) draw; the reference has no f32 weight format)"}
    res["cpu_sample"] = dict(shapes=[(ff, d), (ff, d), (d, ff)], reps=k, fmt=fmt)
    st.close()
    return res


def model_workload(name, steps, warmup, no_graph, branches=False, splits=32):
    """Config 4: greedy decode of the whole synthetic model (24 layers of MLA attention over an FP8 latent cache + 128 seeded
    experts top-8 + a shared expert, tied BF16 LM head over 151936 ids), the cache pre-filled so that the timed steps end at
    the 4096th position.  A step = one token for each of the batch's sequences, all of its launches in one hipGraph."""
    from nanoseedlm_amd import backend, model, moe
    T = int(name[3:])
    cfg = dict(n_layer=24, d=2048, n_head=16, head_dim=128, r=512, rope=64, n_exp=128, top_k=8, ff=768, ff_shared=768, vocab=151936,
               max_ctx=4096, max_rows=T, kv_fmt=backend.KV_FP8, n_splits=splits, eps=1e-6, rope_theta=10000.0)
    if steps + warmup + 8 > cfg["max_ctx"]:
        sys.exit("bench.py: c4 decodes towards position 4096; --steps + --warmup must stay below 4088")
    m = model.DecodeModel(**cfg)
    m.fill_random(seed=20261125, eb=-24)
    m.set_branches(branches)
    start = cfg["max_ctx"] - steps - warmup - 4
    rng = np.random.default_rng(4)
    m.fill_cache(T, start, seed=5)
    m.start(rng.integers(0, cfg["vocab"], T), np.full(T, start))
    stream = moe.new_stream()
    m.step(stream, T)                                                  # warm every kernel before capture
    moe.device_sync()
    g = None if no_graph else m.graph_of_step(stream, T)

    def run():
        if g:
            m.launch(g, stream)
        else:
            m.step(stream, T)
    seen = set()
    for _ in range(warmup):
        run()
    moe.device_sync()
    e0, e1 = moe.Event(), moe.Event()
    t0 = time.perf_counter()
    e0.record(stream)
    for _ in range(steps):
        run()
    e1.record(stream)
    e1.sync()
    moe.device_sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms = e1.ms_since(e0) / steps
    ids, logits = m.ids(T), m.logits(T)           # (both raise when the persistent MoE kernel's error word is set)
    fail_on_kernel_error()
    if not np.isfinite(logits).all():
        raise RuntimeError("the synthetic model's logits are not finite")
    # bytes a step has to read: weight records (top-k experts per row; rows of a batch share some, counted once from the
    # last layer's routing), the latent cache rows up to each sequence's position, the LM head
    mh = C.c_void_p(m.L.nslm_model_moe(m.h))
    ind = np.zeros((T, cfg["top_k"]), dtype=np.int32)
    wt = np.zeros((T, cfg["top_k"]), dtype=np.float32)
    backend.check(m.L.nslm_moe_last_routing(mh, T, ind.ctypes.data_as(C.c_void_p), wt.ctypes.data_as(C.c_void_p)), "nslm_moe_last_routing")
    uniq = len(set(ind.reshape(-1).tolist()))
    m.L.nslm_moe_expert_bytes.restype = C.c_uint64
    eb = int(m.L.nslm_moe_expert_bytes(mh))
    pos_mean = cfg["max_ctx"] - 4 - steps / 2.0
    kv_bytes = T * cfg["n_layer"] * pos_mean * (cfg["r"] + cfg["rope"]) * (1 + 1 / 32.0)
    bytes_step = m.step_bytes() - cfg["n_layer"] * cfg["top_k"] * eb + cfg["n_layer"] * uniq * eb + kv_bytes
    flops = 2.0 * T * (m.step_bytes() - 2 * cfg["vocab"] * cfg["d"]) / 4.5 * 8 + 2.0 * T * cfg["vocab"] * cfg["d"]
    res = dict(ms_per_step=ms, wall_ms_per_step=wall_ms / steps, bytes_per_step=bytes_step, tokens=T, flops_per_step=flops)
    res["roofline"] = dict(bound="hbm", achieved=bytes_step / ms / 1e6, peak=HBM_PEAK_GBS, unit="GB/s", frac=bytes_step / ms / 1e6 / HBM_PEAK_GBS,
                           traffic=None, traffic_source=None, kernel="whole decode step (%s x 24 is the largest share)" % ("k_moe_decode_cu" if T == 1 else "k_moe_decode" if T <= 8 else "k_moe_decode_grouped")
                           if T <= 24 else "whole decode step (grouped k_mm_stream launches are the largest share)",
                           launch_us=ms * 1e3, algorithmic_bytes=bytes_step)
    res["config"] = {"workload": f"C4 full synthetic model greedy decode: 24 layers, hidden 2048, MLA 16 heads (latent 512 + rope 64, FP8 cache), "
                                 f"128 seeded P=4 experts top-8 (intermediate 768) + shared expert, vocab 151936 BF16 LM head, batch {T}, "
                                 f"positions {start + 1 + warmup}..{start + warmup + steps}",
                     "launch": ("stream" if no_graph else "hipGraph per step") + (", side-stream branches" if branches else ""), "unique_experts_last_layer": uniq,
                     "last_ids": [int(v) for v in ids[:4]]}
    res["cpu_sample"] = dict(shapes=[(cfg["ff"], cfg["d"]), (cfg["ff"], cfg["d"]), (cfg["d"], cfg["ff"])], reps=cfg["top_k"], fmt=4)
    m.close()
    return res


def dense_workload(name, steps, warmup, matrices=64):
    from nanoseedlm_amd import backend, moe, packs
    L = backend.hip()
    rng = np.random.default_rng(20261125)
    stream = moe.new_stream()
    e0, e1 = moe.Event(), moe.Event()
    if name == "c0":
        R = K = 4096
        NM = max(1, matrices)   # 64 (604 MB: every launch reads its records from HBM); 1 = the matrix stays in the 256 MB Infinity Cache
        p = packs.seed4p4(rng, NM, R, K, eb=-22)
        ds, dc, de = moe.DevBuf.from_array(p["seeds"]), moe.DevBuf.from_array(p["coefs"]), moe.DevBuf.from_array(p["codes"])
        x = moe.DevBuf.from_array(rng.standard_normal(K).astype(np.float32))
        y = moe.DevBuf(4 * R)
        sl = []
        for i in range(NM):
            w = backend.WSlice()
            w.p[0], w.p[1], w.p[3] = ds.ptr.value + i * R * K // 4, dc.ptr.value + i * R * K // 4, de.ptr.value + i * R * K // 16
            w.eb = -22
            sl.append(w)

        def run(i):
            L.kc_mv(stream, packs.MF_SEED4P4, sl[i % NM], K, R, x.ptr, K, y.ptr, R, 1, 0, None)
        # (the launches of a 9 us kernel are issued by the C host's own loop, the events by the same call: an interpreter between
        # the launches is as slow as the kernel)
        slarr = (backend.WSlice * NM)(*sl)

        def run_seq(first, n, nm=NM, before=None, after=None):
            backend.check(backend.host().nslm_mv_seq(stream, packs.MF_SEED4P4, slarr, nm, first, n, K, R, x.ptr, y.ptr,
                                                     before.e if before else None, after.e if after else None), "nslm_mv_seq")
        bytes_step, flops, T = R * K * 36 / 64.0, 2.0 * R * K, 1
        desc, bound = f"C0 dense seeded GEMV: W 4096x4096 P=4, batch 1, rotating over {NM} matri{'x' if NM == 1 else 'ces'}", "hbm"
        sample = dict(shapes=[(R, K)], reps=1, fmt=packs.MF_SEED4P4)
    elif name == "deq":
        # The weights' form of the decode alone, through a product entry point: kc_slice_deq regenerates the BF16 weights of a
        # 4096 x 4096 P=4 slice (the exact integer sums on v_dot2_i32_i16, one convert and one multiply a weight), rotating over
        # the matrices.  Reads 9.4 MB of records and writes 33.6 MB a launch.
        R = K = 4096
        NM = max(1, matrices)
        p = packs.seed4p4(rng, NM, R, K, eb=-22)
        ds, dc, de = moe.DevBuf.from_array(p["seeds"]), moe.DevBuf.from_array(p["coefs"]), moe.DevBuf.from_array(p["codes"])
        y = moe.DevBuf(2 * R * K)
        sl = []
        for i in range(NM):
            w = backend.WSlice()
            w.p[0], w.p[1], w.p[3] = ds.ptr.value + i * R * K // 4, dc.ptr.value + i * R * K // 4, de.ptr.value + i * R * K // 16
            w.eb = -22
            sl.append(w)

        def run(i):
            L.kc_slice_deq(stream, packs.MF_SEED4P4, sl[i % NM], K, R, y.ptr)
        bytes_step, flops, T = R * K * 36 / 64.0, 0.0, 1
        desc, bound = f"weights of a 4096x4096 P=4 slice regenerated as BF16 (kc_slice_deq), rotating over {NM} matrices", "hbm"
        sample = dict(shapes=[(R, K)], reps=1, fmt=packs.MF_SEED4P4)
    else:
        R, K, T = 14336, 4096, 512
        p = packs.seed4p4(rng, 1, R, K, eb=-22)
        ds, dc, de = moe.DevBuf.from_array(p["seeds"]), moe.DevBuf.from_array(p["coefs"]), moe.DevBuf.from_array(p["codes"])
        x = moe.DevBuf.from_array(packs.f32_to_bf16_bits(rng.standard_normal((T, K)).astype(np.float32)))
        y = moe.DevBuf(4 * T * R)
        w = backend.WSlice()
        w.p[0], w.p[1], w.p[3] = ds.ptr.value, dc.ptr.value, de.ptr.value
        w.eb = -22

        def run(i):
            L.kc_mm_packed(stream, packs.MF_SEED4P4, w, K, R, x.ptr, K, y.ptr, R, T, 0, None)
        bytes_step, flops = R * K * 36 / 64.0, 2.0 * T * R * K
        desc, bound = "C1 seeded prefill GEMM: W 14336x4096 P=4, X bf16 [512 x 4096], bf16 MFMA, fp32 accumulate", "mfma"
        sample = dict(shapes=[(R, K)], reps=1, fmt=packs.MF_SEED4P4)
    t_pre = time.perf_counter()
    while time.perf_counter() - t_pre < PREWARM_S:
        for i in range(256):
            run(i)
        moe.device_sync()
    if name == "c0":
        run_seq(0, warmup)
    else:
        for i in range(warmup):
            run(i)
    moe.device_sync()
    t0 = time.perf_counter()
    if name == "c0":
        run_seq(warmup, steps, NM, e0, e1)
    else:
        e0.record(stream)
        for i in range(steps):
            run(warmup + i)
        e1.record(stream)
    e1.sync()
    moe.device_sync()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms = e1.ms_since(e0) / steps
    fail_on_kernel_error()
    res = dict(ms_per_step=ms, wall_ms_per_step=wall_ms / steps, bytes_per_step=bytes_step, tokens=T, flops_per_step=flops)
    resident = None
    if name == "c0":
        # The same launches on ONE matrix, which then stays in the Infinity Cache (9.4 MB of 256 MB), as the reference's kernel
        # bench offers beside its rotating mode (harness/nslm-mova-kbench.c:8-9,149).  If this is no faster than the rotating
        # figure, HBM is not what bounds the kernel.
        run_seq(0, max(warmup, 64), 1)
        moe.device_sync()
        run_seq(0, steps, 1, e0, e1)
        e1.sync()
        rms = e1.ms_since(e0) / steps
        fail_on_kernel_error()
        resident = dict(launch_us=rms * 1e3, achieved=bytes_step / rms / 1e6, frac=bytes_step / rms / 1e6 / HBM_PEAK_GBS, matrices=1)
    if bound == "hbm":
        res["roofline"] = dict(bound="hbm", achieved=bytes_step / ms / 1e6, peak=HBM_PEAK_GBS, unit="GB/s",
                               frac=bytes_step / ms / 1e6 / HBM_PEAK_GBS, kernel="k_mv_seed<dense>" if name == "c0" else "k_deq_seed",
                               launch_us=ms * 1e3, algorithmic_bytes=bytes_step, cache_resident=resident, **counters_of(name))
    else:
        res["roofline"] = dict(bound="mfma", achieved=flops / ms / 1e9, peak=MFMA_BF16_PEAK_TFLOPS, unit="TFLOP/s",
                               frac=flops / ms / 1e9 / MFMA_BF16_PEAK_TFLOPS, kernel="k_mm_stream<2, 8> (BF16 activations, 512-token tile)",
                               launch_us=ms * 1e3, algorithmic_flops=flops, **counters_of(name))
    res["config"] = {"workload": desc, "launch": "stream"}
    res["cpu_sample"] = sample
    return res


def cpu_baseline(sample, budget_s=12.0):
    """The CPU decode-in-dot-product on this host's cores over the workload's matrices (a bounded sample: the matrices
    one token reads, repeated until about budget_s of CPU time)."""
    from nanoseedlm_amd import packs
    from oracle import oracle as orc
    orc.build()
    ref = orc.ref()
    cores = os.cpu_count() or 1
    threads = min(cores, 16)
    rng = np.random.default_rng(7)
    fmt = sample["fmt"]
    mats = []
    weights = 0
    for (R, K) in sample["shapes"]:
        if R * K > 2 ** 25:          # bound the sample: at most 32 M weights per matrix
            R = 2 ** 25 // K
        p = (packs.seed4p4 if fmt == packs.MF_SEED4P4 else packs.seed4)(rng, 1, R, K, eb=-22)
        mats.append((p, R, K, rng.standard_normal(K).astype(np.float32)))
        weights += R * K
    vp = lambda a: a.ctypes.data_as(C.c_void_p)
    if ref is not None:
        kind = "reference"
        tiled = []
        for p, R, K, x in mats:
            t = ref.ref_tile4(vp(p["seeds"][0]), vp(p["coefs"][0]), vp(p["codes"][0]), -22, R, K // 8) if fmt == packs.MF_SEED4P4 \
                else ref.ref_tile3(vp(p["seeds"][0]), vp(p["nibs"][0]), -22, R, K // 8)
            tiled.append((C.c_void_p(t), x, np.zeros(R, dtype=np.float32)))

        def once():
            for t, x, y in tiled:
                ref.ref_tiled_matmul(t, vp(x), 1, vp(y), threads)
    else:
        kind = "port"
        threads = min(cores, 16)

        def once():
            for p, R, K, x in mats:
                if fmt == packs.MF_SEED4P4:
                    orc.cpu_seed4_matvec(p["seeds"][0], p["coefs"][0], p["codes"][0], -22, x, R, K // 8, threads)
                else:
                    orc.cpu_seed3_matvec(p["seeds"][0], p["nibs"][0], -22, x, R, K // 8, threads)
    once()
    n, t0 = 0, time.perf_counter()
    best = 1e30
    while time.perf_counter() - t0 < budget_s:
        t1 = time.perf_counter()
        once()
        best = min(best, time.perf_counter() - t1)
        n += 1
    bpw = 0.5625 if fmt == packs.MF_SEED4P4 else 0.5
    return dict(value=weights * bpw / best / 1e9, unit="GB/s", cores=threads, kind=kind, gweights_per_s=weights / best / 1e9,
                sample=f"{len(mats)} matrices {[(R, K) for _, R, K, _ in mats]} ({weights / 1e6:.1f} M weights) x {n} passes, best pass "
                       f"{best * 1e3:.2f} ms, host cores visible {cores}, loadavg {open('/proc/loadavg').read().split()[0]}"
                       + ("" if ref is not None else "; scalar C restatement (compiled reference not present)"))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="c2b1")
    ap.add_argument("--layers", type=int, default=4)
    ap.add_argument("--matrices", type=int, default=64, help="c0: matrices the launches rotate over (64: records from HBM; 1: resident in the Infinity Cache)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--q4-gemm-from", type=int, default=9, help="c3: rows from which the Q4 projections take the grouped GEMM launches instead of matvecs")
    ap.add_argument("--no-graph", action="store_true", help="c4: plain stream launches instead of one hipGraph per step (c2 / c3 steps are stream launches unless --graph)")
    ap.add_argument("--graph", action="store_true", help="c2 / c3: one hipGraph per step")
    ap.add_argument("--splits", type=int, default=32, help="c4: pieces the attention of a (row, head group) is split into over the context")
    ap.add_argument("--branches", action="store_true", help="c4: independent launches of a layer on side streams (parallel graph branches; measured slower)")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MiB",
                    help="after the workload, run 20 device-to-device copies of this size: a copy kernel of known traffic "
                         "for scaling rocprofv3's FETCH_SIZE / WRITE_SIZE counters")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build measures one GPU (one process, one MI355X, no collectives); run with --gpus 1")
    from nanoseedlm_amd import backend
    backend.require_gpu()
    if a.workload[:2] in ("c2", "c3"):
        # Layer steps are issued as plain launches on the stream: a step of up to 24 rows of C2 is ONE launch, and around the
        # about ten launches of a batched step (or the five of C3 with its projections) a hipGraph replay a step measured
        # 5 us slower than the launches themselves (C2 at 32 rows 253.9 against 248.4 us, C3 at 1 row 92.2 against 87.1).
        r = moe_workload(a.workload, a.steps, a.warmup, a.layers, a.no_graph or not a.graph, a.q4_gemm_from)
    elif a.workload[:2] == "c4":
        r = model_workload(a.workload, a.steps, a.warmup, a.no_graph, a.branches, a.splits)
    else:
        r = dense_workload(a.workload, a.steps, a.warmup, a.matrices)
    gbs = r["bytes_per_step"] / r["ms_per_step"] / 1e6
    line = {
        "metric": METRIC, "value": gbs, "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic", "config": r["config"], "pct_hbm_peak": 100.0 * gbs / HBM_PEAK_GBS,
        "tokens_per_s": r["tokens"] / r["ms_per_step"] * 1e3, "bytes_per_step": r["bytes_per_step"],
        "tflops": r["flops_per_step"] / r["ms_per_step"] / 1e9, "host_ms_per_step": r["wall_ms_per_step"],
        "roofline": r["roofline"],
        "prewarm_s": 0.0 if a.workload[:2] == "c4" else PREWARM_S,   # untimed steps of the same workload before the W warmup steps
    }
    line["cpu_baseline"] = None if a.no_cpu else cpu_baseline(r["cpu_sample"])
    if a.calibrate_copy > 0:
        from nanoseedlm_amd import moe
        n = a.calibrate_copy << 20
        src, dst = moe.DevBuf(n), moe.DevBuf(n)
        for _ in range(20):
            backend.check(backend.hip().nh_memcpy_d2d(dst.ptr, src.ptr, C.c_size_t(n)), "nh_memcpy_d2d")
        moe.device_sync()
        src.free(); dst.free()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
