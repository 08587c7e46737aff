"""A whole (tiny) synthetic model's greedy decode on the GPU against a reference composition of the oracle's pieces:
embedding, RMSNorm, seeded dense projections, per-head maps, RoPE + latent cache (BF16 and FP8), latent attention, routed
experts + shared expert, LM head, arg-max - several steps, two sequences at different positions, so the caches are read
back.  The reference feeds on the GPU's tokens; logits must agree within the accumulated BF16 rounding of the stack."""
import numpy as np
import pytest

from nanoseedlm_amd import packs
from test_gpu_moe import expert_ref

pytestmark = pytest.mark.gpu
r_ = packs.round_bf16


def f64(a):
    return np.asarray(a, dtype=np.float64)


def dense_ref(orc, p, x, gemm):
    """bf16(W x): exact weights and f32 activations in the matvec, both rounded to BF16 in the MFMA GEMM."""
    W = orc.rows_f32(p["fmt"], orc.make_slice(p["fmt"], p["seeds"][0], p["coefs"][0], None, p["codes"][0], eb=int(p["eb"][0])), p["R"], p["K"])
    if gemm:
        W, x = r_(W), r_(np.asarray(x, dtype=np.float32))
    return r_((f64(W) @ f64(x)).astype(np.float32))


def norm_ref(x, w, eps):
    x = f64(x)
    return (x / np.sqrt(np.mean(x * x) + eps) * (1.0 + f64(w))).astype(np.float32)


@pytest.mark.parametrize("T,branches", [(2, False), (2, True), (12, False), (40, False)])
@pytest.mark.parametrize("kv", ["bf16", "fp8"])
def test_tiny_model_decode(oracle, kv, T, branches):
    from nanoseedlm_amd import backend, model, moe
    backend.require_gpu()
    rng = np.random.default_rng(2024 + T)
    gemm = T > 8                                                       # above 8 rows the experts, router and LM head run the packed GEMMs
    dgemm = T > 32                                                     # the dense projections stay matvecs (exact weights) up to 32 rows
    cfg = dict(n_layer=2, d=128, n_head=2, head_dim=64, r=64, rope=64, n_exp=8, top_k=2, ff=64, ff_shared=64, vocab=96, max_ctx=16,
               max_rows=T, kv_fmt=backend.KV_FP8 if kv == "fp8" else backend.KV_BF16, n_splits=2, eps=1e-6, rope_theta=10000.0)
    m = model.DecodeModel(**cfg)
    m.set_branches(branches)                                           # independent launches of a layer on side streams
    L, d, H, hd, r, rope, E, k = cfg["n_layer"], cfg["d"], cfg["n_head"], cfg["head_dim"], cfg["r"], cfg["rope"], cfg["n_exp"], cfg["top_k"]
    QD, ffs, V = H * hd, cfg["ff_shared"], cfg["vocab"]
    shapes = {model.W_Q: (QD, d), model.W_KVA: (r, d), model.W_KR: (rope, d), model.W_O: (d, QD), model.W_SG: (ffs, d), model.W_SU: (ffs, d),
              model.W_SD: (d, ffs)}
    Wd, Wh, Wn, Wx = {}, {}, {}, {}
    for l in range(L):
        for w, (R, K) in shapes.items():
            Wd[l, w] = packs.seed4p4(rng, 1, R, K, eb=-9, code_max=3)
            m.set_dense(l, w, Wd[l, w])
        for w, (O, I) in ((model.H_QRMIX, (rope, hd)), (model.H_QLAT, (r, hd)), (model.H_VUP, (hd, r))):
            Wh[l, w] = packs.f32_to_bf16_bits((rng.standard_normal((H, O, I)) / np.sqrt(I)).astype(np.float32))
            m.set_heads(l, w, Wh[l, w])
        for w in range(2):
            Wn[l, w] = (0.1 * rng.standard_normal(d)).astype(np.float32)
            m.set_norm(l, w, Wn[l, w])
        gate, up, down = (packs.seed4p4(rng, E, cfg["ff"], d, eb=-9, code_max=3), packs.seed4p4(rng, E, cfg["ff"], d, eb=-10, code_max=3),
                          packs.seed4p4(rng, E, d, cfg["ff"], eb=-9, code_max=3))
        rw = packs.f32_to_bf16_bits((rng.standard_normal((E, d)) * 0.05).astype(np.float32))
        Wx[l] = (gate, up, down, rw)
        m.set_experts(l, gate, up, down, rw)
    Wn[L, 0] = (0.1 * rng.standard_normal(d)).astype(np.float32)
    m.set_norm(L, 0, Wn[L, 0])
    emb = packs.f32_to_bf16_bits((rng.standard_normal((V, d)) * 0.05).astype(np.float32))
    m.set_embed(emb)
    m.finalize()
    embf = packs.bf16_bits_to_f32(emb)
    inv = np.array([cfg["rope_theta"] ** (-2.0 * p / rope) for p in range(rope // 2)]).astype(np.float32)
    scale = np.float32(1.0) / np.sqrt(np.float32(hd + rope))
    ids, pos = rng.integers(0, cfg["vocab"], T).astype(np.int32), rng.integers(0, 6, T).astype(np.int32)
    # the reference's caches [layer][slot][position]; slot 1 starts at position 3 with zeros below it (as the device's)
    lat_c = np.zeros((L, T, cfg["max_ctx"], r), dtype=np.float32)
    kr_c = np.zeros((L, T, cfg["max_ctx"], rope), dtype=np.float32)

    def cache_value(v):
        if kv == "bf16":
            return r_(v)
        c, s = oracle.fp8_row(r_(v)[None])
        return oracle.fp8_decode(c, s)[0]

    m.start(ids, pos)
    worst, moved, seen = 0.0, 0.0, set()
    for step in range(4):
        m.step(None, T)
        got = m.logits(T)
        nxt = m.ids(T)
        for t in range(T):
            x = embf[ids[t]].copy()
            for l in range(L):
                xn = norm_ref(x, Wn[l, 0], cfg["eps"])
                q = dense_ref(oracle, Wd[l, model.W_Q], xn, dgemm)
                c = dense_ref(oracle, Wd[l, model.W_KVA], xn, dgemm)
                kr = dense_ref(oracle, Wd[l, model.W_KR], xn, dgemm)
                qr = oracle.heads_map(packs.bf16_bits_to_f32(Wh[l, model.H_QRMIX]).reshape(H * rope, hd), q[None], H, rope, hd, QD, hd)[0]
                ql = oracle.heads_map(packs.bf16_bits_to_f32(Wh[l, model.H_QLAT]).reshape(H * r, hd), q[None], H, r, hd, QD, hd)[0]
                half = rope // 2
                qrot, krot = np.zeros((H, rope), np.float32), np.zeros(rope, np.float32)
                for i in range(half):
                    for h in range(H):
                        y0, y1 = oracle.rope_pair(float(qr[h, i]), float(qr[h, i + half]), int(pos[t]), float(inv[i]))
                        qrot[h, i], qrot[h, i + half] = r_(np.float32(y0)), r_(np.float32(y1))
                    y0, y1 = oracle.rope_pair(float(kr[i]), float(kr[i + half]), int(pos[t]), float(inv[i]))
                    krot[i], krot[i + half] = y0, y1
                lat_c[l, t, pos[t]] = cache_value(c)
                kr_c[l, t, pos[t]] = cache_value(krot)
                olat = np.stack([oracle.mla_attn(ql[h], qrot[h], lat_c[l, t], kr_c[l, t], int(pos[t]), float(scale)) for h in range(H)])
                o = oracle.heads_map(packs.bf16_bits_to_f32(Wh[l, model.H_VUP]).reshape(H * hd, r), olat.reshape(1, H * r), H, hd, r, H * r, r)[0]
                x = r_(x + dense_ref(oracle, Wd[l, model.W_O], o.reshape(-1), dgemm))
                xn = norm_ref(x, Wn[l, 1], cfg["eps"])
                gate, up, down, rw = Wx[l]
                xe = r_(xn) if gemm else xn
                lg = r_((f64(packs.bf16_bits_to_f32(rw)) @ f64(xe)).astype(np.float32))
                ind, wt = oracle.route_softmax(lg[None], k)
                ys = np.stack([expert_ref(oracle, gate, up, down, int(ind[0, j]), xe, gemm=gemm) for j in range(k)])
                mo = (f64(wt[0])[:, None] * ys).sum(0)
                g = dense_ref(oracle, Wd[l, model.W_SG], xn, dgemm)
                u = dense_ref(oracle, Wd[l, model.W_SU], xn, dgemm)
                sg = r_((1 / (1 + np.exp(-f64(g)))).astype(np.float32))
                a = r_(r_(g * sg) * u)
                sh = dense_ref(oracle, Wd[l, model.W_SD], a, dgemm)
                x = r_(x + r_((mo + f64(sh)).astype(np.float32)))
            xn = norm_ref(x, Wn[L, 0], cfg["eps"])
            want = r_((f64(embf) @ f64(r_(xn) if gemm else xn)).astype(np.float32))
            err = np.max(np.abs(got[t] - want)) / np.max(np.abs(want))
            worst = max(worst, err)
            moved = max(moved, float(np.linalg.norm(x - embf[ids[t]]) / np.linalg.norm(embf[ids[t]])))
            # two layers deep, every tensor boundary rounded to BF16 (a flipped rounding is 2^-8 of a value) and an attention
            # softmax in between: the composed bound is 2e-2 (measured: at most 1e-2); each kernel's own bound is one BF16 ulp
            assert err < 2e-2, (step, t, err)
            assert got[t, nxt[t]] == got[t].max()                      # the next id is the GPU's own arg-max
        seen.update(int(v) for v in nxt)
        ids, pos = nxt.copy(), pos + 1
    m.close()
    print("worst relative logit error", worst, "layers moved the stream by", moved, "tokens seen", sorted(seen))
    assert moved > 0.3, "the layers must matter to the logits for this comparison to test them"


@pytest.mark.parametrize("T", [2, 12])
def test_graph_replay_equals_eager_steps(T):
    """The step captured once in a hipGraph and replayed (positions and ids live on the device) gives the bits of eager
    launches at every step, with eager work and synchronisations of another model between the replays."""
    from nanoseedlm_amd import backend, model, moe
    backend.require_gpu()
    cfg = dict(n_layer=2, d=128, n_head=2, head_dim=64, r=64, rope=64, n_exp=8, top_k=2, ff=64, ff_shared=64, vocab=96, max_ctx=24,
               max_rows=T, kv_fmt=backend.KV_FP8, n_splits=2, eps=1e-6, rope_theta=10000.0)
    rng = np.random.default_rng(5)
    ids, pos = rng.integers(0, cfg["vocab"], T).astype(np.int32), rng.integers(0, 6, T).astype(np.int32)
    ms = []
    for _ in range(2):
        m = model.DecodeModel(**cfg)
        m.fill_random(seed=11, eb=-13)
        m.start(ids, pos)
        ms.append(m)
    eager, replay = ms
    stream = moe.new_stream()
    replay.step(stream, T)                                           # warm every kernel, then rewind and capture
    moe.device_sync()
    replay.start(ids, pos)
    g = replay.graph_of_step(stream, T)
    seen = set()
    for step in range(6):
        eager.step(None, T)
        a, ia = eager.logits(T), eager.ids(T)
        replay.launch(g, stream)
        moe.device_sync()
        b, ib = replay.logits(T), replay.ids(T)
        assert np.isfinite(a).all() and np.array_equal(a.view(np.uint32), b.view(np.uint32)) and np.array_equal(ia, ib), step
        seen.add(a.tobytes())
    assert len(seen) == 6                                            # the steps differ from one another (positions advance)
    for m in ms:
        m.close()


def test_a_full_cache_slot_refuses_the_next_step():
    """A step writes the cache at every row's position and the positions advance on the device: the host refuses the step
    (and the replay of a captured step) that would write past a sequence slot, and the device-side position saturates."""
    from nanoseedlm_amd import backend, model, moe
    backend.require_gpu()
    T = 2
    cfg = dict(n_layer=2, d=128, n_head=2, head_dim=64, r=64, rope=64, n_exp=8, top_k=2, ff=64, ff_shared=64, vocab=96, max_ctx=8,
               max_rows=T, kv_fmt=backend.KV_BF16, n_splits=2, eps=1e-6, rope_theta=10000.0)
    m = model.DecodeModel(**cfg)
    m.fill_random(seed=3, eb=-13)
    with pytest.raises(RuntimeError):
        m.step(None, T)                                              # no start yet
    m.start(np.array([5, 9], dtype=np.int32), np.array([2, cfg["max_ctx"] - 1], dtype=np.int32))
    assert m.steps_left() == 1
    m.step(None, T)                                                  # row 1 writes its slot's last position
    assert np.isfinite(m.logits(T)).all() and m.steps_left() == 0
    with pytest.raises(RuntimeError):
        m.step(None, T)
    m.start(np.array([5, 9], dtype=np.int32), np.array([0, cfg["max_ctx"] - 3], dtype=np.int32))
    stream = moe.new_stream()
    g = m.graph_of_step(stream, T)
    assert m.steps_left() == 3                                       # the capture itself launched nothing
    for _ in range(3):
        m.launch(g, stream)
    moe.device_sync()
    assert np.isfinite(m.logits(T)).all()
    with pytest.raises(RuntimeError):
        m.launch(g, stream)
    m.close()
