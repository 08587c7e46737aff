"""Parity of the MLA decode-attention kernels (per-head maps, RoPE + cache write, FP8 cache codec, latent attention) against
the CPU oracle, through the C ABI, on the GPU.  Bars as the reference's tests/test_mova_kernels.c:786-1036,1233-1330:
maps and attention within one BF16 ulp + 2e-6 of the double-precision result, RoPE within one BF16 ulp + 1e-6, the latent's
cache codes exactly the C codec's, attention over an FP8 cache bit-equal to attention over the decoded cache."""
import numpy as np
import pytest

from nanoseedlm_amd import packs
from test_gpu_kernels import be, close_bf, make_pack, slice_of   # noqa: F401  (be is a fixture)

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fmt", [packs.MF_BF16, packs.MF_Q8, packs.MF_Q4, packs.MF_SEED4P4])
@pytest.mark.parametrize("O,I,gate", [(96, 128, False), (128, 96, True), (512, 128, False)])
def test_heads_mv(be, oracle, fmt, O, I, gate):
    if fmt in (packs.MF_Q8, packs.MF_Q4) and I % 64:
        pytest.skip("affine groups of 64 need I % 64 == 0")
    rng = np.random.default_rng(O + I + fmt)
    H, T = 4, 3
    p = make_pack(rng, fmt, 1, H * O, I)
    x = packs.round_bf16((rng.standard_normal((T, H * I)) * 2).astype(np.float32))
    g = packs.round_bf16((rng.standard_normal((T, H, O)) * 3).astype(np.float32)) if gate else None
    ebias = np.array([-19, -21, -18, -20], dtype=np.int32) if fmt == packs.MF_SEED4P4 else None
    y = be.kt_heads_w(p, H, O, I, x, H * I, I, g=g, ebias=ebias)
    if fmt == packs.MF_SEED4P4:   # head h's rows with head h's exponent bias
        W = np.concatenate([oracle.rows_f32(fmt, oracle.make_slice(fmt, p["seeds"][0][h * O:(h + 1) * O], p["coefs"][0][h * O:(h + 1) * O], None,
                                                                   p["codes"][0][h * O * I // 16:(h + 1) * O * I // 16], eb=int(ebias[h])), O, I)
                            for h in range(H)])
    else:
        # BF16 / Q8 as BF16 values, Q4 unrounded (the matvec form s q + b)
        W = oracle.rows_f32(fmt, slice_of(oracle, p, 0), H * O, I, round_=1 if fmt == packs.MF_Q8 else 0)
    want = oracle.heads_map(W, x, H, O, I, H * I, I, g=g)
    mag = np.einsum("hoi,thi->tho", np.abs(W).reshape(H, O, I).astype(np.float64), np.abs(x).reshape(T, H, I).astype(np.float64))
    assert np.all(close_bf(y, want.astype(np.float64), 2e-6 + 64 * 1.2e-7 * mag * (4.0 if gate else 1.0)))


@pytest.mark.parametrize("rope", [128, 64])
@pytest.mark.parametrize("fmt", ["bf16", "fp8"])
def test_rope_and_cache_write(be, oracle, rope, fmt):
    rng = np.random.default_rng(rope)
    nh, r, P, T = 4, 96, 10, 2
    kvf = be.KV_FP8 if fmt == "fp8" else be.KV_BF16
    qr0 = packs.round_bf16(rng.standard_normal((T, nh, rope)).astype(np.float32))
    kr = packs.round_bf16(rng.standard_normal((T, rope)).astype(np.float32))
    c = packs.round_bf16(rng.standard_normal((T, r)).astype(np.float32))
    inv = (1e7 ** (-2.0 * np.arange(rope // 2) / rope)).astype(np.float32)
    pos, kv0 = [3, 4], [0, 5]
    if fmt == "bf16":
        cache = dict(k=np.zeros((P, rope), np.uint16), v=np.zeros((P, r), np.uint16))
    else:
        cache = dict(k=np.zeros((P, rope), np.uint8), v=np.zeros((P, r), np.uint8), ks=np.zeros((P, rope // 32), np.uint8),
                     vs=np.zeros((P, r // 32), np.uint8))
    qr = be.kt_mla_rope(nh, r, rope, kvf, qr0, kr, c, cache, pos, kv0, inv)
    half = rope // 2
    for t in range(T):
        at = kv0[t] + pos[t]
        krot = np.zeros(rope)
        for i in range(half):
            for h in range(nh):
                y0, y1 = oracle.rope_pair(float(qr0[t, h, i]), float(qr0[t, h, i + half]), pos[t], float(inv[i]))
                assert close_bf(qr[t, h, i], y0, 1e-6) and close_bf(qr[t, h, i + half], y1, 1e-6)
            krot[i], krot[i + half] = oracle.rope_pair(float(kr[t, i]), float(kr[t, i + half]), pos[t], float(inv[i]))
        if fmt == "bf16":
            assert np.all(close_bf(packs.bf16_bits_to_f32(cache["k"][at]), krot, 1e-6))
            assert np.array_equal(packs.bf16_bits_to_f32(cache["v"][at]), c[t])
        else:
            codes, scales = oracle.fp8_row(c[t][None])            # the latent's codes are the C codec's, bit for bit
            assert np.array_equal(cache["v"][at], codes[0]) and np.array_equal(cache["vs"][at], scales[0])
            kdec = oracle.fp8_decode(cache["k"][at][None], cache["ks"][at][None])[0]
            step = 2.0 ** (cache["ks"][at].repeat(32).astype(np.float64) - 127)   # an E4M3 step is at most |v| / 8, plus the subnormal grid
            assert np.all(np.abs(kdec - krot) <= np.abs(krot) / 8.0 + step * 2.0 ** -9 + 1e-6)
    untouched = [i for i in range(P) if i not in (3, 9)]
    assert not cache["k"][untouched].any() and not cache["v"][untouched].any()


def test_kv_f32_decodes_the_codec(be, oracle):
    rng = np.random.default_rng(77)
    x = (rng.standard_normal((5, 512)) * rng.uniform(0.01, 30, (5, 1))).astype(np.float32)
    codes, scales = oracle.fp8_row(x)
    assert np.array_equal(be.kt_kv_f32(be.KV_FP8, codes, scales), oracle.fp8_decode(codes, scales))
    # every code, a range of scales (subnormal codes and the ends of the scale range included)
    allc = np.tile(np.arange(256, dtype=np.uint8), 8).reshape(8, 256)
    sc = np.array([[1, 8, 100, 127, 128, 200, 239, 250]] * 8, dtype=np.uint8).T.copy()
    got = be.kt_kv_f32(be.KV_FP8, allc, sc)
    want = oracle.fp8_decode(allc, sc)
    finite = np.isfinite(want) & (np.abs(want) < 3e38) & ((np.abs(want) > 1.2e-38) | (want == 0))
    assert np.array_equal(got[finite], want[finite])


CASES = [(32, 768, 128, 3, 1, 0), (32, 768, 128, 3, 5, 0), (20, 64, 128, 3, 3, 0), (8, 96, 128, 45, 1, 0), (32, 768, 128, 3, 40, 150),
         (20, 64, 128, 3, 40, 150), (16, 512, 64, 3, 8, 0), (16, 512, 64, 3, 1, 0), (20, 512, 64, 3, 5, 0), (5, 512, 64, 45, 3, 0),
         (40, 512, 64, 3, 40, 150)]


@pytest.mark.parametrize("nh,r,rope,T,ns,lp", CASES)
def test_latent_attention(be, oracle, nh, r, rope, T, ns, lp):
    rng = np.random.default_rng(nh * r + T + ns)
    NP = 640
    pos = [300, 299, 37] if T == 3 else [37 + t for t in range(T)]
    kv0 = [0, 310, 600] if T == 3 else [19] * T
    ql = packs.round_bf16((rng.standard_normal((T, nh, r)) * 0.3).astype(np.float32))
    qr = packs.round_bf16(rng.standard_normal((T, nh, rope)).astype(np.float32))
    lat = packs.round_bf16(rng.standard_normal((NP, r)).astype(np.float32))
    kr = packs.round_bf16(rng.standard_normal((NP, rope)).astype(np.float32))
    scale = float(1 / np.sqrt(128.0))
    cache = dict(k=packs.f32_to_bf16_bits(kr), v=packs.f32_to_bf16_bits(lat))
    o = be.kt_mla_attn(nh, r, rope, be.KV_BF16, ql, qr, cache, pos, kv0, scale, (301 + ns - 1) // ns, ns, long_from=lp)
    for t in range(T):
        for h in range(0, nh, max(1, nh // 6)):
            want = oracle.mla_attn(ql[t, h], qr[t, h], lat[kv0[t]:], kr[kv0[t]:], pos[t], scale)
            assert np.all(close_bf(o[t, h], want.astype(np.float64), 2e-6)), (t, h)
    # the same rows over an FP8 cache: bit-equal to the BF16 kernel on the decoded cache
    kc, ksc = oracle.fp8_row(kr)
    vc, vsc = oracle.fp8_row(lat)
    o8 = be.kt_mla_attn(nh, r, rope, be.KV_FP8, ql, qr, dict(k=kc, v=vc, ks=ksc, vs=vsc), pos, kv0, scale, (301 + ns - 1) // ns, ns, long_from=lp)
    dec = dict(k=packs.f32_to_bf16_bits(oracle.fp8_decode(kc, ksc)), v=packs.f32_to_bf16_bits(oracle.fp8_decode(vc, vsc)))
    od = be.kt_mla_attn(nh, r, rope, be.KV_BF16, ql, qr, dec, pos, kv0, scale, (301 + ns - 1) // ns, ns, long_from=lp)
    assert np.array_equal(o8.view(np.uint32), od.view(np.uint32))


def test_latent_attention_over_any_cache_bytes(be, oracle):
    """Every byte is a code of this codec: a cache of random bytes (0x7F / 0xFF, which the encoder never writes, and scale
    bytes far from 127 included) reads as the decoded cache does."""
    rng = np.random.default_rng(77)
    nh, r, rope, NP, T = 16, 512, 64, 200, 2
    vc, kc = rng.integers(0, 256, (NP, r)).astype(np.uint8), rng.integers(0, 256, (NP, rope)).astype(np.uint8)
    vsc = rng.integers(118, 124, (NP, r // 32)).astype(np.uint8)
    ksc = rng.integers(118, 124, (NP, rope // 32)).astype(np.uint8)
    vsc[rng.random(vsc.shape) < 0.1] = 20                             # outside the range the conversion instruction takes
    vc[::7, 5], vc[3::11, 130], kc[::5, 9] = 0x7F, 0xFF, 0x7F
    ql = packs.round_bf16((rng.standard_normal((T, nh, r)) * 0.05).astype(np.float32))
    qr = packs.round_bf16((rng.standard_normal((T, nh, rope)) * 0.05).astype(np.float32))
    scale = float(1 / np.sqrt(192.0))
    ld, kd = oracle.fp8_decode(vc, vsc), oracle.fp8_decode(kc, ksc)
    assert np.isfinite(ld).all() and np.abs(ld).max() == 480 * 2.0 ** -4
    for ns in (1, 4):
        o8 = be.kt_mla_attn(nh, r, rope, be.KV_FP8, ql, qr, dict(k=kc, v=vc, ks=ksc, vs=vsc), [199, 70], [0, 0], scale, 64, ns)
        od = be.kt_mla_attn(nh, r, rope, be.KV_BF16, ql, qr, dict(k=packs.f32_to_bf16_bits(kd), v=packs.f32_to_bf16_bits(ld)), [199, 70], [0, 0],
                            scale, 64, ns)
        assert np.array_equal(o8.view(np.uint32), od.view(np.uint32))
        for t, p in ((0, 199), (1, 70)):
            for h in (0, 9):
                want = oracle.mla_attn(ql[t, h], qr[t, h], ld, kd, p, scale)
                # P enters the second product as BF16 hi + lo terms (16 bits of P): an absolute slack of 2^-16 of the largest value
                assert np.all(close_bf(o8[t, h], want.astype(np.float64), 30.0 * 2.0 ** -16)), (ns, t, h)


def test_latent_attention_long_context_fp8(be, oracle):
    """The full model's shape: 16 heads, latent 512, RoPE 64, FP8 cache, 4096 positions, 32 splits."""
    rng = np.random.default_rng(4096)
    nh, r, rope, NP = 16, 512, 64, 4096
    lat = packs.round_bf16(rng.standard_normal((NP, r)).astype(np.float32))
    kr = packs.round_bf16(rng.standard_normal((NP, rope)).astype(np.float32))
    kc, ksc = oracle.fp8_row(kr)
    vc, vsc = oracle.fp8_row(lat)
    ql = packs.round_bf16((rng.standard_normal((2, nh, r)) * 0.2).astype(np.float32))
    qr = packs.round_bf16(rng.standard_normal((2, nh, rope)).astype(np.float32))
    scale = float(1 / np.sqrt(192.0))
    o = be.kt_mla_attn(nh, r, rope, be.KV_FP8, ql, qr, dict(k=kc, v=vc, ks=ksc, vs=vsc), [4095, 1000], [0, 0], scale, 128, 32)
    ld, kd = oracle.fp8_decode(vc, vsc), oracle.fp8_decode(kc, ksc)
    for t, p in ((0, 4095), (1, 1000)):
        for h in (0, 7, 15):
            want = oracle.mla_attn(ql[t, h], qr[t, h], ld, kd, p, scale)
            assert np.all(close_bf(o[t, h], want.astype(np.float64), 2e-6)), (t, h)


@pytest.mark.parametrize("kvf", ["bf16", "fp8"])
@pytest.mark.parametrize("H,hd,r,rope,T", [(16, 128, 512, 64, 3), (5, 64, 128, 128, 2)])
def test_query_maps_rope_and_cache_write_in_one_launch(be, kvf, H, hd, r, rope, T):
    """kc_mla_qmaps_rope == kc_heads_mv (RoPE mix) + kc_heads_mv (latent query) + kc_mla_rope: the same bits in qr, ql and
    the cache rows."""
    import ctypes as C
    from nanoseedlm_amd import moe
    L = be.hip()
    rng = np.random.default_rng(H * r + T)
    fmt = be.KV_FP8 if kvf == "fp8" else be.KV_BF16
    es, NP = (1 if fmt == be.KV_FP8 else 2), 40
    q = moe.DevBuf.from_array(packs.round_bf16(rng.standard_normal((T, H * hd)).astype(np.float32)))
    kr = moe.DevBuf.from_array(packs.round_bf16(rng.standard_normal((T, rope)).astype(np.float32)))
    c = moe.DevBuf.from_array(packs.round_bf16(rng.standard_normal((T, r)).astype(np.float32)))
    wq = moe.DevBuf.from_array(packs.f32_to_bf16_bits((rng.standard_normal((H, rope, hd)) / np.sqrt(hd)).astype(np.float32)))
    wl = moe.DevBuf.from_array(packs.f32_to_bf16_bits((rng.standard_normal((H, r, hd)) / np.sqrt(hd)).astype(np.float32)))
    inv = moe.DevBuf.from_array(np.array([10000.0 ** (-2.0 * p / rope) for p in range(rope // 2)], dtype=np.float32))
    ri = (be.RowInfo * T)()
    for t in range(T):
        ri[t].pos, ri[t].kv0 = 3 + 5 * t, 10 * t
    rib = moe.DevBuf(C.sizeof(ri))
    be.check(L.nh_memcpy_h2d(rib.ptr, ri, C.c_size_t(C.sizeof(ri))), "h2d")
    Wq, Wl = be.WSlice(), be.WSlice()
    Wq.p[0], Wl.p[0] = wq.ptr.value, wl.ptr.value
    a = be.MlaArgs(H, r, 128, 1, 0.1)
    a.pad[0] = rope
    hq, hl = be.HmvArgs(H, rope, hd, H * hd, hd, 0), be.HmvArgs(H, r, hd, H * hd, hd, 0)
    L.kc_heads_mv.argtypes = [C.c_void_p, be.HmvArgs, C.c_int, be.WSlice, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
    L.kc_mla_rope.argtypes = [C.c_void_p, be.MlaArgs, C.c_void_p, C.c_void_p, C.c_void_p, be.KvView, C.c_void_p, C.c_void_p, C.c_int]
    L.kc_mla_qmaps_rope.argtypes = [C.c_void_p, be.MlaArgs, be.HmvArgs, be.HmvArgs, C.c_int, be.WSlice, be.WSlice, C.c_void_p, C.c_void_p, C.c_void_p,
                                    C.c_void_p, C.c_void_p, be.KvView, C.c_void_p, C.c_void_p, C.c_int]
    outs = []
    for fused in (False, True):
        kc, vc = moe.DevBuf(NP * rope * es), moe.DevBuf(NP * r * es)
        ks, vs = moe.DevBuf(NP * rope // 32 + 16), moe.DevBuf(NP * r // 32 + 16)
        for b in (kc, vc, ks, vs):
            be.check(L.nh_memset(b.ptr, 0, C.c_size_t(b.nbytes)), "memset")
        kv = be.KvView(be.KvSeg(kc.ptr, vc.ptr, ks.ptr, vs.ptr), be.KvSeg(None, None, None, None), NP, fmt)
        qr, ql = moe.DevBuf(4 * T * H * rope), moe.DevBuf(4 * T * H * r)
        if fused:
            assert L.kc_mla_qmaps_rope(None, a, hq, hl, packs.MF_BF16, Wq, Wl, q.ptr, qr.ptr, ql.ptr, kr.ptr, c.ptr, kv, rib.ptr, inv.ptr, T) == 0
        else:
            L.kc_heads_mv(None, hq, packs.MF_BF16, Wq, None, q.ptr, None, qr.ptr, T)
            L.kc_heads_mv(None, hl, packs.MF_BF16, Wl, None, q.ptr, None, ql.ptr, T)
            L.kc_mla_rope(None, a, qr.ptr, kr.ptr, c.ptr, kv, rib.ptr, inv.ptr, T)
        moe.device_sync()
        assert L.kc_last_error() == 0
        outs.append([qr.to_array(np.uint32, (T, H, rope)), ql.to_array(np.uint32, (T, H, r)), kc.to_array(np.uint8, (NP * rope * es,)),
                     vc.to_array(np.uint8, (NP * r * es,)), ks.to_array(np.uint8, (NP * rope // 32,)), vs.to_array(np.uint8, (NP * r // 32,))])
    assert outs[0][0].any() and outs[0][1].any() and outs[0][2].any() and outs[0][3].any()
    for x, y in zip(*outs):
        assert np.array_equal(x, y)


@pytest.mark.parametrize("kvf,H,hd,r,rope,ns", [("fp8", 16, 128, 512, 64, 32), ("bf16", 16, 128, 512, 64, 5), ("bf16", 6, 64, 128, 128, 3)])
def test_attention_with_reduce_and_value_map_in_one_launch(be, oracle, kvf, H, hd, r, rope, ns):
    """kc_mla_attn_vup == kc_mla_attn + kc_heads_mv (latent -> value): the same bits."""
    import ctypes as C
    from nanoseedlm_amd import moe
    L = be.hip()
    rng = np.random.default_rng(H + r + ns)
    T, NP = 3, 700
    fmt = be.KV_FP8 if kvf == "fp8" else be.KV_BF16
    lat = packs.round_bf16(rng.standard_normal((NP, r)).astype(np.float32))
    krr = packs.round_bf16(rng.standard_normal((NP, rope)).astype(np.float32))
    if fmt == be.KV_FP8:
        kc, ksc = oracle.fp8_row(krr)
        vc, vsc = oracle.fp8_row(lat)
        bufs = [moe.DevBuf.from_array(x) for x in (kc, vc, ksc, vsc)]
    else:
        bufs = [moe.DevBuf.from_array(packs.f32_to_bf16_bits(krr)), moe.DevBuf.from_array(packs.f32_to_bf16_bits(lat)), moe.DevBuf(16), moe.DevBuf(16)]
    kv = be.KvView(be.KvSeg(*[b.ptr for b in bufs]), be.KvSeg(None, None, None, None), NP, fmt)
    ql = moe.DevBuf.from_array(packs.round_bf16((rng.standard_normal((T, H, r)) * 0.3).astype(np.float32)))
    qr = moe.DevBuf.from_array(packs.round_bf16(rng.standard_normal((T, H, rope)).astype(np.float32)))
    wv = moe.DevBuf.from_array(packs.f32_to_bf16_bits((rng.standard_normal((H, hd, r)) / np.sqrt(r)).astype(np.float32)))
    ri = (be.RowInfo * T)()
    for t, (p, k0) in enumerate(((650, 0), (37, 20), (300, 310))):
        ri[t].pos, ri[t].kv0 = p, k0
    rib = moe.DevBuf(C.sizeof(ri))
    be.check(L.nh_memcpy_h2d(rib.ptr, ri, C.c_size_t(C.sizeof(ri))), "h2d")
    a = be.MlaArgs(H, r, 128, ns, float(1 / np.sqrt(hd + rope)))
    a.pad[0] = rope
    W = be.WSlice()
    W.p[0] = wv.ptr.value
    hv = be.HmvArgs(H, hd, r, H * r, r, 0)
    part, olat = moe.DevBuf(4 * T * H * ns * (r + 2)), moe.DevBuf(4 * T * H * r)
    ya, yb = moe.DevBuf(4 * T * H * hd), moe.DevBuf(4 * T * H * hd)
    L.kc_mla_attn.argtypes = [C.c_void_p, be.MlaArgs, C.c_void_p, C.c_void_p, be.KvView, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
    L.kc_heads_mv.argtypes = [C.c_void_p, be.HmvArgs, C.c_int, be.WSlice, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
    L.kc_mla_attn_vup.argtypes = [C.c_void_p, be.MlaArgs, C.c_void_p, C.c_void_p, be.KvView, C.c_void_p, C.c_void_p, be.HmvArgs, C.c_int, be.WSlice,
                                  C.c_void_p, C.c_int]
    L.kc_mla_attn(None, a, ql.ptr, qr.ptr, kv, rib.ptr, part.ptr, olat.ptr, T)
    L.kc_heads_mv(None, hv, packs.MF_BF16, W, None, olat.ptr, None, ya.ptr, T)
    assert L.kc_mla_attn_vup(None, a, ql.ptr, qr.ptr, kv, rib.ptr, part.ptr, hv, packs.MF_BF16, W, yb.ptr, T) == 0
    moe.device_sync()
    assert L.kc_last_error() == 0
    A, B = ya.to_array(np.uint32, (T, H, hd)), yb.to_array(np.uint32, (T, H, hd))
    assert A.any() and np.array_equal(A, B)
