"""Pins of the CPU oracle (oracle/nslm_oracle.c): the reference's own golden vectors and known-answer tests, what the
mathematics fixes (closed forms in Python big integers / fractions, brute force), the committed fixtures made from the
compiled reference (tests/golden/), and - where oracle/_ref is built - the compiled reference itself, live."""
import ctypes as C
import os
from fractions import Fraction

import numpy as np
import pytest

from nanoseedlm_amd import packs

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


# ---- independent big-integer restatement used as "what the mathematics fixes" -----------------------------------------

def py_states(seed, n):
    """x^16 + x^12 + x^3 + x + 1 as a bit recurrence on an unbounded Python int: x[n+16] = x[n]^x[n+1]^x[n+3]^x[n+12]."""
    x = seed
    for i in range(n):
        b = ((x >> i) ^ (x >> (i + 1)) ^ (x >> (i + 3)) ^ (x >> (i + 12))) & 1
        x |= b << (i + 16)
    return [(x >> k) & 0xFFFF for k in range(1, n + 1)]


def rne_bf16(fr):
    """Exact rational -> BF16 bits via f32 RNE then BF16 RNE (the spec rounds twice: nslm/lfsr.h:9-10)."""
    f = np.float32(float(fr))  # float(Fraction) is correctly rounded to double; isum*R32*2^e needs the f32 product:
    return f


def q4(v):
    v &= 15
    return v - 16 if v >= 8 else v


# ---- LFSR --------------------------------------------------------------------------------------------------------------

def test_lfsr_hand_states_and_period(oracle):
    # tests/test_lfsr.c:25 hand-computed states after seed 1
    assert list(oracle.lfsr_states(1, 6)) == [0x8000, 0x4000, 0x2000, 0x1000, 0x8800, 0x4400]
    # tests/test_lfsr.c:14-22 period 65535, zero never visited
    L = oracle.lib()
    s, n, seen = 1, 0, set()
    while True:
        assert s not in seen
        seen.add(s)
        s = L.or_lfsr_step(s)
        n += 1
        if s == 1:
            break
    assert n == 65535 and 0 not in seen
    # seed semantics: the first state is the one AFTER the seed (tests/test_lfsr.c:30-35)
    assert oracle.lfsr_states(0xACE1, 24)[0] == L.or_lfsr_step(0xACE1) != 0xACE1


def test_lfsr_fnv_golden(oracle):
    # tests/test_lfsr.c:41-56: FNV-1a over the 24 states of every seed locks the definition
    assert oracle.lib().or_lfsr_fnv24() == 0x740E86E513D34463


def test_lfsr_bigint_and_stream_tables(oracle):
    rng = np.random.default_rng(1)
    for seed in [1, 2, 0x8000, 0xFFFF, 0xACE1] + list(rng.integers(1, 65536, 200)):
        assert list(oracle.lfsr_states(int(seed), 48)) == py_states(int(seed), 48)
    t24, t32 = oracle.stream_table(24), oracle.stream_table(32)
    assert np.array_equal(t24, t32 & 0xFFFFFF)
    s = np.arange(65536)
    # GF(2) linearity (tests/test_lfsr.c:86-91)
    assert np.array_equal(t32, t32[s & 0xFF] ^ t32[s & 0xFF00])
    # state k = bits k..k+15 of seed | table << 16 (engine/kernels_moe.cu:49-51)
    for seed in rng.integers(1, 65536, 50):
        st = int(seed) | (int(t32[seed]) << 16)
        assert [(st >> k) & 0xFFFF for k in range(1, 33)] == list(oracle.lfsr_states(int(seed), 32))


def test_lfsr_vs_reference_all_seeds(oracle, ref):
    t32 = oracle.stream_table(32)
    t24 = oracle.stream_table(24)
    for s in range(0, 65536, 1):
        if s % 257 == 0 or s < 300:  # a dense prefix and a stride over the rest keeps this to a second
            assert ref.ref_lfsr_stream32(s) == t32[s] and ref.ref_lfsr_stream24(s) == t24[s]
            assert ref.ref_lfsr_step(s) == oracle.lib().or_lfsr_step(s)
    out = np.zeros(48, dtype=np.uint16)
    for s in (1, 77, 65535, 0x1234):
        ref.ref_lfsr_states_wordpar(C.c_uint16(s), 48, out.ctypes.data_as(C.c_void_p))
        assert np.array_equal(out, oracle.lfsr_states(s, 48))


# ---- block decode ------------------------------------------------------------------------------------------------------

def exact_block(seed, qs, P):
    st = py_states(seed, 8 * P)
    return [sum((st[c * P + p] - 32768) * qs[p] for p in range(P)) for c in range(8)]


def bf16_of_isum(isum, e):
    r32 = np.float32(1.0) / np.float32(32767.0)
    sc = np.float32(r32 * np.float32(2.0 ** e))  # exact power-of-two scaling of R32
    return int(packs.f32_to_bf16_bits(np.float32(np.float32(isum) * sc)))


def test_decode_closed_form(oracle):
    rng = np.random.default_rng(2)
    for _ in range(300):
        seed = int(rng.integers(1, 65536))
        w = int(rng.integers(0, 65536))
        e = int(rng.integers(-30, 1))
        q = [q4(w), q4(w >> 4), q4(w >> 8), q4(w >> 12)]
        isum = exact_block(seed, q, 4)
        assert list(oracle.isum_p4(seed, w)) == isum
        assert max(abs(v) for v in isum) < 2 ** 20
        assert list(oracle.decode_p4(seed, w, e)) == [bf16_of_isum(v, e) for v in isum]
        q3 = [q4(w >> 4), q4(w >> 8), q4(w >> 12)]
        isum3 = exact_block(seed, q3, 3)
        assert list(oracle.isum_p3(seed, w)) == isum3
        assert list(oracle.decode_p3(seed, w, e)) == [bf16_of_isum(v, e + (w & 15)) for v in isum3]


def test_decode_exactness_identity(oracle):
    # fl(isum * fl(R32 2^e)) == ldexp(fl(isum * R32), e) (tests/test_lfsr.c:67-85)
    rng = np.random.default_rng(3)
    r32 = np.float32(1.0) / np.float32(32767.0)
    L = oracle.lib()
    for _ in range(2000):
        isum = int(rng.integers(-786431, 786432))
        e = int(rng.integers(-30, 1))
        a = np.float32(np.float32(isum) * np.float32(L.or_scale(e)))
        b = np.float32(np.ldexp(np.float32(np.float32(isum) * r32), e))
        assert a == b
    assert np.float32(L.or_scale(0)) == r32


def test_int4_fields_exhaustive(oracle, ref):
    # pack/unpack of every nibble position, against the reference's nslm4_q / nslm_q (tests/test_lfsr.c:58-66)
    for w in range(0, 65536, 7):
        for p in range(4):
            assert ref.ref_nslm4_q(w, p) == q4(w >> (4 * p))
        for p in range(3):
            assert ref.ref_nslm_q(w, p) == q4(w >> (4 + 4 * p))


def test_decode_vs_reference_live(oracle, ref):
    rng = np.random.default_rng(4)
    out = np.zeros(8, dtype=np.uint16)
    for _ in range(2000):
        seed, w, e = int(rng.integers(1, 65536)), int(rng.integers(0, 65536)), int(rng.integers(-30, -5))
        ref.nslm4_decode_block(C.c_uint16(seed), C.c_uint16(w), C.c_int(e), out.ctypes.data_as(C.c_void_p))
        assert np.array_equal(out, oracle.decode_p4(seed, w, e))
        ref.ref_nslm_decode_block(C.c_uint16(seed), C.c_uint16(w), C.c_int(e), out.ctypes.data_as(C.c_void_p))
        assert np.array_equal(out, oracle.decode_p3(seed, w, e))


def test_decode_golden_fixture(oracle):
    g = np.load(os.path.join(GOLD, "blocks.npz"))
    for i in range(g["seed"].size):
        assert np.array_equal(oracle.decode_p4(int(g["seed"][i]), int(g["word"][i]), int(g["e"][i])), g["p4"][i])
        assert np.array_equal(oracle.decode_p3(int(g["seed"][i]), int(g["word"][i]), int(g["e"][i])), g["p3"][i])


# ---- rows / matrices ---------------------------------------------------------------------------------------------------

def _slice_of(oracle, p, s=0):
    f = p["fmt"]
    if f == packs.MF_SEED4P4:
        return oracle.make_slice(f, p["seeds"][s], p["coefs"][s], None, p["codes"][s], eb=p["eb"][s])
    if f == packs.MF_SEED4:
        return oracle.make_slice(f, p["seeds"][s], p["nibs"][s], eb=p["eb"][s])
    if f in (packs.MF_Q4, packs.MF_Q8):
        return oracle.make_slice(f, p["words"][s], p["scales"][s], p["biases"][s], gs={32: 5, 64: 6}[p["group"]])
    return oracle.make_slice(f, p["w"][s])


def test_rows_equal_block_decode(oracle):
    rng = np.random.default_rng(5)
    R, K = 6, 64
    p4 = packs.seed4p4(rng, 1, R, K, eb=-20)
    w = oracle.rows_f32(packs.MF_SEED4P4, _slice_of(oracle, p4), R, K)
    codes = packs.unpack_nibbles(p4["codes"][0], R * K // 8).reshape(R, K // 8)
    for r in range(R):
        for j in range(K // 8):
            want = oracle.decode_p4(int(p4["seeds"][0, r, j]), int(p4["coefs"][0, r, j]), -20 + int(codes[r, j]))
            assert np.array_equal(packs.f32_to_bf16_bits(w[r, 8 * j:8 * j + 8]), want)
    assert np.array_equal(oracle.slice_bf16(packs.MF_SEED4P4, _slice_of(oracle, p4), R, K), packs.f32_to_bf16_bits(w))
    p3 = packs.seed4(rng, 1, R, K, eb=-19)
    w3 = oracle.rows_f32(packs.MF_SEED4, _slice_of(oracle, p3), R, K)
    for r in range(R):
        for j in range(K // 8):
            want = oracle.decode_p3(int(p3["seeds"][0, r, j]), int(p3["nibs"][0, r, j]), -19)
            assert np.array_equal(packs.f32_to_bf16_bits(w3[r, 8 * j:8 * j + 8]), want)


def test_rows_vs_reference_live(oracle, ref):
    rng = np.random.default_rng(6)
    R, K = 5, 128
    out = np.zeros(K, dtype=np.float32)
    for fmt, p in ((packs.MF_SEED4P4, packs.seed4p4(rng, 1, R, K, eb=-21)), (packs.MF_SEED4, packs.seed4(rng, 1, R, K, eb=-18)),
                   (packs.MF_Q4, packs.affine(rng, 1, R, K, 4)), (packs.MF_Q8, packs.affine(rng, 1, R, K, 8)),
                   (packs.MF_Q4, packs.affine(rng, 1, R, K, 4, group=32))):
        sl = _slice_of(oracle, p)
        for rnd in (0, 1):
            mine = oracle.rows_f32(fmt, sl, R, K, rnd)
            for r in range(R):
                if fmt == packs.MF_SEED4P4:
                    a = (p["seeds"][0], p["coefs"][0], p["codes"][0], int(p["eb"][0]), 0)
                elif fmt == packs.MF_SEED4:
                    a = (p["seeds"][0], p["nibs"][0], None, int(p["eb"][0]), 0)
                else:
                    a = (p["words"][0], p["scales"][0], p["biases"][0], 0, p["group"])
                ref.ref_row_f32(C.c_int(fmt), a[0].ctypes.data_as(C.c_void_p), a[1].ctypes.data_as(C.c_void_p),
                                None if a[2] is None else a[2].ctypes.data_as(C.c_void_p), C.c_int32(a[3]), C.c_int(a[4]),
                                C.c_int(R), C.c_int(K), C.c_int(r), C.c_int(rnd), out.ctypes.data_as(C.c_void_p))
                assert np.array_equal(out.view(np.uint32), mine[r].view(np.uint32)), (fmt, rnd, r)


def test_affine_closed_form(oracle, ref):
    rng = np.random.default_rng(7)
    for bits in (4, 8):
        p = packs.affine(rng, 1, 4, 128, bits)
        n = 4 * 128
        got = oracle.affine_dequant(p["words"][0], p["scales"][0], p["biases"][0], n, bits, 64)
        per = 32 // bits
        q = np.stack([(p["words"][0] >> np.uint32(bits * i)) & np.uint32((1 << bits) - 1) for i in range(per)], -1).reshape(-1)
        s = np.repeat(packs.bf16_bits_to_f32(p["scales"][0]).reshape(-1), 64)
        b = np.repeat(packs.bf16_bits_to_f32(p["biases"][0]).reshape(-1), 64)
        want = packs.f32_to_bf16_bits((s * q.astype(np.float32)).astype(np.float32) + b)
        assert np.array_equal(got, want)
        out = np.zeros(n, dtype=np.uint16)
        ref.nslm_affine_dequantize(p["words"][0].ctypes.data_as(C.c_void_p), p["scales"][0].ctypes.data_as(C.c_void_p),
                                   p["biases"][0].ctypes.data_as(C.c_void_p), 4, 128, bits, out.ctypes.data_as(C.c_void_p))
        assert np.array_equal(out, got)


# ---- CPU decode-in-dot-product -----------------------------------------------------------------------------------------

@pytest.mark.parametrize("rows,kb,bias", [(40, 8, -20), (37, 30, -24), (64, 96, -22)])
def test_cpu_matvec_vs_double(oracle, rows, kb, bias):
    # tests/test_cpu_seed4.c:27-63: < 2e-6 of max |ref| against the double dot over exact weights
    rng = np.random.default_rng(rows)
    p = packs.seed4p4(rng, 1, rows, kb * 8, eb=bias)
    x = ((rng.integers(0, 20001, kb * 8) - 10000) / 10000.0).astype(np.float32)
    y = oracle.cpu_seed4_matvec(p["seeds"][0], p["coefs"][0], p["codes"][0], bias, x, rows, kb, threads=3)
    w = oracle.rows_f32(packs.MF_SEED4P4, _slice_of(oracle, p), rows, kb * 8).astype(np.float64)
    want = w @ x.astype(np.float64)
    assert np.max(np.abs(y - want)) / np.max(np.abs(want)) < 2e-6
    yd, _ = oracle.mv_double(packs.MF_SEED4P4, _slice_of(oracle, p), rows, kb * 8, x)
    assert np.allclose(yd[0], want, rtol=1e-12, atol=1e-12)
    p3 = packs.seed4(rng, 1, rows, kb * 8, eb=bias)
    y3 = oracle.cpu_seed3_matvec(p3["seeds"][0], p3["nibs"][0], bias, x, rows, kb, threads=2)
    w3 = oracle.rows_f32(packs.MF_SEED4, _slice_of(oracle, p3), rows, kb * 8).astype(np.float64)
    assert np.max(np.abs(y3 - w3 @ x)) / np.max(np.abs(w3 @ x)) < 2e-6


def test_cpu_matvec_bit_equal_reference(oracle, ref):
    rng = np.random.default_rng(11)
    for rows, kb in ((53, 24), (16, 10), (7, 6)):
        p = packs.seed4p4(rng, 1, rows, kb * 8, eb=-21)
        x = rng.standard_normal(kb * 8).astype(np.float32)
        mine = oracle.cpu_seed4_matvec(p["seeds"][0], p["coefs"][0], p["codes"][0], -21, x, rows, kb)
        y = np.zeros(rows, dtype=np.float32)
        ref.ref_matvec(p["seeds"][0].ctypes.data_as(C.c_void_p), p["coefs"][0].ctypes.data_as(C.c_void_p),
                       p["codes"][0].ctypes.data_as(C.c_void_p), -21, x.ctypes.data_as(C.c_void_p), rows, kb,
                       y.ctypes.data_as(C.c_void_p), 2)
        assert np.array_equal(y.view(np.uint32), mine.view(np.uint32))
        t = ref.ref_tile4(p["seeds"][0].ctypes.data_as(C.c_void_p), p["coefs"][0].ctypes.data_as(C.c_void_p),
                          p["codes"][0].ctypes.data_as(C.c_void_p), -21, rows, kb)
        yt = np.zeros(rows, dtype=np.float32)
        ref.ref_tiled_matmul(C.c_void_p(t), x.ctypes.data_as(C.c_void_p), 1, yt.ctypes.data_as(C.c_void_p), 2)
        ref.ref_tile_free(C.c_void_p(t))
        assert np.array_equal(yt.view(np.uint32), mine.view(np.uint32))
        p3 = packs.seed4(rng, 1, rows, kb * 8, eb=-20)
        mine3 = oracle.cpu_seed3_matvec(p3["seeds"][0], p3["nibs"][0], -20, x, rows, kb)
        t = ref.ref_tile3(p3["seeds"][0].ctypes.data_as(C.c_void_p), p3["nibs"][0].ctypes.data_as(C.c_void_p), -20, rows, kb)
        ref.ref_tiled_matmul(C.c_void_p(t), x.ctypes.data_as(C.c_void_p), 1, yt.ctypes.data_as(C.c_void_p), 1)
        ref.ref_tile_free(C.c_void_p(t))
        assert np.array_equal(yt.view(np.uint32), mine3.view(np.uint32))


def test_matvec_golden_fixture(oracle):
    g = np.load(os.path.join(GOLD, "matvec_p4.npz"))
    rows, kb = int(g["rows"]), int(g["kb"])
    mine = oracle.cpu_seed4_matvec(g["seeds"], g["coefs"], g["codes"], int(g["bias"]), g["x"], rows, kb)
    assert np.array_equal(mine.view(np.uint32), g["y_ref"].view(np.uint32))
    sl = oracle.make_slice(packs.MF_SEED4P4, g["seeds"], g["coefs"], None, g["codes"], eb=int(g["bias"]))
    w = oracle.rows_f32(packs.MF_SEED4P4, sl, rows, kb * 8)
    assert np.array_equal(w.view(np.uint32), g["rows_ref"].view(np.uint32))


# ---- routers -----------------------------------------------------------------------------------------------------------

def test_route_softmax(oracle):
    # tests/test_qwen4_kernels.c:233-245: an engineered tie goes to the higher index
    rng = np.random.default_rng(8)
    E, k = 512, 10
    lg = rng.standard_normal((3, E)).astype(np.float32)
    lg[0, 7] = lg[0, 300] = 9.0
    ind, wt = oracle.route_softmax(lg, k)
    assert ind[0, 0] == 300 and ind[0, 1] == 7
    for t in range(3):
        p = np.exp(lg[t].astype(np.float64) - lg[t].max())
        order = sorted(range(E), key=lambda e: (-p[e], -e))[:k]
        assert list(ind[t]) == order
        assert np.allclose(wt[t], p[order] / p[order].sum(), rtol=1e-6)
        assert abs(wt[t].sum() - 1) < 1e-5


def test_route_softmax_vs_reference(oracle, ref):
    rng = np.random.default_rng(9)
    E, k = 128, 8
    lg = np.round(rng.standard_normal((20, E)) * 2).astype(np.float32) / 2  # many exact ties
    ind, wt = oracle.route_softmax(lg, k)
    ri, rw = np.zeros(k, dtype=np.int32), np.zeros(k, dtype=np.float32)
    for t in range(20):
        ref.ref_qwen4_route(E, k, lg[t].ctypes.data_as(C.c_void_p), ri.ctypes.data_as(C.c_void_p), rw.ctypes.data_as(C.c_void_p))
        assert np.array_equal(ri, ind[t]) and np.array_equal(rw, wt[t])


def test_route_sigmoid(oracle):
    # tests/test_mova_kernels.c:376-445: brute-force k-round arg-max, ties to the lowest id, a many-ties case
    rng = np.random.default_rng(10)
    n, k, T = 128, 8, 4
    score = rng.uniform(0, 1, (T, n)).astype(np.float32)
    sel = score + rng.standard_normal((T, n)).astype(np.float32) * 0.1
    sel[1] = np.round(sel[1] * 4) / 4  # many ties
    sel[2, :] = 0.5                    # all tied: picks 0..k-1
    inds, wts = oracle.topk_sigmoid(score, sel, k, 2.5)
    assert list(inds[2]) == list(range(k))
    for t in range(T):
        order = sorted(range(n), key=lambda e: (-sel[t, e], e))[:k]
        assert list(inds[t]) == order
        s = np.float32(0)
        for e in order:
            s = np.float32(s + score[t, e])
        assert np.array_equal(wts[t], (score[t, order] / s * np.float32(2.5)).astype(np.float32))
    d = 64
    W = packs.f32_to_bf16_bits((rng.standard_normal((n, d)) * 0.05).astype(np.float32))
    bias = packs.f32_to_bf16_bits((rng.standard_normal(n) * 0.01).astype(np.float32))
    x = packs.round_bf16(rng.standard_normal((T, d)).astype(np.float32))
    sc, se, inds, wts = oracle.route_sigmoid(W, bias, x, k, d // 2, 1.0)
    Wf = packs.bf16_bits_to_f32(W).astype(np.float64)
    s0 = packs.round_bf16((x[:, :d // 2].astype(np.float64) @ Wf[:, :d // 2].T).astype(np.float32))
    s1 = packs.round_bf16((x[:, d // 2:].astype(np.float64) @ Wf[:, d // 2:].T).astype(np.float32))
    want = 1.0 / (1.0 + np.exp(-(s0 + s1).astype(np.float64)))
    assert np.allclose(sc, want, rtol=1e-6)
    assert np.array_equal(se, sc + packs.bf16_bits_to_f32(bias)[None, :])


# ---- elementwise, grouping, slot table ---------------------------------------------------------------------------------

def test_swiglu_and_combines(oracle):
    rng = np.random.default_rng(12)
    r = packs.round_bf16
    g = r(rng.standard_normal(500).astype(np.float32) * 3)
    u = r(rng.standard_normal(500).astype(np.float32))
    a = oracle.swiglu(g, u)
    sig = r((1.0 / (1.0 + np.exp(-g.astype(np.float64)))).astype(np.float32))
    want = r(r(g * sig) * u)
    # expf vs exp: at most one BF16 flip of the sigmoid
    assert np.mean(a != want) < 0.02 and np.allclose(a, want, rtol=1.6e-2, atol=1e-6)
    T, k, d = 3, 4, 32
    D = r(rng.standard_normal((T * k, d)).astype(np.float32))
    w = rng.uniform(0, 1, (T, k)).astype(np.float32)
    sh = r(rng.standard_normal((T, d)).astype(np.float32))
    x = r(rng.standard_normal((T, d)).astype(np.float32))
    got = oracle.moe_combine(D, w, sh, x)
    s = np.zeros((T, d), dtype=np.float32)
    for j in range(k):
        s = (s + r(D.reshape(T, k, d)[:, j] * r(w[:, j])[:, None])).astype(np.float32)
    assert np.array_equal(got, r(x + r(r(s) + sh)))
    sg = rng.standard_normal((T, 1)).astype(np.float32)
    got = oracle.q4_moe_combine(D, w, sh, sg)
    acc = (1.0 / (1.0 + np.exp(-sg.astype(np.float64)))) * sh
    want = acc + np.einsum("tk,tkd->td", w.astype(np.float64), D.reshape(T, k, d).astype(np.float64))
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6)


def test_bucket(oracle):
    # tests/test_qwen4_engine.c:33-61: skewed selections (half the pairs on expert 0), n = 512 experts
    rng = np.random.default_rng(13)
    n, count, bn = 512, 1000, 128
    inds = rng.integers(0, n, count).astype(np.int32)
    inds[::2] = 0
    perm, tiles = oracle.bucket(inds, n, bn)
    assert sorted(perm.tolist()) == list(range(count))
    assert np.array_equal(perm, np.argsort(inds, kind="stable"))
    pos = 0
    for e, start, cnt, _ in tiles:
        assert start == pos and 0 < cnt <= bn and np.all(inds[perm[start:start + cnt]] == e)
        pos += cnt
    assert pos == count
    runs = {}
    for e, start, cnt, _ in tiles:
        runs.setdefault(int(e), []).append(int(cnt))
    for e, c in runs.items():
        assert all(v == bn for v in c[:-1]) and sum(c) == int(np.sum(inds == e))


def test_cache_admit_lru(oracle):
    per_layer, layers, slots = 16, 2, 12
    unit_slot = np.full(per_layer * layers, -1, dtype=np.int32)
    slot_unit = np.full(slots, -1, dtype=np.int32)
    slot_last = np.zeros(slots, dtype=np.uint32)
    tick = np.array([0x40000000, 0, 0, 0], dtype=np.uint32)
    # first admit: 4 misses take the never-used slots 0..3 in expert order
    jobs, h, m = oracle.cache_admit(unit_slot, slot_unit, slot_last, tick, per_layer, 0, [5, 3, 9, 3, 12])
    assert (h, m) == (0, 4) and jobs.tolist() == [[3, 0], [5, 1], [9, 2], [12, 3]]
    # second admit on layer 1: hits none, takes slots 4..7
    jobs, h, m = oracle.cache_admit(unit_slot, slot_unit, slot_last, tick, per_layer, 1, [0, 1, 2, 3])
    assert jobs[:, 1].tolist() == [4, 5, 6, 7] and jobs[:, 0].tolist() == [16, 17, 18, 19]
    # third: layer 0 again, two hits (3, 5) and 6 misses: 4 free slots, then the LRU (layer 0's untouched 9, 12)
    jobs, h, m = oracle.cache_admit(unit_slot, slot_unit, slot_last, tick, per_layer, 0, [3, 5, 0, 1, 2, 4, 6, 7])
    assert (h, m) == (2, 6)
    assert jobs[:, 1].tolist() == [8, 9, 10, 11, 2, 3]
    assert unit_slot[9] == -1 and unit_slot[12] == -1
    for u in (3, 5, 0, 1, 2, 4, 6, 7):
        assert unit_slot[u] >= 0 and slot_unit[unit_slot[u]] == u
    # all resident: slots == units degenerates to hits only
    unit_slot = np.arange(per_layer, dtype=np.int32)
    slot_unit = np.arange(per_layer, dtype=np.int32)
    slot_last = np.zeros(per_layer, dtype=np.uint32)
    jobs, h, m = oracle.cache_admit(unit_slot, slot_unit, slot_last, tick, per_layer, 0, [1, 2, 3])
    assert jobs.size == 0 and (h, m) == (3, 0)


def test_gnorm_closed_form(oracle):
    # tests/test_mova_kernels.c:355-374: per-group double sum, close_bf(1e-6) of bf16(w * (x * r))
    rng = np.random.default_rng(7)
    T, d = 3, 256
    x = packs.round_bf16((rng.standard_normal((T, d)) * 3).astype(np.float32))
    wb = packs.f32_to_bf16_bits((1 + 0.3 * rng.standard_normal(d)).astype(np.float32))
    y = oracle.gnorm(x, wb, 1e-6)
    w = packs.bf16_bits_to_f32(wb).astype(np.float64)
    for t in range(T):
        for g in range(2):
            sl = slice(g * d // 2, (g + 1) * d // 2)
            r = 1.0 / np.sqrt(np.mean(x[t, sl].astype(np.float64) ** 2) + 1e-6)
            want = w[sl] * (x[t, sl].astype(np.float64) * r)
            # one BF16 ulp (2^-8 relative) around the unrounded value, plus the f32 slack of the inner product
            assert np.all(np.abs(y[t, sl] - want) <= np.abs(want) * (2.0 ** -8 + 1e-6) + 1e-30)
            assert np.array_equal(y[t, sl], packs.round_bf16(y[t, sl]))           # every output is a BF16 value
    # a constant row: r = 1 / sqrt(c^2 + eps) exactly, so y = bf16(w * fl(c * fl(r)))
    c = np.float32(0.5)
    xc = np.full((1, d), c, dtype=np.float32)
    r = np.float32(1.0 / np.sqrt(float(c) ** 2 + 1e-6))
    want = packs.round_bf16((packs.bf16_bits_to_f32(wb) * (c * r)).astype(np.float32))
    assert np.array_equal(oracle.gnorm(xc, wb, 1e-6)[0], want)


def test_norm1p(oracle):
    rng = np.random.default_rng(8)
    T, ln = 3, 512
    x = rng.standard_normal((T, ln)).astype(np.float32)
    w = (0.1 * rng.standard_normal(ln)).astype(np.float32)
    for g in (ln, 128):
        y = oracle.norm1p(x, g, w, 1e-6)
        xs = x.astype(np.float64).reshape(T, ln // g, g)
        r = 1.0 / np.sqrt((xs ** 2).mean(-1, keepdims=True) + 1e-6)
        want = (xs * r).reshape(T, ln) * (1.0 + w.astype(np.float64))
        assert np.allclose(y, want, rtol=1e-6, atol=0)
    # a row of ones with w = 0: y = 1 / sqrt(1 + eps)
    y = oracle.norm1p(np.ones((1, 64), np.float32), 64, np.zeros(64, np.float32), 1e-6)
    assert np.all(y == np.float32(1.0 / np.sqrt(1.0 + 1e-6)))


def test_norm1p_vs_reference(oracle, ref):
    rng = np.random.default_rng(9)
    ln = 768
    x = rng.standard_normal(ln).astype(np.float32)
    w = (0.2 * rng.standard_normal(ln)).astype(np.float32)
    for g in (768, 256, 64):
        y = np.zeros(ln, dtype=np.float32)
        ref.ref_norm1p(x.ctypes.data_as(C.c_void_p), ln, g, w.ctypes.data_as(C.c_void_p), C.c_float(1e-6), y.ctypes.data_as(C.c_void_p))
        assert np.array_equal(oracle.norm1p(x[None], g, w, 1e-6)[0].view(np.uint32), y.view(np.uint32))


def test_argmax_reference_vector(oracle):
    # tests/test_mova_kernels.c:563-572: a tie goes to the lowest id
    rng = np.random.default_rng(10)
    V = 250624
    lg = packs.round_bf16((rng.standard_normal((2, V)) * 3).astype(np.float32))
    lg[0, 123456] = 50
    lg[0, 200000] = 50
    lg[1, 99] = 60
    out, prob = oracle.argmax(lg, with_prob=True)
    assert out.tolist() == [123456, 99]
    z = lg.astype(np.float64)
    want = 1.0 / np.exp(z - z.max(1, keepdims=True)).sum(1)
    assert np.allclose(prob, want, rtol=1e-12)
    assert oracle.argmax(np.full((1, 17), -np.inf, dtype=np.float32)).tolist() == [0]


def test_fp8_codec(oracle):
    L = oracle.lib()
    L.or_e4m3_dec.restype = C.c_float
    L.or_e4m3_enc_abs.restype = C.c_uint8
    L.or_fp8_scale.restype = C.c_uint8
    dec = [L.or_e4m3_dec(C.c_uint8(c)) for c in range(256)]
    # tests/test_kvq.c:30-35: every finite code round-trips and is exact in BF16; three hand values
    for c in range(0x7F):
        assert L.or_e4m3_enc_abs(C.c_float(dec[c])) == c
        assert packs.round_bf16(np.float32(dec[c])) == np.float32(dec[c])
    assert dec[0x7E] == 448 and dec[0x01] == 0.001953125 and dec[0xB8] == -1
    # the closed form of the value table: (1 + m / 8) 2^(e - 7), subnormals m 2^-9
    for c in range(0x7F):
        e, m = c >> 3, c & 7
        assert dec[c] == ((1 + m / 8) * 2.0 ** (e - 7) if e else m * 2.0 ** -9)
    # rounding: nearest value, midpoints to the even code (:36-45), saturation at 448
    rng = np.random.default_rng(5)
    vals = np.array(dec[:0x7F], dtype=np.float64)
    for a in np.concatenate([rng.uniform(0, 500, 2000), rng.uniform(0, 0.05, 500), (vals[:-1] + vals[1:]) / 2]).astype(np.float32):
        got = L.or_e4m3_enc_abs(C.c_float(float(a)))
        if a >= 448:
            assert got == 0x7E
            continue
        d = np.abs(vals - float(a))
        best = np.flatnonzero(d == d.min())
        want = best[0] if len(best) == 1 else [b for b in best if b % 2 == 0][0]
        assert got == want, (a, got, want)
    # the scale: the smallest power of two s with 448 s >= amax
    for amax in np.concatenate([rng.uniform(1e-6, 1e4, 500), 448.0 * 2.0 ** np.arange(-20, 20)]).astype(np.float32):
        e = L.or_fp8_scale(C.c_float(float(amax))) - 127
        assert 448.0 * 2.0 ** e >= amax and 448.0 * 2.0 ** (e - 1) < amax
    assert L.or_fp8_scale(C.c_float(0.0)) == 127
    # a row: decode(encode(x)) within half a step of the block's E4M3 grid
    x = rng.standard_normal((3, 96)).astype(np.float32)
    codes, scales = oracle.fp8_row(x)
    y = oracle.fp8_decode(codes, scales)
    assert np.all(np.abs(y - x) <= np.abs(x) * 2.0 ** -4 + 2.0 ** (scales.repeat(32, 1).astype(np.float64) - 127 - 10))


def test_fp8_codec_vs_reference(oracle, ref):
    L = oracle.lib()
    for f in (L.or_e4m3_dec, ref.ref_e4m3_dec, ref.ref_fp8_get):
        f.restype = C.c_float
    for f in (L.or_e4m3_enc_abs, ref.ref_e4m3_enc_abs, L.or_fp8_scale, ref.ref_fp8_scale):
        f.restype = C.c_uint8
    rng = np.random.default_rng(6)
    for c in range(256):
        assert L.or_e4m3_dec(C.c_uint8(c)) == ref.ref_e4m3_dec(C.c_uint8(c))
    for a in np.abs(np.concatenate([rng.standard_normal(3000) * 100, rng.standard_normal(1000) * 0.01])).astype(np.float32):
        assert L.or_e4m3_enc_abs(C.c_float(float(a))) == ref.ref_e4m3_enc_abs(C.c_float(float(a)))
        assert L.or_fp8_scale(C.c_float(float(a))) == ref.ref_fp8_scale(C.c_float(float(a)))
    x = (rng.standard_normal((4, 128)) * rng.uniform(0.01, 50, (4, 1))).astype(np.float32)
    codes, scales = oracle.fp8_row(x)
    for i in range(4):
        rc, rs = np.zeros(128, np.uint8), np.zeros(4, np.uint8)
        ref.ref_fp8_row(x[i].ctypes.data_as(C.c_void_p), 128, rc.ctypes.data_as(C.c_void_p), rs.ctypes.data_as(C.c_void_p))
        assert np.array_equal(rc, codes[i]) and np.array_equal(rs, scales[i])


def test_mla_reference_forms(oracle):
    rng = np.random.default_rng(12)
    r, rope, npos = 64, 64, 9
    lat = packs.round_bf16(rng.standard_normal((npos, r)).astype(np.float32))
    kr = packs.round_bf16(rng.standard_normal((npos, rope)).astype(np.float32))
    ql = (rng.standard_normal(r) * 0.3).astype(np.float32)
    qr = rng.standard_normal(rope).astype(np.float32)
    # one position: that position's latent; zero queries: equal scores, the mean latent
    assert np.array_equal(oracle.mla_attn(ql, qr, lat, kr, 0, 0.1), lat[0])
    o = oracle.mla_attn(np.zeros(r, np.float32), np.zeros(rope, np.float32), lat, kr, npos - 1, 0.1)
    assert np.array_equal(o, packs.round_bf16(lat.astype(np.float64).mean(0).astype(np.float32)))
    # the general case against numpy in float64 (tests/test_mova_kernels.c:1006-1024)
    s = (lat[:6].astype(np.float64) @ ql + kr[:6].astype(np.float64) @ qr) * 0.125
    p = np.exp(s - s.max())
    want = packs.round_bf16(((p[:, None] * lat[:6]).sum(0) / p.sum()).astype(np.float32))
    assert np.array_equal(oracle.mla_attn(ql, qr, lat, kr, 5, 0.125), want)
    # rope: a rotation (norm kept), angle (float) pos * inv
    y0, y1 = oracle.rope_pair(0.3, -0.7, 11, 0.01)
    th = float(np.float32(np.float32(11) * np.float32(0.01)))
    assert abs(y0 - (0.3 * np.cos(th) + 0.7 * np.sin(th))) < 1e-15 and abs(y1 - (-0.7 * np.cos(th) + 0.3 * np.sin(th))) < 1e-15
    # per-head maps: bf16 of the double dot; with the gate, times bf16(softplus_ln2(g)), softplus_ln2(0) = 1
    H, O, I, T = 2, 3, 16, 2
    W = packs.round_bf16((rng.standard_normal((H * O, I)) * 0.1).astype(np.float32))
    x = packs.round_bf16(rng.standard_normal((T, H * I)).astype(np.float32))
    y = oracle.heads_map(W, x, H, O, I, H * I, I)
    want = packs.round_bf16(np.einsum("hoi,thi->tho", W.reshape(H, O, I).astype(np.float64), x.reshape(T, H, I).astype(np.float64)).astype(np.float32))
    assert np.array_equal(y, want)
    assert np.array_equal(oracle.heads_map(W, x, H, O, I, H * I, I, g=np.zeros((T, H, O), np.float32)), want)
