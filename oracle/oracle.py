"""ctypes view of the CPU oracle (oracle/nslm_oracle.c) and, when built, of the compiled reference (oracle/_ref).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg as the
checker.  The shipped package (nanoseedlm_amd/) never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboracle.so")
REF_PATH = os.path.join(HERE, "_ref", "libnslm_ref.so")

BF16, SEED4, Q8, Q4, SEED4P4 = 0, 1, 2, 3, 4


class OrSlice(C.Structure):
    _fields_ = [("p", C.c_void_p * 4), ("eb", C.c_int32), ("gs", C.c_int32)]


def build(force=False):
    """Compile liboracle.so (gcc) and, when the reference tree is present, oracle/_ref/libnslm_ref.so."""
    if force or not os.path.exists(LIB_PATH):
        subprocess.check_call(["make", "-C", HERE, "liboracle.so"] + (["-B"] if force else []))
    if os.path.isdir("/root/reference/nslm") and (force or not os.path.exists(REF_PATH)):
        subprocess.check_call(["make", "-C", HERE, "ref"] + (["-B"] if force else []))


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        L.or_lfsr_step.restype = C.c_uint16
        L.or_lfsr_step.argtypes = [C.c_uint16]
        L.or_lfsr_stream.restype = C.c_uint32
        L.or_lfsr_stream.argtypes = [C.c_uint16, C.c_int]
        L.or_lfsr_fnv24.restype = C.c_uint64
        L.or_scale.restype = C.c_float
        L.or_scale.argtypes = [C.c_int]
        L.or_f2bf.restype = C.c_uint16
        L.or_f2bf.argtypes = [C.c_float]
        L.or_silu_bf.restype = C.c_float
        L.or_silu_bf.argtypes = [C.c_float]
        L.or_bucket.restype = C.c_int
        L.or_cache_admit.restype = C.c_int
        _lib = L
    return _lib


def ref():
    """The compiled reference library, or None when it was not built (no reference tree, no prebuilt file)."""
    global _ref
    if _ref is None and os.path.exists(REF_PATH):
        R = C.CDLL(REF_PATH)
        R.ref_lfsr_step.restype = C.c_uint16
        R.ref_lfsr_step.argtypes = [C.c_uint16]
        R.ref_lfsr_stream24.restype = C.c_uint32
        R.ref_lfsr_stream24.argtypes = [C.c_uint16]
        R.ref_lfsr_stream32.restype = C.c_uint32
        R.ref_lfsr_stream32.argtypes = [C.c_uint16]
        R.ref_nslm_scale.restype = C.c_float
        R.ref_nslm_scale.argtypes = [C.c_int]
        R.ref_tile4.restype = C.c_void_p
        R.ref_tile3.restype = C.c_void_p
        R.ref_tile_free.argtypes = [C.c_void_p]
        _ref = R
    return _ref


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


# ---- numpy helpers -----------------------------------------------------------------------------------------------

def bf16_bits(x):
    """f32 array -> BF16 bits (round to nearest even), numpy restatement of nslm/lfsr.h:95-100."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return ((u >> 16) & 0xFFFF).astype(np.uint16)


def bf16_to_f32(h):
    return (np.asarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def bfr(x):
    return bf16_to_f32(bf16_bits(x))


def make_slice(fmt, p0=None, p1=None, p2=None, p3=None, eb=0, gs=0):
    s = OrSlice()
    keep = []
    for i, a in enumerate((p0, p1, p2, p3)):
        if a is not None:
            keep.append(a)
            s.p[i] = a.ctypes.data
    s.eb = int(eb)
    s.gs = int(gs)
    s._keep = keep
    return s


# ---- wrappers ----------------------------------------------------------------------------------------------------

def lfsr_states(seed, n):
    out = np.zeros(n, dtype=np.uint16)
    lib().or_lfsr_states(C.c_uint16(seed), C.c_int(n), _p(out))
    return out


def stream_table(nbits):
    t = np.zeros(65536, dtype=np.uint32)
    lib().or_lfsr_stream_table(C.c_int(nbits), _p(t))
    return t


def decode_p4(seed, coef, e):
    out = np.zeros(8, dtype=np.uint16)
    lib().or_decode_p4(C.c_uint16(seed), C.c_uint16(coef), C.c_int(e), _p(out))
    return out


def decode_p3(seed, nib, exp_bias):
    out = np.zeros(8, dtype=np.uint16)
    lib().or_decode_p3(C.c_uint16(seed), C.c_uint16(nib), C.c_int(exp_bias), _p(out))
    return out


def isum_p4(seed, coef):
    out = np.zeros(8, dtype=np.int32)
    lib().or_isum_p4(C.c_uint16(seed), C.c_uint16(coef), _p(out))
    return out


def isum_p3(seed, nib):
    out = np.zeros(8, dtype=np.int32)
    lib().or_isum_p3(C.c_uint16(seed), C.c_uint16(nib), _p(out))
    return out


def rows_f32(fmt, sl, R, K, round_=0):
    """All R rows of a slice as f32 [R, K] (seeds unrounded; affine rounded to BF16 when round_)."""
    out = np.zeros((R, K), dtype=np.float32)
    L = lib()
    for r in range(R):
        L.or_row_f32(C.c_int(fmt), C.byref(sl), C.c_int(R), C.c_int(K), C.c_int(r), C.c_int(round_), _p(out[r]))
    return out


def slice_bf16(fmt, sl, R, K):
    out = np.zeros((R, K), dtype=np.uint16)
    lib().or_slice_bf16(C.c_int(fmt), C.byref(sl), C.c_int(R), C.c_int(K), _p(out))
    return out


def mv_double(fmt, sl, R, K, x, qmv=1):
    """y[T, R] in double over the row decoder, and mag = sum |w x|."""
    x = _c(x, np.float32).reshape(-1, K)
    T = x.shape[0]
    y = np.zeros((T, R), dtype=np.float64)
    mag = np.zeros((T, R), dtype=np.float64)
    lib().or_mv_double(C.c_int(fmt), C.byref(sl), C.c_int(R), C.c_int(K), _p(x), C.c_int(K), C.c_int(T), C.c_int(qmv),
                       _p(y), _p(mag))
    return y, mag


def affine_dequant(words, scales, biases, n, bits, group=64):
    out = np.zeros(n, dtype=np.uint16)
    lib().or_affine_dequant(_p(words), _p(scales), _p(biases), C.c_int64(n), C.c_int(bits), C.c_int(group), _p(out))
    return out


def cpu_seed4_matvec(seeds, coefs, codes, bias, x, rows, kb, threads=1):
    y = np.zeros(rows, dtype=np.float32)
    lib().or_cpu_seed4_matvec(_p(seeds), _p(coefs), _p(codes), C.c_int(bias), _p(_c(x, np.float32)), C.c_int(rows),
                              C.c_int(kb), _p(y), C.c_int(threads))
    return y


def cpu_seed3_matvec(seeds, nibs, bias, x, rows, kb, threads=1):
    y = np.zeros(rows, dtype=np.float32)
    lib().or_cpu_seed3_matvec(_p(seeds), _p(nibs), C.c_int(bias), _p(_c(x, np.float32)), C.c_int(rows), C.c_int(kb),
                              _p(y), C.c_int(threads))
    return y


def route_softmax(logits, k):
    logits = _c(logits, np.float32)
    T, E = logits.shape
    ind = np.zeros((T, k), dtype=np.int32)
    wt = np.zeros((T, k), dtype=np.float32)
    for t in range(T):
        lib().or_route_softmax(C.c_int(E), C.c_int(k), _p(logits[t]), _p(ind[t]), _p(wt[t]))
    return ind, wt


def route_sigmoid(W, bias, x, k, hw, scale):
    W = _c(W, np.uint16)
    bias = _c(bias, np.uint16)
    x = _c(x, np.float32)
    n, d = W.shape
    T = x.shape[0]
    score = np.zeros((T, n), dtype=np.float32)
    sel = np.zeros((T, n), dtype=np.float32)
    inds = np.zeros((T, k), dtype=np.int32)
    wts = np.zeros((T, k), dtype=np.float32)
    lib().or_route_sigmoid(C.c_int(d), C.c_int(n), C.c_int(k), C.c_int(hw), C.c_float(scale), _p(W), _p(bias), _p(x),
                           C.c_int(T), _p(score), _p(sel), _p(inds), _p(wts))
    return score, sel, inds, wts


def topk_sigmoid(score, sel, k, scale):
    score = _c(score, np.float32)
    sel = _c(sel, np.float32)
    T, n = score.shape
    inds = np.zeros((T, k), dtype=np.int32)
    wts = np.zeros((T, k), dtype=np.float32)
    lib().or_topk_sigmoid(C.c_int(n), C.c_int(k), C.c_float(scale), _p(score), _p(sel), C.c_int(T), _p(inds), _p(wts))
    return inds, wts


def swiglu(g, u):
    g = _c(g, np.float32)
    u = _c(u, np.float32)
    a = np.zeros_like(g)
    lib().or_swiglu(_p(g), _p(u), _p(a), C.c_int(g.size))
    return a


def moe_combine(D, w, shared, x):
    """x[T, d] updated as engine/kernels_moe.cu:780-788; returns the new x."""
    D = _c(D, np.float32)
    w = _c(w, np.float32)
    shared = _c(shared, np.float32)
    x = np.array(x, dtype=np.float32, copy=True)
    T, d = x.shape
    k = w.shape[1]
    lib().or_moe_combine(_p(D), _p(w), _p(shared), _p(x), C.c_int(d), C.c_int(k), C.c_int(T))
    return x


def q4_moe_combine(D, wt, sh, sg):
    D = _c(D, np.float32)
    wt = _c(wt, np.float32)
    sh = _c(sh, np.float32)
    sg = _c(sg, np.float32)
    T, d = sh.shape
    k = wt.shape[1]
    out = np.zeros((T, d), dtype=np.float32)
    sgld = sg.shape[1] if sg.ndim == 2 else 1
    lib().or_q4_moe_combine(C.c_int(d), C.c_int(k), _p(D), _p(wt), _p(sh), _p(sg), C.c_int(sgld), _p(out), C.c_int(T))
    return out


def bucket(inds, n, bn):
    inds = _c(inds, np.int32).reshape(-1)
    count = inds.size
    perm = np.zeros(count, dtype=np.int32)
    tiles = np.zeros((count + n, 4), dtype=np.int32)
    nt = lib().or_bucket(_p(inds), C.c_int(count), C.c_int(n), C.c_int(bn), _p(perm), _p(tiles))
    return perm, tiles[:nt].copy()


def cache_admit(unit_slot, slot_unit, slot_last, tick, per_layer, sl, inds, protect_prev=0):
    """In-place host model of one admit; returns (jobs[nj,2], hits, misses)."""
    inds = _c(inds, np.int32).reshape(-1)
    jobs = np.zeros((per_layer, 2), dtype=np.int32)
    hits = C.c_uint32(0)
    misses = C.c_uint32(0)
    nj = lib().or_cache_admit(_p(unit_slot), _p(slot_unit), _p(slot_last), _p(tick), C.c_int(slot_unit.size),
                              C.c_int(per_layer), C.c_int(sl), _p(inds), C.c_int(inds.size), C.c_int(protect_prev),
                              _p(jobs), C.byref(hits), C.byref(misses))
    return jobs[:nj].copy(), hits.value, misses.value


def gnorm(x, w_bits, eps):
    """Grouped RMSNorm (2 groups): x [T, d] f32, w BF16 bits [d]."""
    x = _c(x, np.float32)
    w_bits = _c(w_bits, np.uint16)
    T, d = x.shape
    y = np.zeros_like(x)
    lib().or_gnorm(C.c_int(d), C.c_float(eps), _p(x), _p(w_bits), _p(y), C.c_int(T))
    return y


def norm1p(x, g, w, eps):
    """y = x r (1 + w) per group of g values of each row of x [T, len]."""
    x = _c(x, np.float32)
    w = _c(w, np.float32)
    T, ln = x.shape
    y = np.zeros_like(x)
    lib().or_norm1p(_p(x), C.c_int(ln), C.c_int(g), _p(w), C.c_float(eps), _p(y), C.c_int(T))
    return y


def argmax(logits, with_prob=False):
    logits = _c(logits, np.float32)
    n, V = logits.shape
    out = np.zeros(n, dtype=np.int32)
    prob = np.zeros(n, dtype=np.float64)
    lib().or_argmax(_p(logits), C.c_int(V), C.c_int(n), _p(out), _p(prob) if with_prob else None)
    return (out, prob) if with_prob else out


def fp8_row(x):
    """FP8 cache rows of x [rows, n] (n a multiple of 32): codes u8 [rows, n], scales u8 [rows, n / 32]."""
    x = _c(x, np.float32)
    rows, n = x.shape
    codes = np.zeros((rows, n), dtype=np.uint8)
    scales = np.zeros((rows, n // 32), dtype=np.uint8)
    for i in range(rows):
        lib().or_fp8_row(_p(x[i]), C.c_int(n), codes[i].ctypes.data_as(C.c_void_p), scales[i].ctypes.data_as(C.c_void_p))
    return codes, scales


def fp8_decode(codes, scales):
    codes = _c(codes, np.uint8)
    scales = _c(scales, np.uint8)
    lib().or_fp8_get.restype = C.c_float
    rows, n = codes.shape
    y = np.zeros((rows, n), dtype=np.float32)
    for i in range(rows):
        for j in range(n):
            y[i, j] = lib().or_fp8_get(codes[i].ctypes.data_as(C.c_void_p), scales[i].ctypes.data_as(C.c_void_p), C.c_int(j))
    return y


def heads_map(W, x, H, O, I, xs, hs, g=None):
    """W f32 [H * O, I] (exact weights), x [T, xs] -> y [T, H, O]."""
    W = _c(W, np.float32)
    x = _c(x, np.float32)
    T = x.shape[0]
    y = np.zeros((T, H, O), dtype=np.float32)
    gg = _c(g, np.float32) if g is not None else None
    lib().or_heads_map(C.c_int(H), C.c_int(O), C.c_int(I), _p(W), _p(x), C.c_int(xs), C.c_int(hs), _p(gg) if gg is not None else None,
                       _p(y), C.c_int(T))
    return y


def rope_pair(x0, x1, pos, inv):
    y0, y1 = C.c_double(0), C.c_double(0)
    lib().or_rope_pair(C.c_double(x0), C.c_double(x1), C.c_int(pos), C.c_float(inv), C.byref(y0), C.byref(y1))
    return y0.value, y1.value


def mla_attn(ql, qr, lat, kr, pos, scale):
    """One (row, head): ql [r], qr [rope], lat [npos, r], kr [npos, rope] (f32 values) -> olat [r]."""
    ql, qr, lat, kr = _c(ql, np.float32), _c(qr, np.float32), _c(lat, np.float32), _c(kr, np.float32)
    r, rope = ql.size, qr.size
    o = np.zeros(r, dtype=np.float32)
    lib().or_mla_attn(C.c_int(r), C.c_int(rope), C.c_double(scale), _p(ql), _p(qr), _p(lat), _p(kr), C.c_int(pos), _p(o))
    return o
