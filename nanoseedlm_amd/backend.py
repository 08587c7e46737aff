"""ctypes bindings of the gfx950 libraries: libnslm_hip.so (kc_* / kq4_* kernels and the nh_* runtime layer), libnslm_host.so
(the C99 host side: nslm_moe_*, nslm_model_*, nsf_*) and, for tests, tests/kt/libnslm_kt.so (the kernel-test binding, kt_*).
There is no CPU fallback: a missing library or GPU raises."""
import ctypes as C
import os
import subprocess

import numpy as np

from . import packs

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
HIP_SO = os.path.join(HERE, "libnslm_hip.so")
HOST_SO = os.path.join(HERE, "libnslm_host.so")
KT_SO = os.path.join(os.path.dirname(HERE), "tests", "kt", "libnslm_kt.so")


class WSlice(C.Structure):
    _fields_ = [("p", C.c_void_p * 4), ("eb", C.c_int32), ("gs", C.c_int32), ("pad", C.c_int32 * 2)]


class RowInfo(C.Structure):
    _fields_ = [("pos", C.c_int), ("kv0", C.c_int), ("pad", C.c_int * 2)]


class MlaArgs(C.Structure):
    _fields_ = [("n_head", C.c_int), ("r", C.c_int), ("chunk", C.c_int), ("n_splits", C.c_int), ("scale", C.c_float),
                ("pad", C.c_int * 3)]


KV_BF16, KV_FP8 = 0, 2


class HmvArgs(C.Structure):
    _fields_ = [("H", C.c_int), ("O", C.c_int), ("I", C.c_int), ("xs", C.c_int), ("hs", C.c_int), ("gate", C.c_int), ("pad", C.c_int * 2)]


class KvSeg(C.Structure):
    _fields_ = [("k", C.c_void_p), ("v", C.c_void_p), ("ks", C.c_void_p), ("vs", C.c_void_p)]


class KvView(C.Structure):
    _fields_ = [("a", KvSeg), ("b", KvSeg), ("nv", C.c_int32), ("fmt", C.c_int32)]


class RouterArgs(C.Structure):
    _fields_ = [("d", C.c_int), ("n", C.c_int), ("top_k", C.c_int), ("hw", C.c_int), ("scale", C.c_float)]


class MmTile(C.Structure):
    _fields_ = [("slice", C.c_int), ("start", C.c_int), ("count", C.c_int), ("pad", C.c_int)]


class CachePool(C.Structure):
    _fields_ = [("unit_slot", C.c_void_p), ("slot_unit", C.c_void_p), ("slot_last", C.c_void_p), ("tick", C.c_void_p),
                ("stats", C.c_void_p), ("jobs", C.c_void_p), ("njobs", C.c_void_p), ("vram", C.c_void_p),
                ("host", C.c_void_p), ("unit_bytes", C.c_uint64), ("slots", C.c_int32), ("per_layer", C.c_int32),
                ("ntens", C.c_int32), ("tab", C.c_void_p), ("off", (C.c_uint32 * 4) * 3), ("hits", C.c_uint64),
                ("misses", C.c_uint64)]


class Qwen4Cfg(C.Structure):
    _fields_ = ([(n, C.c_int) for n in ("n_layer", "d", "vocab", "eos", "hc", "hc_rank", "n_head", "n_kv", "head_dim", "rot_dim")]
                + [("rope_theta", C.c_float), ("eps", C.c_float)]
                + [(n, C.c_int) for n in ("ix_heads", "ix_dim", "ix_budget", "ix_ratio", "lin_hk", "lin_hv", "lin_dk", "lin_dv",
                                          "lin_conv", "n_exp", "top_k", "ff_exp", "ff_shared", "ple_dim", "ple_conv", "ngram",
                                          "heads_per_ngram", "ngram_parts")]
                + [("ngram_base", C.c_int64), ("ngram_div", C.c_int64), ("seed", C.c_int64), ("attn", C.c_uint8 * 128),
                   ("ple", C.c_int8 * 128)])


class KtWeight(C.Structure):
    _fields_ = [("fmt", C.c_int), ("S", C.c_int), ("R", C.c_int), ("K", C.c_int), ("w", C.c_void_p), ("s", C.c_void_p),
                ("b", C.c_void_p), ("e", C.c_void_p), ("wn", C.c_size_t), ("sn", C.c_size_t), ("bn", C.c_size_t),
                ("en", C.c_size_t), ("group", C.c_int)]


def build(force=False):
    """Compile both libraries in-tree (hipcc --offload-arch=gfx950, gcc)."""
    subprocess.check_call(["make", "-C", CSRC, "-j8", "all"] + (["-B"] if force else []))


_hip = None
_kt = None
_host = None


def hip():
    """libnslm_hip.so; raises when it has not been built."""
    global _hip
    if _hip is None:
        if not os.path.exists(HIP_SO):
            raise RuntimeError(f"{HIP_SO} is missing: build it with nanoseedlm_amd.backend.build() "
                               "(hipcc --offload-arch=gfx950); there is no CPU fallback")
        L = C.CDLL(HIP_SO, mode=C.RTLD_GLOBAL)
        L.nh_error_string.restype = C.c_char_p
        _hip = L
    return _hip


def host():
    """libnslm_host.so, the C99 host side (MoE layer, model step, model folder; links libnslm_hip.so); raises when missing."""
    global _host
    if _host is None:
        hip()
        if not os.path.exists(HOST_SO):
            raise RuntimeError(f"{HOST_SO} is missing: build it with nanoseedlm_amd.backend.build()")
        _host = C.CDLL(HOST_SO)
    return _host


def kt():
    """tests/kt/libnslm_kt.so, the kernel-test binding (kt_*: host arrays in, one kc_* call, host arrays out; links
    libnslm_hip.so).  Test infrastructure, not part of the product libraries; raises when missing."""
    global _kt
    if _kt is None:
        hip()
        if not os.path.exists(KT_SO):
            raise RuntimeError(f"{KT_SO} is missing: build it with nanoseedlm_amd.backend.build()")
        L = C.CDLL(KT_SO)
        L.kt_name.restype = C.c_char_p
        _kt = L
    return _kt


def require_gpu():
    n = C.c_int(0)
    if hip().nh_device_count(C.byref(n)) != 0 or n.value < 1:
        raise RuntimeError("no HIP device visible: this backend runs on an MI355X only")
    return n.value


def check(err, what="HIP call"):
    if err != 0:
        raise RuntimeError(f"{what} failed: {hip().nh_error_string(err).decode()} ({err})")


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


# ---- KtWeight from a pack (nanoseedlm_amd.packs) -------------------------------------------------------------------------

def kt_weight(p):
    """A KtWeight over the pack's host arrays (kept alive on the returned object)."""
    w = KtWeight()
    f = p["fmt"]
    w.fmt, w.S, w.R, w.K = f, p["S"], p["R"], p["K"]
    keep = []

    def put(field, nfield, arr):
        arr = np.ascontiguousarray(arr)
        keep.append(arr)
        setattr(w, field, arr.ctypes.data)
        setattr(w, nfield, arr.nbytes)

    if f == packs.MF_SEED4P4:
        put("w", "wn", p["seeds"]); put("s", "sn", p["coefs"]); put("b", "bn", p["eb"]); put("e", "en", p["codes"])
    elif f == packs.MF_SEED4:
        put("w", "wn", p["seeds"]); put("s", "sn", p["nibs"]); put("b", "bn", p["eb"])
    elif f in (packs.MF_Q4, packs.MF_Q8):
        put("w", "wn", p["words"]); put("s", "sn", p["scales"]); put("b", "bn", p["biases"])
        w.group = p["group"]
    else:
        put("w", "wn", p["w"])
    w._keep = keep
    return w


def _chk(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what} returned {rc}")


# ---- kt_* wrappers on numpy arrays ----------------------------------------------------------------------------------------

def kt_mv(p, x, T=None, add=0, y0=None):
    x = _c(x, np.float32).reshape(-1, p["K"])
    T = x.shape[0] if T is None else T
    y = np.zeros((T, p["R"]), dtype=np.float32) if y0 is None else np.array(y0, dtype=np.float32, copy=True)
    _chk(kt().kt_mv(C.byref(kt_weight(p)), T, add, _p(x), _p(y)), "kt_mv")
    return y


def kt_mv_sel(p, sel, x, xdiv):
    sel = _c(sel, np.int32)
    x = _c(x, np.float32)
    y = np.zeros((sel.size, p["R"]), dtype=np.float32)
    _chk(kt().kt_mv_sel(C.byref(kt_weight(p)), sel.size, xdiv, _p(sel), _p(x), _p(y)), "kt_mv_sel")
    return y


def kt_mv_gu(p, sel, x, xdiv):
    sel = _c(sel, np.int32)
    x = _c(x, np.float32)
    a = np.zeros((sel.size, p["R"]), dtype=np.float32)
    _chk(kt().kt_mv_gu(C.byref(kt_weight(p)), sel.size, xdiv, _p(sel), _p(x), _p(a)), "kt_mv_gu")
    return a


def kt_mm(p, x, y0):
    x = _c(x, np.float32).reshape(-1, p["K"])
    y = np.array(y0, dtype=np.float32, copy=True)
    _chk(kt().kt_mm(C.byref(kt_weight(p)), x.shape[0], _p(x), _p(y)), "kt_mm")
    return y


def kt_mm_plain(p, x, packed=0):
    x = _c(x, np.float32).reshape(-1, p["K"])
    y = np.zeros((x.shape[0], p["R"]), dtype=np.float32)
    _chk(kt().kt_mm_plain(C.byref(kt_weight(p)), x.shape[0], packed, _p(x), _p(y)), "kt_mm_plain")
    return y


def kt_mm_grouped(p, perm, tiles, x, xdiv):
    perm = _c(perm, np.int32)
    tiles = _c(tiles, np.int32).reshape(-1, 4)
    x = _c(x, np.float32)
    y = np.zeros((perm.size, p["R"]), dtype=np.float32)
    _chk(kt().kt_mm_grouped(C.byref(kt_weight(p)), perm.size, xdiv, _p(perm), _p(tiles), tiles.shape[0], _p(x), _p(y)),
         "kt_mm_grouped")
    return y


def kt_mm_bucketed(p, inds, x, xdiv, packed=0):
    inds = _c(inds, np.int32).reshape(-1)
    x = _c(x, np.float32)
    n = p["S"]
    y = np.zeros((inds.size, p["R"]), dtype=np.float32)
    perm = np.zeros(inds.size, dtype=np.int32)
    tiles = np.zeros((inds.size // 128 + n + 1, 4), dtype=np.int32)
    nt = np.zeros(1, dtype=np.int32)
    _chk(kt().kt_mm_bucketed(C.byref(kt_weight(p)), inds.size, xdiv, _p(inds), packed, _p(x), _p(y), _p(perm), _p(tiles),
                             _p(nt)), "kt_mm_bucketed")
    return y, perm, tiles[:int(nt[0])].copy()


def kt_bucket(inds, n):
    inds = _c(inds, np.int32).reshape(-1)
    perm = np.zeros(inds.size, dtype=np.int32)
    tiles = np.zeros((inds.size // 128 + n + 1, 4), dtype=np.int32)
    nt = np.zeros(1, dtype=np.int32)
    _chk(kt().kt_bucket(_p(inds), inds.size, n, _p(perm), _p(tiles), _p(nt)), "kt_bucket")
    return perm, tiles[:int(nt[0])].copy()


def kt_router(W, bias, x, k, hw, scale):
    W = _c(W, np.uint16)
    bias = _c(bias, np.uint16)
    x = _c(x, np.float32)
    n, d = W.shape
    T = x.shape[0]
    a = RouterArgs(d, n, k, hw, scale)
    ind = np.zeros((T, k), dtype=np.int32)
    wt = np.zeros((T, k), dtype=np.float32)
    _chk(kt().kt_router(a, _p(W), _p(bias), _p(x), T, _p(ind), _p(wt)), "kt_router")
    return ind, wt


def kt_router_topk(score, sel, k, scale):
    score = _c(score, np.float32)
    sel = _c(sel, np.float32)
    T, n = score.shape
    a = RouterArgs(0, n, k, 0, scale)
    ind = np.zeros((T, k), dtype=np.int32)
    wt = np.zeros((T, k), dtype=np.float32)
    _chk(kt().kt_router_topk(a, _p(score), _p(sel), T, _p(ind), _p(wt)), "kt_router_topk")
    return ind, wt


def kt_q4_route(logits, k):
    logits = _c(logits, np.float32)
    T, E = logits.shape
    ind = np.zeros((T, k), dtype=np.int32)
    wt = np.zeros((T, k), dtype=np.float32)
    _chk(kt().kt_q4_route(E, k, _p(logits), _p(ind), _p(wt), T), "kt_q4_route")
    return ind, wt


def kt_swiglu(g, u):
    g = _c(g, np.float32)
    u = _c(u, np.float32)
    a = np.zeros_like(g)
    _chk(kt().kt_swiglu(_p(g), _p(u), _p(a), g.size), "kt_swiglu")
    return a


def kt_combine(D, w, shared, x):
    D, w, shared = _c(D, np.float32), _c(w, np.float32), _c(shared, np.float32)
    x = np.array(x, dtype=np.float32, copy=True)
    T, d = x.shape
    _chk(kt().kt_combine(_p(D), _p(w), _p(shared), _p(x), d, w.shape[1], T), "kt_combine")
    return x


def kt_q4_combine(D, wt, sh, sg):
    D, wt, sh, sg = _c(D, np.float32), _c(wt, np.float32), _c(sh, np.float32), _c(sg, np.float32)
    T, d = sh.shape
    out = np.zeros((T, d), dtype=np.float32)
    sgld = sg.shape[1] if sg.ndim == 2 else 1
    _chk(kt().kt_q4_combine(d, wt.shape[1], _p(D), _p(wt), _p(sh), _p(sg), sgld, _p(out), T), "kt_q4_combine")
    return out


def kt_gnorm(x, w_bits, eps):
    x, w_bits = _c(x, np.float32), _c(w_bits, np.uint16)
    T, d = x.shape
    y = np.zeros_like(x)
    _chk(kt().kt_gnorm(d, C.c_float(eps), _p(x), _p(w_bits), _p(y), T), "kt_gnorm")
    return y


def kt_q4_norm1p(x, g, w, eps):
    x, w = _c(x, np.float32), _c(w, np.float32)
    T, ln = x.shape
    y = np.zeros_like(x)
    _chk(kt().kt_q4_norm1p(_p(x), ln, g, _p(w), C.c_float(eps), _p(y), T), "kt_q4_norm1p")
    return y


def kt_embed(p, ids):
    """Rows ids of slice 0 of a BF16 / Q8 / Q4 / seed pack as BF16-valued f32 [n, K]."""
    ids = _c(ids, np.int32)
    x = np.zeros((ids.size, p["K"]), dtype=np.float32)
    if p["fmt"] in (packs.MF_SEED4P4, packs.MF_SEED4):
        _chk(kt().kt_embed_seed(C.byref(kt_weight(p)), _p(ids), ids.size, _p(x)), "kt_embed_seed")
    elif p["fmt"] == packs.MF_BF16:
        E = _c(p["w"][0], np.uint16)
        _chk(kt().kt_embed(packs.MF_BF16, _p(E), None, None, None, p["R"], p["K"], _p(ids), ids.size, _p(x)), "kt_embed")
    else:
        q, s_, b = _c(p["words"][0], np.uint32), _c(p["scales"][0], np.uint16), _c(p["biases"][0], np.uint16)
        _chk(kt().kt_embed(p["fmt"], None, _p(q), _p(s_), _p(b), p["R"], p["K"], _p(ids), ids.size, _p(x)), "kt_embed")
    return x


def kt_argmax(logits, with_prob=False):
    logits = _c(logits, np.float32)
    n, V = logits.shape
    out = np.zeros(n, dtype=np.int32)
    if not with_prob:
        _chk(kt().kt_argmax(_p(logits), V, n, _p(out)), "kt_argmax")
        return out
    prob = np.zeros(n, dtype=np.float32)
    _chk(kt().kt_argmax_p(_p(logits), V, n, _p(out), _p(prob)), "kt_argmax_p")
    return out, prob


def kt_heads_w(p, H, O, I, x, xs, hs, g=None, ebias=None):
    """Per-head maps with W = slice 0 of pack p (R = H * O, K = I): y [T, H, O]."""
    x = _c(x, np.float32)
    T = x.shape[0]
    y = np.zeros((T, H, O), dtype=np.float32)
    gg = _c(g, np.float32) if g is not None else None
    eb = _c(ebias, np.int32) if ebias is not None else None
    _chk(kt().kt_heads_w(C.byref(kt_weight(p)), H, O, I, _p(eb) if eb is not None else None, _p(x), xs, hs,
                         _p(gg) if gg is not None else None, _p(y), T), "kt_heads_w")
    return y


def _ri(pos, kv0):
    ri = (RowInfo * len(pos))()
    for i, (a, b) in enumerate(zip(pos, kv0)):
        ri[i].pos, ri[i].kv0 = int(a), int(b)
    return ri


def kt_mla_rope(n_head, r, rope, fmt, qr, kr, c, cache, pos, kv0, inv):
    """cache = dict(k, v[, ks, vs]) of npos positions, updated in place; returns the rotated qr."""
    qr = np.array(qr, dtype=np.float32, copy=True)
    kr, c, inv = _c(kr, np.float32), _c(c, np.float32), _c(inv, np.float32)
    T = kr.shape[0]
    a = MlaArgs(n_head, r, 128, 1, 0.0)
    a.pad[0] = rope
    npos = cache["k"].shape[0]
    _chk(kt().kt_mla_rope_f(a, fmt, _p(qr), _p(kr), _p(c), _p(cache["k"]), _p(cache["v"]), _p(cache["ks"]) if fmt == KV_FP8 else None,
                            _p(cache["vs"]) if fmt == KV_FP8 else None, npos, _ri(pos, kv0), _p(inv), T), "kt_mla_rope_f")
    return qr


def kt_mla_attn(n_head, r, rope, fmt, ql, qr, cache, pos, kv0, scale, chunk, n_splits, long_from=0):
    ql, qr = _c(ql, np.float32), _c(qr, np.float32)
    T = len(pos)
    a = MlaArgs(n_head, r, chunk, n_splits, scale)
    a.pad[0], a.pad[2] = rope, long_from
    npos = cache["k"].shape[0]
    o = np.zeros((T, n_head, r), dtype=np.float32)
    _chk(kt().kt_mla_attn_f(a, fmt, _p(ql), _p(qr), _p(cache["k"]), _p(cache["v"]), _p(cache["ks"]) if fmt == KV_FP8 else None,
                            _p(cache["vs"]) if fmt == KV_FP8 else None, npos, _ri(pos, kv0), _p(o), T), "kt_mla_attn_f")
    return o


def kt_kv_f32(fmt, codes, scales):
    codes = np.ascontiguousarray(codes)
    rows, n = codes.shape
    y = np.zeros((rows, n), dtype=np.float32)
    _chk(kt().kt_kv_f32(fmt, _p(codes), _p(np.ascontiguousarray(scales)) if scales is not None else None, n, rows, _p(y)), "kt_kv_f32")
    return y


def kt_slice_deq(p, s=0):
    out = np.zeros((p["R"], p["K"]), dtype=np.uint16)
    _chk(kt().kt_slice_deq(C.byref(kt_weight(p)), s, _p(out)), "kt_slice_deq")
    return out


def kt_heads_deq_p4(seeds, coefs, ebias, codes, H, O, I):
    seeds, coefs, codes = _c(seeds, np.uint16), _c(coefs, np.uint16), _c(codes, np.uint8)
    ebias = _c(ebias, np.int32)
    out = np.zeros((H, O, I), dtype=np.uint16)
    _chk(kt().kt_heads_deq(packs.MF_SEED4P4, H, O, I, _p(seeds), C.c_size_t(seeds.nbytes), _p(coefs), C.c_size_t(coefs.nbytes),
                           _p(ebias), _p(codes), C.c_size_t(codes.nbytes), 0, _p(out)), "kt_heads_deq")
    return out


def kt_cache_admit(unit_slot, slot_unit, slot_last, tick, stats, per_layer, sl, inds, flags=0):
    """One admit on host-side state (updated in place); returns jobs [nj, 2]."""
    inds = _c(inds, np.int32).reshape(-1)
    jobs = np.zeros((per_layer, 2), dtype=np.int32)
    nj = kt().kt_cache_admit(_p(unit_slot), _p(slot_unit), _p(slot_last), _p(tick), _p(stats), unit_slot.size, slot_unit.size,
                             per_layer, sl, _p(inds), inds.size, flags, _p(jobs))
    if nj < 0:
        raise RuntimeError("kt_cache_admit failed")
    return jobs[:nj].copy()


def kt_cache_roundtrip(arena, slots, per_layer, inds):
    arena = _c(arena, np.uint8)
    units, unit_bytes = arena.shape
    inds = _c(inds, np.int32).reshape(-1)
    pool = np.zeros((slots, unit_bytes), dtype=np.uint8)
    unit_slot = np.zeros(units, dtype=np.int32)
    _chk(kt().kt_cache_roundtrip(_p(arena), units, slots, C.c_uint64(unit_bytes), per_layer, _p(inds), inds.size, _p(pool),
                                 _p(unit_slot)), "kt_cache_roundtrip")
    return pool, unit_slot
