/* kernel_backend_hip.c - kernel_backend.h on the gfx950 library, as a C99 engine would drive it: plain C, no HIP header,
 * device memory and copies through the nh_ layer (include/nslm_rt.h), kernels through kc_ / kq4_ (include/kernels_hip.h).
 * Mirrors the reference's tests/kernel_backend_cuda.c call pattern: fresh allocations per call, default stream, sync,
 * copy back, free. */
#include "kernel_backend.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "nslm_rt.h"

static void* g_live[64]; /* this call's device allocations */
static int g_nlive;
static int g_bad;        /* an allocation or copy of this call failed */

static void* dev(const void* p, size_t n) { /* a device copy of n bytes (zeros when p is NULL) */
    void* d = NULL;
    if (g_nlive >= 64 || nh_malloc(&d, n ? n : 16)) { g_bad = 1; return NULL; }
    if (p ? nh_memcpy_h2d(d, p, n) : nh_memset(d, 0, n ? n : 16)) g_bad = 1;
    g_live[g_nlive++] = d;
    return d;
}
static int done(const char* what, void* host, const void* d, size_t n) { /* sync, copy back, free */
    int e = g_bad ? -1 : nh_device_sync();
    if (!e && host) e = nh_memcpy_d2h(host, d, n);
    if (!e) e = nh_last_error();
    if (!e) e = kc_last_error();
    for (int i = 0; i < g_nlive; ++i) nh_free(g_live[i]);
    g_nlive = 0;
    if (e) { printf("FAIL: %s: %s\n", what, g_bad ? "allocation or upload failed" : nh_error_string(e)); g_bad = 0; return -1; }
    return 0;
}
static int fetch(const char* what, void* host, const void* d, size_t n) { /* an output before the last one */
    if (!g_bad && !nh_device_sync() && !nh_memcpy_d2h(host, d, n)) return 0;
    done(what, NULL, NULL, 0);
    return -1;
}

int kt_open(char* err, int errlen) {
    int n = 0;
    if (nh_device_count(&n) || n < 1) { snprintf(err, (size_t) errlen, "no HIP device"); return -1; }
    return 0;
}
void kt_close(void) {}
const char* kt_name(void) { return "HIP gfx950"; }
int kt_mm_tile(void) { return MMT_BN; }
int kt_seed_gemm_exact(int on) { kc_seed_gemm_f32(on); return 1; }
int kt_has_fmt(int fmt) { return fmt >= MF_BF16 && fmt <= MF_SEED4P4; }
void kt_store_f32(int on) { kc_store_f32(on); }

/* the weight's slices (device addresses in freshly uploaded streams) */
static void slices(const KtWeight* w, WSlice* out) {
    const uint8_t* W = (const uint8_t*) dev(w->w, w->wn);
    const uint8_t* S = w->s ? (const uint8_t*) dev(w->s, w->sn) : NULL;
    const uint8_t* B = (w->b && (w->fmt == MF_Q8 || w->fmt == MF_Q4)) ? (const uint8_t*) dev(w->b, w->bn) : NULL;
    const uint8_t* E = w->e ? (const uint8_t*) dev(w->e, w->en) : NULL;
    const size_t rk = (size_t) w->R * w->K;
    const int group = w->group ? w->group : 64;
    for (int s = 0; s < w->S; ++s) {
        WSlice* o = &out[s];
        memset(o, 0, sizeof *o);
        switch (w->fmt) {
        case MF_BF16: o->p[0] = W + s * rk * 2; break;
        case MF_Q8: case MF_Q4:
            o->p[0] = W + s * rk / (w->fmt == MF_Q8 ? 1 : 2);
            o->p[1] = S + s * rk / group * 2;
            o->p[2] = B + s * rk / group * 2;
            o->gs = group == 32 ? 5 : 6;
            break;
        default: /* seeds */
            o->p[0] = W + s * rk / 8 * 2;
            o->p[1] = S + s * rk / 8 * 2;
            if (w->fmt == MF_SEED4P4) o->p[3] = E + s * rk / 16;
            o->eb = ((const int32_t*) w->b)[s];
        }
    }
}
#define MAXS 1024
static WSlice g_ws[MAXS];

int kt_mv(const KtWeight* w, int T, int add, const float* x, float* y) {
    if (w->S > MAXS) return -1;
    slices(w, g_ws);
    const size_t yn = sizeof(float) * (size_t) T * w->R;
    float* dy = (float*) dev(y, yn);
    const float* dx = (const float*) dev(x, sizeof(float) * (size_t) T * w->K);
    if (!g_bad) kc_mv(0, w->fmt, g_ws[0], w->K, w->R, dx, w->K, dy, w->R, T, add, NULL);
    return done("kc_mv", y, dy, yn);
}
int kt_mv_sel(const KtWeight* w, int P, int xdiv, const int32_t* sel, const float* x, float* y) {
    if (w->S > MAXS) return -1;
    slices(w, g_ws);
    const size_t yn = sizeof(float) * (size_t) P * w->R;
    float* dy = (float*) dev(NULL, yn);
    const WSlice* d = (const WSlice*) dev(g_ws, sizeof(WSlice) * (size_t) w->S);
    const float* dx = (const float*) dev(x, sizeof(float) * (size_t) ((P + xdiv - 1) / xdiv) * w->K);
    const int32_t* ds = (const int32_t*) dev(sel, 4 * (size_t) P);
    if (!g_bad) kc_mv_sel(0, w->fmt, d, w->K, w->R, dx, w->K, dy, w->R, ds, P, xdiv, NULL);
    return done("kc_mv_sel", y, dy, yn);
}
int kt_mv_gu(const KtWeight* w, int P, int xdiv, const int32_t* sel, const float* x, float* a) {
    if (w->S > MAXS) return -1;
    slices(w, g_ws);
    const size_t yn = sizeof(float) * (size_t) P * w->R;
    float* da = (float*) dev(NULL, yn);
    const WSlice* d = (const WSlice*) dev(g_ws, sizeof(WSlice) * (size_t) w->S);
    const float* dx = (const float*) dev(x, sizeof(float) * (size_t) ((P + xdiv - 1) / xdiv) * w->K);
    const int32_t* ds = (const int32_t*) dev(sel, 4 * (size_t) P);
    if (!g_bad) kc_mv_gu(0, w->fmt, d, d + 1, w->K, w->R, dx, w->K, da, w->R, ds, P, xdiv, NULL);   /* up = slice sel + 1 */
    return done("kc_mv_gu", a, da, yn);
}
int kt_mm(const KtWeight* w, int T, const float* x, float* y) {
    if (w->S > MAXS) return -1;
    slices(w, g_ws);
    const size_t yn = sizeof(float) * (size_t) T * w->R;
    float* dy = (float*) dev(y, yn);
    const float* dx = (const float*) dev(x, sizeof(float) * (size_t) T * w->K);
    if (!g_bad) kc_mm(0, w->fmt, g_ws[0], w->K, w->R, dx, w->K, dy, w->R, T, 1, NULL);
    return done("kc_mm", y, dy, yn);
}
int kt_mm_plain(const KtWeight* w, int T, int packed, const float* x, float* y) {
    if (w->S > MAXS) return -1;
    slices(w, g_ws);
    const size_t yn = sizeof(float) * (size_t) T * w->R, xn = (size_t) T * w->K;
    float* dy = (float*) dev(NULL, yn);
    const float* dx = (const float*) dev(x, sizeof(float) * xn);
    if (packed) {
        uint16_t* dp = (uint16_t*) dev(NULL, 2 * xn);
        if (!g_bad) {
            kc_pack_input_bf16(0, dx, dp, xn);
            kc_mm_packed(0, w->fmt, g_ws[0], w->K, w->R, dp, w->K, dy, w->R, T, 0, NULL);
        }
    } else if (!g_bad) kc_mm(0, w->fmt, g_ws[0], w->K, w->R, dx, w->K, dy, w->R, T, 0, NULL);
    return done("kc_mm", y, dy, yn);
}
int kt_mm_grouped(const KtWeight* w, int P, int xdiv, const int32_t* perm, const MmTile* tiles, int nt, const float* x,
                  float* y) {
    if (w->S > MAXS) return -1;
    slices(w, g_ws);
    const size_t yn = sizeof(float) * (size_t) P * w->R;
    float* dy = (float*) dev(NULL, yn);
    const WSlice* d = (const WSlice*) dev(g_ws, sizeof(WSlice) * (size_t) w->S);
    const float* dx = (const float*) dev(x, sizeof(float) * (size_t) ((P + xdiv - 1) / xdiv) * w->K);
    const int32_t* dp = (const int32_t*) dev(perm, 4 * (size_t) P);
    const MmTile* dt = (const MmTile*) dev(tiles, sizeof(MmTile) * (size_t) nt);
    if (!g_bad) kc_mm_grouped(0, w->fmt, d, w->K, w->R, dx, w->K, dy, w->R, xdiv, dp, dt, nt, NULL);
    return done("kc_mm_grouped", y, dy, yn);
}
int kt_bucket(const int32_t* inds, int count, int n, int32_t* perm, MmTile* tiles, int32_t* ntiles) {
    const int maxt = count / MMT_BN + n + 1;
    const int32_t* di = (const int32_t*) dev(inds, 4 * (size_t) count);
    int32_t* dp = (int32_t*) dev(NULL, 4 * (size_t) count);
    MmTile* dt = (MmTile*) dev(NULL, sizeof(MmTile) * (size_t) maxt);
    int32_t* dn = (int32_t*) dev(NULL, 4 * (size_t) (2 * n + 3));
    if (!g_bad) kc_bucket(0, di, count, n, dp, dt, dn);
    if (fetch("kc_bucket", perm, dp, 4 * (size_t) count)) return -1;
    if (fetch("kc_bucket", ntiles, dn, 4)) return -1;
    return done("kc_bucket", tiles, dt, sizeof(MmTile) * (size_t) (ntiles[0] < maxt ? ntiles[0] : maxt));
}
int kt_mm_bucketed(const KtWeight* w, int count, int xdiv, const int32_t* inds, int packed, const float* x, float* y,
                   int32_t* perm, MmTile* tiles, int32_t* ntiles) {
    if (w->S > MAXS) return -1;
    slices(w, g_ws);
    const int n = w->S, maxt = count / MMT_BN + n + 1;
    const size_t yn = sizeof(float) * (size_t) count * w->R, xn = (size_t) ((count + xdiv - 1) / xdiv) * w->K;
    float* dy = (float*) dev(NULL, yn);
    const WSlice* d = (const WSlice*) dev(g_ws, sizeof(WSlice) * (size_t) w->S);
    const float* dx = (const float*) dev(x, sizeof(float) * xn);
    const int32_t* di = (const int32_t*) dev(inds, 4 * (size_t) count);
    int32_t* dp = (int32_t*) dev(NULL, 4 * (size_t) count);
    MmTile* dt = (MmTile*) dev(NULL, sizeof(MmTile) * (size_t) maxt);
    int32_t* dn = (int32_t*) dev(NULL, 4 * (size_t) (2 * n + 3));
    if (!g_bad) {
        kc_bucket(0, di, count, n, dp, dt, dn);
        if (packed) {
            uint16_t* dxp = (uint16_t*) dev(NULL, 2 * xn);
            if (!g_bad) {
                kc_pack_input_bf16(0, dx, dxp, xn);
                kc_mm_grouped_packed(0, w->fmt, d, w->K, w->R, dxp, w->K, dy, w->R, xdiv, dp, dt, dn, maxt, NULL);
            }
        } else kc_mm_grouped_dev(0, w->fmt, d, w->K, w->R, dx, w->K, dy, w->R, xdiv, dp, dt, dn, maxt, NULL);
    }
    int32_t nt0 = 0;
    if (perm && fetch("kc_bucket", perm, dp, 4 * (size_t) count)) return -1;
    if (fetch("kc_bucket", &nt0, dn, 4)) return -1;
    if (ntiles) *ntiles = nt0;
    if (tiles && fetch("kc_bucket", tiles, dt, sizeof(MmTile) * (size_t) (nt0 < maxt ? nt0 : maxt))) return -1;
    return done("kc_mm_grouped_dev", y, dy, yn);
}
int kt_router(RouterArgs a, const uint16_t* W, const uint16_t* bias, const float* x, int T, int32_t* ind, float* wt) {
    const uint16_t* dW = (const uint16_t*) dev(W, 2 * (size_t) a.n * a.d);
    const uint16_t* db = (const uint16_t*) dev(bias, 2 * (size_t) a.n);
    const float* dx = (const float*) dev(x, 4 * (size_t) T * a.d);
    float* sc = (float*) dev(NULL, 4 * (size_t) T * a.n), *se = (float*) dev(NULL, 4 * (size_t) T * a.n);
    int32_t* di = (int32_t*) dev(NULL, 4 * (size_t) T * a.top_k);
    float* dw = (float*) dev(NULL, 4 * (size_t) T * a.top_k);
    if (!g_bad) kc_router(0, a, dW, db, dx, sc, se, di, dw, T);
    if (fetch("kc_router", ind, di, 4 * (size_t) T * a.top_k)) return -1;
    return done("kc_router", wt, dw, 4 * (size_t) T * a.top_k);
}
int kt_router_topk(RouterArgs a, const float* score, const float* sel, int T, int32_t* ind, float* wt) {
    const float* sc = (const float*) dev(score, 4 * (size_t) T * a.n), *se = (const float*) dev(sel, 4 * (size_t) T * a.n);
    int32_t* di = (int32_t*) dev(NULL, 4 * (size_t) T * a.top_k);
    float* dw = (float*) dev(NULL, 4 * (size_t) T * a.top_k);
    if (!g_bad) kc_router_topk(0, a, sc, se, di, dw, T);
    if (fetch("kc_router_topk", ind, di, 4 * (size_t) T * a.top_k)) return -1;
    return done("kc_router_topk", wt, dw, 4 * (size_t) T * a.top_k);
}
int kt_q4_route(int n_exp, int top_k, const float* logits, int32_t* ind, float* wt, int T) {
    Qwen4Cfg c;
    memset(&c, 0, sizeof c);
    c.n_exp = n_exp;
    c.top_k = top_k;
    const float* dl = (const float*) dev(logits, 4 * (size_t) T * n_exp);
    int32_t* di = (int32_t*) dev(NULL, 4 * (size_t) T * top_k);
    float* dw = (float*) dev(NULL, 4 * (size_t) T * top_k);
    if (!g_bad) kq4_route(0, &c, dl, di, dw, T);
    if (fetch("kq4_route", ind, di, 4 * (size_t) T * top_k)) return -1;
    return done("kq4_route", wt, dw, 4 * (size_t) T * top_k);
}
int kt_swiglu(const float* g, const float* u, float* a, int n) {
    const float* dg = (const float*) dev(g, 4 * (size_t) n), *du = (const float*) dev(u, 4 * (size_t) n);
    float* da = (float*) dev(NULL, 4 * (size_t) n);
    if (!g_bad) kc_swiglu(0, dg, du, da, n);
    return done("kc_swiglu", a, da, 4 * (size_t) n);
}
int kt_combine(const float* D, const float* w, const float* shared, float* x, int d, int k, int T) {
    const float* dD = (const float*) dev(D, 4 * (size_t) T * k * d), *dw = (const float*) dev(w, 4 * (size_t) T * k);
    const float* ds = (const float*) dev(shared, 4 * (size_t) T * d);
    float* dx = (float*) dev(x, 4 * (size_t) T * d);
    if (!g_bad) kc_moe_combine(0, dD, dw, ds, dx, d, k, T);
    return done("kc_moe_combine", x, dx, 4 * (size_t) T * d);
}
int kt_q4_combine(int d, int k, const float* D, const float* wt, const float* sh, const float* sg, int sgld, float* out, int T) {
    const float* dD = (const float*) dev(D, 4 * (size_t) T * k * d), *dw = (const float*) dev(wt, 4 * (size_t) T * k);
    const float* ds = (const float*) dev(sh, 4 * (size_t) T * d), *dg = (const float*) dev(sg, 4 * (size_t) T * sgld);
    float* dout = (float*) dev(NULL, 4 * (size_t) T * d);
    if (!g_bad) kq4_moe_combine(0, d, k, dD, dw, ds, dg, sgld, dout, T);
    return done("kq4_moe_combine", out, dout, 4 * (size_t) T * d);
}
int kt_gnorm(int d, float eps, const float* x, const uint16_t* w, float* y, int T) {
    const float* dx = (const float*) dev(x, 4 * (size_t) T * d);
    const uint16_t* dw = (const uint16_t*) dev(w, 2 * (size_t) d);
    float* dy = (float*) dev(NULL, 4 * (size_t) T * d);
    if (!g_bad) kc_gnorm(0, d, eps, dx, dw, dy, T);
    return done("kc_gnorm", y, dy, 4 * (size_t) T * d);
}
int kt_q4_norm1p(const float* x, int len, int g, const float* w, float eps, float* y, int T) {
    const float* dx = (const float*) dev(x, 4 * (size_t) T * len), *dw = (const float*) dev(w, 4 * (size_t) len);
    float* dy = (float*) dev(NULL, 4 * (size_t) T * len);
    if (!g_bad) kq4_norm1p(0, dx, len, g, dw, eps, dy, T);
    return done("kq4_norm1p", y, dy, 4 * (size_t) T * len);
}
int kt_embed(int fmt, const uint16_t* E, const uint32_t* q8, const uint16_t* s8, const uint16_t* b8, int V, int d,
             const int32_t* ids, int n, float* x) {
    WSlice w;
    memset(&w, 0, sizeof w);
    if (fmt == MF_BF16) {
        w.p[0] = dev(E, 2 * (size_t) V * d);
    } else {   /* Q8 (or Q4) with one group per 64 values */
        const size_t per = fmt == MF_Q8 ? 4 : 8;
        w.p[0] = dev(q8, 4 * (size_t) V * d / per);
        w.p[1] = dev(s8, 2 * (size_t) V * d / 64);
        w.p[2] = dev(b8, 2 * (size_t) V * d / 64);
    }
    const int32_t* di = (const int32_t*) dev(ids, 4 * (size_t) n);
    float* dx = (float*) dev(NULL, 4 * (size_t) n * d);
    if (!g_bad) kc_embed(0, fmt, w, d, di, dx, n);
    return done("kc_embed", x, dx, 4 * (size_t) n * d);
}
int kt_embed_seed(const KtWeight* w, const int32_t* ids, int n, float* x) {
    if (w->S > MAXS || (w->fmt != MF_SEED4P4 && w->fmt != MF_SEED4)) return 1;
    slices(w, g_ws);
    const int32_t* di = (const int32_t*) dev(ids, 4 * (size_t) n);
    float* dx = (float*) dev(NULL, 4 * (size_t) n * w->K);
    if (!g_bad) kc_embed(0, w->fmt, g_ws[0], w->K, di, dx, n);
    return done("kc_embed", x, dx, 4 * (size_t) n * w->K);
}
int kt_argmax(const float* logits, int V, int n, int32_t* out) {
    const float* dl = (const float*) dev(logits, 4 * (size_t) V * n);
    int32_t* dout = (int32_t*) dev(NULL, 4 * (size_t) n);
    if (!g_bad) kc_argmax(0, dl, dout, V, n);
    return done("kc_argmax", out, dout, 4 * (size_t) n);
}
int kt_argmax_p(const float* logits, int V, int n, int32_t* out, float* prob) {
    const float* dl = (const float*) dev(logits, 4 * (size_t) V * n);
    int32_t* dout = (int32_t*) dev(NULL, 4 * (size_t) n);
    float* dp = (float*) dev(NULL, 4 * (size_t) n);
    if (!g_bad) kc_argmax_p(0, dl, dout, dp, V, n);
    if (fetch("kc_argmax_p", prob, dp, 4 * (size_t) n)) return -1;
    return done("kc_argmax_p", out, dout, 4 * (size_t) n);
}
/* ---- MLA decode attention (tests/kernel_backend.h:79-81,97-104,123-137) ---- */
int kt_heads_w(const KtWeight* w, int H, int O, int I, const int32_t* ebias, const float* x, int xs, int hs, const float* g,
               float* y, int T) {
    /* W stacked [H][O][I] = slice 0 of w with R = H * O, K = I; seed maps: an exponent bias per head */
    if (w->S > MAXS) return -1;
    slices(w, g_ws);
    WSlice W = g_ws[0];
    if (w->fmt == MF_SEED4P4 && ebias) W.p[2] = dev(ebias, 4 * (size_t) H);
    else if (w->fmt == MF_SEED4P4) {   /* one bias for every head: the slice's own */
        int32_t eb[64];
        if (H > 64) return -1;
        for (int h = 0; h < H; ++h) eb[h] = g_ws[0].eb;
        W.p[2] = dev(eb, 4 * (size_t) H);
    }
    const size_t xn = (size_t) (T - 1) * xs + (size_t) (H - 1) * hs + I;
    const float* dx = (const float*) dev(x, 4 * xn);
    const float* dg = g ? (const float*) dev(g, 4 * (size_t) T * H * O) : NULL;
    float* dy = (float*) dev(NULL, 4 * (size_t) T * H * O);
    HmvArgs a = {H, O, I, xs, hs, g != NULL, {0, 0}};
    if (!g_bad) kc_heads_mv(0, a, w->fmt, W, NULL, dx, dg, dy, T);
    return done("kc_heads_mv", y, dy, 4 * (size_t) T * H * O);
}
/* caches of npos positions: BF16 (Kc / Vc as u16) or FP8 (codes + scale bytes); fmt KV_BF16 / KV_FP8 */
static KvView mla_view(int fmt, int r, int rope, int npos, void* k, void* v, void* ks, void* vs, void** dk, void** dv, void** dks, void** dvs) {
    KvView kv;
    memset(&kv, 0, sizeof kv);
    const size_t e = fmt == KV_BF16 ? 2 : 1;
    *dk = dev(k, e * (size_t) npos * rope);
    *dv = dev(v, e * (size_t) npos * r);
    *dks = fmt == KV_FP8 ? dev(ks, (size_t) npos * rope / 32) : NULL;
    *dvs = fmt == KV_FP8 ? dev(vs, (size_t) npos * r / 32) : NULL;
    kv.a.k = *dk; kv.a.v = *dv; kv.a.ks = (float*) *dks; kv.a.vs = (float*) *dvs;
    kv.nv = npos;   /* everything in segment a */
    kv.fmt = fmt;
    return kv;
}
int kt_mla_rope_f(MlaArgs a, int fmt, float* qr, const float* kr, const float* c, void* k, void* v, void* ks, void* vs, int npos,
                  const RowInfo* ri, const float* inv, int T) {
    const int rope = a.pad[0] > 0 ? a.pad[0] : ATT_HD;
    void *dk, *dv, *dks, *dvs;
    const KvView kv = mla_view(fmt, a.r, rope, npos, k, v, ks, vs, &dk, &dv, &dks, &dvs);
    float* dq = (float*) dev(qr, 4 * (size_t) T * a.n_head * rope);
    const float* dkr = (const float*) dev(kr, 4 * (size_t) T * rope), *dc = (const float*) dev(c, 4 * (size_t) T * a.r);
    const RowInfo* dri = (const RowInfo*) dev(ri, sizeof(RowInfo) * (size_t) T);
    const float* dinv = (const float*) dev(inv, 4 * (size_t) (rope / 2));
    if (!g_bad) kc_mla_rope(0, a, dq, dkr, dc, kv, dri, dinv, T);
    const size_t e = fmt == KV_BF16 ? 2 : 1;
    if (fetch("kc_mla_rope", k, dk, e * (size_t) npos * rope) || fetch("kc_mla_rope", v, dv, e * (size_t) npos * a.r)) return -1;
    if (fmt == KV_FP8 && (fetch("kc_mla_rope", ks, dks, (size_t) npos * rope / 32) || fetch("kc_mla_rope", vs, dvs, (size_t) npos * a.r / 32)))
        return -1;
    return done("kc_mla_rope", qr, dq, 4 * (size_t) T * a.n_head * rope);
}
int kt_mla_attn_f(MlaArgs a, int fmt, const float* ql, const float* qr, void* k, void* v, void* ks, void* vs, int npos,
                  const RowInfo* ri, float* olat, int T) {
    const int rope = a.pad[0] > 0 ? a.pad[0] : ATT_HD;
    void *dk, *dv, *dks, *dvs;
    const KvView kv = mla_view(fmt, a.r, rope, npos, k, v, ks, vs, &dk, &dv, &dks, &dvs);
    const float* dql = (const float*) dev(ql, 4 * (size_t) T * a.n_head * a.r), *dqr = (const float*) dev(qr, 4 * (size_t) T * a.n_head * rope);
    const RowInfo* dri = (const RowInfo*) dev(ri, sizeof(RowInfo) * (size_t) T);
    float* part = (float*) dev(NULL, 4 * (size_t) T * a.n_head * a.n_splits * (a.r + 2));
    float* dol = (float*) dev(NULL, 4 * (size_t) T * a.n_head * a.r);
    if (!g_bad) kc_mla_attn(0, a, dql, dqr, kv, dri, part, dol, T);
    return done("kc_mla_attn", olat, dol, 4 * (size_t) T * a.n_head * a.r);
}
int kt_kv_f32(int fmt, const uint8_t* codes, const uint8_t* scales, int len, int rows, float* y) {
    const uint8_t* dc = (const uint8_t*) dev(codes, (fmt == KV_BF16 ? 2 : 1) * (size_t) len * rows);
    const uint8_t* ds = fmt == KV_FP8 ? (const uint8_t*) dev(scales, (size_t) rows * len / 32) : NULL;
    float* dy = (float*) dev(NULL, 4 * (size_t) len * rows);
    if (!g_bad) kc_kv_f32(0, fmt, dc, ds, len, rows, dy);
    return done("kc_kv_f32", y, dy, 4 * (size_t) len * rows);
}
int kt_slice_deq(const KtWeight* w, int slice, uint16_t* out) {
    if (w->S > MAXS || slice >= w->S) return -1;
    slices(w, g_ws);
    const size_t on = 2 * (size_t) w->R * w->K;
    uint16_t* dout = (uint16_t*) dev(NULL, on);
    if (!g_bad) kc_slice_deq(0, w->fmt, g_ws[slice], w->K, w->R, dout);
    return done("kc_slice_deq", out, dout, on);
}
int kt_heads_deq(int fmt, int H, int O, int I, const void* p0, size_t n0, const void* p1, size_t n1, const int32_t* ebias,
                 const void* p3, size_t n3, int group, uint16_t* out) {
    WSlice W;
    memset(&W, 0, sizeof W);
    W.p[0] = dev(p0, n0);
    W.p[1] = dev(p1, n1);
    if (fmt == MF_SEED4P4) { W.p[2] = dev(ebias, 4 * (size_t) H); W.p[3] = dev(p3, n3); }
    else { W.p[2] = dev(p3, n3); W.gs = group == 32 ? 5 : 6; }
    const size_t on = 2 * (size_t) H * O * I;
    uint16_t* dout = (uint16_t*) dev(NULL, on);
    if (!g_bad) kc_heads_deq(0, fmt, W, NULL, H, O, I, dout);
    return done("kc_heads_deq", out, dout, on);
}
int kt_cache_admit(int32_t* unit_slot, int32_t* slot_unit, uint32_t* slot_last, uint32_t* tick, uint32_t* stats, int units,
                   int slots, int per_layer, int sl, const int32_t* inds, int count, int flags, int32_t* jobs) {
    CachePool p;
    memset(&p, 0, sizeof p);
    p.unit_slot = (int32_t*) dev(unit_slot, 4 * (size_t) units);
    p.slot_unit = (int32_t*) dev(slot_unit, 4 * (size_t) slots);
    p.slot_last = (uint32_t*) dev(slot_last, 4 * (size_t) slots);
    p.tick = (uint32_t*) dev(tick, 16);
    p.stats = (uint32_t*) dev(stats, 8);
    p.jobs = (int32_t*) dev(NULL, 8 * (size_t) per_layer);
    p.njobs = (int32_t*) dev(NULL, 4);
    p.slots = slots; p.per_layer = per_layer; p.ntens = 0; p.unit_bytes = 16;
    const int32_t* di = (const int32_t*) dev(inds, 4 * (size_t) count);
    if (!g_bad) kc_cache_admit(0, &p, sl, di, count, flags);
    int32_t nj = 0;
    if (fetch("kc_cache_admit", unit_slot, p.unit_slot, 4 * (size_t) units) || fetch("kc_cache_admit", slot_unit, p.slot_unit, 4 * (size_t) slots) ||
        fetch("kc_cache_admit", slot_last, p.slot_last, 4 * (size_t) slots) || fetch("kc_cache_admit", tick, p.tick, 16) ||
        fetch("kc_cache_admit", stats, p.stats, 8) || fetch("kc_cache_admit", &nj, p.njobs, 4)) return -1;
    if (done("kc_cache_admit", jobs, p.jobs, 8 * (size_t) (nj < per_layer ? nj : per_layer))) return -1;
    return nj;
}
int kt_cache_roundtrip(const uint8_t* arena, int units, int slots, uint64_t unit_bytes, int per_layer, const int32_t* inds,
                       int count, uint8_t* pool_out, int32_t* unit_slot_out) {
    CachePool p;
    memset(&p, 0, sizeof p);
    int32_t* us = (int32_t*) malloc(4 * (size_t) units), *su = (int32_t*) malloc(4 * (size_t) slots);
    for (int i = 0; i < units; ++i) us[i] = -1;
    for (int i = 0; i < slots; ++i) su[i] = -1;
    uint32_t tick[4] = {CACHE_TICK_BASE, 0, 0, 0};
    p.unit_slot = (int32_t*) dev(us, 4 * (size_t) units);
    p.slot_unit = (int32_t*) dev(su, 4 * (size_t) slots);
    p.slot_last = (uint32_t*) dev(NULL, 4 * (size_t) slots);
    p.tick = (uint32_t*) dev(tick, 16);
    p.stats = (uint32_t*) dev(NULL, 8);
    p.jobs = (int32_t*) dev(NULL, 8 * (size_t) per_layer);
    p.njobs = (int32_t*) dev(NULL, 4);
    p.vram = (uint8_t*) dev(NULL, (size_t) slots * unit_bytes);
    p.host = (const uint8_t*) dev(arena, (size_t) units * unit_bytes);
    p.unit_bytes = unit_bytes; p.slots = slots; p.per_layer = per_layer; p.ntens = 0;
    free(us); free(su);
    const int32_t* di = (const int32_t*) dev(inds, 4 * (size_t) count);
    if (!g_bad) { kc_cache_admit(0, &p, 0, di, count, 0); kc_cache_copy(0, &p, 64); }
    if (fetch("kc_cache_copy", unit_slot_out, p.unit_slot, 4 * (size_t) units)) return -1;
    return done("kc_cache_copy", pool_out, p.vram, (size_t) slots * unit_bytes);
}
