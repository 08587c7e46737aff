/* moe_layer.c - see moe_layer.h.  Plain C99 over the kc_ / kq4_ / nh_ entry points. */
#include "moe_layer.h"
#include "model_folder.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "nslm_rt.h"

struct NslmMoe {
    NslmMoeCfg c;
    int units, resident, final;
    uint64_t unit_bytes, stream_len[3][4];
    CachePool pool;             /* device pointers inside */
    uint8_t* arena;             /* every unit: device memory, or (host_units) the device address of pinned host memory */
    uint8_t* arena_host;        /* host_units: the same memory as the host sees it */
    CachePool pool_pre;         /* prefetch: the pool with job lists and statistics of its own (two producers never share a list) */
    nh_stream_t cst;            /* prefetch: the copy stream */
    nh_event_t ev_admit, *ev_pred;   /* prefetch: admit done on the step's stream; layer l's predicted experts copied */
    int pred_pending;           /* layer whose predicted experts are being copied, or -1 */
    float *plogit, *pscore, *pwt;
    int32_t* pind;
    uint8_t* unit_host;         /* staging for one unit */
    int32_t* eb;                /* host: [units][3] exponent biases */
    uint16_t *rw, *rb;          /* device: router weights [layer][n_exp][d], biases [layer][n_exp] */
    uint16_t* px;               /* device: BF16 view of the step's activations [max_rows][d] (batched path) */
    float *logit, *score, *wt, *A, *G, *U, *D, *zero;
    int32_t *ind, *perm, *ntiles;
    MmTile* tiles;
    int max_tiles;
    uint32_t* sync;             /* device: the fused decode kernel's barrier words */
    int fused;                  /* 1: steps of the softmax composition up to kc_moe_decode_max_rows() rows take kc_moe_decode;
                                   2: the same, and every such step is checked and redone by the separate launchers if it failed */
    int fallbacks;              /* checked steps that were redone */
    long fused_steps;           /* steps the persistent kernel took */
};

static uint64_t pad256(uint64_t n) { return (n + 255) & ~(uint64_t) 255; }

NslmMoe* nslm_moe_open(const NslmMoeCfg* c, char* err, int errlen) {
    if (c->n_exp > CACHE_MAX_PER_LAYER || c->top_k > 32 || c->n_exp < c->top_k || (c->fmt != MF_SEED4P4 && c->fmt != MF_SEED4) ||
        c->d % 8 || c->ff % 8 || c->max_rows < 1) {
        snprintf(err, (size_t) errlen, "moe: unsupported configuration");
        return NULL;
    }
    NslmMoe* m = (NslmMoe*) calloc(1, sizeof *m);
    m->c = *c;
    m->units = c->n_layer * c->n_exp;
    /* unit layout: tensor i's stream s at a 256-byte aligned offset (engine/mova_cuda.c:318-327) */
    uint64_t cur = 0;
    for (int i = 0; i < 3; ++i)
        for (int s = 0; s < 4; ++s) {
            const uint64_t nblk = (uint64_t) c->d * c->ff / 8;
            uint64_t len = 0;
            if (s == 0 || s == 1) len = nblk * 2;
            else if (s == 3 && c->fmt == MF_SEED4P4) len = (nblk + 1) / 2;
            m->stream_len[i][s] = len;
            m->pool.off[i][s] = 0xFFFFFFFFu;
            if (!len) continue;
            m->pool.off[i][s] = (uint32_t) cur;
            cur += pad256(len);
        }
    m->unit_bytes = m->pool.unit_bytes = cur;
    m->pool.per_layer = c->n_exp;
    m->pool.ntens = 3;
    m->pool.slots = (c->slots <= 0 || c->slots >= m->units) ? m->units : c->slots;
    m->resident = m->pool.slots == m->units;
    if (!m->resident && m->pool.slots < 2 * c->top_k * c->max_rows && m->pool.slots < c->n_exp) {
        snprintf(err, (size_t) errlen, "moe: a pool of %d slots cannot hold one step's experts", m->pool.slots);
        free(m);
        return NULL;
    }
    const int P = c->max_rows * (c->top_k + 1);   /* + 1: the shared expert's pair in nslm_moe_step_layer */
    m->max_tiles = P / MMT_BN + c->n_exp + 1;
    int bad = 0;
    if (c->host_units) bad |= nh_host_alloc_mapped((void**) &m->arena_host, (void**) &m->arena, cur * (uint64_t) m->units);
    else bad |= nh_malloc((void**) &m->arena, cur * (uint64_t) m->units);
    if (m->resident) m->pool.vram = m->arena;
    else bad |= nh_malloc((void**) &m->pool.vram, cur * (uint64_t) m->pool.slots);
    m->pool.host = m->arena;
    bad |= nh_malloc((void**) &m->pool.unit_slot, 4 * (size_t) m->units);
    bad |= nh_malloc((void**) &m->pool.slot_unit, 4 * (size_t) m->pool.slots);
    bad |= nh_malloc((void**) &m->pool.slot_last, 4 * (size_t) m->pool.slots);
    bad |= nh_malloc((void**) &m->pool.tick, 16);
    bad |= nh_malloc((void**) &m->pool.stats, 16);
    bad |= nh_malloc((void**) &m->pool.jobs, 8 * (size_t) c->n_exp);
    bad |= nh_malloc((void**) &m->pool.njobs, 16);
    bad |= nh_malloc((void**) &m->pool.tab, sizeof(WSlice) * (size_t) m->units * 3);
    bad |= nh_malloc((void**) &m->rw, 2 * (size_t) c->n_layer * c->n_exp * c->d);
    bad |= nh_malloc((void**) &m->rb, 2 * (size_t) c->n_layer * c->n_exp);
    bad |= nh_malloc((void**) &m->logit, 4 * (size_t) c->max_rows * c->n_exp);
    bad |= nh_malloc((void**) &m->score, 4 * (size_t) c->max_rows * c->n_exp);
    bad |= nh_malloc((void**) &m->wt, 4 * (size_t) P);
    bad |= nh_malloc((void**) &m->ind, 4 * (size_t) P);
    bad |= nh_malloc((void**) &m->A, 4 * (size_t) P * c->ff);
    bad |= nh_malloc((void**) &m->G, 4 * (size_t) P * c->ff);
    bad |= nh_malloc((void**) &m->px, 2 * (size_t) c->max_rows * c->d);
    bad |= nh_malloc((void**) &m->U, 4 * (size_t) P * c->ff);
    bad |= nh_malloc((void**) &m->D, 4 * (size_t) P * c->d);
    bad |= nh_malloc((void**) &m->zero, 4 * (size_t) c->max_rows * c->d);
    bad |= nh_malloc((void**) &m->perm, 4 * (size_t) P);
    bad |= nh_malloc((void**) &m->tiles, sizeof(MmTile) * (size_t) m->max_tiles);
    bad |= nh_malloc((void**) &m->ntiles, 4 * (size_t) (2 * c->n_exp + 4));   /* + kq4_route_bucket's ticket word */
    bad |= nh_malloc((void**) &m->sync, 4 * kc_moe_decode_sync_words(kc_moe_decode_max_rows(), c->d));
    m->fused = 1;
    m->pred_pending = -1;
    if (c->prefetch && !m->resident && c->router == NSLM_ROUTE_SIGMOID) {
        m->pool_pre = m->pool;   /* the table and the slots are shared; filled in again by nslm_moe_finalize */
        bad |= nh_malloc((void**) &m->pool_pre.jobs, 8 * (size_t) c->n_exp);
        bad |= nh_malloc((void**) &m->pool_pre.njobs, 16);
        bad |= nh_malloc((void**) &m->pool_pre.stats, 16);
        bad |= nh_malloc((void**) &m->plogit, 4 * (size_t) c->max_rows * c->n_exp);
        bad |= nh_malloc((void**) &m->pscore, 4 * (size_t) c->max_rows * c->n_exp);
        bad |= nh_malloc((void**) &m->pwt, 4 * (size_t) P);
        bad |= nh_malloc((void**) &m->pind, 4 * (size_t) P);
        bad |= nh_stream_create_prio(&m->cst, 0);
        bad |= nh_event_create_untimed(&m->ev_admit);
        m->ev_pred = (nh_event_t*) calloc((size_t) c->n_layer, sizeof(nh_event_t));
        for (int l = 0; m->ev_pred && l < c->n_layer; ++l) bad |= nh_event_create_untimed(&m->ev_pred[l]);
        if (!m->ev_pred) bad = 1;
    }
    m->unit_host = (uint8_t*) calloc(1, cur);
    m->eb = (int32_t*) calloc((size_t) m->units * 3, 4);
    if (bad || !m->unit_host || !m->eb) {
        snprintf(err, (size_t) errlen, "moe: out of memory (%.2f GB of experts)", (double) cur * m->units / 1e9);
        nslm_moe_close(m);
        return NULL;
    }
    nh_memset(m->zero, 0, 4 * (size_t) c->max_rows * c->d);
    nh_memset(m->sync, 0, 4 * kc_moe_decode_sync_words(kc_moe_decode_max_rows(), c->d));
    nh_memset(m->rb, 0, 2 * (size_t) c->n_layer * c->n_exp);
    nh_memset(m->ntiles, 0, 4 * (size_t) (2 * c->n_exp + 4));
    return m;
}

void nslm_moe_close(NslmMoe* m) {
    if (!m) return;
    if (m->cst) {
        nh_stream_sync(m->cst);
        nh_stream_destroy(m->cst);
        nh_event_destroy(m->ev_admit);
        for (int l = 0; m->ev_pred && l < m->c.n_layer; ++l)
            if (m->ev_pred[l]) nh_event_destroy(m->ev_pred[l]);
        free(m->ev_pred);
        void* pd[] = {m->pool_pre.jobs, m->pool_pre.njobs, m->pool_pre.stats, m->plogit, m->pscore, m->pwt, m->pind};
        for (size_t i = 0; i < sizeof pd / sizeof pd[0]; ++i)
            if (pd[i]) nh_free(pd[i]);
    }
    if (m->arena_host) {
        nh_host_free(m->arena_host);
        m->arena = NULL;
    }
    void* d[] = {m->arena, m->resident ? NULL : m->pool.vram, m->pool.unit_slot, m->pool.slot_unit, m->pool.slot_last, m->pool.tick,
                 m->pool.stats, m->pool.jobs, m->pool.njobs, m->pool.tab, m->rw, m->rb, m->logit, m->score, m->wt, m->ind, m->A,
                 m->G, m->U, m->D, m->zero, m->perm, m->tiles, m->ntiles, m->sync, m->px};
    for (size_t i = 0; i < sizeof d / sizeof d[0]; ++i)
        if (d[i]) nh_free(d[i]);
    free(m->unit_host);
    free(m->eb);
    free(m);
}

/* host bytes into the arena: a copy to the device, or a plain copy where the arena is host memory */
static int arena_write(NslmMoe* m, uint8_t* dst, const void* src, uint64_t n) {
    if (!m->arena_host) return nh_memcpy_h2d(dst, src, n);
    memcpy(m->arena_host + (dst - m->arena), src, n);
    return 0;
}

int nslm_moe_set_expert(NslmMoe* m, int layer, int expert, int tensor, const uint16_t* seeds, const uint16_t* words,
                        const uint8_t* codes, int eb) {
    if (layer < 0 || layer >= m->c.n_layer || expert < 0 || expert >= m->c.n_exp || tensor < 0 || tensor > 2) return -1;
    const int u = layer * m->c.n_exp + expert;
    uint8_t* base = m->arena + (uint64_t) u * m->unit_bytes;
    int e = arena_write(m, base + m->pool.off[tensor][0], seeds, m->stream_len[tensor][0]);
    e |= arena_write(m, base + m->pool.off[tensor][1], words, m->stream_len[tensor][1]);
    if (m->c.fmt == MF_SEED4P4) e |= arena_write(m, base + m->pool.off[tensor][3], codes, m->stream_len[tensor][3]);
    m->eb[u * 3 + tensor] = eb;
    return e ? -1 : 0;
}

int nslm_moe_set_router(NslmMoe* m, int layer, const uint16_t* W, const uint16_t* bias) {
    if (layer < 0 || layer >= m->c.n_layer) return -1;
    int e = nh_memcpy_h2d(m->rw + (size_t) layer * m->c.n_exp * m->c.d, W, 2 * (size_t) m->c.n_exp * m->c.d);
    if (bias) e |= nh_memcpy_h2d(m->rb + (size_t) layer * m->c.n_exp, bias, 2 * (size_t) m->c.n_exp);
    return e ? -1 : 0;
}

/* A model folder's stacked expert tensor [experts][rows][cols / 8] into the arena: expert e's share of each stream is
 * contiguous in the file, its exponent bias is entry e of the exp_bias stream. */
int nslm_moe_load_experts(NslmMoe* m, int layer, int which, const NsfTensor* t) {
    const int rows = which == 2 ? m->c.d : m->c.ff, cols = which == 2 ? m->c.ff : m->c.d;
    if (!t || layer < 0 || layer >= m->c.n_layer || which < 0 || which > 2 || t->enc != m->c.fmt || t->slices != m->c.n_exp || t->rows != rows ||
        t->cols != cols)
        return -1;
    int bad = 0;
    for (int e = 0; e < m->c.n_exp && !bad; ++e) {
        const int u = layer * m->c.n_exp + e;
        uint8_t* base = m->arena + (uint64_t) u * m->unit_bytes;
        for (int s = 0; s < 4; ++s) {
            if (s == 2 || !m->stream_len[which][s]) continue;
            const uint64_t n = m->stream_len[which][s];
            if (t->s[s].len != n * (uint64_t) m->c.n_exp) return -1;
            if (m->arena_host) memcpy(m->arena_host + (base - m->arena) + m->pool.off[which][s], t->s[s].p + (uint64_t) e * n, n);
            else bad |= nsf_upload(base + m->pool.off[which][s], &t->s[s], (uint64_t) e * n, n);
        }
        int32_t eb;
        memcpy(&eb, t->s[2].p + 4 * (size_t) e, 4);
        m->eb[u * 3 + which] = eb;
    }
    return bad ? -1 : 0;
}
int nslm_moe_load_router(NslmMoe* m, int layer, const NsfTensor* w, const NsfTensor* bias) {
    if (!w || layer < 0 || layer >= m->c.n_layer || w->enc != NSF_BF16 || w->slices != 1 || w->rows != m->c.n_exp || w->cols != m->c.d) return -1;
    if (bias && (bias->enc != NSF_BF16 || bias->s[0].len != 2 * (uint64_t) m->c.n_exp)) return -1;
    int bad = nsf_upload(m->rw + (size_t) layer * m->c.n_exp * m->c.d, &w->s[0], 0, w->s[0].len);
    if (bias) bad |= nsf_upload(m->rb + (size_t) layer * m->c.n_exp, &bias->s[0], 0, bias->s[0].len);
    return bad ? -1 : 0;
}

int nslm_moe_fill_random(NslmMoe* m, uint64_t seed, int eb, float router_scale) {
    kc_fill_random(0, m->arena, m->unit_bytes * (uint64_t) m->units, seed);
    kc_fill_bf16(0, m->rw, (size_t) m->c.n_layer * m->c.n_exp * m->c.d, seed ^ 0x5151, router_scale);
    for (int i = 0; i < m->units * 3; ++i) m->eb[i] = eb;
    return nh_device_sync() || kc_last_error() ? -1 : 0;
}

/* initial residency round-robin over the layers, expert-major, and the slice tables (engine/mova_cuda.c:372-392) */
int nslm_moe_finalize(NslmMoe* m) {
    const int units = m->units, slots = m->pool.slots, E = m->c.n_exp, nl = m->c.n_layer;
    int32_t* us = (int32_t*) malloc(4 * (size_t) units);
    int32_t* su = (int32_t*) malloc(4 * (size_t) slots);
    WSlice* tab = (WSlice*) calloc((size_t) units * 3, sizeof(WSlice));
    const uint32_t tick0[4] = {CACHE_TICK_BASE, 0, 0, 0};
    int bad = 0, s = 0;
    for (int u = 0; u < units; ++u) us[u] = -1;
    for (int i = 0; i < slots; ++i) su[i] = -1;
    if (m->resident) {
        for (int u = 0; u < units; ++u) us[u] = su[u] = u;   /* the arena is the pool */
    } else {
        for (int x = 0; x < E && s < slots; ++x)
            for (int sl = 0; sl < nl && s < slots; ++sl, ++s) {
                const int u = sl * E + x;
                us[u] = s;
                su[s] = u;
                if (m->arena_host) bad |= nh_memcpy_h2d(m->pool.vram + (uint64_t) s * m->unit_bytes, m->arena_host + (uint64_t) u * m->unit_bytes, m->unit_bytes);
                else bad |= nh_memcpy_d2d(m->pool.vram + (uint64_t) s * m->unit_bytes, m->arena + (uint64_t) u * m->unit_bytes, m->unit_bytes);
            }
    }
    for (int sl = 0; sl < nl; ++sl)
        for (int i = 0; i < 3; ++i)
            for (int x = 0; x < E; ++x) {
                WSlice* t = &tab[((size_t) sl * 3 + i) * E + x];
                const int u = sl * E + x;
                t->eb = m->eb[u * 3 + i];
                if (us[u] < 0) continue;
                for (int st = 0; st < 4; ++st)
                    if (m->pool.off[i][st] != 0xFFFFFFFFu) t->p[st] = m->pool.vram + (uint64_t) us[u] * m->unit_bytes + m->pool.off[i][st];
            }
    bad |= nh_memcpy_h2d(m->pool.unit_slot, us, 4 * (size_t) units);
    bad |= nh_memcpy_h2d(m->pool.slot_unit, su, 4 * (size_t) slots);
    bad |= nh_memset(m->pool.slot_last, 0, 4 * (size_t) slots);
    bad |= nh_memcpy_h2d(m->pool.tick, tick0, 16);
    bad |= nh_memset(m->pool.njobs, 0, 16);
    bad |= nh_memset(m->pool.stats, 0, 16);
    bad |= nh_memcpy_h2d(m->pool.tab, tab, sizeof(WSlice) * (size_t) units * 3);
    if (m->cst) {   /* the prefetch's view: the same table and slots, its own job list and counters */
        CachePool pre = m->pool;
        pre.jobs = m->pool_pre.jobs; pre.njobs = m->pool_pre.njobs; pre.stats = m->pool_pre.stats;
        m->pool_pre = pre;
        bad |= nh_memset(pre.njobs, 0, 16);
        bad |= nh_memset(pre.stats, 0, 16);
    }
    bad |= nh_device_sync();
    free(us); free(su); free(tab);
    m->final = !bad;
    return bad ? -1 : 0;
}

/* The layer's whole expert block in the one persistent launch: routed experts + a shared expert of their shape + the
 * residual (out = bf16(res + bf16(sum)), res may be out).  0 done, 1 not available for this stack / shape (nothing
 * launched: compose nslm_moe_step with kc_mv_gu / kc_mv / kc_residual_add), -1 error. */
int nslm_moe_step_layer(NslmMoe* m, kc_stream_t s, int layer, const float* xn, int T, const WSlice* shared, const float* res, float* out,
                        const float* norm_w, float norm_eps) {
    const NslmMoeCfg* c = &m->c;
    if (!m->final || T < 1 || T > c->max_rows || layer < 0 || layer >= c->n_layer) return -1;
    const int E = c->n_exp;
    const WSlice* tab = m->pool.tab + (size_t) layer * 3 * E;
    /* (a checked stack composes the block from nslm_moe_step, which can redo its part: this launch updates out in place) */
    if (!(m->fused == 1 && m->resident && c->router == NSLM_ROUTE_SOFTMAX && T <= kc_moe_decode_max_rows())) return 1;
    if (kc_moe_decode_layer(s, c->fmt, m->rw + (size_t) layer * E * c->d, tab, tab + E, tab + 2 * E, E, c->top_k, c->d, c->ff, xn, c->d, T, out,
                            c->d, m->logit, m->ind, m->wt, m->A, m->D, m->sync, shared, res, norm_w, norm_eps))
        return 1;
    m->fused_steps++;
    return kc_last_error() ? -1 : 0;
}

int nslm_moe_step(NslmMoe* m, kc_stream_t s, int layer, const float* xn, int T, float* io) {
    const NslmMoeCfg* c = &m->c;
    if (!m->final || T < 1 || T > c->max_rows || layer < 0 || layer >= c->n_layer) return -1;
    const int E = c->n_exp, k = c->top_k, d = c->d, ff = c->ff, P = T * k;
    const WSlice* gate = m->pool.tab + ((size_t) layer * 3 + 0) * E;
    const WSlice* up = m->pool.tab + ((size_t) layer * 3 + 1) * E;
    const WSlice* down = m->pool.tab + ((size_t) layer * 3 + 2) * E;
    if (m->fused && m->resident && c->router == NSLM_ROUTE_SOFTMAX && T <= kc_moe_decode_max_rows() &&
        !kc_moe_decode(s, c->fmt, m->rw + (size_t) layer * E * d, gate, up, down, E, k, d, ff, xn, d, T, io, d, m->logit, m->ind,
                       m->wt, m->A, m->D, m->sync)) {   /* the whole step in one persistent kernel */
        m->fused_steps++;
        if (m->fused != 2) return kc_last_error() ? -1 : 0;
        /* checked: the kernel's workgroups wait for each other, and a wait that gave up (the grid was not resident at once:
           another stream's kernel held the CUs) has left void results and the sync words in no defined state.  Then the words
           are zeroed, the stack goes back to the separate launchers (until nslm_moe_set_fused turns the kernel on again) and
           the step is redone by them: xn is untouched and io only written. */
        uint32_t w = 0;
        if (kc_last_error() || nh_stream_sync((nh_stream_t) s) || nh_memcpy_d2h(&w, m->sync + kc_moe_decode_error_word(), 4)) return -1;
        if (!w) return 0;
        if (nh_memset_async(m->sync, 0, 4 * kc_moe_decode_sync_words(kc_moe_decode_max_rows(), c->d), (nh_stream_t) s)) return -1;   /* on s: ordered before the stack's next kernel there */
        m->fused = 0;
        m->fallbacks++;
    }
    int routed_and_grouped = 0;
    if (c->router == NSLM_ROUTE_SOFTMAX) {
        WSlice rw;
        memset(&rw, 0, sizeof rw);
        rw.p[0] = m->rw + (size_t) layer * E * d;
        Qwen4Cfg qc;
        memset(&qc, 0, sizeof qc);
        qc.n_exp = E;
        qc.top_k = k;
        if (T <= MV_MAXT) {
            kc_mv(s, MF_BF16, rw, d, E, xn, d, m->logit, E, T, 0, NULL);
            kq4_route(s, &qc, m->logit, m->ind, m->wt, T);
        } else {
            /* The batched path: the logits by the decode path's row sums over the input rounded to BF16, as the GEMM
               multiplies it (a 128-row GEMM is two workgroups: 16 us where this takes 5), the BF16 view of xn that the
               three GEMMs read made by the same launch;
               then routing and grouping in one launch.  Shapes the folded launches do not take go the reference's way
               (engine/qwen4_cuda.c:1033-1034, 1058-1061: router matvec or GEMM, route, bucket). */
            const int packed = d % 8 == 0 && ff % 8 == 0;
            if (!(packed && T <= 64 && !kc_mv_pack(s, MF_BF16, rw, d, E, xn, d, m->logit, E, T, m->px))) {
                if (packed) {
                    kc_pack_input_bf16(s, xn, m->px, (size_t) T * d);
                    kc_mm_packed(s, MF_BF16, rw, d, E, m->px, d, m->logit, E, T, 0, NULL);
                } else {
                    kc_mm(s, MF_BF16, rw, d, E, xn, d, m->logit, E, T, 0, NULL);
                }
            }
            kq4_route_bucket(s, &qc, m->logit, m->ind, m->wt, T, m->perm, m->tiles, m->ntiles);
            routed_and_grouped = 1;
        }
    } else {
        RouterArgs ra = {d, E, k, d / 2, c->route_scale};
        kc_router(s, ra, m->rw + (size_t) layer * E * d, m->rb + (size_t) layer * E, xn, m->logit, m->score, m->ind, m->wt, T);
    }
    if (!m->resident) {   /* with every expert resident the table never changes: nothing to admit, nothing to copy */
        if (m->pred_pending >= 0) {   /* the predicted experts' copies land before the table is consulted - or changed: a caller
                                         that does not go on with the predicted layer must not meet copies in flight either */
            nh_stream_wait_event((nh_stream_t) s, m->ev_pred[m->pred_pending]);
            m->pred_pending = -1;
        }
        kc_cache_admit(s, &m->pool, layer, m->ind, P, 0);
        kc_cache_copy(s, &m->pool, 64);
        if (m->cst && T <= MV_MAXT && layer + 1 < c->n_layer) {
            /* decode: the next layer's likely experts, from its router on this layer's input; their slots may not be the ones
               this layer's gathers are about to read (CACHE_PROTECT_PREV), and their copies run beside those gathers */
            RouterArgs ra = {d, E, k, d / 2, c->route_scale};
            kc_router(s, ra, m->rw + (size_t) (layer + 1) * E * d, m->rb + (size_t) (layer + 1) * E, xn, m->plogit, m->pscore, m->pind, m->pwt, T);
            kc_cache_admit(s, &m->pool_pre, layer + 1, m->pind, P, CACHE_PROTECT_PREV);
            nh_event_record(m->ev_admit, (nh_stream_t) s);
            nh_stream_wait_event(m->cst, m->ev_admit);
            kc_cache_copy((kc_stream_t) m->cst, &m->pool_pre, 8);
            nh_event_record(m->ev_pred[layer + 1], m->cst);
            m->pred_pending = layer + 1;
        }
    }
    if (T <= MV_MAXT) {   /* decode: one gather pass per (token, expert) pair (engine/mova_cuda.c:1301-1307) */
        kc_mv_gu(s, c->fmt, gate, up, d, ff, xn, d, m->A, ff, m->ind, P, k, NULL);
        kc_mv_sel(s, c->fmt, down, ff, d, m->A, ff, m->D, d, m->ind, P, 1, NULL);
    } else {              /* batched: pairs grouped by expert, three grouped GEMMs (engine/mova_cuda.c:1308-1317) */
        /* BF16 views of the activations feed the MFMA path, as the reference's packed_layer() case does
           (engine/mova_cuda.c:1012-1035,1229,1308-1317): SwiGLU writes A as that view directly */
        const int packed = d % 8 == 0 && ff % 8 == 0;
        if (!routed_and_grouped) kc_bucket(s, m->ind, P, E, m->perm, m->tiles, m->ntiles);
        if (packed) {
            if (c->router != NSLM_ROUTE_SOFTMAX) kc_pack_input_bf16(s, xn, m->px, (size_t) T * d);   /* else: made for the router */
            /* a step of T rows chooses no expert more than T times: no tile holds more than T pairs */
            /* gate, up and SwiGLU in one launch (else: the two GEMMs in one launch, then SwiGLU) */
            if (kc_mm_grouped_swiglu(s, c->fmt, gate, up, d, ff, m->px, d, (uint16_t*) m->A, ff, k, m->perm, m->tiles, m->ntiles, m->max_tiles, T)) {
                kc_mm_grouped_packed_pair(s, c->fmt, gate, up, d, ff, m->px, d, m->G, m->U, ff, k, m->perm, m->tiles, m->ntiles, m->max_tiles, T);
                kc_swiglu_pack(s, m->G, m->U, (uint16_t*) m->A, (size_t) P * ff);
            }
            kc_mm_grouped_packed_rows(s, c->fmt, down, ff, d, (const uint16_t*) m->A, ff, m->D, d, 1, m->perm, m->tiles, m->ntiles,
                                      m->max_tiles, T);
        } else {
            kc_mm_grouped_dev(s, c->fmt, gate, d, ff, xn, d, m->G, ff, k, m->perm, m->tiles, m->ntiles, m->max_tiles, NULL);
            kc_mm_grouped_dev(s, c->fmt, up, d, ff, xn, d, m->U, ff, k, m->perm, m->tiles, m->ntiles, m->max_tiles, NULL);
            kc_swiglu(s, m->G, m->U, m->A, P * ff);
            kc_mm_grouped_dev(s, c->fmt, down, ff, d, m->A, ff, m->D, d, 1, m->perm, m->tiles, m->ntiles, m->max_tiles, NULL);
        }
    }
    if (c->router == NSLM_ROUTE_SOFTMAX) kq4_moe_combine(s, d, k, m->D, m->wt, m->zero, m->zero, 0, io, T);
    else kc_moe_combine(s, m->D, m->wt, m->zero, io, d, k, T);
    return kc_last_error() ? -1 : 0;
}

void nslm_moe_set_fused(NslmMoe* m, int on) { m->fused = on; }
int nslm_moe_fused_mode(const NslmMoe* m) { return m->fused; }
int nslm_moe_step_seq(NslmMoe* m, kc_stream_t s, int n, const int* layers, const float* const* xn, int T, float* io, void* before,
                      void* after) {
    if (before && nh_event_record((nh_event_t) before, (nh_stream_t) s)) return -1;
    for (int i = 0; i < n; ++i)
        if (nslm_moe_step(m, s, layers[i], xn[i], T, io)) return -1;
    if (after && nh_event_record((nh_event_t) after, (nh_stream_t) s)) return -1;
    return 0;
}
int nslm_mv_seq(kc_stream_t s, int fmt, const WSlice* ws, int nw, int first, int n, int K, int R, const float* x, float* y, void* before,
                void* after) {
    if (nw < 1 || first < 0) return -1;
    if (before && nh_event_record((nh_event_t) before, (nh_stream_t) s)) return -1;
    for (int i = 0; i < n; ++i) kc_mv(s, fmt, ws[(first + i) % nw], K, R, x, K, y, R, 1, 0, NULL);
    if (after && nh_event_record((nh_event_t) after, (nh_stream_t) s)) return -1;
    return kc_last_error() ? -1 : 0;
}
int nslm_moe_fallbacks(const NslmMoe* m) { return m->fallbacks; }
long nslm_moe_fused_steps(const NslmMoe* m) { return m->fused_steps; }
void* nslm_moe_sync_ptr(NslmMoe* m) { return m->sync; }
const uint16_t* nslm_moe_router_w(const NslmMoe* m, int layer) { return m->rw + (size_t) layer * m->c.n_exp * m->c.d; }
int nslm_moe_fused_error(NslmMoe* m) {
    uint32_t w = 0;
    if (nh_device_sync() || nh_memcpy_d2h(&w, m->sync + kc_moe_decode_error_word(), 4)) return -1;
    return (int) w;
}

int nslm_moe_fused_words(NslmMoe* m, int first, int n, uint32_t* out) {
    if (first < 0 || n < 0 || (size_t) first + (size_t) n > kc_moe_decode_sync_words(kc_moe_decode_max_rows(), m->c.d)) return -1;
    return nh_device_sync() || nh_memcpy_d2h(out, m->sync + first, 4 * (size_t) n) ? -1 : 0;
}

int nslm_moe_last_routing(NslmMoe* m, int T, int32_t* ind, float* wt) {
    if (nh_device_sync()) return -1;
    return (nh_memcpy_d2h(ind, m->ind, 4 * (size_t) T * m->c.top_k) | nh_memcpy_d2h(wt, m->wt, 4 * (size_t) T * m->c.top_k)) ? -1 : 0;
}
int nslm_moe_last_logits(NslmMoe* m, int T, float* logits) {
    if (T < 1 || T > m->c.max_rows || nh_device_sync()) return -1;
    return nh_memcpy_d2h(logits, m->logit, 4 * (size_t) T * m->c.n_exp) ? -1 : 0;
}
int nslm_moe_last_pairs(NslmMoe* m, int pairs, float* A, float* D) {
    if (nh_device_sync()) return -1;
    return (nh_memcpy_d2h(A, m->A, 4 * (size_t) pairs * m->c.ff) | nh_memcpy_d2h(D, m->D, 4 * (size_t) pairs * m->c.d)) ? -1 : 0;
}
int nslm_moe_prefetch_stats(NslmMoe* m, uint32_t* hits, uint32_t* misses) {
    uint32_t st[2] = {0, 0};
    if (!m->cst) return -1;
    if (nh_device_sync() || nh_memcpy_d2h(st, m->pool_pre.stats, 8)) return -1;
    *hits = st[0];
    *misses = st[1];
    return 0;
}
int nslm_moe_cache_stats(NslmMoe* m, uint32_t* hits, uint32_t* misses) {
    uint32_t st[2] = {0, 0};
    if (nh_device_sync() || nh_memcpy_d2h(st, m->pool.stats, 8)) return -1;
    *hits = st[0];
    *misses = st[1];
    return 0;
}
const WSlice* nslm_moe_tab(const NslmMoe* m, int layer, int tensor) { return m->pool.tab + ((size_t) layer * 3 + tensor) * m->c.n_exp; }
uint64_t nslm_moe_unit_bytes(const NslmMoe* m) { return m->unit_bytes; }
uint64_t nslm_moe_expert_bytes(const NslmMoe* m) {
    uint64_t n = 0;
    for (int i = 0; i < 3; ++i)
        for (int s = 0; s < 4; ++s) n += m->stream_len[i][s];
    return n;
}

