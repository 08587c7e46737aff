/* decode_model.c - see decode_model.h.  C99, no HIP headers: everything goes through the kc_* / kq4_* launchers and nh_*. */
#include "decode_model.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "nslm_rt.h"

typedef struct {
    WSlice w;
    int R, K;
} Dense;

struct NslmModel {
    NslmModelCfg c;
    NslmMoe* moe;
    uint8_t* dense_arena;              /* every layer's seeded dense matrices */
    uint64_t dense_layer_bytes;
    Dense* dense;                      /* [n_layer][NSLM_W_COUNT], host copies of the slices */
    WSlice* shared_tab;                /* device: [n_layer][3] slices of the shared expert (gate, up, down) */
    uint16_t* heads[NSLM_H_COUNT];     /* device: [n_layer][H][O][I] BF16 */
    float* norm;                       /* device: [n_layer * 2 + 1][d] */
    uint16_t* embed;                   /* device: [vocab][d] BF16, also the LM head */
    uint8_t *kc, *vc, *ks, *vs;        /* device caches: [n_layer][rows][...] */
    float* inv;                        /* device: rope / 2 inverse frequencies */
    RowInfo* ri;                       /* device: [max_rows] */
    int32_t *ids, *sel0;               /* device: [max_rows] */
    float *x, *xn, *q, *cl, *kr, *qr, *ql, *olat, *o, *part, *mo, *as, *gs, *us, *sh, *logits;
    uint16_t *px, *pa;                 /* BF16 views of activations for the GEMM path */
    int final;
    int next_pos;                      /* the largest position the next step writes (host-side bound; -1 before nslm_model_start) */
    int branches;                      /* independent launches of a layer on side streams (parallel graph branches) */
    nh_stream_t side[2];
    nh_event_t ev[4];
};

/* side stream i starts after everything queued on s so far / s continues after everything queued on side stream i */
static void fork_to(NslmModel* m, kc_stream_t s, int i) {
    nh_event_record(m->ev[0], (nh_stream_t) s);
    nh_stream_wait_event(m->side[i], m->ev[0]);
}
static void join_from(NslmModel* m, kc_stream_t s, int i) {
    nh_event_record(m->ev[1 + i], m->side[i]);
    nh_stream_wait_event((nh_stream_t) s, m->ev[1 + i]);
}
int nslm_model_set_branches(NslmModel* m, int on) {
    if (on && !m->side[0]) {
        int bad = nh_stream_create(&m->side[0]) | nh_stream_create(&m->side[1]);
        for (int i = 0; i < 4; ++i) bad |= nh_event_create(&m->ev[i]);
        if (bad) return -1;
    }
    m->branches = on != 0;
    return 0;
}

static uint64_t pad256(uint64_t n) { return (n + 255) & ~(uint64_t) 255; }
static int qd(const NslmModelCfg* c) { return c->n_head * c->head_dim; }
static size_t cache_rows(const NslmModelCfg* c) { return (size_t) c->max_rows * c->max_ctx; }
static size_t kv_elem(const NslmModelCfg* c) { return c->kv_fmt == KV_BF16 ? 2 : 1; }

void nslm_model_dense_shape(const NslmModel* m, int which, int* R, int* K) {
    const NslmModelCfg* c = &m->c;
    const int shapes[NSLM_W_COUNT][2] = {{qd(c), c->d}, {c->r, c->d}, {c->rope, c->d}, {c->d, qd(c)},
                                         {c->ff_shared, c->d}, {c->ff_shared, c->d}, {c->d, c->ff_shared}};
    *R = shapes[which][0];
    *K = shapes[which][1];
}
void nslm_model_heads_shape(const NslmModel* m, int which, int* O, int* I) {
    const NslmModelCfg* c = &m->c;
    *O = which == NSLM_H_QRMIX ? c->rope : which == NSLM_H_QLAT ? c->r : c->head_dim;
    *I = which == NSLM_H_VUP ? c->r : c->head_dim;
}
static size_t heads_elems(const NslmModel* m, int which) {
    int O, I;
    nslm_model_heads_shape(m, which, &O, &I);
    return (size_t) m->c.n_head * O * I;
}

NslmModel* nslm_model_open(const NslmModelCfg* c, char* err, int errlen) {
    if (c->d % 64 || qd(c) % 64 || c->r % 64 || (c->rope != 64 && c->rope != 128) || c->ff_shared % 64 || c->head_dim % 8 ||
        c->max_rows < 1 || c->vocab < 1 || (c->kv_fmt != KV_BF16 && c->kv_fmt != KV_FP8)) {
        snprintf(err, (size_t) errlen, "model: unsupported configuration");
        return NULL;
    }
    NslmModel* m = (NslmModel*) calloc(1, sizeof *m);
    if (!m) {
        snprintf(err, (size_t) errlen, "model: out of memory");
        return NULL;
    }
    m->next_pos = -1;
    m->c = *c;
    if (m->c.n_splits <= 0) m->c.n_splits = 32;
    NslmMoeCfg mc = {c->n_layer, c->n_exp, c->top_k, c->d, c->ff, MF_SEED4P4, NSLM_ROUTE_SOFTMAX, c->max_rows, 0, 1.0f, 0, 0};
    m->moe = nslm_moe_open(&mc, err, errlen);
    if (!m->moe) { free(m); return NULL; }
    /* the dense seeded matrices of a layer, each stream at a 256-byte aligned offset of the layer's block */
    m->dense = (Dense*) calloc((size_t) c->n_layer * NSLM_W_COUNT, sizeof(Dense));
    uint64_t off[NSLM_W_COUNT][3], cur = 0;
    for (int w = 0; w < NSLM_W_COUNT; ++w) {
        int R, K;
        nslm_model_dense_shape(m, w, &R, &K);
        const uint64_t nb = (uint64_t) R * K / 8;
        off[w][0] = cur; cur += pad256(nb * 2);
        off[w][1] = cur; cur += pad256(nb * 2);
        off[w][2] = cur; cur += pad256((nb + 1) / 2);
    }
    m->dense_layer_bytes = cur;
    const int T = c->max_rows, H = c->n_head;
    const size_t rows = cache_rows(c), e = kv_elem(c);
    int bad = 0;
    bad |= nh_malloc((void**) &m->dense_arena, cur * (uint64_t) c->n_layer);
    for (int l = 0; l < c->n_layer && !bad; ++l)
        for (int w = 0; w < NSLM_W_COUNT; ++w) {
            Dense* dn = &m->dense[l * NSLM_W_COUNT + w];
            nslm_model_dense_shape(m, w, &dn->R, &dn->K);
            uint8_t* base = m->dense_arena + (uint64_t) l * cur;
            dn->w.p[0] = base + off[w][0];
            dn->w.p[1] = base + off[w][1];
            dn->w.p[3] = base + off[w][2];
            dn->w.eb = -22;
        }
    bad |= nh_malloc((void**) &m->shared_tab, sizeof(WSlice) * 3 * (size_t) c->n_layer);
    for (int w = 0; w < NSLM_H_COUNT; ++w) bad |= nh_malloc((void**) &m->heads[w], 2 * heads_elems(m, w) * (size_t) c->n_layer);
    bad |= nh_malloc((void**) &m->norm, 4 * (size_t) (2 * c->n_layer + 1) * c->d);
    bad |= nh_malloc((void**) &m->embed, 2 * (size_t) c->vocab * c->d);
    bad |= nh_malloc((void**) &m->kc, e * rows * c->rope * (size_t) c->n_layer);
    bad |= nh_malloc((void**) &m->vc, e * rows * c->r * (size_t) c->n_layer);
    bad |= nh_malloc((void**) &m->ks, rows * (c->rope / 32) * (size_t) c->n_layer + 16);
    bad |= nh_malloc((void**) &m->vs, rows * (c->r / 32) * (size_t) c->n_layer + 16);
    bad |= nh_malloc((void**) &m->inv, 4 * (size_t) (c->rope / 2));
    bad |= nh_malloc((void**) &m->ri, sizeof(RowInfo) * (size_t) T);
    bad |= nh_malloc((void**) &m->ids, 4 * (size_t) T);
    bad |= nh_malloc((void**) &m->sel0, 4 * (size_t) T);
    const size_t wide = (size_t) (H * c->r > qd(c) ? H * c->r : qd(c)) > (size_t) c->d ? (size_t) (H * c->r > qd(c) ? H * c->r : qd(c)) : (size_t) c->d;
    float** fb[] = {&m->x, &m->xn, &m->q, &m->cl, &m->kr, &m->qr, &m->ql, &m->olat, &m->o, &m->mo, &m->as, &m->gs, &m->us, &m->sh};
    const size_t fn[] = {(size_t) c->d, (size_t) c->d, (size_t) qd(c), (size_t) c->r, (size_t) c->rope, (size_t) H * c->rope, (size_t) H * c->r,
                         (size_t) H * c->r, (size_t) qd(c), (size_t) c->d, (size_t) c->ff_shared, (size_t) c->ff_shared, (size_t) c->ff_shared,
                         (size_t) c->d};
    for (size_t i = 0; i < sizeof fb / sizeof fb[0]; ++i) bad |= nh_malloc((void**) fb[i], 4 * fn[i] * (size_t) T);
    bad |= nh_malloc((void**) &m->part, 4 * (size_t) T * H * m->c.n_splits * (size_t) (c->r + 2));
    bad |= nh_malloc((void**) &m->logits, 4 * (size_t) T * c->vocab);
    bad |= nh_malloc((void**) &m->px, 2 * (size_t) T * wide);
    bad |= nh_malloc((void**) &m->pa, 2 * (size_t) T * wide);
    if (bad) {
        snprintf(err, (size_t) errlen, "model: out of device memory");
        nslm_model_close(m);
        return NULL;
    }
    float* inv = (float*) malloc(4 * (size_t) (c->rope / 2));
    for (int p = 0; p < c->rope / 2; ++p) inv[p] = (float) pow((double) c->rope_theta, -2.0 * p / c->rope);
    bad |= nh_memcpy_h2d(m->inv, inv, 4 * (size_t) (c->rope / 2));
    free(inv);
    bad |= nh_memset(m->sel0, 0, 4 * (size_t) T);
    bad |= nh_memset(m->norm, 0, 4 * (size_t) (2 * c->n_layer + 1) * c->d);   /* y = x r (1 + 0) */
    bad |= nh_memset(m->kc, 0, e * rows * c->rope * (size_t) c->n_layer);
    bad |= nh_memset(m->vc, 0, e * rows * c->r * (size_t) c->n_layer);
    bad |= nh_memset(m->ks, 0, rows * (c->rope / 32) * (size_t) c->n_layer);
    bad |= nh_memset(m->vs, 0, rows * (c->r / 32) * (size_t) c->n_layer);
    if (bad) {
        snprintf(err, (size_t) errlen, "model: device initialisation failed");
        nslm_model_close(m);
        return NULL;
    }
    return m;
}

void nslm_model_close(NslmModel* m) {
    if (!m) return;
    nslm_moe_close(m->moe);
    void* d[] = {m->dense_arena, m->shared_tab, m->heads[0], m->heads[1], m->heads[2], m->norm, m->embed, m->kc, m->vc, m->ks, m->vs, m->inv,
                 m->ri, m->ids, m->sel0, m->x, m->xn, m->q, m->cl, m->kr, m->qr, m->ql, m->olat, m->o, m->part, m->mo, m->as, m->gs, m->us,
                 m->sh, m->logits, m->px, m->pa};
    for (size_t i = 0; i < sizeof d / sizeof d[0]; ++i)
        if (d[i]) nh_free(d[i]);
    for (int i = 0; i < 2; ++i)
        if (m->side[i]) nh_stream_destroy(m->side[i]);
    for (int i = 0; i < 4; ++i)
        if (m->ev[i]) nh_event_destroy(m->ev[i]);
    free(m->dense);
    free(m);
}

NslmMoe* nslm_model_moe(NslmModel* m) { return m->moe; }

int nslm_model_set_dense(NslmModel* m, int layer, int which, const uint16_t* seeds, const uint16_t* coefs, const uint8_t* codes, int eb) {
    if (layer < 0 || layer >= m->c.n_layer || which < 0 || which >= NSLM_W_COUNT) return -1;
    Dense* dn = &m->dense[layer * NSLM_W_COUNT + which];
    const size_t nb = (size_t) dn->R * dn->K / 8;
    int e = nh_memcpy_h2d((void*) dn->w.p[0], seeds, nb * 2);
    e |= nh_memcpy_h2d((void*) dn->w.p[1], coefs, nb * 2);
    e |= nh_memcpy_h2d((void*) dn->w.p[3], codes, (nb + 1) / 2);
    dn->w.eb = eb;
    return e ? -1 : 0;
}
int nslm_model_set_heads(NslmModel* m, int layer, int which, const uint16_t* w) {
    if (layer < 0 || layer >= m->c.n_layer || which < 0 || which >= NSLM_H_COUNT) return -1;
    const size_t n = heads_elems(m, which);
    return nh_memcpy_h2d(m->heads[which] + (size_t) layer * n, w, 2 * n) ? -1 : 0;
}
int nslm_model_set_norm(NslmModel* m, int layer, int which, const float* w) {
    if (layer < 0 || layer > m->c.n_layer || which < 0 || which > 1) return -1;
    const size_t row = layer == m->c.n_layer ? 2 * (size_t) m->c.n_layer : 2 * (size_t) layer + which;
    return nh_memcpy_h2d(m->norm + row * m->c.d, w, 4 * (size_t) m->c.d) ? -1 : 0;
}
int nslm_model_set_embed(NslmModel* m, const uint16_t* w) { return nh_memcpy_h2d(m->embed, w, 2 * (size_t) m->c.vocab * m->c.d) ? -1 : 0; }

int nslm_model_finalize(NslmModel* m) {
    WSlice* tab = (WSlice*) calloc(3 * (size_t) m->c.n_layer, sizeof(WSlice));
    for (int l = 0; l < m->c.n_layer; ++l)
        for (int i = 0; i < 3; ++i) tab[l * 3 + i] = m->dense[l * NSLM_W_COUNT + NSLM_W_SG + i].w;
    int bad = nh_memcpy_h2d(m->shared_tab, tab, sizeof(WSlice) * 3 * (size_t) m->c.n_layer);
    free(tab);
    bad |= nslm_moe_finalize(m->moe);
    m->final = !bad;
    return bad ? -1 : 0;
}

int nslm_model_fill_random(NslmModel* m, uint64_t seed, int eb) {
    const NslmModelCfg* c = &m->c;
    kc_fill_random(0, m->dense_arena, m->dense_layer_bytes * (uint64_t) c->n_layer, seed ^ 1);
    for (int i = 0; i < c->n_layer * NSLM_W_COUNT; ++i) m->dense[i].w.eb = eb;
    for (int w = 0; w < NSLM_H_COUNT; ++w) {
        int O, I;
        nslm_model_heads_shape(m, w, &O, &I);
        kc_fill_bf16(0, m->heads[w], heads_elems(m, w) * (size_t) c->n_layer, seed ^ (uint64_t) (2 + w), 1.7f / sqrtf((float) I));
    }
    kc_fill_bf16(0, m->embed, (size_t) c->vocab * c->d, seed ^ 7, 0.05f);
    if (nslm_moe_fill_random(m->moe, seed ^ 9, eb, 0.035f)) return -1;
    if (nh_device_sync() || kc_last_error()) return -1;
    return nslm_model_finalize(m);
}

int nslm_model_start(NslmModel* m, int T, const int32_t* ids, const int32_t* pos) {
    if (T < 1 || T > m->c.max_rows) return -1;
    RowInfo ri[64];
    int hi = 0;
    if (T > 64) return -1;
    memset(ri, 0, sizeof ri);
    for (int t = 0; t < T; ++t) {
        if (pos[t] < 0 || pos[t] >= m->c.max_ctx || ids[t] < 0 || ids[t] >= m->c.vocab) return -1;
        ri[t].pos = pos[t];
        ri[t].kv0 = t * m->c.max_ctx;
        ri[t].pad[0] = m->c.max_ctx;   /* kc_rows_advance never moves a row past its slot's last position */
        if (pos[t] > hi) hi = pos[t];
    }
    m->next_pos = hi;
    int bad = nh_device_sync();
    bad |= nh_memcpy_h2d(m->ri, ri, sizeof(RowInfo) * (size_t) T);
    bad |= nh_memcpy_h2d(m->ids, ids, 4 * (size_t) T);
    return bad ? -1 : 0;
}

int nslm_model_fill_cache(NslmModel* m, int T, int upto, uint64_t seed) {
    const NslmModelCfg* c = &m->c;
    if (T < 1 || T > c->max_rows || upto < 0 || upto > c->max_ctx) return -1;
    const size_t rows = cache_rows(c), e = kv_elem(c);
    for (int l = 0; l < c->n_layer; ++l)
        for (int t = 0; t < T; ++t) {
            const size_t r0 = (size_t) l * rows + (size_t) t * c->max_ctx;
            if (c->kv_fmt == KV_BF16) {
                kc_fill_bf16(0, (uint16_t*) m->kc + r0 * c->rope, (size_t) upto * c->rope, seed ^ (uint64_t) (l * 64 + t), 1.0f);
                kc_fill_bf16(0, (uint16_t*) m->vc + r0 * c->r, (size_t) upto * c->r, seed ^ (uint64_t) (l * 64 + t + 4096), 1.0f);
            } else {   /* codes as kc_mla_rope's encoder writes them (it saturates at 0x7E, nslm/kvq.h:19-23); scales 2^-6 */
                kc_fill_fp8_codes(0, m->kc + (r0 * c->rope) * e, (size_t) upto * c->rope, seed ^ (uint64_t) (l * 64 + t));
                kc_fill_fp8_codes(0, m->vc + (r0 * c->r) * e, (size_t) upto * c->r, seed ^ (uint64_t) (l * 64 + t + 4096));
                nh_memset(m->ks + r0 * (c->rope / 32), 121, (size_t) upto * (c->rope / 32));
                nh_memset(m->vs + r0 * (c->r / 32), 121, (size_t) upto * (c->r / 32));
            }
        }
    return nh_device_sync() || kc_last_error() ? -1 : 0;
}

/* y[T][R] (+)= W x.  The reference takes the matvec up to MV_MAXT rows and the packed MFMA GEMM above
 * (engine/mova_cuda.c:1020-1028).  Here the matvec (exact weights, f32 activations, four rows a workgroup) stays the choice
 * up to DENSE_MV_ROWS rows: a 2048 x 2048 projection is a 32-workgroup grid for the GEMM's 64-row tiles (22 us at 16 rows),
 * the matvec's 1024 workgroups take 14 us (24 us at 32 rows). */
#define DENSE_MV_ROWS 32
static void dense(const NslmModel* m, kc_stream_t s, const Dense* dn, const float* x, const uint16_t* xp, int xs, float* y, int T, int add) {
    (void) m;
    if (T <= DENSE_MV_ROWS) kc_mv(s, MF_SEED4P4, dn->w, dn->K, dn->R, x, xs, y, dn->R, T, add, NULL);
    else kc_mm_packed(s, MF_SEED4P4, dn->w, dn->K, dn->R, xp, xs, y, dn->R, T, add, NULL);
}

int nslm_model_step(NslmModel* m, kc_stream_t s, int T) {
    const NslmModelCfg* c = &m->c;
    if (!m->final || T < 1 || T > c->max_rows) return -1;
    /* a step writes the cache at each row's position: refused once a sequence slot is full (the positions advance on the
       device, so the host keeps the bound: nslm_model_start's largest position + the steps issued since) */
    if (m->next_pos < 0 || m->next_pos >= c->max_ctx) return -1;
    const int d = c->d, H = c->n_head, hd = c->head_dim, r = c->r, rope = c->rope, QD = qd(c), ffs = c->ff_shared;
    const int big = T > MV_MAXT, bigd = T > DENSE_MV_ROWS;   /* rows above which the experts / the dense projections take the GEMMs */
    const size_t rows = cache_rows(c), e = kv_elem(c);
    MlaArgs ma;
    memset(&ma, 0, sizeof ma);
    ma.n_head = H; ma.r = r; ma.chunk = 128; ma.n_splits = c->n_splits;
    ma.scale = 1.0f / sqrtf((float) (hd + rope));
    ma.pad[0] = rope;
    kc_seed_gemm_f32(0);
    WSlice emb;
    memset(&emb, 0, sizeof emb);
    emb.p[0] = m->embed;
    kc_embed(s, MF_BF16, emb, d, m->ids, m->x, T);
    for (int l = 0; l < c->n_layer; ++l) {
        const Dense* dn = m->dense + (size_t) l * NSLM_W_COUNT;
        /* ---- attention: x += W_o v_up(attn(q_lat(q), q_rope_mix(q); c, k_rope)) ---- */
        WSlice hw;
        memset(&hw, 0, sizeof hw);
        HmvArgs hq = {H, rope, hd, QD, hd, 0, {0, 0}}, hl = {H, r, hd, QD, hd, 0, {0, 0}}, hv = {H, hd, r, H * r, r, 0, {0, 0}};
        const int par = m->branches && !big;
        kc_stream_t s1 = par ? (kc_stream_t) m->side[0] : s, s2 = par ? (kc_stream_t) m->side[1] : s;
        int one = 0;   /* steps of up to 8 rows on one stream: the norm and the three projections of its output as one launch */
        const WSlice w3[3] = {dn[NSLM_W_Q].w, dn[NSLM_W_KVA].w, dn[NSLM_W_KR].w};
        const int R3[3] = {QD, r, rope}, a3[3] = {0, 0, 0};
        float* const y3[3] = {m->q, m->cl, m->kr};
        if (!big && !par) one = !kc_mv_multi(s, MF_SEED4P4, 3, w3, R3, y3, R3, a3, d, m->x, d, T, m->norm + (size_t) (2 * l) * d, c->eps);
        if (!one) {
            kq4_norm1p(s, m->x, d, d, m->norm + (size_t) (2 * l) * d, c->eps, m->xn, T);
            /* more than 8 rows: the norm stays a launch (every workgroup of a pass would redo 8 rows' sums), the three
               projections still go as one launch per 8 rows */
            if (big && !bigd) one = !kc_mv_multi(s, MF_SEED4P4, 3, w3, R3, y3, R3, a3, d, m->xn, d, T, NULL, 0.0f);
        }
        if (!one) {
            if (bigd) kc_pack_input_bf16(s, m->xn, m->px, (size_t) T * d);
            /* with branches: [Q -> q RoPE mix] | [KV down, then q -> latent] | [K rope] */
            if (par) { fork_to(m, s, 0); fork_to(m, s, 1); }
            dense(m, s, &dn[NSLM_W_Q], m->xn, m->px, d, m->q, T, 0);
            if (par) nh_event_record(m->ev[3], (nh_stream_t) s);
            dense(m, s1, &dn[NSLM_W_KVA], m->xn, m->px, d, m->cl, T, 0);
            dense(m, s2, &dn[NSLM_W_KR], m->xn, m->px, d, m->kr, T, 0);
        }
        WSlice hwq = hw, hwl = hw, hwv = hw;
        hwq.p[0] = m->heads[NSLM_H_QRMIX] + (size_t) l * H * rope * hd;
        hwl.p[0] = m->heads[NSLM_H_QLAT] + (size_t) l * H * r * hd;
        hwv.p[0] = m->heads[NSLM_H_VUP] + (size_t) l * H * hd * r;
        KvView kv;
        memset(&kv, 0, sizeof kv);
        kv.a.k = m->kc + (size_t) l * rows * rope * e;
        kv.a.v = m->vc + (size_t) l * rows * r * e;
        kv.a.ks = (float*) (m->ks + (size_t) l * rows * (rope / 32));
        kv.a.vs = (float*) (m->vs + (size_t) l * rows * (r / 32));
        kv.nv = (int32_t) rows;
        kv.fmt = c->kv_fmt;
        /* the query's two maps + RoPE + cache write as one launch, and the splits' reduce + value-up map as one, where the
           shapes allow (single stream); else the reference's sequence of five launches */
        int fusedq = 0;
        if (!par) fusedq = !kc_mla_qmaps_rope(s, ma, hq, hl, MF_BF16, hwq, hwl, m->q, m->qr, m->ql, m->kr, m->cl, kv, m->ri, m->inv, T);
        if (!fusedq) {
            kc_heads_mv(s, hq, MF_BF16, hwq, NULL, m->q, NULL, m->qr, T);
            if (par) nh_stream_wait_event(m->side[0], m->ev[3]);
            kc_heads_mv(s1, hl, MF_BF16, hwl, NULL, m->q, NULL, m->ql, T);
            if (par) { join_from(m, s, 0); join_from(m, s, 1); }
            kc_mla_rope(s, ma, m->qr, m->kr, m->cl, kv, m->ri, m->inv, T);
        }
        /* (above 8 rows the fused reduce re-reads the partials from too many workgroups: 19 us against 13 for the two kernels) */
        if (big || kc_mla_attn_vup(s, ma, m->ql, m->qr, kv, m->ri, m->part, hv, MF_BF16, hwv, m->o, T)) {
            kc_mla_attn(s, ma, m->ql, m->qr, kv, m->ri, m->part, m->olat, T);
            kc_heads_mv(s, hv, MF_BF16, hwv, NULL, m->olat, NULL, m->o, T);
        }
        if (bigd) kc_pack_input_bf16(s, m->o, m->pa, (size_t) T * QD);
        dense(m, s, &dn[NSLM_W_O], m->o, m->pa, QD, m->x, T, 1);   /* x = bf16(x + bf16(W_o o)) */
        /* ---- experts: x = bf16(x + bf16(sum_k wt_k y_k + shared(xn))) ---- */
        const WSlice* st = m->shared_tab + (size_t) l * 3;
        const float* nw2 = m->norm + (size_t) (2 * l + 1) * d;
        if (T <= kc_moe_decode_max_rows() && !par && ffs == c->ff) {   /* norm + routed + shared + residual: the whole expert block in the one persistent launch */
            const WSlice sh3[3] = {dn[NSLM_W_SG].w, dn[NSLM_W_SU].w, dn[NSLM_W_SD].w};
            const int rc = nslm_moe_step_layer(m->moe, s, l, m->x, T, sh3, m->x, m->x, nw2, c->eps);
            if (rc < 0) return -1;
            if (rc == 0) continue;
        }
        kq4_norm1p(s, m->x, d, d, nw2, c->eps, m->xn, T);
        if (!big) {   /* the shared expert through the gather entry points with every pair on slice 0 (engine/qwen4_cuda.c:1029),
                         beside the routed experts when branches are on (as the reference runs it on its second stream, :1026-1032) */
            if (par) fork_to(m, s, 0);
            kc_mv_gu(s1, MF_SEED4P4, st, st + 1, d, ffs, m->xn, d, m->as, ffs, m->sel0, T, 1, NULL);
            kc_mv(s1, MF_SEED4P4, dn[NSLM_W_SD].w, ffs, d, m->as, ffs, m->sh, d, T, 0, NULL);
            if (nslm_moe_step(m->moe, s, l, m->xn, T, m->mo)) return -1;
            if (par) join_from(m, s, 0);
        } else {
            if (nslm_moe_step(m->moe, s, l, m->xn, T, m->mo)) return -1;
            int two = 0;   /* the shared expert's gate and up as one launch per 8 rows */
            if (!bigd) {
                const WSlice w2[2] = {dn[NSLM_W_SG].w, dn[NSLM_W_SU].w};
                const int R2[2] = {ffs, ffs}, a2[2] = {0, 0};
                float* const y2[2] = {m->gs, m->us};
                two = !kc_mv_multi(s, MF_SEED4P4, 2, w2, R2, y2, R2, a2, d, m->xn, d, T, NULL, 0.0f);
            }
            if (!two) {
                if (bigd) kc_pack_input_bf16(s, m->xn, m->px, (size_t) T * d);
                dense(m, s, &dn[NSLM_W_SG], m->xn, m->px, d, m->gs, T, 0);
                dense(m, s, &dn[NSLM_W_SU], m->xn, m->px, d, m->us, T, 0);
            }
            if (bigd && ffs % 8 == 0) kc_swiglu_pack(s, m->gs, m->us, m->pa, (size_t) T * ffs);   /* the GEMM reads the BF16 view only */
            else {
                kc_swiglu(s, m->gs, m->us, m->as, T * ffs);
                if (bigd) kc_pack_input_bf16(s, m->as, m->pa, (size_t) T * ffs);
            }
            dense(m, s, &dn[NSLM_W_SD], m->as, m->pa, ffs, m->sh, T, 0);
        }
        kc_residual_add(s, m->x, m->mo, m->sh, (size_t) T * d);
    }
    kq4_norm1p(s, m->x, d, d, m->norm + (size_t) (2 * c->n_layer) * d, c->eps, m->xn, T);
    if (!big) kc_mv(s, MF_BF16, emb, d, c->vocab, m->xn, d, m->logits, c->vocab, T, 0, NULL);
    else {
        kc_pack_input_bf16(s, m->xn, m->px, (size_t) T * d);
        kc_mm_packed(s, MF_BF16, emb, d, c->vocab, m->px, d, m->logits, c->vocab, T, 0, NULL);
    }
    kc_argmax(s, m->logits, m->ids, c->vocab, T);
    kc_rows_advance(s, m->ri, T);
    if (kc_last_error()) return -1;            /* (a launch failed: the host's bound stays) */
    if (!nslm_stream_capturing(s)) m->next_pos += 1;   /* a captured step launched nothing: its replays are counted when launched */
    return 0;
}

int nslm_model_steps_left(const NslmModel* m) { return m->next_pos < 0 ? 0 : m->c.max_ctx - m->next_pos; }
int nslm_model_launch(NslmModel* m, NslmGraph* g, kc_stream_t s) {
    if (!g || m->next_pos < 0 || m->next_pos >= m->c.max_ctx) return -1;
    if (nslm_graph_launch(g, s)) return -1;
    m->next_pos += 1;
    return 0;
}
int nslm_model_account(NslmModel* m, int steps) {
    if (m->next_pos < 0 || m->next_pos + steps > m->c.max_ctx || m->next_pos + steps < 0) return -1;
    m->next_pos += steps;
    return 0;
}

/* (both synchronise, and report -1 when a wait inside the persistent expert kernel gave up since open: its results are void) */
int nslm_model_ids(NslmModel* m, int T, int32_t* ids) {
    return nh_device_sync() || nh_memcpy_d2h(ids, m->ids, 4 * (size_t) T) || nslm_moe_fused_error(m->moe) ? -1 : 0;
}
int nslm_model_logits(NslmModel* m, int T, float* logits) {
    return nh_device_sync() || nh_memcpy_d2h(logits, m->logits, 4 * (size_t) T * m->c.vocab) || nslm_moe_fused_error(m->moe) ? -1 : 0;
}
int nslm_model_hidden(NslmModel* m, int T, float* h) { return nh_device_sync() || nh_memcpy_d2h(h, m->xn, 4 * (size_t) T * m->c.d) ? -1 : 0; }
int nslm_model_get_embed(NslmModel* m, int first, int rows, uint16_t* w) {
    if (first < 0 || rows < 0 || first + rows > m->c.vocab) return -1;
    return nh_device_sync() || nh_memcpy_d2h(w, m->embed + (size_t) first * m->c.d, 2 * (size_t) rows * m->c.d) ? -1 : 0;
}
uint64_t nslm_model_step_bytes(const NslmModel* m) {
    const NslmModelCfg* c = &m->c;
    uint64_t b = 0;
    for (int w = 0; w < NSLM_W_COUNT; ++w) b += (uint64_t) m->dense[w].R * m->dense[w].K / 16 * 9;   /* 4.5 bytes per 8 weights */
    for (int w = 0; w < NSLM_H_COUNT; ++w) b += 2 * (uint64_t) heads_elems(m, w);
    b += (uint64_t) c->top_k * nslm_moe_expert_bytes(m->moe) + 2 * (uint64_t) c->n_exp * c->d;
    return b * (uint64_t) c->n_layer + 2 * (uint64_t) c->vocab * c->d;
}
