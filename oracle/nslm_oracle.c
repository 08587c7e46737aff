/* oracle/nslm_oracle.c - CPU restatement of the SeedLM decode-in-matmul arithmetic (see nslm_oracle.h).
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP path.  Never linked into the shipped library.
 * Build: gcc -O2 -ffp-contract=off (no FMA contraction: the reference builds its C with the same flag,
 * CMakeLists.txt:7-8; explicit fmaf() calls below are the reference's explicit FMAs).
 *
 * What pins each function (tests/test_oracle.py):
 *   or_lfsr_*            hand-computed states after seed 1 (tests/test_lfsr.c:25), period 65535 (:14-22), the FNV-1a
 *                        golden over 24 states of all seeds 0x740e86e513d34463 (:41-56), GF(2) linearity of the stream
 *                        tables (:86-91); also bit-compared with the compiled reference (oracle/_ref) when present.
 *   or_decode_p3/p4      integer closed form recomputed in Python big-ints from or_lfsr_states + exact rational
 *                        scaling and RNE; exhaustive pack/unpack of the int4 fields; compiled reference's
 *                        nslm_decode_block / nslm4_decode_block on random blocks (golden fixture + live).
 *   or_row_f32           equals or_decode_* before rounding; compiled reference ns_row_f32 (golden fixture + live).
 *   or_affine_dequant    closed form bf16(s*q+b); compiled reference nslm_affine_dequantize.
 *   or_cpu_seed4_matvec  double-precision dot over exact weights, < 2e-6 of max |y| (tests/test_cpu_seed4.c:49-63);
 *                        bit-equal with the compiled reference's cpu_seed4_matvec_mt (live + golden fixture).
 *   or_route_softmax     engineered tie lg[7]=lg[300] -> 300 first (tests/test_qwen4_kernels.c:233-245), weights sum
 *                        to 1, brute-force argsort; compiled reference qwen4_route.
 *   or_route_sigmoid / or_topk_sigmoid   brute-force k-round arg-max with ties to the lowest id incl. a many-ties case
 *                        (tests/test_mova_kernels.c:376-445).
 *   or_swiglu / or_moe_combine / or_q4_moe_combine   closed forms recomputed in numpy float64 with BF16 rounding.
 *   or_gnorm             the reference test's own closed form (tests/test_mova_kernels.c:361-374): per-group double sum, within
 *                        its close_bf(1e-6) of bf16(w * (x * r)); a constant row has r = 1 / sqrt(c^2 + eps) exactly.
 *   or_norm1p            compiled reference qwen4_norm1p (live); closed form on a constant row; g == len and g < len.
 *   or_argmax            the reference test's vector: lg[123456] = lg[200000] = 50 -> 123456, lg[V + 99] = 60 -> 99
 *                        (tests/test_mova_kernels.c:563-572); prob against numpy's softmax in float64.
 *   or_e4m3_* / or_fp8_*  every finite E4M3 code round-trips and decodes exactly to BF16, 0x7E = 448, 0x01 = 2^-9, 0xB8 = -1,
 *                        midpoints go to the even code (tests/test_kvq.c:30-45); the scale is the smallest power of two s
 *                        with 448 s >= amax (nslm/kvq.h:4-5); bit-compared with the compiled reference's kvq.h (live).
 *   or_heads_map / or_rope_pair / or_mla_attn   the reference tests' own double-precision forms
 *                        (tests/test_mova_kernels.c:800-812, 962-979, 1004-1031); softmax of equal scores gives the mean
 *                        latent; one position gives that position's latent.
 *   or_bucket            host regrouping is the definition (tests/test_qwen4_engine.c:33-61): stable sort by expert.
 *   or_cache_admit       invariants (every selected unit resident afterwards, LRU victim = smallest tick, ties to the
 *                        lowest slot); the reference holds no standalone vector for it.
 */
#include "nslm_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------------------------------------------------ */
/* LFSR: x^16 + x^12 + x^3 + x + 1, Fibonacci, shift right, feedback into bit 15 (nslm/lfsr.h:4-8,20-23).            */

uint16_t or_lfsr_step(uint16_t s) {
    unsigned fb = (s ^ (s >> 1) ^ (s >> 3) ^ (s >> 12)) & 1u;
    return (uint16_t) ((s >> 1) | (fb << 15));
}

void or_lfsr_states(uint16_t s, int n, uint16_t* out) {
    for (int i = 0; i < n; ++i) {
        s = or_lfsr_step(s);
        out[i] = s;
    }
}

/* bit k of the result = top bit of state k+1 = stream bit 16+k (nslm/lfsr.h:41-59) */
uint32_t or_lfsr_stream(uint16_t s, int nbits) {
    uint32_t g = 0;
    for (int k = 0; k < nbits; ++k) {
        s = or_lfsr_step(s);
        g |= (uint32_t) (s >> 15) << k;
    }
    return g;
}

void or_lfsr_stream_table(int nbits, uint32_t* table) {
    for (uint32_t s = 0; s < 65536; ++s) table[s] = or_lfsr_stream((uint16_t) s, nbits);
}

uint64_t or_lfsr_fnv24(void) {
    uint64_t h = 1469598103934665603ull;
    uint16_t st[24];
    for (uint32_t s = 1; s <= 65535; ++s) {
        or_lfsr_states((uint16_t) s, 24, st);
        for (int k = 0; k < 24; ++k) h = (h ^ st[k]) * 1099511628211ull;
    }
    return h;
}

/* ------------------------------------------------------------------------------------------------------------------ */
/* scalar helpers */

static float bits2f(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static uint32_t f2bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static const float kR32 = 1.0f / 32767.0f; /* nslm/lfsr.h:18 */

float or_scale(int e) { return kR32 * bits2f((uint32_t) (e + 127) << 23); } /* nslm/lfsr.h:87-93 */

uint16_t or_f2bf(float f) { /* nslm/lfsr.h:95-100 */
    uint32_t u = f2bits(f);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t) (u >> 16);
}
float or_bf2f(uint16_t h) { return bits2f((uint32_t) h << 16); }
float or_bfr(float f) { return or_bf2f(or_f2bf(f)); }

static int sext4(unsigned v) { return (int) (v & 15u) - (int) ((v & 8u) << 1); }

/* ------------------------------------------------------------------------------------------------------------------ */
/* block decode */

static void isum_block(uint16_t seed, const int* q, int P, int32_t out[8]) {
    uint16_t st[32];
    or_lfsr_states(seed, 8 * P, st);
    for (int c = 0; c < 8; ++c) {
        int32_t acc = 0;
        for (int p = 0; p < P; ++p) acc += ((int32_t) st[c * P + p] - 32768) * q[p];
        out[c] = acc;
    }
}

void or_isum_p3(uint16_t seed, uint16_t nib, int32_t out[8]) { /* nslm/lfsr.h:80-84,116-128 */
    int q[3] = {sext4(nib >> 4), sext4(nib >> 8), sext4(nib >> 12)};
    isum_block(seed, q, 3, out);
}
void or_isum_p4(uint16_t seed, uint16_t coef, int32_t out[8]) { /* nslm/search4.h:27, nslm/lib_search4.c:22-31 */
    int q[4] = {sext4(coef), sext4(coef >> 4), sext4(coef >> 8), sext4(coef >> 12)};
    isum_block(seed, q, 4, out);
}

void or_decode_p3(uint16_t seed, uint16_t nib, int exp_bias, uint16_t out[8]) {
    int32_t is[8];
    or_isum_p3(seed, nib, is);
    const float sc = or_scale(exp_bias + (nib & 15));
    for (int c = 0; c < 8; ++c) out[c] = or_f2bf((float) is[c] * sc);
}
void or_decode_p4(uint16_t seed, uint16_t coef, int e, uint16_t out[8]) {
    int32_t is[8];
    or_isum_p4(seed, coef, is);
    const float sc = or_scale(e);
    for (int c = 0; c < 8; ++c) out[c] = or_f2bf((float) is[c] * sc);
}

/* ------------------------------------------------------------------------------------------------------------------ */
/* rows */

static int group_shift(const OrSlice* w) { return w->gs ? w->gs : 6; }

void or_row_f32(int fmt, const OrSlice* w, int R, int K, int row, int round, float* out) {
    (void) R;
    const size_t base = (size_t) row * (size_t) K;
    if (fmt == OR_BF16) {
        const uint16_t* v = (const uint16_t*) w->p[0] + base;
        for (int c = 0; c < K; ++c) out[c] = or_bf2f(v[c]);
        return;
    }
    if (fmt == OR_Q8 || fmt == OR_Q4) { /* nslm/lib_rows.c:36-48 */
        const uint32_t* q = (const uint32_t*) w->p[0];
        const uint16_t* S = (const uint16_t*) w->p[1];
        const uint16_t* B = (const uint16_t*) w->p[2];
        const int sh = group_shift(w);
        for (int c = 0; c < K; ++c) {
            const size_t i = base + (size_t) c;
            const float s = or_bf2f(S[i >> sh]), b = or_bf2f(B[i >> sh]);
            const uint32_t code = fmt == OR_Q8 ? (q[i >> 2] >> (8 * (i & 3))) & 255u : (q[i >> 3] >> (4 * (i & 7))) & 15u;
            const float v = s * (float) code + b;
            out[c] = round ? or_bfr(v) : v;
        }
        return;
    }
    /* seeds (nslm/lib_rows.c:49-76): block g = row * K/8 + j; P=4 exponent code = nibble g&1 of codes[g>>1] */
    const int nbk = K / 8;
    const uint16_t* seeds = (const uint16_t*) w->p[0];
    const uint16_t* cw = (const uint16_t*) w->p[1];
    const uint8_t* codes = (const uint8_t*) w->p[3];
    for (int j = 0; j < nbk; ++j) {
        const size_t g = (size_t) row * (size_t) nbk + (size_t) j;
        int32_t is[8];
        int e;
        if (fmt == OR_SEED4P4) {
            or_isum_p4(seeds[g], cw[g], is);
            e = w->eb + ((codes[g >> 1] >> ((g & 1) * 4)) & 15);
        } else {
            or_isum_p3(seeds[g], cw[g], is);
            e = w->eb + (cw[g] & 15);
        }
        const float sc = or_scale(e);
        for (int c = 0; c < 8; ++c) out[j * 8 + c] = (float) is[c] * sc;
    }
}

void or_slice_bf16(int fmt, const OrSlice* w, int R, int K, uint16_t* out) {
    float* row = (float*) malloc(sizeof(float) * (size_t) K);
    for (int r = 0; r < R; ++r) {
        or_row_f32(fmt, w, R, K, r, 1, row);
        for (int c = 0; c < K; ++c) out[(size_t) r * K + c] = or_f2bf(row[c]);
    }
    free(row);
}

void or_affine_dequant(const uint32_t* words, const uint16_t* scales, const uint16_t* biases, int64_t n, int bits,
                       int group, uint16_t* out) {
    const int per = 32 / bits;
    const uint32_t mask = (1u << bits) - 1u;
    for (int64_t i = 0; i < n; ++i) {
        const uint32_t q = (words[i / per] >> (bits * (int) (i % per))) & mask;
        out[i] = or_f2bf(or_bf2f(scales[i / group]) * (float) q + or_bf2f(biases[i / group]));
    }
}

/* ------------------------------------------------------------------------------------------------------------------ */
/* CPU decode-in-dot-product.  Algebra (nslm/cpu_seed4.h:5-8): with v = 1 + state/2^16 (exact in f32) and X = sum_c x_c,
 *   sum_c x_c isum_c / 2^16 = sum_p q_p A_p - 1.5 (sum_p q_p) X,  A_p = sum_c x_c v[c][p]
 * A_p by FMAs in c order, the combine without contraction, one FMA into the row accumulator per block.             */

typedef struct {
    const uint16_t *seeds, *cw;
    const uint8_t* codes;
    int bias, kb, P, r0, r1;
    const uint32_t* table;
    const float *x, *xsum;
    float* y;
} MvJob;

static void* mv_rows(void* arg) {
    const MvJob* j = (const MvJob*) arg;
    const int P = j->P;
    for (int r = j->r0; r < j->r1; ++r) {
        float acc = 0.0f;
        for (int b = 0; b < j->kb; ++b) {
            const size_t g = (size_t) r * (size_t) j->kb + (size_t) b;
            const uint32_t s = j->seeds[g], t = j->table[s], word = j->cw[g];
            const uint64_t stream = (uint64_t) s | ((uint64_t) t << 16);
            float a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            for (int c = 0; c < 8; ++c)
                for (int p = 0; p < P; ++p) {
                    const uint32_t st = (uint32_t) (stream >> (c * P + p + 1)) & 0xFFFFu;
                    a[p] = fmaf(j->x[8 * b + c], bits2f(0x3F800000u | (st << 7)), a[p]);
                }
            float d, qsum;
            int code;
            if (P == 4) {
                const float q0 = (float) sext4(word), q1 = (float) sext4(word >> 4), q2 = (float) sext4(word >> 8),
                            q3 = (float) sext4(word >> 12);
                qsum = ((q0 + q1) + q2) + q3;
                d = ((a[0] * q0 + a[1] * q1) + a[2] * q2) + a[3] * q3;
                code = (j->codes[g >> 1] >> ((g & 1) * 4)) & 15;
            } else {
                const float q0 = (float) sext4(word >> 4), q1 = (float) sext4(word >> 8), q2 = (float) sext4(word >> 12);
                qsum = (q0 + q1) + q2;
                d = (a[0] * q0 + a[1] * q1) + a[2] * q2;
                code = (int) (word & 15u);
            }
            d = d - (1.5f * qsum) * j->xsum[b];
            acc = fmaf(d, bits2f((uint32_t) (j->bias + 16 + 127 + code) << 23) * kR32, acc);
        }
        j->y[r] = acc;
    }
    return NULL;
}

static void seed_matvec(const uint16_t* seeds, const uint16_t* cw, const uint8_t* codes, int bias, int P, const float* x,
                        int rows, int kb, float* y, int threads) {
    static uint32_t* tab; /* the 32-bit stream table serves both P: P=3 reads its low 24 bits */
    if (!tab) {
        uint32_t* t = (uint32_t*) malloc(65536 * sizeof(uint32_t));
        or_lfsr_stream_table(32, t);
        tab = t;
    }
    float* xsum = (float*) malloc(sizeof(float) * (size_t) kb);
    for (int b = 0; b < kb; ++b) {
        float s = 0.0f;
        for (int c = 0; c < 8; ++c) s += x[8 * b + c];
        xsum[b] = s;
    }
    if (threads < 1) threads = 1;
    if (threads > 64) threads = 64;
    MvJob jobs[64];
    pthread_t th[64];
    const int per = (rows + threads - 1) / threads;
    int n = 0;
    for (int i = 0; i < threads; ++i) {
        const int r0 = i * per, r1 = r0 + per < rows ? r0 + per : rows;
        if (r0 >= r1) break;
        jobs[n] = (MvJob){seeds, cw, codes, bias, kb, P, r0, r1, tab, x, xsum, y};
        ++n;
    }
    for (int i = 1; i < n; ++i) pthread_create(&th[i], NULL, mv_rows, &jobs[i]);
    if (n) mv_rows(&jobs[0]);
    for (int i = 1; i < n; ++i) pthread_join(th[i], NULL);
    free(xsum);
}

void or_cpu_seed4_matvec(const uint16_t* seeds, const uint16_t* coefs, const uint8_t* codes, int bias, const float* x,
                         int rows, int kb, float* y, int threads) {
    seed_matvec(seeds, coefs, codes, bias, 4, x, rows, kb, y, threads);
}
void or_cpu_seed3_matvec(const uint16_t* seeds, const uint16_t* nibs, int bias, const float* x, int rows, int kb,
                         float* y, int threads) {
    seed_matvec(seeds, nibs, NULL, bias, 3, x, rows, kb, y, threads);
}

/* ------------------------------------------------------------------------------------------------------------------ */
/* GEMV in double.  qmv != 0: Q4 weights unrounded s*q+b (MLX's qmv form); BF16 and Q8 as their BF16 values, seeds exact
 * (tests/test_mova_kernels.c:146-158).                                                                               */

void or_mv_double(int fmt, const OrSlice* w, int R, int K, const float* x, int xs, int T, int qmv, double* y,
                  double* mag) {
    float* row = (float*) malloc(sizeof(float) * (size_t) K);
    const int seed = fmt == OR_SEED4 || fmt == OR_SEED4P4;
    for (int r = 0; r < R; ++r) {
        or_row_f32(fmt, w, R, K, r, !seed, row);
        for (int t = 0; t < T; ++t) {
            double acc = 0, m = 0;
            if (qmv && fmt == OR_Q4) {
                /* exact products of the unrounded affine value: recompute s*q+b in double */
                const uint32_t* q = (const uint32_t*) w->p[0];
                const uint16_t* S = (const uint16_t*) w->p[1];
                const uint16_t* B = (const uint16_t*) w->p[2];
                const int sh = group_shift(w);
                for (int c = 0; c < K; ++c) {
                    const size_t i = (size_t) r * K + c;
                    const uint32_t code = (q[i >> 3] >> (4 * (i & 7))) & 15u;
                    const double wv = (double) or_bf2f(S[i >> sh]) * (double) code + (double) or_bf2f(B[i >> sh]);
                    const double v = wv * (double) x[(size_t) t * xs + c];
                    acc += v;
                    m += fabs(v);
                }
            } else {
                for (int c = 0; c < K; ++c) {
                    const double v = (double) row[c] * (double) x[(size_t) t * xs + c];
                    acc += v;
                    m += fabs(v);
                }
            }
            y[(size_t) t * R + r] = acc;
            if (mag) mag[(size_t) t * R + r] = m;
        }
    }
    free(row);
}

/* ------------------------------------------------------------------------------------------------------------------ */
/* routers */

void or_route_softmax(int E, int k, const float* logits, int32_t* ind, float* wt) {
    double mx = -INFINITY, top = 0;
    for (int e = 0; e < E; ++e)
        if (logits[e] > mx) mx = logits[e];
    double* p = (double*) malloc(sizeof(double) * (size_t) E);
    char* taken = (char*) calloc((size_t) E, 1);
    for (int e = 0; e < E; ++e) p[e] = exp((double) logits[e] - mx);
    /* k rounds of arg-max over the probabilities: larger value first, equal values to the higher index */
    for (int r = 0; r < k; ++r) {
        int best = -1;
        for (int e = 0; e < E; ++e) {
            if (taken[e]) continue;
            if (best < 0 || p[e] > p[best] || (p[e] == p[best] && e > best)) best = e;
        }
        taken[best] = 1;
        ind[r] = best;
        top += p[best];
    }
    for (int r = 0; r < k; ++r) wt[r] = (float) (p[ind[r]] / top);
    free(p);
    free(taken);
}

void or_topk_sigmoid(int n, int k, float scale, const float* score, const float* sel, int T, int32_t* inds, float* wts) {
    char* taken = (char*) malloc((size_t) n);
    for (int t = 0; t < T; ++t) {
        const float* sc = score + (size_t) t * n;
        const float* se = sel + (size_t) t * n;
        memset(taken, 0, (size_t) n);
        float sum = 0;
        for (int j = 0; j < k; ++j) {
            int best = -1;
            for (int e = 0; e < n; ++e)
                if (!taken[e] && (best < 0 || se[e] > se[best])) best = e; /* strict >: ties keep the lowest id */
            taken[best] = 1;
            inds[t * k + j] = best;
            sum += sc[best];
        }
        for (int j = 0; j < k; ++j) wts[t * k + j] = sc[inds[t * k + j]] / sum * scale;
    }
    free(taken);
}

void or_route_sigmoid(int d, int n, int k, int hw, float scale, const uint16_t* W, const uint16_t* bias, const float* x,
                      int T, float* score, float* sel, int32_t* inds, float* wts) {
    for (int t = 0; t < T; ++t)
        for (int e = 0; e < n; ++e) {
            double s0 = 0, s1 = 0;
            for (int c = 0; c < d; ++c) {
                const double v = (double) or_bf2f(W[(size_t) e * d + c]) * (double) x[(size_t) t * d + c];
                if (c < hw) s0 += v;
                else s1 += v;
            }
            const float sg = 1.0f / (1.0f + expf(-(or_bfr((float) s0) + or_bfr((float) s1))));
            score[(size_t) t * n + e] = sg;
            sel[(size_t) t * n + e] = sg + or_bf2f(bias[e]);
        }
    or_topk_sigmoid(n, k, scale, score, sel, T, inds, wts);
}

/* ------------------------------------------------------------------------------------------------------------------ */
/* elementwise */

float or_silu_bf(float g) { /* engine/kernels_moe.cu:28-31: sigmoid and product each rounded to BF16 */
    const float s = or_bfr(1.0f / (1.0f + expf(-g)));
    return or_bfr(g * s);
}
void or_swiglu(const float* g, const float* u, float* a, int n) {
    for (int i = 0; i < n; ++i) a[i] = or_bfr(or_silu_bf(g[i]) * u[i]);
}
void or_moe_combine(const float* D, const float* w, const float* shared, float* x, int d, int k, int T) {
    for (int t = 0; t < T; ++t)
        for (int c = 0; c < d; ++c) {
            float s = 0;
            for (int j = 0; j < k; ++j) s += or_bfr(D[((size_t) t * k + j) * d + c] * or_bfr(w[t * k + j]));
            const size_t i = (size_t) t * d + c;
            x[i] = or_bfr(x[i] + or_bfr(or_bfr(s) + shared[i]));
        }
}
void or_q4_moe_combine(int d, int k, const float* D, const float* wt, const float* sh, const float* sg, int sgld,
                       float* out, int T) {
    for (int t = 0; t < T; ++t) {
        const float gate = 1.0f / (1.0f + expf(-sg[(size_t) t * sgld]));
        for (int i = 0; i < d; ++i) {
            float a = gate * sh[(size_t) t * d + i];
            for (int j = 0; j < k; ++j) a += wt[t * k + j] * D[((size_t) t * k + j) * d + i];
            out[(size_t) t * d + i] = a;
        }
    }
}

/* ------------------------------------------------------------------------------------------------------------------ */
/* grouping: pairs by expert (ascending pair id inside an expert), runs of at most bn pairs */

int or_bucket(const int32_t* inds, int count, int n, int bn, int32_t* perm, int32_t* tiles) {
    int np = 0, nt = 0;
    for (int e = 0; e < n; ++e) {
        const int first = np;
        for (int i = 0; i < count; ++i)
            if (inds[i] == e) perm[np++] = i;
        for (int o = first; o < np; o += bn) {
            tiles[4 * nt + 0] = e;
            tiles[4 * nt + 1] = o;
            tiles[4 * nt + 2] = np - o < bn ? np - o : bn;
            tiles[4 * nt + 3] = 0;
            ++nt;
        }
    }
    return nt;
}

/* ------------------------------------------------------------------------------------------------------------------ */
/* slot table: one admit call.  Hits take the new tick; misses, in expert order, take the least recently used slot not
 * touched by this call (nor, with protect_prev, by the previous one); ties to the lowest slot index.               */

int or_cache_admit(int32_t* unit_slot, int32_t* slot_unit, uint32_t* slot_last, uint32_t* tick, int slots,
                   int per_layer, int sl, const int32_t* inds, int count, int protect_prev, int32_t* jobs,
                   uint32_t* hits, uint32_t* misses) {
    const uint32_t prev = tick[0], now = prev + 1;
    char* need = (char*) calloc((size_t) per_layer, 1);
    for (int i = 0; i < count; ++i) need[inds[i]] = 1;
    int nneed = 0, nmiss = 0, nj = 0;
    for (int x = 0; x < per_layer; ++x) {
        if (!need[x]) continue;
        ++nneed;
        const int s = unit_slot[sl * per_layer + x];
        if (s >= 0) slot_last[s] = now;
        else ++nmiss;
    }
    tick[0] = now;
    if (hits) *hits += (uint32_t) (nneed - nmiss);
    if (misses) *misses += (uint32_t) nmiss;
    for (int x = 0; x < per_layer; ++x) {
        if (!need[x] || unit_slot[sl * per_layer + x] >= 0) continue;
        uint32_t best = 0xFFFFFFFFu;
        int bs = -1;
        for (int s = 0; s < slots; ++s) {
            const uint32_t l = slot_last[s];
            if (l == now || (protect_prev && l == prev)) continue;
            if (l < best) {
                best = l;
                bs = s;
            }
        }
        if (bs < 0) break; /* nothing replaceable: stop admitting */
        const int u = sl * per_layer + x, old = slot_unit[bs];
        if (old >= 0) unit_slot[old] = -1;
        slot_unit[bs] = u;
        unit_slot[u] = bs;
        slot_last[bs] = now;
        jobs[2 * nj] = u;
        jobs[2 * nj + 1] = bs;
        ++nj;
    }
    free(need);
    return nj;
}

/* ------------------------------------------------------------------------------------------------------------------ */
/* the small kernels either side of the matmuls                                                                        */

void or_gnorm(int d, float eps, const float* x, const uint16_t* w, float* y, int T) {
    const int hw = d / 2;
    for (int t = 0; t < T; ++t) {
        const float* xr = x + (size_t) t * d;
        double a = 0, b = 0;
        for (int c = 0; c < d; ++c) {
            if (c < hw) a += (double) xr[c] * xr[c];
            else b += (double) xr[c] * xr[c];
        }
        const float r0 = (float) (1.0 / sqrt(a / hw + eps)), r1 = (float) (1.0 / sqrt(b / hw + eps));
        for (int c = 0; c < d; ++c) y[(size_t) t * d + c] = or_bfr(or_bf2f(w[c]) * (xr[c] * (c < hw ? r0 : r1)));
    }
}

void or_norm1p(const float* x, int len, int g, const float* w, float eps, float* y, int T) {
    for (int t = 0; t < T; ++t)
        for (int a = 0; a + g <= len; a += g) {
            const float* xi = x + (size_t) t * len + a;
            double ss = 0;
            for (int k = 0; k < g; ++k) ss += (double) xi[k] * xi[k];
            const double s = 1.0 / sqrt(ss / g + eps);
            for (int k = 0; k < g; ++k) y[(size_t) t * len + a + k] = (float) (xi[k] * s * (1.0 + w[a + k]));
        }
}

void or_argmax(const float* logits, int V, int n, int32_t* out, double* prob) {
    for (int t = 0; t < n; ++t) {
        const float* l = logits + (size_t) t * V;
        float best = -INFINITY;
        int idx = 0;
        for (int i = 0; i < V; ++i)
            if (l[i] > best) { best = l[i]; idx = i; }   /* strict: the first of equal maxima stays */
        out[t] = idx;
        if (prob) {
            double s = 0;
            for (int i = 0; i < V; ++i) s += exp((double) l[i] - (double) best);
            prob[t] = 1.0 / s;
        }
    }
}

/* ------------------------------------------------------------------------------------------------------------------ */
/* FP8 KV cache codec (nslm/kvq.h)                                                                                     */

float or_e4m3_dec(uint8_t c) {
    const int e = (c >> 3) & 15, m = c & 7;
    const float v = e ? ldexpf(1.0f + (float) m / 8, e - 7) : ldexpf((float) m, -9);
    return c & 0x80 ? -v : v;
}
uint8_t or_e4m3_enc_abs(float a) {
    if (!(a < 448.0f)) return 0x7E;
    if (a < 0.015625f) return (uint8_t) rintf(a * 512.0f);
    int e;
    const float f = frexpf(a, &e);
    int E = e - 1, m = (int) rintf((2 * f - 1) * 8);
    if (m == 8) { ++E; m = 0; }
    const int c = ((E + 7) << 3) | m;
    return (uint8_t) (c > 0x7E ? 0x7E : c);
}
uint8_t or_fp8_scale(float amax) {
    if (!(amax > 0)) return 127;
    int k;
    frexpf(amax, &k);
    int e = amax <= ldexpf(448.0f, k - 9) ? k - 9 : k - 8;
    if (e < -126) e = -126;
    if (e > 127) e = 127;
    return (uint8_t) (e + 127);
}
void or_fp8_row(const float* x, int n, uint8_t* codes, uint8_t* scales) {
    for (int b = 0; b < n; b += 32) {
        float amax = 0;
        for (int i = 0; i < 32; ++i) amax = fmaxf(amax, fabsf(x[b + i]));
        scales[b / 32] = or_fp8_scale(amax);
        const int e = (int) scales[b / 32] - 127;
        for (int i = 0; i < 32; ++i) {
            const uint8_t c = or_e4m3_enc_abs(ldexpf(fabsf(x[b + i]), -e));
            codes[b + i] = (uint8_t) (c && x[b + i] < 0 ? c | 0x80 : c);
        }
    }
}
float or_fp8_get(const uint8_t* codes, const uint8_t* scales, int i) { return ldexpf(or_e4m3_dec(codes[i]), (int) scales[i / 32] - 127); }

/* ------------------------------------------------------------------------------------------------------------------ */
/* MLA decode attention                                                                                                */

static float or_softplus_gate(float g) {   /* softplus(x, beta = ln 2) in f32, then BF16 */
    const float gx = g * 0.69314718055994531f;
    return or_bfr((fmaxf(gx, 0.0f) + logf(1.0f + expf(-fabsf(gx)))) / 0.69314718055994531f);
}
void or_heads_map(int H, int O, int I, const float* W, const float* x, int xs, int hs, const float* g, float* y, int T) {
    for (int t = 0; t < T; ++t)
        for (int h = 0; h < H; ++h)
            for (int o = 0; o < O; ++o) {
                double s = 0;
                for (int i = 0; i < I; ++i) s += (double) W[((size_t) h * O + o) * I + i] * x[(size_t) t * xs + (size_t) h * hs + i];
                const size_t yi = ((size_t) t * H + h) * O + o;
                float v = or_bfr((float) s);
                if (g) v = or_bfr(v * or_softplus_gate(g[yi]));
                y[yi] = v;
            }
}
void or_rope_pair(double x0, double x1, int pos, float inv, double* y0, double* y1) {
    const double th = (double) (float) ((float) pos * inv), cs = cos(th), sn = sin(th);
    *y0 = x0 * cs - x1 * sn;
    *y1 = x1 * cs + x0 * sn;
}
void or_mla_attn(int r, int rope, double scale, const float* ql, const float* qr, const float* lat, const float* kr, int pos,
                 float* olat) {
    double* s = (double*) malloc(sizeof(double) * (size_t) (pos + 1));
    double* acc = (double*) calloc((size_t) r, sizeof(double));
    double m = -INFINITY, l = 0;
    for (int p = 0; p <= pos; ++p) {
        double v = 0;
        for (int i = 0; i < r; ++i) v += (double) ql[i] * lat[(size_t) p * r + i];
        for (int i = 0; i < rope; ++i) v += (double) qr[i] * kr[(size_t) p * rope + i];
        s[p] = v * scale;
        if (s[p] > m) m = s[p];
    }
    for (int p = 0; p <= pos; ++p) {
        const double e = exp(s[p] - m);
        l += e;
        for (int i = 0; i < r; ++i) acc[i] += e * lat[(size_t) p * r + i];
    }
    for (int i = 0; i < r; ++i) olat[i] = or_bfr((float) (acc[i] / l));
    free(s);
    free(acc);
}
