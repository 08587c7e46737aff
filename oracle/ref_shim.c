/* oracle/ref_shim.c - exports the reference's header-only spec functions from the compiled reference library.
 *
 * TEST INFRASTRUCTURE ONLY.  Compiled together with the reference's own nslm/lib_*.c, from where they lie, into
 * oracle/_ref/libnslm_ref.so (see oracle/Makefile).  It contains no arithmetic of its own: each wrapper forwards to the
 * reference's inline function of the same name (nslm/lfsr.h, nslm/search4.h) or fills the reference's NsTensor struct
 * (nslm/model_st.h:44-50) around caller streams so ns_row_f32 (nslm/lib_rows.c:27) can be called from ctypes.
 */
#include <stdlib.h>
#include <string.h>

#include "cpu_seed4.h"
#include "kvq.h"
#include "lfsr.h"
#include "qwen4_ops.h"
#include "rows.h"
#include "search4.h"

uint16_t ref_lfsr_step(uint16_t s) { return lfsr_step(s); }
void ref_lfsr_states(uint16_t s, int n, uint16_t* out) { lfsr_states(s, n, out); }
void ref_lfsr_states_wordpar(uint16_t s, int n, uint16_t* out) { lfsr_states_wordpar(s, n, out); }
uint32_t ref_lfsr_stream24(uint16_t s) { return lfsr_stream24(s); }
uint32_t ref_lfsr_stream32(uint16_t s) { return lfsr_stream32(s); }
float ref_nslm_scale(int e) { return nslm_scale(e); }
uint16_t ref_nslm_f2bf(float f) { return nslm_f2bf(f); }
void ref_nslm_decode_block(uint16_t seed, uint16_t nib, int exp_bias, uint16_t* out) { nslm_decode_block(seed, nib, exp_bias, out); }
int ref_nslm4_q(uint16_t coef, int p) { return nslm4_q(coef, p); }
int ref_nslm_q(uint16_t nib, int p) { return nslm_q(nib, p); }

static NsRows g_rows;
static int g_rows_ready;

/* one row of a single-slice tensor given as raw streams; eb: the slice's exponent bias */
void ref_row_f32(int enc, const void* p0, const void* p1, const void* p3, int32_t eb, int group, int rows, int cols,
                 int row, int round, float* out) {
    if (!g_rows_ready) { ns_rows_init(&g_rows); g_rows_ready = 1; }
    NsTensor t;
    memset(&t, 0, sizeof t);
    t.enc = enc; t.slices = 1; t.rows = rows; t.cols = cols; t.group = group;
    t.s[0].p = (const uint8_t*) p0;
    t.s[1].p = (const uint8_t*) p1;
    if (enc == NS_Q8 || enc == NS_Q4) t.s[2].p = (const uint8_t*) p3;   /* biases */
    else { t.s[2].p = (const uint8_t*) &eb; t.s[3].p = (const uint8_t*) p3; }
    ns_row_f32(&g_rows, &t, 0, row, round, out);
}

void ref_qwen4_route(int n_exp, int top_k, const float* logits, int32_t* ind, float* wt) {
    Qwen4Cfg c;
    memset(&c, 0, sizeof c);
    c.n_exp = n_exp; c.top_k = top_k;
    qwen4_route(&c, logits, ind, wt);
}

float ref_e4m3_dec(uint8_t c) { return kvq_e4m3_dec(c); }
uint8_t ref_e4m3_enc_abs(float a) { return kvq_e4m3_enc_abs(a); }
uint8_t ref_fp8_scale(float amax) { return kvq_fp8_scale(amax); }
void ref_fp8_row(const float* x, int n, uint8_t* codes, uint8_t* scales) { kvq_row(x, n, n, codes, scales); }
float ref_fp8_get(const uint8_t* codes, const uint8_t* scales, int i) { return kvq_fp8_get(codes, scales, i); }

void ref_norm1p(const float* x, int len, int g, const float* w, float eps, float* y) { qwen4_norm1p(x, len, g, w, eps, y); }

/* the tiled CPU mat-vec / mat-mul as the reference's own bench drives it (harness/nslm-cpu-seed-bench.c:50-75) */
void* ref_tile4(const uint16_t* seeds, const uint16_t* coefs, const uint8_t* codes, int bias, int rows, int kb) {
    CpuSeed4Tiled* t = (CpuSeed4Tiled*) malloc(sizeof *t);
    cpu_seed4_tile(t, seeds, coefs, codes, bias, rows, kb);
    return t;
}
void* ref_tile3(const uint16_t* seeds, const uint16_t* nibs, int bias, int rows, int kb) {
    CpuSeed4Tiled* t = (CpuSeed4Tiled*) malloc(sizeof *t);
    cpu_seed3_tile(t, seeds, nibs, bias, rows, kb);
    return t;
}
void ref_tiled_matmul(void* t, const float* x, int ntok, float* y, int threads) {
    cpu_seed4_tiled_matmul_mt((const CpuSeed4Tiled*) t, cpu_seed4_table(), x, ntok, y, threads);
}
void ref_tile_free(void* t) { cpu_seed4_tiled_free((CpuSeed4Tiled*) t); free(t); }
void ref_matvec(const uint16_t* seeds, const uint16_t* coefs, const uint8_t* codes, int bias, const float* x, int rows,
                int kb, float* y, int threads) {
    cpu_seed4_matvec_mt(seeds, coefs, codes, bias, cpu_seed4_table(), x, rows, kb, y, threads);
}
