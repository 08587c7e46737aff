/* oracle/nslm_oracle.h - CPU restatement of the SeedLM decode-in-matmul arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or calls this file: it is the checker the
 * parity tests, the smoke test and the benchmark's CPU-baseline leg compare the HIP path against.
 *
 * Every function names the reference file:line whose arithmetic it restates (paths relative to the reference tree).
 * Pins: see the header comment of nslm_oracle.c.
 */
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* weight formats, numbered as the reference (engine/kernels_moe.metal:17) */
enum { OR_BF16 = 0, OR_SEED4 = 1, OR_Q8 = 2, OR_Q4 = 3, OR_SEED4P4 = 4 };

/* one slice's streams, in the reference's stream order (engine/kernels_cuda.h:4-7, nslm/model_st.h:42-43) */
typedef struct {
    const void* p[4];
    int32_t eb; /* seeds: exponent bias */
    int32_t gs; /* Q8/Q4: log2 group, 0 means 64 */
} OrSlice;

/* ---- LFSR (nslm/lfsr.h:20-59) ---- */
uint16_t or_lfsr_step(uint16_t s);
void or_lfsr_states(uint16_t s, int n, uint16_t* out);
uint32_t or_lfsr_stream(uint16_t s, int nbits); /* nbits 24 or 32: bit k = top bit of state k+1 */
void or_lfsr_stream_table(int nbits, uint32_t* table /* [65536] */);
uint64_t or_lfsr_fnv24(void); /* FNV-1a over the 24 states after every seed 1..65535 (tests/test_lfsr.c:41-56) */

/* ---- scalar helpers (nslm/lfsr.h:87-112) ---- */
float or_scale(int e);          /* fl(R32 * 2^e) */
uint16_t or_f2bf(float f);      /* round to nearest even */
float or_bf2f(uint16_t h);
float or_bfr(float f);          /* f32 value of the BF16 rounding */

/* ---- block decode to BF16 bits: P=3 (nslm/lfsr.h:116-128) and P=4 (nslm/lib_search4.c:22-31) ---- */
void or_decode_p3(uint16_t seed, uint16_t nib, int exp_bias, uint16_t out[8]);
void or_decode_p4(uint16_t seed, uint16_t coef, int e, uint16_t out[8]);
/* the exact integer sums of a block (|isum| < 2^20) */
void or_isum_p3(uint16_t seed, uint16_t nib, int32_t out[8]);
void or_isum_p4(uint16_t seed, uint16_t coef, int32_t out[8]);

/* ---- one weight row as f32 (nslm/lib_rows.c:27-76): seeds unrounded, affine rounded to BF16 when round != 0 ---- */
void or_row_f32(int fmt, const OrSlice* w, int R, int K, int row, int round, float* out);
/* rows [0,R) of a slice rounded to BF16 bits: the prefill GEMM's weight definition (engine/kernels_moe.cu:357-403,
 * 1325-1335) */
void or_slice_bf16(int fmt, const OrSlice* w, int R, int K, uint16_t* out);

/* ---- affine dequantize (nslm/lib_affine.c:54-63), group = 1 << gs ---- */
void or_affine_dequant(const uint32_t* words, const uint16_t* scales, const uint16_t* biases, int64_t n, int bits,
                       int group, uint16_t* out);

/* ---- CPU decode-in-dot-product, P=4 (nslm/cpu_seed4.h:1-8, nslm/lib_cpu_seed4.c:76-101 scalar form) ----
 * y[r] for rows [0,rows); threads > 1 splits the rows over pthreads.  x has kb*8 floats. */
void or_cpu_seed4_matvec(const uint16_t* seeds, const uint16_t* coefs, const uint8_t* codes, int bias, const float* x,
                         int rows, int kb, float* y, int threads);
/* the same for P=3 nibble words (nslm/lib_cpu_seed4.c:351-394 scalar form) */
void or_cpu_seed3_matvec(const uint16_t* seeds, const uint16_t* nibs, int bias, const float* x, int rows, int kb,
                         float* y, int threads);

/* ---- GEMV reference in double over the row decoder, unrounded (tests/test_mova_kernels.c:186-193) ----
 * y[t*R + r] = sum_c w[r][c] * x[t*xs + c];  mag (may be NULL) = sum |w x| */
void or_mv_double(int fmt, const OrSlice* w, int R, int K, const float* x, int xs, int T, int qmv, double* y,
                  double* mag);

/* ---- routers ---- */
/* softmax top-k, ties to the higher index, weights renormalised over the k (nslm/lib_qwen4_ops.c:107-122) */
void or_route_softmax(int E, int k, const float* logits, int32_t* ind, float* wt);
/* sigmoid router (nslm/lib_mova_ref.c:171-201): W, bias BF16; two partial sums each rounded to BF16 */
void or_route_sigmoid(int d, int n, int k, int hw, float scale, const uint16_t* W, const uint16_t* bias, const float* x,
                      int T, float* score, float* sel, int32_t* inds, float* wts);
/* its top-k step alone from score / sel (engine/kernels_moe.cu:742-772: ties to the lowest id) */
void or_topk_sigmoid(int n, int k, float scale, const float* score, const float* sel, int T, int32_t* inds, float* wts);

/* ---- elementwise (engine/kernels_moe.cu:28-31, 775-788; engine/kernels_qwen4.cu:506-515) ---- */
float or_silu_bf(float g);
void or_swiglu(const float* g, const float* u, float* a, int n);
void or_moe_combine(const float* D, const float* w, const float* shared, float* x, int d, int k, int T);
void or_q4_moe_combine(int d, int k, const float* D, const float* wt, const float* sh, const float* sg, int sgld,
                       float* out, int T);

/* ---- the small kernels either side of the matmuls ---- */
/* grouped RMSNorm, 2 groups (nslm/lib_mova_ref.c:158-168): sums in double, r as float, y = bf16(w * (x * r)) */
void or_gnorm(int d, float eps, const float* x, const uint16_t* w, float* y, int T);
/* y = x r (1 + w) per group of g (nslm/lib_qwen4_ops.c:11-18): all in double, one rounding to float */
void or_norm1p(const float* x, int len, int g, const float* w, float eps, float* y, int T);
/* greedy arg-max, ties to the lowest index (engine/kernels_moe.cu:2115-2136), and prob = 1 / sum exp(l - max) (:2137-2150) */
void or_argmax(const float* logits, int V, int n, int32_t* out, double* prob);

/* ---- FP8 KV cache codec (nslm/kvq.h:19-34,48-57,70-79,109-111): E4M3 codes, one E8M0 scale byte per 32 values ---- */
float or_e4m3_dec(uint8_t c);
uint8_t or_e4m3_enc_abs(float a);              /* a >= 0: round to nearest even, saturated at 448 */
uint8_t or_fp8_scale(float amax);              /* the smallest 2^e with 448 2^e >= amax, as byte e + 127 */
void or_fp8_row(const float* x, int n, uint8_t* codes, uint8_t* scales);   /* n a multiple of 32 */
float or_fp8_get(const uint8_t* codes, const uint8_t* scales, int i);

/* ---- MLA decode attention (nslm/lib_mova_ref.c:280-345; engine/kernels_moe.cu:1147-1323) ---- */
/* per-head maps y[t][h][o] = bf16(W_h[o] . x[t*xs + h*hs ..]) over exact weights W [H*O][I] given as f32 rows; with g:
 * bf16(that * bf16(softplus_ln2(g))) (engine/kernels_moe.cu:215-218,1170-1174).  Sums in double. */
void or_heads_map(int H, int O, int I, const float* W, const float* x, int xs, int hs, const float* g, float* y, int T);
/* RoPE of pair (p, p + rope/2) at angle (float) pos * inv[p] (engine/kernels_moe.cu:1188-1196), in double */
void or_rope_pair(double x0, double x1, int pos, float inv, double* y0, double* y1);
/* latent attention of one (row, head) over positions 0..pos: lat [npos][r], kr [npos][rope] as f32 values; olat[r] =
 * bf16(sum softmax(scale (ql . c + qr . k)) c), all sums in double */
void or_mla_attn(int r, int rope, double scale, const float* ql, const float* qr, const float* lat, const float* kr, int pos,
                 float* olat);

/* ---- grouping (engine/kernels_moe.cu:527-573; tests/test_qwen4_engine.c:33-61 host regrouping) ----
 * tiles: int32 quads {slice,start,count,0}; returns the tile count */
int or_bucket(const int32_t* inds, int count, int n, int bn, int32_t* perm, int32_t* tiles);

/* ---- expert slot table, host model of engine/kernels_moe.cu:2025-2102 ----
 * unit_slot[units], slot_unit[slots], slot_last[slots], tick[1]; returns the number of (unit,slot) jobs written */
int or_cache_admit(int32_t* unit_slot, int32_t* slot_unit, uint32_t* slot_last, uint32_t* tick, int slots,
                   int per_layer, int sl, const int32_t* inds, int count, int protect_prev, int32_t* jobs,
                   uint32_t* hits, uint32_t* misses);

#ifdef __cplusplus
}
#endif
