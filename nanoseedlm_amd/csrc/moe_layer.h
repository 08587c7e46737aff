/* moe_layer.h - host side of one routed-expert MoE layer stack on the gfx950 kernels, in C99: the expert slot table
 * (layout and initial residency as the reference's build_pool, engine/mova_cuda.c:311-404) and the per-layer launch
 * sequence of the reference's engines (engine/mova_cuda.c:1279-1325 encode_layer; engine/qwen4_cuda.c:1023-1083 moe).
 * All experts of all layers live in one HBM arena; with slots == units (the default on a 288 GB GPU) the arena is the
 * pool, every expert is resident, and the admit / copy kernels are skipped.  A smaller pool exercises the LRU table.
 */
#pragma once
#include <stdint.h>

#include "kernels_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

enum { NSLM_ROUTE_SOFTMAX = 0, NSLM_ROUTE_SIGMOID = 1 };

typedef struct {
    int n_layer, n_exp, top_k, d, ff;
    int fmt;       /* MF_SEED4P4 or MF_SEED4: the experts' format */
    int router;    /* NSLM_ROUTE_SOFTMAX: logits = bf16(W x) by kc_mv on a BF16 router weight, kq4_route, kq4_moe_combine
                      (f32 sums; the Qwen composition).  NSLM_ROUTE_SIGMOID: kc_router, kc_moe_combine (BF16 rounding at
                      every tensor boundary; the MoVA composition) */
    int max_rows;  /* most tokens a step takes */
    int slots;     /* pool slots; 0 or >= n_layer * n_exp: all resident */
    float route_scale;
    int host_units; /* 1: the experts' units live in pinned host memory that the GPU reads (the reference's layout where the expert
                      set exceeds device memory, engine/mova_cuda.c:340-360); the pool's slots are the only copies in HBM */
    int prefetch;   /* 1 (sigmoid composition, a pool smaller than the expert set, decode steps): after a layer's own experts are
                      admitted, the next layer's router is run on this layer's input, its likely experts are admitted with
                      CACHE_PROTECT_PREV and copied on a second stream, and the next layer's admit waits for that copy
                      (engine/mova_cuda.c:1283-1303) */
} NslmMoeCfg;

typedef struct NslmMoe NslmMoe;

NslmMoe* nslm_moe_open(const NslmMoeCfg* c, char* err, int errlen);
void nslm_moe_close(NslmMoe* m);
/* tensor: 0 gate [ff][d], 1 up [ff][d], 2 down [d][ff].  Host streams of ONE expert: seeds, words (coefficient or nibble
 * words), codes (P = 4 only), exponent bias.  Call for every (layer, expert, tensor) before nslm_moe_finalize. */
int nslm_moe_set_expert(NslmMoe* m, int layer, int expert, int tensor, const uint16_t* seeds, const uint16_t* words,
                        const uint8_t* codes, int eb);
/* router weight [n_exp][d] as BF16 bits; bias [n_exp] BF16 bits (sigmoid router only, else NULL) */
int nslm_moe_set_router(NslmMoe* m, int layer, const uint16_t* W, const uint16_t* bias);
int nslm_moe_finalize(NslmMoe* m);
/* benchmarks: every expert's records filled on the device from a reproducible generator (any bytes are valid seed records),
 * one exponent bias for all, router weights BF16 uniform in [-router_scale, router_scale].  Call before nslm_moe_finalize. */
int nslm_moe_fill_random(NslmMoe* m, uint64_t seed, int eb, float router_scale);
/* One MoE layer for T rows, asynchronous on stream s (launches only, capturable into a graph).
 * xn: the layer input [T][d] (device).  io [T][d] (device): softmax composition: receives sum_k wt_k y_k;
 * sigmoid composition: the residual stream, updated in place x = bf16(x + bf16(bf16(sum) + 0)). */
int nslm_moe_step(NslmMoe* m, kc_stream_t s, int layer, const float* xn, int T, float* io);
/* n steps one after the other on s from one call (step i: layer layers[i], input xn[i], all into io): what a C host's decode
 * loop issues, without a caller's interpreter between the launches.  before / after (nh_event_t, or NULL): events recorded on s
 * directly before the first and after the last step, for a caller that times the steps.  Stops at the first step that fails (-1). */
int nslm_moe_step_seq(NslmMoe* m, kc_stream_t s, int n, const int* layers, const float* const* xn, int T, float* io, void* before,
                      void* after);
/* The same for the dense one-row matvec: n launches of kc_mv(fmt, ws[(first + i) % nw], K, R, x -> y) on s, with the events around them. */
int nslm_mv_seq(kc_stream_t s, int fmt, const WSlice* ws, int nw, int first, int n, int K, int R, const float* x, float* y, void* before,
                void* after);
/* routed experts + a shared expert (3 host slices: gate, up, down of the routed experts' shape) + residual in the one persistent launch:
 * out = bf16(res + bf16(sum_j wt_j y_j + y_shared)).  0 done, 1 not available (nothing launched), -1 error. */
int nslm_moe_step_layer(NslmMoe* m, kc_stream_t s, int layer, const float* xn, int T, const WSlice* shared, const float* res, float* out,
                        const float* norm_w, float norm_eps);   /* norm_w: xn is the raw stream, normalised inside (kq4_norm1p's values) */
/* 1 (default): decode steps of the softmax composition with every expert resident run as one persistent kernel
 * (kc_moe_decode); 0: always the separate launchers.  The results are the same bits either way.
 * 2: as 1, checked - for hosts that run other streams beside the steps (the reference engine copies experts on a second
 * stream, engine/mova_cuda.c:136-146): the kernel's workgroups wait for each other, and if they cannot all be resident a
 * bounded wait gives up and the results are void.  In this mode nslm_moe_step synchronises s after the kernel, reads its
 * error word and, if set, zeroes the sync words, redoes the step through the separate launchers and leaves the stack at
 * mode 0; nslm_moe_fallbacks() counts these.  Not capturable (it synchronises); nslm_moe_step_layer answers 1 (not
 * available) so that the caller composes the block around nslm_moe_step. */
void nslm_moe_set_fused(NslmMoe* m, int on);
int nslm_moe_fused_mode(const NslmMoe* m);
int nslm_moe_fallbacks(const NslmMoe* m);
long nslm_moe_fused_steps(const NslmMoe* m);   /* steps that the persistent kernel took (launched, not necessarily without error) */
/* 0, or non-zero when a grid barrier of the fused kernel gave up since open (synchronises) */
int nslm_moe_fused_error(NslmMoe* m);
/* n words of the persistent kernels' sync area from word `first`, copied to the host (synchronises): behind the error word
 * (kc_moe_decode_error_word()) lie which wait gave up (word + 1) and workgroup 0's phase timeline (64-bit wall-clock ticks, 100 MHz,
 * from word + 2) */
int nslm_moe_fused_words(NslmMoe* m, int first, int n, uint32_t* out);
/* the last step's routing, copied to the host (synchronises the device): ind [T][top_k], wt [T][top_k] */
int nslm_moe_last_routing(NslmMoe* m, int T, int32_t* ind, float* wt);
/* the last step's router logits [T][n_exp] as the kernels formed them (softmax router: the BF16-rounded values the selection
 * was made on), copied to the host (synchronises) */
int nslm_moe_last_logits(NslmMoe* m, int T, float* logits);
/* the last step's intermediates per (token, expert) pair, copied to the host (synchronises): A [pairs][ff] = the SwiGLU outputs
 * the down projections read, D [pairs][d] = the experts' outputs the combine sums.  Pair t * top_k + j of nslm_moe_step (the
 * batched path's A is the packed BF16 view: read it as uint16 [pairs][ff] in the first half of the buffer). */
int nslm_moe_last_pairs(NslmMoe* m, int pairs, float* A, float* D);
/* the slot table's counters and state (synchronises): hits, misses since open */
int nslm_moe_cache_stats(NslmMoe* m, uint32_t* hits, uint32_t* misses);
/* the prefetch's own counters (synchronises): predicted experts already resident, predicted experts copied ahead */
int nslm_moe_prefetch_stats(NslmMoe* m, uint32_t* hits, uint32_t* misses);
/* the device slice table [n_exp] of a layer's tensor (0 gate, 1 up, 2 down): what kc_mv_gu / kc_mv_sel take */
const WSlice* nslm_moe_tab(const NslmMoe* m, int layer, int tensor);
/* the device address of a layer's BF16 router weight [n_exp][d] */
const uint16_t* nslm_moe_router_w(const NslmMoe* m, int layer);
uint64_t nslm_moe_unit_bytes(const NslmMoe* m);
/* compressed bytes one expert's three matrices occupy (without alignment padding) */
uint64_t nslm_moe_expert_bytes(const NslmMoe* m);

/* ---- capture / replay of a launch sequence (hipGraph), and event timing, for hosts without HIP headers ---- */
typedef struct NslmGraph NslmGraph;
int nslm_graph_begin(kc_stream_t s);                 /* start capturing s */
NslmGraph* nslm_graph_end(kc_stream_t s);            /* end capture and instantiate; NULL on failure */
int nslm_graph_launch(NslmGraph* g, kc_stream_t s);
int nslm_stream_capturing(kc_stream_t s);           /* 1 while s records into a graph */
void nslm_graph_free(NslmGraph* g);

#ifdef __cplusplus
}
#endif
