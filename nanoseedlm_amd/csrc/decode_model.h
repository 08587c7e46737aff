/* decode_model.h - host side (C99) of a whole synthetic seeded-MoE model's greedy decode on the gfx950 kernels: the
 * benchmark configuration "24 layers, hidden 2048, MLA attention with 16 heads, latent 512 + RoPE 64, 8-bit KV cache,
 * 128 seeded P=4 experts top-8 plus one shared expert per layer, BF16 LM head over 151936 tokens".  The launch sequence
 * per layer follows the reference engines (attention: engine/mova_cuda.c:1229-1278 with the absorbed-MLA maps of
 * nslm/lib_mova_ref.c:392-450; experts: engine/qwen4_cuda.c:1023-1083 through moe_layer.c); what the benchmark leaves open
 * is fixed here and stated at each step in decode_model.c.  Everything a step needs lives on the device - token ids,
 * positions, caches - so one step is a pure launch sequence and can be captured into a graph and replayed.
 */
#pragma once
#include <stdint.h>

#include "moe_layer.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
    int n_layer, d, n_head, head_dim, r, rope;
    int n_exp, top_k, ff, ff_shared;
    int vocab, max_ctx, max_rows;
    int kv_fmt;        /* KV_BF16 or KV_FP8 */
    int n_splits;      /* attention key splits (0: 32) */
    float eps, rope_theta;
} NslmModelCfg;

typedef struct NslmModel NslmModel;

/* the seeded dense matrices of a layer */
enum { NSLM_W_Q = 0, NSLM_W_KVA = 1, NSLM_W_KR = 2, NSLM_W_O = 3, NSLM_W_SG = 4, NSLM_W_SU = 5, NSLM_W_SD = 6, NSLM_W_COUNT = 7 };
/* the BF16 per-head maps of a layer */
enum { NSLM_H_QRMIX = 0, NSLM_H_QLAT = 1, NSLM_H_VUP = 2, NSLM_H_COUNT = 3 };

NslmModel* nslm_model_open(const NslmModelCfg* c, char* err, int errlen);
void nslm_model_close(NslmModel* m);
/* every weight filled on the device from a reproducible generator: random seed records (exponent bias eb), BF16 maps,
 * router and embedding uniform in small ranges, unit norms.  For benchmarks; finalizes the model. */
int nslm_model_fill_random(NslmModel* m, uint64_t seed, int eb);
/* tests: upload weights.  Dense seeded matrix `which` of `layer` [R][K] (P = 4 streams); per-head map (BF16 bits);
 * norm weights (f32 [d]; layer n_layer: the final norm; which 0 attention, 1 experts); the embedding = LM head (BF16
 * bits [vocab][d]); the experts through nslm_model_moe().  Then nslm_model_finalize(). */
int nslm_model_set_dense(NslmModel* m, int layer, int which, const uint16_t* seeds, const uint16_t* coefs, const uint8_t* codes, int eb);
int nslm_model_set_heads(NslmModel* m, int layer, int which, const uint16_t* w);
int nslm_model_set_norm(NslmModel* m, int layer, int which, const float* w);
int nslm_model_set_embed(NslmModel* m, const uint16_t* w);
NslmMoe* nslm_model_moe(NslmModel* m);
int nslm_model_finalize(NslmModel* m);
void nslm_model_dense_shape(const NslmModel* m, int which, int* R, int* K);
void nslm_model_heads_shape(const NslmModel* m, int which, int* O, int* I);

/* T sequences (slot t at cache rows [t * max_ctx, ...)): their next input tokens and positions (synchronises) */
int nslm_model_start(NslmModel* m, int T, const int32_t* ids, const int32_t* pos);
/* cache rows [0, upto) of every slot filled with reproducible pseudo-random entries (benchmarks: a context without
 * having decoded it) */
int nslm_model_fill_cache(NslmModel* m, int T, int upto, uint64_t seed);
/* one greedy decode step for the T sequences, asynchronous on s: reads the ids, appends to the caches at the positions,
 * leaves the arg-max tokens as the next ids and advances the positions.  Launches only. */
/* on: a layer's independent launches (the three projections of the normed input, the two maps of the query, the shared
 * expert beside the routed ones - the reference runs that one on a second stream, engine/qwen4_cuda.c:1026-1032) go to
 * two side streams joined by events, which a captured step turns into parallel graph branches.  Steps of up to 8 rows. */
int nslm_model_set_branches(NslmModel* m, int on);
/* -1 (nothing launched) when a sequence slot is full: a step writes the cache at every row's position, and the positions
 * advance on the device, so the host keeps the bound - the largest position given to nslm_model_start plus the steps that
 * ran since.  A step that succeeds on a stream that is not capturing counts one; a step recorded into a graph counts
 * nothing (it launched nothing), and every replay through nslm_model_launch counts one (-1, nothing launched: it would run
 * past max_ctx).  A caller that replays the graph by other means (as a child of its own graph) accounts with
 * nslm_model_account(m, n) before it launches (-1: the n steps would run past max_ctx; n < 0 takes steps back).  On the
 * device the positions saturate at max_ctx - 1, so even an unaccounted replay stays inside the cache. */
int nslm_model_step(NslmModel* m, kc_stream_t s, int T);
int nslm_model_steps_left(const NslmModel* m);
int nslm_model_launch(NslmModel* m, NslmGraph* g, kc_stream_t s);
int nslm_model_account(NslmModel* m, int steps);
/* synchronising reads: the current ids, the last step's logits [T][vocab]; -1 also when a wait inside the persistent expert
 * kernel gave up since open (the results are void then) */
int nslm_model_ids(NslmModel* m, int T, int32_t* ids);
int nslm_model_logits(NslmModel* m, int T, float* logits);
/* for tests (both synchronise): the last step's final hidden rows [T][d] after the closing norm - what the LM head multiplies -
 * and rows [first, first + rows) of the BF16 embedding / LM-head matrix */
int nslm_model_hidden(NslmModel* m, int T, float* h);
int nslm_model_get_embed(NslmModel* m, int first, int rows, uint16_t* w);
/* compressed weight bytes one decode step of one token reads: experts selected + shared expert + dense + maps + LM head */
uint64_t nslm_model_step_bytes(const NslmModel* m);

#ifdef __cplusplus
}
#endif
