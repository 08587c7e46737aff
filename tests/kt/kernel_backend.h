/* kernel_backend.h - the host side of the kernel tests: one call per kernel (or fused group) on HOST arrays.  Each call
 * uploads its inputs into fresh device allocations, runs the kc_ / kq4_ launcher the engine runs, on the default stream,
 * copies the outputs back and frees - the call pattern of the reference's tests/kernel_backend_cuda.c, whose kt_
 * functions these mirror by name, argument meaning and return convention for the seed-matmul path
 * (reference tests/kernel_backend.h:14-56, 241).  Returns 0, -1 after printing what failed, or 1 for "not in this backend".
 */
#pragma once
#include <stddef.h>
#include <stdint.h>

#include "kernels_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* A stacked weight: S slices of R x K in the model's streams, slice after slice in each stream
 * (reference tests/kernel_backend.h:19-30): BF16 w = values; Q8 / Q4 w = packed words, s = scales, b = biases;
 * SEED4 w = seeds, s = nibble words, b = int32 exponent bias per slice; SEED4P4 w = seeds, s = coefficient words,
 * b = int32 exponent bias per slice, e = exponent codes (two blocks per byte, low first). */
typedef struct {
    int fmt, S, R, K;
    const void *w, *s, *b, *e;
    size_t wn, sn, bn, en; /* bytes */
    int group;             /* Q8 / Q4: 32 or 64 (0 is 64) */
} KtWeight;

int kt_open(char* err, int errlen);
void kt_close(void);
const char* kt_name(void);
int kt_mm_tile(void);
int kt_seed_gemm_exact(int on);
int kt_has_fmt(int fmt);
void kt_store_f32(int on); /* this backend: unrounded f32 stores from the matvec family and the GEMM */

int kt_mv(const KtWeight* w, int T, int add, const float* x, float* y);
int kt_mv_sel(const KtWeight* w, int P, int xdiv, const int32_t* sel, const float* x, float* y);
int kt_mv_gu(const KtWeight* w, int P, int xdiv, const int32_t* sel, const float* x, float* a);
int kt_mm(const KtWeight* w, int T, const float* x, float* y);
/* the same without the residual, optionally through kc_pack_input_bf16 + kc_mm_packed */
int kt_mm_plain(const KtWeight* w, int T, int packed, const float* x, float* y);
int kt_mm_grouped(const KtWeight* w, int P, int xdiv, const int32_t* perm, const MmTile* tiles, int nt, const float* x,
                  float* y);
/* kc_bucket on inds[count] (n experts), then kc_mm_grouped_dev (packed: kc_mm_grouped_packed) with the device tile
 * count; perm / tiles / ntiles (may be NULL) receive the grouping */
int kt_mm_bucketed(const KtWeight* w, int count, int xdiv, const int32_t* inds, int packed, const float* x, float* y,
                   int32_t* perm, MmTile* tiles, int32_t* ntiles);
int kt_bucket(const int32_t* inds, int count, int n, int32_t* perm, MmTile* tiles, int32_t* ntiles);
int kt_router(RouterArgs a, const uint16_t* W, const uint16_t* bias, const float* x, int T, int32_t* ind, float* wt);
int kt_router_topk(RouterArgs a, const float* score, const float* sel, int T, int32_t* ind, float* wt);
int kt_q4_route(int n_exp, int top_k, const float* logits, int32_t* ind, float* wt, int T);
int kt_swiglu(const float* g, const float* u, float* a, int n);
int kt_combine(const float* D, const float* w, const float* shared, float* x, int d, int k, int T);
int kt_q4_combine(int d, int k, const float* D, const float* wt, const float* sh, const float* sg, int sgld, float* out, int T);
/* slice `slice` of w decoded to BF16 bits [R][K] (kc_slice_deq) */
/* the small kernels of a full decode step (tests/kernel_backend.h:51,139-143,155) */
int kt_gnorm(int d, float eps, const float* x, const uint16_t* w, float* y, int T);
int kt_q4_norm1p(const float* x, int len, int g, const float* w, float eps, float* y, int T);
int kt_embed(int fmt, const uint16_t* E, const uint32_t* q8, const uint16_t* s8, const uint16_t* b8, int V, int d,
             const int32_t* ids, int n, float* x);
int kt_embed_seed(const KtWeight* w, const int32_t* ids, int n, float* x);   /* 1 for formats this backend lacks */
int kt_argmax(const float* logits, int V, int n, int32_t* out);
int kt_argmax_p(const float* logits, int V, int n, int32_t* out, float* prob);   /* ours: kc_argmax_p has no kt_ in the reference */
/* MLA decode attention (tests/kernel_backend.h:79-104,123-137).  The reference splits these by format (kt_heads_mv /
 * kt_heads_q / kt_heads_seed, kt_mla_rope / kt_mla_rope_q, kt_mla_attn / kt_mla_attn_q); here the format is an argument:
 * per-head maps with W = slice 0 of w (R = H * O, K = I; ebias: a seed map's exponent bias per head, or NULL); caches of
 * npos positions in fmt KV_BF16 (k, v: u16) or KV_FP8 (k, v: codes, ks, vs: scale bytes), all in one segment. */
int kt_heads_w(const KtWeight* w, int H, int O, int I, const int32_t* ebias, const float* x, int xs, int hs, const float* g,
               float* y, int T);
int kt_mla_rope_f(MlaArgs a, int fmt, float* qr, const float* kr, const float* c, void* k, void* v, void* ks, void* vs, int npos,
                  const RowInfo* ri, const float* inv, int T);
int kt_mla_attn_f(MlaArgs a, int fmt, const float* ql, const float* qr, void* k, void* v, void* ks, void* vs, int npos,
                  const RowInfo* ri, float* olat, int T);
int kt_kv_f32(int fmt, const uint8_t* codes, const uint8_t* scales, int len, int rows, float* y);
int kt_slice_deq(const KtWeight* w, int slice, uint16_t* out);
/* a SEED4P4 / Q8 / Q4 per-head map [H][O][I] decoded to BF16 (kc_heads_deq); seeds: ebias one per head */
int kt_heads_deq(int fmt, int H, int O, int I, const void* p0, size_t n0, const void* p1, size_t n1, const int32_t* ebias,
                 const void* p3, size_t n3, int group, uint16_t* out);
/* One slot-table admit (+ copy) on host-side state: arrays are updated in place.  tab: [ntens][per_layer] WSlice of
 * sparse layer 0 (device pointers are rewritten relative to a pool base of 0: offsets).  Returns njobs or -1. */
int kt_cache_admit(int32_t* unit_slot, int32_t* slot_unit, uint32_t* slot_last, uint32_t* tick, uint32_t* stats, int units,
                   int slots, int per_layer, int sl, const int32_t* inds, int count, int flags, int32_t* jobs);
/* fills a pool of `slots` units of unit_bytes from an arena of `units`, admits inds and copies; pool_out receives the pool */
int kt_cache_roundtrip(const uint8_t* arena, int units, int slots, uint64_t unit_bytes, int per_layer, const int32_t* inds,
                       int count, uint8_t* pool_out, int32_t* unit_slot_out);

#ifdef __cplusplus
}
#endif
