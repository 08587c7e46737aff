/* include/kernels_hip.h - C entry points of the MI355X (gfx950) SeedLM decode-in-matmul backend.
 *
 * This is the drop-in boundary: every kc_ and kq4_ function below keeps the name, argument order, argument meaning and error
 * behaviour of the reference's launcher of the same name (engine/kernels_cuda.h, engine/kernels_qwen4.h), so the
 * reference's C99 engine (engine/mova_cuda.c encode_layer :1218-1327, engine/qwen4_cuda.c moe :1023-1083) and its
 * kernel tests (tests/kernel_backend_cuda.c) can call this library in place of engine/kernels_moe.cu.
 * Differences a host must know:
 *   - the first argument is a kc_stream_t: an opaque pointer that carries a hipStream_t (0 = the default stream), where
 *     the reference takes a cudaStream_t;
 *   - the stream table argument G is accepted and ignored (the kernels hold the 512-entry GF(2) basis themselves);
 *   - launchers are asynchronous, allocate nothing and keep no per-call state, so whole forwards can be captured into
 *     graphs as the reference does (engine/mova_cuda.c:1402-1406).
 * The structs are layout-identical to the reference's (engine/kernels_cuda.h:19-48, engine/kernels_moe.metal:96-130).
 * Plain C99: no HIP header is needed to include this file.
 */
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* kc_stream_t; /* holds a hipStream_t; replaces cudaStream_t in every signature */

/* weight formats = the reference's MF_ and NS_ codes (engine/kernels_moe.metal:17, nslm/model_st.h:31) */
enum { MF_BF16 = 0, MF_SEED4 = 1, MF_Q8 = 2, MF_Q4 = 3, MF_SEED4P4 = 4 };
#define MV_MAXT 8 /* dense matvec: tokens per call (engine/kernels_moe.metal:20) */

/* One slice's device stream addresses (engine/kernels_cuda.h:19-24).  Stream order (engine/kernels_cuda.h:4-7):
 * BF16 0 values; Q8/Q4 0 packed words, 1 scales, 2 biases; SEED4 0 seeds, 1 nibble words; SEED4P4 0 seeds,
 * 1 coefficient words, 3 exponent codes (block g of the slice in nibble g&1 of byte g>>1). */
typedef struct {
    const void* p[4];
    int32_t eb;     /* seeds: the slice's exponent bias */
    int32_t gs;     /* Q8 / Q4: log2 of the affine group (5: 32, 6: 64); 0 is 64 */
    int32_t pad[2];
} WSlice;

typedef struct { /* engine/kernels_moe.metal:104-108 */
    int d, n, top_k;
    int hw;      /* router partition width (d / 2) */
    float scale; /* router_scaling_factor */
} RouterArgs;

typedef struct { int slice, start, count, pad; } MmTile; /* engine/kernels_moe.metal:130 */

/* the expert slot table (engine/kernels_cuda.h:32-48) */
typedef struct {
    int32_t* unit_slot;  /* [units]: slot, or -1 */
    int32_t* slot_unit;  /* [slots]: unit, or -1 */
    uint32_t* slot_last; /* [slots]: the admit tick of the last use */
    uint32_t* tick;      /* [4]: the admit tick (from CACHE_TICK_BASE), unused */
    uint32_t* stats;     /* [2]: hits, misses */
    int32_t* jobs;       /* [2 * per_layer]: (unit, slot) pairs queued by the last admit */
    int32_t* njobs;      /* [1] */
    uint8_t* vram;       /* the pool */
    const uint8_t* host; /* device address of the arena that holds every unit */
    uint64_t unit_bytes;
    int32_t slots, per_layer, ntens;
    WSlice* tab;         /* [sparse layer][ntens][per_layer] */
    uint32_t off[3][4];  /* byte offset of tensor i's stream s in a unit (0xFFFFFFFF: no stream) */
    uint64_t hits, misses;
} CachePool;
#define CACHE_TICK_BASE 0x40000000u
enum { CACHE_PROTECT_PREV = 2 };
#define CACHE_MAX_PER_LAYER 1024

/* ---- seed / affine / BF16 matvec family ------------------------------------------------------------------------- */
/* engine/kernels_cuda.h:78-79, engine/kernels_moe.cu:2308-2316.  Dense matvec, T <= MV_MAXT tokens:
 * y[t][r] = bf16(W[r] . x[t]), or with add: bf16(y + bf16(W[r] . x[t])).  Token t's rows do not depend on T. */
void kc_mv(kc_stream_t s, int fmt, WSlice w, int K, int R, const float* x, int xs, float* y, int ys, int T, int add,
           const uint32_t* G);
/* engine/kernels_cuda.h:81-82, engine/kernels_moe.cu:2317-2323.  Gather matvec over P (token, expert) pairs: pair p
 * uses slice sel[p] and input row p / xdiv. */
/* No counterpart in the reference (its hosts launch kc_mv once per matrix): n <= 4 dense seed matrices w[j] ([R[j]][K]) against
 * the same T <= 64 rows of x in ONE launch per 8 rows, y[j][t * ys[j] + r] (+)= as kc_mv writes it, bit for bit.  0, or -1 when the
 * shapes are outside the seed fast path (K % 64, K > 6144, unaligned x): nothing is launched, call kc_mv per matrix.
 * norm_w (f32 [K], K <= 4096) or NULL: the rows of x are normalised first, exactly as kq4_norm1p(x, K, K, norm_w, norm_eps) would
 * have stored them (each workgroup recomputes the row's scale; the launch of the norm is saved).
 * BF16 / Q8 / Q4 matrices (fmt as for kc_mv): the same in one launch for T <= MV_MAXT rows, K % 8 == 0, x 16-byte aligned,
 * without norm_w (-1 with it). */
int kc_mv_multi(kc_stream_t s, int fmt, int n, const WSlice* w, const int* R, float* const* y, const int* ys, const int* add, int K,
                const float* x, int xs, int T, const float* norm_w, float norm_eps);
void kc_mv_sel(kc_stream_t s, int fmt, const WSlice* ws, int K, int R, const float* x, int xs, float* y, int ys,
               const int32_t* sel, int P, int xdiv, const uint32_t* G);
/* engine/kernels_cuda.h:84-85, engine/kernels_moe.cu:2324-2328.  Routed experts' gate + up + SwiGLU in one pass:
 * a[p][r] = bf16(silu_bf(bf16(g . x)) * bf16(u . x)). */
void kc_mv_gu(kc_stream_t s, int fmt, const WSlice* wg, const WSlice* wu, int K, int R, const float* x, int xs, float* a,
              int ys, const int32_t* sel, int P, int xdiv, const uint32_t* G);

/* ---- prefill GEMM ------------------------------------------------------------------------------------------------- */
/* engine/kernels_cuda.h:95, engine/kernels_moe.cu:2354-2355: seed weights exact in f32 (three BF16 terms) instead of
 * rounded to BF16.  Process-global, as in the reference. */
void kc_seed_gemm_f32(int on);
/* engine/kernels_cuda.h:96-97, engine/kernels_moe.cu:2360-2364 */
void kc_mm(kc_stream_t s, int fmt, WSlice w, int K, int R, const float* x, int xs, float* y, int ys, int T, int add,
           const uint32_t* G);
/* engine/kernels_cuda.h:98-99, engine/kernels_moe.cu:2365-2372 */
void kc_mm_grouped(kc_stream_t s, int fmt, const WSlice* ws, int K, int R, const float* x, int xs, float* y, int ys,
                   int xdiv, const int32_t* perm, const MmTile* tiles, int ntiles, const uint32_t* G);
/* engine/kernels_cuda.h:103-108, engine/kernels_moe.cu:2373-2383, 2396-2399 */
#define BUCKET_MAX_EXPERTS 1024
void kc_bucket(kc_stream_t s, const int32_t* inds, int count, int n, int32_t* perm, MmTile* tiles, int32_t* ntiles);
void kc_mm_grouped_dev(kc_stream_t s, int fmt, const WSlice* ws, int K, int R, const float* x, int xs, float* y, int ys,
                       int xdiv, const int32_t* perm, const MmTile* tiles, const int32_t* ntiles, int max_tiles,
                       const uint32_t* G);
/* engine/kernels_cuda.h:110-114, engine/kernels_moe.cu:2384-2395 */
void kc_pack_input_bf16(kc_stream_t s, const float* x, uint16_t* y, size_t n);
void kc_mm_packed(kc_stream_t s, int fmt, WSlice w, int K, int R, const uint16_t* x, int xs, float* y, int ys, int T,
                  int add, const uint32_t* G);
void kc_mm_grouped_packed(kc_stream_t s, int fmt, const WSlice* ws, int K, int R, const uint16_t* x, int xs, float* y,
                          int ys, int xdiv, const int32_t* perm, const MmTile* tiles, const int32_t* nt, int max_tiles,
                          const uint32_t* G);
/* pairs per tile of the grouped GEMM: MmTile.count <= MMT_BN (engine/kernels_cuda.h:116) */
#define MMT_BN 128

/* ---- routers, elementwise ------------------------------------------------------------------------------------------ */
/* engine/kernels_cuda.h:120-123, engine/kernels_moe.cu:2400-2407: sigmoid scores, selection scores, top-k, weights */
void kc_router(kc_stream_t s, RouterArgs a, const uint16_t* W, const uint16_t* bias, const float* x, float* score,
               float* sel, int32_t* inds, float* wts, int T);
void kc_router_topk(kc_stream_t s, RouterArgs a, const float* score, const float* sel, int32_t* inds, float* wts, int T);
/* engine/kernels_qwen4.h:53-54, engine/kernels_qwen4.cu:417-422: softmax top-k (ties to the higher index), n_exp <= 1024,
 * top_k <= 32.  Qwen4Cfg is the reference's configuration struct (nslm/qwen4_cfg.h:9-26), layout-identical here; the
 * kernels read only n_exp and top_k. */
#define QWEN4_MAX_LAYERS 128
typedef struct {
    int n_layer, d, vocab, eos;
    int hc, hc_rank;
    int n_head, n_kv, head_dim, rot_dim;
    float rope_theta, eps;
    int ix_heads, ix_dim, ix_budget, ix_ratio;
    int lin_hk, lin_hv, lin_dk, lin_dv, lin_conv;
    int n_exp, top_k, ff_exp, ff_shared;
    int ple_dim, ple_conv, ngram, heads_per_ngram, ngram_parts;
    int64_t ngram_base, ngram_div, seed;
    uint8_t attn[QWEN4_MAX_LAYERS];
    int8_t ple[QWEN4_MAX_LAYERS];
} Qwen4Cfg;
void kq4_route(kc_stream_t s, const Qwen4Cfg* c, const float* logits, int32_t* ind, float* wt, int T);
void kq4_route_ld(kc_stream_t s, const Qwen4Cfg* c, const float* logits, int ld, int32_t* ind, float* wt, int T);
/* engine/kernels_cuda.h:124-125, engine/kernels_moe.cu:2408-2413 */
void kc_swiglu(kc_stream_t s, const float* g, const float* u, float* a, int n);
/* kc_swiglu + kc_pack_input_bf16 in one pass (no counterpart in the reference): y = the BF16 bits of kc_swiglu's values,
 * n % 8 == 0, g / u / y 16-byte aligned, y distinct from g and u */
void kc_swiglu_pack(kc_stream_t s, const float* g, const float* u, uint16_t* y, size_t n);
/* The batched step's first two launches folded (no counterpart in the reference, which routes, packs and groups in four):
 * kc_mv_pack = kc_mv of a BF16 / Q8 / Q4 matrix (add = 0) for up to 64 rows in ONE launch, on the rows rounded to BF16 as the
 * GEMM it stands in for multiplies them (engine/kernels_moe.cu:455-470; kc_mv's row sums over those values), that also
 * leaves the rows' BF16 view px [T][K] (kc_pack_input_bf16's bits) for the GEMMs that follow; returns -1 (nothing launched)
 * where kc_mv would not take its wave-a-row path (K % 8, x or px not 16-byte aligned, xs % 4, K > 4096 rows' worth of LDS).
 * kq4_route_bucket = kq4_route + kc_bucket in one launch: ind / wt as kq4_route's, perm / tiles / ntiles as kc_bucket's for
 * count = T * top_k; ntiles holds 2 * n_exp + 4 ints here, the last one zero before the first call (the launch leaves it zero). */
int kc_mv_pack(kc_stream_t s, int fmt, WSlice w, int K, int R, const float* x, int xs, float* y, int ys, int T, uint16_t* px);
void kq4_route_bucket(kc_stream_t s, const Qwen4Cfg* c, const float* logits, int32_t* ind, float* wt, int T, int32_t* perm,
                      MmTile* tiles, int32_t* ntiles);
void kc_moe_combine(kc_stream_t s, const float* D, const float* w, const float* shared, float* x, int d, int k, int T);
/* engine/kernels_qwen4.h:71, engine/kernels_qwen4.cu:514-516 */
void kq4_moe_combine(kc_stream_t s, int d, int k, const float* D, const float* wt, const float* sh, const float* sg,
                     int sgld, float* out, int T);

/* ---- expert slot table (engine/kernels_cuda.h:53-55, engine/kernels_moe.cu:2710-2722) ------------------------------ */
void kc_cache_admit(kc_stream_t s, const CachePool* p, int sl, const int32_t* inds, int count, int flags);
void kc_cache_copy(kc_stream_t s, const CachePool* p, int blocks);

/* ---- weights to BF16 in memory (engine/kernels_cuda.h:161, engine/kernels_moe.cu:2441-2444) ------------------------
 * A per-head map [H][O][I] in fmt decoded to BF16 bits: SEED4P4 with W.p = seeds, coefficients, exponent biases [H]
 * (int32, device), exponent codes; Q8 / Q4 as bf16(scale * code + bias). */
void kc_heads_deq(kc_stream_t s, int fmt, WSlice W, const uint32_t* G, int H, int O, int I, uint16_t* out);

/* ---- additions of this backend (no counterpart in the reference) --------------------------------------------------- */
/* Rows [0,R) of one slice of any format decoded to BF16 bits [R][K] (seeds with the slice's own eb; SEED4 too):
 * the bit-exact weight regeneration check. */
void kc_slice_deq(kc_stream_t s, int fmt, WSlice w, int K, int R, uint16_t* out);
/* kc_mm_grouped_packed for a caller that knows an upper bound of MmTile.count: a decode step of T rows chooses no expert
 * more than T times, so no tile holds more than tile_rows = T pairs.  Up to 32 the launch uses workgroups with one
 * multiplying wave (four a CU instead of two; the tiles are decode-bound).  The bound is a promise: pairs of a tile beyond
 * it are not computed, and their results are stored as NaN so that a broken promise shows.  tile_rows < 1 or > 32: as kc_mm_grouped_packed. */
void kc_mm_grouped_packed_rows(kc_stream_t s, int fmt, const WSlice* ws, int K, int R, const uint16_t* x, int xs, float* y,
                               int ys, int xdiv, const int32_t* perm, const MmTile* tiles, const int32_t* nt, int max_tiles,
                               int tile_rows);
/* Two grouped GEMMs of one shape over the same tiles and activations in one launch (an expert's gate and up matrices: ya = the
 * ws_a slices' product, yb = the ws_b slices'), each bit for bit what kc_mm_grouped_packed_rows gives alone: one launch's ramp
 * and tail instead of two.  No counterpart in the reference (two launches, engine/mova_cuda.c:1308-1311). */
void kc_mm_grouped_packed_pair(kc_stream_t s, int fmt, const WSlice* ws_a, const WSlice* ws_b, int K, int R, const uint16_t* x, int xs,
                               float* ya, float* yb, int ys, int xdiv, const int32_t* perm, const MmTile* tiles, const int32_t* nt,
                               int max_tiles, int tile_rows);
/* The gate GEMM, the up GEMM and kc_swiglu_pack in one launch: a workgroup's 64 weight rows are 32 gate rows and the same 32 up
 * rows of the tile's expert, so a lane holds both sums of a (pair, row) and stores a16[pair][row] = the BF16 bits kc_swiglu_pack
 * would have stored from the two GEMMs' outputs (bit for bit).  R = the expert width, ys = a16's row stride.  -1 (nothing
 * launched) where kc_mm_grouped_packed would not take its streamed kernel (K % 64, alignment) or kc_store_f32(1) is set.
 * No counterpart in the reference (three launches, engine/mova_cuda.c:1308-1312). */
int kc_mm_grouped_swiglu(kc_stream_t s, int fmt, const WSlice* gate, const WSlice* up, int K, int R, const uint16_t* x, int xs, uint16_t* a16,
                         int ys, int xdiv, const int32_t* perm, const MmTile* tiles, const int32_t* nt, int max_tiles, int tile_rows);
/* 1: the matvec family stores unrounded f32 instead of BF16-rounded values (for comparison with CPU references that do
 * not round, nslm/lib_cpu_seed4.c).  Process-global like kc_seed_gemm_f32; default 0 = the reference's store. */
void kc_store_f32(int on);
/* ---- the small kernels either side of the seed matmuls in a full decode step ------------------------------------------ */
/* engine/kernels_cuda.h:74-75, engine/kernels_moe.cu:676-692,2302-2304.  x[t][:] = the embedding row ids[t] of w as BF16
 * values: BF16, Q8, Q4 (bf16(s q + b)) and, as tests/kernel_backend.h:141-142 asks of a backend, seed rows (the BF16-rounded
 * exact weights).  d % 8 == 0. */
void kc_embed(kc_stream_t s, int fmt, WSlice w, int d, const int32_t* ids, float* x, int T);
/* engine/kernels_cuda.h:76-77, engine/kernels_moe.cu:694-713.  Grouped RMSNorm, 2 groups of d / 2:
 * y = bf16(w * (x * rsqrt(mean_group(x^2) + eps))), w BF16 [d]. */
void kc_gnorm(kc_stream_t s, int d, float eps, const float* x, const uint16_t* w, float* y, int T);
/* engine/kernels_qwen4.h:24-25, engine/kernels_qwen4.cu:205-236 (nslm/lib_qwen4_ops.c:11-18).  y[t] = x r (1 + w) per
 * group of g values of a row of len (g == len: the plain RMSNorm of a full model), f32 weights, no rounding; y may be x. */
void kq4_norm1p(kc_stream_t s, const float* x, int len, int g, const float* w, float eps, float* y, int T);
/* engine/kernels_cuda.h:177-178, engine/kernels_moe.cu:2115-2151,2714-2719.  Greedy arg-max of n rows of V logits (ties:
 * the lowest index), and with its softmax probability 1 / sum exp(l - max). */
void kc_argmax(kc_stream_t s, const float* logits, int32_t* out, int V, int n);
void kc_argmax_p(kc_stream_t s, const float* logits, int32_t* out, float* prob, int V, int n);

/* ---- decode attention over a latent KV cache (absorbed MLA) ------------------------------------------------------------ */
/* The KV cache view, engine/kernels_cuda.h:57-72: per layer, positions [0, nv) in segment a and [nv, ...) in segment b
 * (row 0 of b = position nv).  MLA: k holds the RoPE key, v the latent; BF16 (u16 values), or FP8 (nslm/kvq.h: E4M3 codes
 * in k / v, one E8M0 scale byte per 32 values in ks / vs).  KV_Q8 and KV_FP4 are not built (the launchers refuse them). */
enum { KV_BF16 = 0, KV_Q8 = 1, KV_FP8 = 2, KV_FP4 = 3 };
typedef struct {
    void* k;
    void* v;
    float* ks; /* FP8: the block scale bytes [rows][n / 32] */
    float* vs;
} KvSeg;
typedef struct {
    KvSeg a, b;
    int32_t nv, fmt;
} KvView;
typedef struct { int pos, kv0; int pad[2]; } RowInfo; /* kv0: the cache row of the sequence slot's position 0 (kernels_moe.metal:86) */
#define ATT_HD 128
/* engine/kernels_moe.metal:100-104.  chunk: target keys per split; each row splits its own 0..pos into
 * min(n_splits, ceil((pos + 1) / chunk)) parts.  pad[0] (ours; the reference leaves it 0): the RoPE key's width, 64 or 128,
 * 0 = 128 (the reference hard-codes ATT_HD).  pad[2] > 0: at most 32 splits, as the reference's one-pass kernel takes it. */
typedef struct {
    int n_head, r, chunk, n_splits;
    float scale;
    int pad[3];
} MlaArgs;
/* per-head maps, engine/kernels_moe.metal:112-115: y[t][h][o] = W_h[o] . x[t * xs + h * hs ..] */
typedef struct {
    int H, O, I, xs, hs, gate;
    int pad[2];
} HmvArgs;
/* engine/kernels_cuda.h:136-142, engine/kernels_moe.cu:1147-1176,2437-2440.  y[t][h][o] = bf16(W_h[o] . x), with g (y's layout)
 * bf16(that * bf16(softplus_ln2(g))).  W stacked [H][O][I] in fmt; SEED4P4 takes head h's exponent bias from W.p[2][h]. */
void kc_heads_mv(kc_stream_t s, HmvArgs a, int fmt, WSlice W, const uint32_t* G, const float* x, const float* g, float* y, int T);
/* engine/kernels_cuda.h:154-156, engine/kernels_moe.cu:1177-1208.  RoPE of the query RoPE parts qr [T][n_head][rope] (in place,
 * BF16-rounded) and of kr [T][rope] into kv.k; the latent c [T][r] into kv.v, at cache row ri[t].kv0 + ri[t].pos. */
void kc_mla_rope(kc_stream_t s, MlaArgs a, float* qr, const float* kr, const float* c, KvView kv, const RowInfo* ri,
                 const float* inv, int T);
/* engine/kernels_cuda.h:157-161, engine/kernels_moe.cu:1217-1323,2459-2489.  olat[t][h] = bf16(sum_p softmax_p(scale (ql_th .
 * c_p + qr_th . k_p)) c_p) over p <= pos_t; n_splits > 1 splits the keys (partials in part: T x n_head x n_splits x (r + 2)
 * floats) and reduces.  r % 8 == 0, r <= 1024.  (r = 512, rope = 64: the matrix-core kernel, a workgroup a (split, 16 heads, row); a
 * launch of at most 256 such workgroups runs two groups of four waves a workgroup over a split's keys and uses 149 KB of LDS a workgroup.) */
/* No counterpart in the reference (three launches there): kc_heads_mv(hq: query -> RoPE mix, O = rope) + kc_heads_mv(hl: query
 * -> latent, O = r) + kc_mla_rope in ONE launch, the same bits.  Both maps in fmt over the same query rows (equal I, xs, hs, no
 * gate).  0, or -1 when the shapes are outside it (r % 64, I / 8 not a power of two <= 64 ...): nothing is launched. */
int kc_mla_qmaps_rope(kc_stream_t s, MlaArgs a, HmvArgs hq, HmvArgs hl, int fmt, WSlice Wq, WSlice Wl, const float* q, float* qr, float* ql,
                      const float* kr, const float* c, KvView kv, const RowInfo* ri, const float* inv, int T);
void kc_mla_attn(kc_stream_t s, MlaArgs a, const float* ql, const float* qr, KvView kv, const RowInfo* ri, float* part,
                 float* olat, int T);
/* No counterpart in the reference: kc_mla_attn (n_splits >= 2) followed by kc_heads_mv(hv: latent -> value, I = r) with the
 * splits' reduce and the map in one launch; y[t][h][o] gets the same bits as the two calls write.  0, or -1 (nothing launched). */
int kc_mla_attn_vup(kc_stream_t s, MlaArgs a, const float* ql, const float* qr, KvView kv, const RowInfo* ri, float* part, HmvArgs hv, int fmt,
                    WSlice W, float* y, int T);
/* engine/kernels_cuda.h:173-176.  y[i] = value i of `rows` cache rows of n values in fmt (KV_BF16 / KV_FP8): the decode the
 * attention reads, for tests */
void kc_kv_f32(kc_stream_t s, int fmt, const uint8_t* codes, const uint8_t* scales, int n, int rows, float* y);

/* ---- additions for a host that runs a whole synthetic model (no counterpart in the reference's header) -------------------- */
/* x = bf16(x + bf16(a + b)) (b may be NULL): the residual stream takes a block's branch outputs, BF16 at the boundary */
void kc_residual_add(kc_stream_t s, float* x, const float* a, const float* b, size_t n);
/* ri[t].pos += 1 for t < T: positions live on the device so that a captured decode step replays.  ri[t].pad[0] > 0 is the
 * length of the row's cache slot: the position saturates at pad[0] - 1 (0: no bound, the reference's RowInfo leaves it 0) */
void kc_rows_advance(kc_stream_t s, RowInfo* ri, int T);
/* reproducible pseudo-random fills for synthetic packs: bytes (any bytes are valid seed records; nbytes rounded down to 8),
 * and BF16 values uniform in [-scale, scale] */
void kc_fill_random(kc_stream_t s, void* p, size_t nbytes, uint64_t seed);
void kc_fill_bf16(kc_stream_t s, uint16_t* p, size_t n, uint64_t seed, float scale);
void kc_fill_fp8_codes(kc_stream_t s, void* p, size_t nbytes, uint64_t seed);   /* random E4M3 codes the cache's encoder can write (no 0x7F / 0xFF) */

/* A whole routed-expert decode step for T <= kc_moe_decode_max_rows() tokens in ONE persistent kernel: router logits bf16(W x) on a BF16
 * router weight [n_exp][d], softmax top-k, gate + up + SwiGLU gather, down gather, out[t] = sum_j wt_j y_j - the same
 * bits as kc_mv(MF_BF16) + kq4_route + kc_mv_gu + kc_mv_sel + kq4_moe_combine(sh = 0), without the four launch gaps.
 * Scratch (caller-owned device memory): logits [T][n_exp], ind / wt [T][top_k] (the routing, also an output), A [T*k][ff],
 * D [T*k][d], sync: kc_moe_decode_sync_words(T, d) uint32 that must be zero before the first call (the kernel keeps them
 * consistent from launch to launch; sync[kc_moe_decode_error_word()] != 0 afterwards reports a wait between workgroups that gave up,
 * after which the caller must zero sync again).
 * The grid spans the whole device and its workgroups wait for each other: nothing else may run on the GPU beside it.
 * Up to MV_MAXT tokens every (token, expert) pair is a pass of its own (the reference's decode composition, bit for bit);
 * above that and up to kc_moe_decode_max_rows() the pairs of one expert share each decoded block, two at a time, with
 * the same per-token arithmetic (exact weights, the row-sum order of kc_mv_sel) - where the reference switches to its grouped
 * GEMM on BF16-rounded weights (engine/mova_cuda.c:1308-1317), so results there differ from the GEMM path's by that rounding
 * (shapes whose gate+up row sums do not fit a wave shuffle are refused above MV_MAXT tokens: the grouped GEMMs are faster there).
 * Returns 0, or -1 when the shape has no fused kernel (nothing launched: use the separate launchers). */
size_t kc_moe_decode_sync_words(int T, int d);
int kc_moe_decode_max_rows(void);
int kc_moe_decode_error_word(void);
/* polls a wait between workgroups makes before it gives up (0: the default, 2^21 - seconds).  A host that shares the GPU
 * between streams may want a shorter bound; tests set a tiny one to drive the error path while every kernel still exits. */
void kc_moe_decode_spin_limit(unsigned polls);
/* Which of the library's two persistent kernels a step of up to MV_MAXT tokens takes (the same bits either way): 0 (default) the
 * one with a workgroup per CU at 1 token, and at 2 where it measured faster (the format P = 3, or the 64-weight chunks of a hidden row a power of two <= 32 and top_k * d * ff >= 24 Mi) where the shape fits it (T * pairs * ff <= 65536, T * n_exp <= 1024, the tokens' staged inputs within
 * a CU's LDS), else the one with a workgroup per (pair, row tile); 1 always the latter; 2 the former wherever the shape fits
 * it.  Process-global, for comparisons. */
void kc_moe_decode_kernel(int which);
int kc_moe_decode(kc_stream_t s, int fmt, const uint16_t* router_w, const WSlice* gate, const WSlice* up, const WSlice* down,
                  int n_exp, int top_k, int d, int ff, const float* x, int xs, int T, float* out, int os, float* logits,
                  int32_t* ind, float* wt, float* A, float* D, uint32_t* sync);
/* kc_moe_decode with the rest of the layer's expert block folded in (no counterpart in the reference, which runs the shared
 * expert as kc_mv_gu + kc_mv on a second stream and adds the residual in its combine, engine/qwen4_cuda.c:1026-1083).
 * shared (host pointer to 3 slices: gate [ff][d], up [ff][d], down [d][ff]) or NULL: an always-on expert of the routed experts'
 * shape, pair top_k of every token with weight 1.  res or NULL: out = bf16(res + bf16(sum)), res may be out.  A and D then
 * hold T * (top_k + 1) rows.  norm_w (f32 [d], d <= 4096) or NULL: x is normalised first, as kq4_norm1p(x, d, d, norm_w, norm_eps)
 * would have stored it (res stays the raw stream).  Same results as the separate launches: sum = f32 sum_j wt_j bf16(y_j) +
 * bf16(y_shared).  With a shared expert the expert-sharing form of the kernel is used from 5 tokens on (every token brings a
 * pair on that expert); the rows are the same bits either way. */
int kc_moe_decode_layer(kc_stream_t s, int fmt, const uint16_t* router_w, const WSlice* gate, const WSlice* up, const WSlice* down,
                        int n_exp, int top_k, int d, int ff, const float* x, int xs, int T, float* out, int os, float* logits,
                        int32_t* ind, float* wt, float* A, float* D, uint32_t* sync, const WSlice* shared, const float* res, const float* norm_w,
                        float norm_eps);
/* kc_moe_decode without a workspace argument.  No counterpart in the reference: it is for callers that cannot allocate device
 * memory or carry a workspace around - code under stream capture, tight serving loops, harnesses that forbid hipMalloc.  What
 * kc_moe_decode's caller owns as scratch (logits, A, D, the sync words) lives in one array inside the library's code object
 * (5.3 MB of device memory on every GPU the library runs on, held until the process ends); the call allocates and frees nothing.
 * ind / wt [T][top_k] (the routing) and out stay the caller's.  Results: kc_moe_decode's, bit for bit.
 * status (device, 4 bytes) or NULL: receives the error word after the step (non-zero: a wait between workgroups gave up, the
 * results are void) - one more one-thread launch.  clear != 0: the sync words are zeroed first (a fill kernel on s); needed
 * only after such an error.
 * Limits: T <= kc_moe_decode_max_rows(); T * n_exp + T * top_k * (ff + d) floats (each part rounded up to 64) <= 2^20;
 * T * ceil(d / (256 / (ff / 64))) <= 24576.  Returns 0; -1 as kc_moe_decode (no fused kernel for the shape, nothing launched);
 * -2 the shape is beyond the limits above (nothing launched, kc_last_error() reports an invalid value); -3 the array's address
 * could not be obtained on the current device.
 * All calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams, two threads) race - serialise them.
 * The first call on a device looks the address up (hipGetSymbolAddress): make it outside a capture. */
int kc_moe_decode_static(kc_stream_t s, int fmt, const uint16_t* router_w, const WSlice* gate, const WSlice* up, const WSlice* down,
                         int n_exp, int top_k, int d, int ff, const float* x, int xs, int T, float* out, int os, int32_t* ind, float* wt,
                         uint32_t* status, int clear);
/* last launch-configuration error of this library on the calling thread's device: 0 none, else a hipError_t value */
int kc_last_error(void);

#ifdef __cplusplus
}
#endif
