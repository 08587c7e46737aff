// nslm_misc.hip - the small kernels around the seed matmuls: both routers, SwiGLU, the two MoE combines, pair grouping
// for the grouped GEMM, the expert slot table, weights-to-BF16, and the BF16 input pack.  Wave64 throughout.
// Reference kernels: engine/kernels_moe.cu:527-573 (bucket), 717-788 (router, swiglu, combine), 1325-1335 (heads_deq),
// 2025-2112 (slot table), 2196-2201 (input pack); engine/kernels_qwen4.cu:385-416 (softmax route), 506-515 (combine).
#include "nslm_dev.h"

using namespace nslm;

namespace {

__device__ __forceinline__ float wave_sum(float v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
#define NEG_INF __uint_as_float(0xFF800000u)

// ---- sigmoid router: one wave per (expert, token) ---------------------------------------------------------------------
// logits as two partial sums over [0,hw) and [hw,d), each rounded to BF16 before the add (the model's two-partition
// router), sigmoid, selection score = sigmoid + bias.
__global__ void __launch_bounds__(256) k_router_logits(RouterArgs a, const uint16_t* W, const uint16_t* bias, const float* x,
                                                       float* score, float* selout) {
    const int lane = threadIdx.x & 63, e = (int) blockIdx.x * 4 + (threadIdx.x >> 6), t = (int) blockIdx.y;
    if (e >= a.n) return;
    const float* xr = x + (size_t) t * a.d;
    const uint16_t* wr = W + (size_t) e * a.d;
    float s0 = 0.0f, s1 = 0.0f;
    for (int c = lane * 4; c < a.d; c += 256) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (c + i >= a.d) break;
            const float v = bf(wr[c + i]) * xr[c + i];
            if (c + i < a.hw) s0 += v;
            else s1 += v;
        }
    }
    s0 = wave_sum(s0);
    s1 = wave_sum(s1);
    if (lane == 0) {
        const float sg = 1.0f / (1.0f + expf(-(bfr(s0) + bfr(s1))));
        score[(size_t) t * a.n + e] = sg;
        selout[(size_t) t * a.n + e] = sg + bf(bias[e]);
    }
}
// k rounds of a wave arg-max over the selection scores (ties to the lowest expert id), weights = score / sum * scale.
// n <= 1024 experts (16 a lane), top_k <= 32.
#define RT_PER 16
__global__ void __launch_bounds__(64) k_router_topk(RouterArgs a, const float* score, const float* sel, int32_t* inds, float* wts) {
    const int t = (int) blockIdx.x, lane = threadIdx.x;
    const float* sc = score + (size_t) t * a.n;
    const float* se = sel + (size_t) t * a.n;
    float v[RT_PER];
#pragma unroll
    for (int j = 0; j < RT_PER; ++j) v[j] = lane + 64 * j < a.n ? se[lane + 64 * j] : NEG_INF;
    int mine = 0;          // round r's winner is kept by lane r (top_k <= 32)
    float mine_sc = 0.0f, sum = 0.0f;
    for (int k = 0; k < a.top_k; ++k) {
        float bv = NEG_INF;
        int bi = 1 << 20;
#pragma unroll
        for (int j = 0; j < RT_PER; ++j) {   // ascending ids: strict > keeps the lowest id of equal values
            const int e = lane + 64 * j;
            if (e < a.n && (v[j] > bv || bi == (1 << 20))) { bv = v[j]; bi = e; }
        }
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o);
            const int oi = __shfl_xor(bi, o);
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
#pragma unroll
        for (int j = 0; j < RT_PER; ++j)
            if (lane + 64 * j == bi) v[j] = NEG_INF;
        const float s = sc[bi];
        sum += s;
        if (lane == k) { mine = bi; mine_sc = s; }
    }
    if (lane < a.top_k) {
        inds[t * a.top_k + lane] = mine;
        wts[t * a.top_k + lane] = mine_sc / sum * a.scale;
    }
}

// ---- softmax router: top k by logit (ties to the HIGHER index), weights = softmax renormalised over the k picked ------
// Round r's winner is kept by lane r (k <= 32 < 64 lanes), so nothing is indexed dynamically.
__global__ void __launch_bounds__(64) k_q4_route(int E, int k, const float* logits, int ld, int32_t* ind, float* wt) {
    const int t = (int) blockIdx.x, lane = threadIdx.x;
    const float* l = logits + (size_t) t * ld;
    float v[RT_PER], mx = NEG_INF, top = 0.0f, mine = 0.0f;
    int mine_id = 0;
#pragma unroll
    for (int j = 0; j < RT_PER; ++j) {
        v[j] = lane + 64 * j < E ? l[lane + 64 * j] : NEG_INF;
        mx = fmaxf(mx, v[j]);
    }
    mx = wave_max(mx);
    for (int r = 0; r < k; ++r) {
        float bv = NEG_INF;
        int bi = -1;
#pragma unroll
        for (int j = 0; j < RT_PER; ++j) {
            const int e = lane + 64 * j;
            if (e < E && (v[j] > bv || (v[j] == bv && e > bi))) { bv = v[j]; bi = e; }
        }
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o);
            const int oi = __shfl_xor(bi, o);
            if (ov > bv || (ov == bv && oi > bi)) { bv = ov; bi = oi; }
        }
#pragma unroll
        for (int j = 0; j < RT_PER; ++j)
            if (lane + 64 * j == bi) v[j] = NEG_INF;
        const float w = expf(bv - mx);
        top += w;
        if (lane == r) { mine = w; mine_id = bi; }
    }
    if (lane < k) {
        ind[(size_t) t * k + lane] = mine_id;
        wt[(size_t) t * k + lane] = mine / top;
    }
}

// ---- elementwise --------------------------------------------------------------------------------------------------------
__global__ void k_swiglu(const float* g, const float* u, float* a, int n) {
    const int i = (int) (blockIdx.x * blockDim.x + threadIdx.x);
    if (i < n) a[i] = bfr(silu_bf(g[i]) * u[i]);
}
// the same values as BF16 bits (they are BF16 values already), eight a thread: k_swiglu + k_pack_input_bf16 in one pass for
// the GEMMs that take a BF16 view of their activations
__global__ void k_swiglu_pack(const float* g, const float* u, uint16_t* y, size_t n) {
    const size_t b = (size_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= n / 8) return;
    const float4 g0 = ((const float4*) g)[2 * b], g1 = ((const float4*) g)[2 * b + 1];
    const float4 u0 = ((const float4*) u)[2 * b], u1 = ((const float4*) u)[2 * b + 1];
    ((uint4*) y)[b] = make_uint4(pack_bf2(bfr(silu_bf(g0.x) * u0.x), bfr(silu_bf(g0.y) * u0.y)),
                                 pack_bf2(bfr(silu_bf(g0.z) * u0.z), bfr(silu_bf(g0.w) * u0.w)),
                                 pack_bf2(bfr(silu_bf(g1.x) * u1.x), bfr(silu_bf(g1.y) * u1.y)),
                                 pack_bf2(bfr(silu_bf(g1.z) * u1.z), bfr(silu_bf(g1.w) * u1.w)));
}
// x[t][c] = bf16(x + bf16(bf16(sum_j bf16(D[t,j][c] * bf16(w[t,j]))) + shared[t][c]))
__global__ void k_moe_combine(const float* D, const float* w, const float* shared, float* x, int d, int k) {
    const int c = (int) (blockIdx.x * blockDim.x + threadIdx.x), t = (int) blockIdx.y;
    if (c >= d) return;
    float s = 0.0f;
    for (int j = 0; j < k; ++j) s += bfr(D[((size_t) t * k + j) * d + c] * bfr(w[t * k + j]));
    const size_t i = (size_t) t * d + c;
    x[i] = bfr(x[i] + bfr(bfr(s) + shared[i]));
}
// out[t][i] = sigmoid(sg[t * sgld]) * sh[t][i] + sum_j wt[t][j] D[t,j][i], all f32
__global__ void k_q4_moe_combine(int d, int k, const float* D, const float* wt, const float* sh, const float* sg, int sgld, float* out) {
    const int i = (int) (blockIdx.x * blockDim.x + threadIdx.x), t = (int) blockIdx.y;
    if (i >= d) return;
    float acc = (1.0f / (1.0f + expf(-sg[(size_t) t * sgld]))) * sh[(size_t) t * d + i];
    for (int j = 0; j < k; ++j) acc = fmaf(wt[t * k + j], D[((size_t) t * k + j) * d + i], acc);
    out[(size_t) t * d + i] = acc;
}
__global__ void k_pack_input_bf16(const float* x, uint16_t* y, size_t n) {
    const size_t b = (size_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= n / 8) return;
    const float4 a = ((const float4*) x)[2 * b], c = ((const float4*) x)[2 * b + 1];
    ((uint4*) y)[b] = make_uint4(pack_bf2(a.x, a.y), pack_bf2(a.z, a.w), pack_bf2(c.x, c.y), pack_bf2(c.z, c.w));
}

// ---- grouping: selections -> pair ids by expert (ascending inside an expert), tiles of <= MMT_BN pairs ----------------
// work (= the ntiles buffer, 2n + 3 ints): [0] tile count, [1 .. n+1] pair offsets, [n+2 .. 2n+2] tile offsets.
__global__ void __launch_bounds__(1024) k_bucket_count(const int32_t* inds, int count, int n, int32_t* work) {
    __shared__ int cnt[BUCKET_MAX_EXPERTS];
    for (int x = threadIdx.x; x < n; x += 1024) cnt[x] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < count; i += 1024) atomicAdd(&cnt[inds[i]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int o = 0, to = 0;
        for (int x = 0; x < n; ++x) {
            work[1 + x] = o;
            work[2 + n + x] = to;
            o += cnt[x];
            to += (cnt[x] + MMT_BN - 1) / MMT_BN;
        }
        work[1 + n] = o;
        work[2 + 2 * n] = to;
        work[0] = to;
    }
}
// one workgroup per expert: an ordered compaction of its pairs (wave ballots + a prefix over the 16 waves)
__global__ void __launch_bounds__(1024) k_bucket_place(const int32_t* inds, int count, const int32_t* work, int32_t* perm, MmTile* tiles) {
    __shared__ int wcount[16];
    const int x = (int) blockIdx.x, n = (int) gridDim.x, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    int base = work[1 + x];
    for (int c0 = 0; c0 < count; c0 += 1024) {
        const int i = c0 + tid;
        const bool hit = i < count && inds[i] == x;
        const unsigned long long m = __ballot(hit);
        if (lane == 0) wcount[wv] = __popcll(m);
        __syncthreads();
        int before = 0, total = 0;
        for (int k = 0; k < 16; ++k) {
            if (k < wv) before += wcount[k];
            total += wcount[k];
        }
        if (hit) perm[base + before + __popcll(m & ((1ull << lane) - 1ull))] = i;
        base += total;
        __syncthreads();
    }
    const int o = work[1 + x], cnt = work[2 + x] - o, t0 = work[2 + n + x];
    for (int t = tid; t * MMT_BN < cnt; t += 1024) {
        MmTile tl;
        tl.slice = x;
        tl.start = o + t * MMT_BN;
        tl.count = min(MMT_BN, cnt - t * MMT_BN);
        tl.pad = 0;
        tiles[t0 + t] = tl;
    }
}

// ---- expert slot table --------------------------------------------------------------------------------------------------
// One workgroup, one thread per expert of the layer.  Hits take the new tick; misses, in expert order, take the least
// recently used slot that this call (and, with CACHE_PROTECT_PREV, the previous one) did not touch, ties to the lowest
// slot index; the unit's slice tables are pointed at the slot and a (unit, slot) copy job is queued.  With every expert
// resident (slots == units, as on a 288 GB GPU) there are no misses and the loop below never runs.
__global__ void __launch_bounds__(CACHE_MAX_PER_LAYER) k_cache_admit(CachePool p, int sl, const int32_t* inds, int count, int flags) {
    __shared__ int need[CACHE_MAX_PER_LAYER];
    __shared__ int miss[CACHE_MAX_PER_LAYER];
    __shared__ int wmiss[16], wneed[16];
    __shared__ unsigned int bestv[16];
    __shared__ int besti[16];
    __shared__ int nmiss, victim;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const uint32_t prev_tick = p.tick[0], now = prev_tick + 1;
    const bool protect = (flags & CACHE_PROTECT_PREV) != 0;
    need[tid] = 0;
    __syncthreads();
    for (int i = tid; i < count; i += CACHE_MAX_PER_LAYER) need[inds[i]] = 1;
    __syncthreads();
    const bool isneed = tid < p.per_layer && need[tid];
    const int s0 = isneed ? p.unit_slot[sl * p.per_layer + tid] : -1;
    const bool ismiss = isneed && s0 < 0;
    if (isneed && s0 >= 0) p.slot_last[s0] = now;
    const unsigned long long mb = __ballot(ismiss), nb = __ballot(isneed);
    if (lane == 0) { wmiss[wv] = __popcll(mb); wneed[wv] = __popcll(nb); }
    __syncthreads();
    if (ismiss) {
        int before = __popcll(mb & ((1ull << lane) - 1ull));
        for (int k = 0; k < wv; ++k) before += wmiss[k];
        miss[before] = tid;
    }
    if (tid == 0) {
        int nm = 0, nn = 0;
        for (int k = 0; k < 16; ++k) { nm += wmiss[k]; nn += wneed[k]; }
        nmiss = nm;
        p.tick[0] = now;
        p.stats[1] += (uint32_t) nm;
        p.stats[0] += (uint32_t) (nn - nm);
        *p.njobs = nm;
    }
    __syncthreads();
    const int total = nmiss;
    for (int m = 0; m < total; ++m) {
        uint32_t best = 0xFFFFFFFFu;
        int bs = 0x7FFFFFFF;
        for (int s = tid; s < p.slots; s += CACHE_MAX_PER_LAYER) {   // ascending s: strict < keeps the lowest index
            const uint32_t l = p.slot_last[s];
            if (l != now && !(protect && l == prev_tick) && l < best) { best = l; bs = s; }
        }
        for (int o = 32; o > 0; o >>= 1) {
            const uint32_t b2 = __shfl_xor(best, o);
            const int s2 = __shfl_xor(bs, o);
            if (b2 < best || (b2 == best && s2 < bs)) { best = b2; bs = s2; }
        }
        if (lane == 0) { bestv[wv] = best; besti[wv] = bs; }
        __syncthreads();
        if (tid == 0) {
            for (int i = 1; i < 16; ++i)
                if (bestv[i] < best || (bestv[i] == best && besti[i] < bs)) { best = bestv[i]; bs = besti[i]; }
            victim = bs < p.slots ? bs : -1;
            if (victim >= 0) {
                const int x = miss[m], u = sl * p.per_layer + x, old = p.slot_unit[bs];
                if (old >= 0) p.unit_slot[old] = -1;
                p.slot_unit[bs] = u;
                p.unit_slot[u] = bs;
                p.slot_last[bs] = now;
                p.jobs[2 * m] = u;
                p.jobs[2 * m + 1] = bs;
                uint8_t* base = p.vram + (uint64_t) bs * p.unit_bytes;
                for (int i = 0; i < p.ntens; ++i) {
                    WSlice* t = p.tab + ((size_t) sl * p.ntens + i) * p.per_layer + x;
                    for (int st = 0; st < 4; ++st)
                        if (p.off[i][st] != 0xFFFFFFFFu) t->p[st] = base + p.off[i][st];
                }
            } else {
                *p.njobs = m;   // nothing may be replaced (a pool smaller than two layers): stop admitting
            }
        }
        __syncthreads();   // also orders tid 0's slot_last update before the next scan
        if (victim < 0) break;
    }
}
// the queued units, arena -> pool slots, 16 bytes per thread per step
__global__ void __launch_bounds__(512) k_cache_copy(CachePool p) {
    const int nj = *p.njobs;
    const uint64_t words = p.unit_bytes / 16, stride = (uint64_t) gridDim.x * blockDim.x;
    for (int j = 0; j < nj; ++j) {
        const uint4* src = (const uint4*) (p.host + (uint64_t) p.jobs[2 * j] * p.unit_bytes);
        uint4* dst = (uint4*) (p.vram + (uint64_t) p.jobs[2 * j + 1] * p.unit_bytes);
        for (uint64_t i = (uint64_t) blockIdx.x * blockDim.x + threadIdx.x; i < words; i += stride) dst[i] = src[i];
    }
}

// ---- weights to BF16 bits: one thread per 8-weight block ---------------------------------------------------------------
// heads: W.p[2] holds an int32 exponent bias per head (SEED4P4 per-head maps); otherwise the slice's own eb.
__global__ void __launch_bounds__(256) k_deq(int fmt, WSlice W, int rows_per_head, int K, int nblocks, int heads, uint16_t* out) {
    __shared__ uint32_t tab[NSLM_TAB_WORDS];
    load_tables(tab);
    __syncthreads();
    const int b = (int) (blockIdx.x * blockDim.x + threadIdx.x);
    if (b >= nblocks) return;
    const int nbk = K / 8, row = b / nbk;
    float o[8];
    if (fmt == MF_SEED4P4 || fmt == MF_SEED4) {
        const uint32_t seed = gp<uint16_t>(W.p[0])[b], word = gp<uint16_t>(W.p[1])[b];
        const int eb = heads ? gp<int32_t>(W.p[2])[row / rows_per_head] : W.eb;
        int is[8], code;
        if (fmt == MF_SEED4P4) {
            block_isum<4>(tab, seed, word, is);
            code = (gp<uint8_t>(W.p[3])[b >> 1] >> ((b & 1) * 4)) & 15;
        } else {
            block_isum<3>(tab, seed, word, is);
            code = (int) (word & 15u);
        }
        const float sc = pow2f(eb + code) * NSLM_R32;   // exact: a power-of-two scaling of R32
#pragma unroll
        for (int c = 0; c < 8; ++c) o[c] = (float) is[c] * sc;
    } else if (fmt == MF_BF16) {
#pragma unroll
        for (int c = 0; c < 8; ++c) o[c] = bf(gp<uint16_t>(W.p[0])[(size_t) b * 8 + c]);
    } else {
        const size_t e0 = (size_t) b * 8, gi = e0 >> group_shift(W);
        const float s = bf(gp<uint16_t>(W.p[1])[gi]), bb = bf(gp<uint16_t>(W.p[2])[gi]);
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const uint32_t q = fmt == MF_Q8 ? (gp<uint32_t>(W.p[0])[e0 / 4 + (c >> 2)] >> (8 * (c & 3))) & 255u
                                            : (gp<uint32_t>(W.p[0])[e0 / 8] >> (4 * c)) & 15u;
            o[c] = s * (float) q + bb;
        }
    }
    uint16_t* dst = out + (size_t) b * 8;
#pragma unroll
    for (int c = 0; c < 8; ++c) dst[c] = (uint16_t) tobf(o[c]);
}

}   // namespace

extern "C" {

void kc_router(kc_stream_t s, RouterArgs a, const uint16_t* W, const uint16_t* bias, const float* x, float* score,
               float* sel, int32_t* inds, float* wts, int T) {
    if (T < 1) return;
    hipLaunchKernelGGL(k_router_logits, dim3((unsigned) (a.n + 3) / 4, (unsigned) T), dim3(256), 0, (hipStream_t) s, a, W, bias, x, score, sel);
    hipLaunchKernelGGL(k_router_topk, dim3((unsigned) T), dim3(64), 0, (hipStream_t) s, a, score, sel, inds, wts);
}
void kc_router_topk(kc_stream_t s, RouterArgs a, const float* score, const float* sel, int32_t* inds, float* wts, int T) {
    if (T < 1) return;
    hipLaunchKernelGGL(k_router_topk, dim3((unsigned) T), dim3(64), 0, (hipStream_t) s, a, score, sel, inds, wts);
}
void kq4_route_ld(kc_stream_t s, const Qwen4Cfg* c, const float* logits, int ld, int32_t* ind, float* wt, int T) {
    if (T < 1) return;
    hipLaunchKernelGGL(k_q4_route, dim3((unsigned) T), dim3(64), 0, (hipStream_t) s, c->n_exp, c->top_k, logits, ld, ind, wt);
}
void kq4_route(kc_stream_t s, const Qwen4Cfg* c, const float* logits, int32_t* ind, float* wt, int T) {
    kq4_route_ld(s, c, logits, c->n_exp, ind, wt, T);
}
void kc_swiglu(kc_stream_t s, const float* g, const float* u, float* a, int n) {
    if (n < 1) return;
    hipLaunchKernelGGL(k_swiglu, dim3((unsigned) (n + 255) / 256), dim3(256), 0, (hipStream_t) s, g, u, a, n);
}
void kc_swiglu_pack(kc_stream_t s, const float* g, const float* u, uint16_t* y, size_t n) {
    if (n < 8) return;
    hipLaunchKernelGGL(k_swiglu_pack, dim3((unsigned) ((n / 8 + 255) / 256)), dim3(256), 0, (hipStream_t) s, g, u, y, n);
}
void kc_moe_combine(kc_stream_t s, const float* D, const float* w, const float* shared, float* x, int d, int k, int T) {
    if (T < 1) return;
    hipLaunchKernelGGL(k_moe_combine, dim3((unsigned) (d + 255) / 256, (unsigned) T), dim3(256), 0, (hipStream_t) s, D, w, shared, x, d, k);
}
void kq4_moe_combine(kc_stream_t s, int d, int k, const float* D, const float* wt, const float* sh, const float* sg,
                     int sgld, float* out, int T) {
    if (T < 1) return;
    hipLaunchKernelGGL(k_q4_moe_combine, dim3((unsigned) (d + 255) / 256, (unsigned) T), dim3(256), 0, (hipStream_t) s, d, k, D, wt, sh, sg, sgld, out);
}
void kc_pack_input_bf16(kc_stream_t s, const float* x, uint16_t* y, size_t n) {
    if (n < 8) return;
    hipLaunchKernelGGL(k_pack_input_bf16, dim3((unsigned) ((n / 8 + 255) / 256)), dim3(256), 0, (hipStream_t) s, x, y, n);
}
void kc_bucket(kc_stream_t s, const int32_t* inds, int count, int n, int32_t* perm, MmTile* tiles, int32_t* ntiles) {
    hipLaunchKernelGGL(k_bucket_count, dim3(1), dim3(1024), 0, (hipStream_t) s, inds, count, n, ntiles);
    hipLaunchKernelGGL(k_bucket_place, dim3((unsigned) n), dim3(1024), 0, (hipStream_t) s, inds, count, ntiles, perm, tiles);
}
void kc_cache_admit(kc_stream_t s, const CachePool* p, int sl, const int32_t* inds, int count, int flags) {
    hipLaunchKernelGGL(k_cache_admit, dim3(1), dim3(CACHE_MAX_PER_LAYER), 0, (hipStream_t) s, *p, sl, inds, count, flags);
}
void kc_cache_copy(kc_stream_t s, const CachePool* p, int blocks) {
    hipLaunchKernelGGL(k_cache_copy, dim3((unsigned) (blocks > 0 ? blocks : 1)), dim3(512), 0, (hipStream_t) s, *p);
}
void kc_heads_deq(kc_stream_t s, int fmt, WSlice W, const uint32_t* G, int H, int O, int I, uint16_t* out) {
    (void) G;
    const int nb = H * O * (I / 8);
    if (nb < 1) return;
    hipLaunchKernelGGL(k_deq, dim3((unsigned) (nb + 255) / 256), dim3(256), 0, (hipStream_t) s, fmt, W, O, I, nb,
                       fmt == MF_SEED4P4 ? 1 : 0, out);
}
void kc_slice_deq(kc_stream_t s, int fmt, WSlice w, int K, int R, uint16_t* out) {
    const int nb = R * (K / 8);
    if (nb < 1) return;
    hipLaunchKernelGGL(k_deq, dim3((unsigned) (nb + 255) / 256), dim3(256), 0, (hipStream_t) s, fmt, w, R, K, nb, 0, out);
}

}   // extern "C"
