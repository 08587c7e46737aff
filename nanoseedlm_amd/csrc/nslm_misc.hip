// nslm_misc.hip - the small kernels around the seed matmuls: both routers, SwiGLU, the two MoE combines, pair grouping
// for the grouped GEMM, the expert slot table, weights-to-BF16, and the BF16 input pack.  Wave64 throughout.
// What they compute is fixed by the reference's kernels of the same entry points - engine/kernels_moe.cu:527-573 (bucket),
// 717-788 (router, swiglu, combine), 1325-1335 (heads_deq), 2025-2112 (slot table), 2196-2201 (input pack);
// engine/kernels_qwen4.cu:385-416 (softmax route), 506-515 (combine) - how they compute it is this file's own: selection
// by counting instead of arg-max rounds, a one-launch counting sort for the grouping, victims of the slot table by
// bisection on the key instead of one scan per miss.
#include "nslm_dev.h"

using namespace nslm;

namespace {

__device__ __forceinline__ float wave_sum(float v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// ---- sigmoid router logits: one wave per expert, every token of the call --------------------------------------------------
// The wave reads each 16-byte piece of its weight row once for up to RL_TOK tokens (a token per grid row re-read the whole
// router weight per token).  Two partial sums over [0, hw) and [hw, d), each rounded to BF16 before the add (the model's
// two-partition router), sigmoid, selection score = sigmoid + bias.
#define RL_TOK 4
__global__ void __launch_bounds__(256) k_router_logits(RouterArgs a, const uint16_t* W, const uint16_t* bias, const float* x, int T,
                                                       float* score, float* selout) {
    const int lane = threadIdx.x & 63, e = (int) blockIdx.x * 4 + (threadIdx.x >> 6);
    if (e >= a.n) return;   // whole waves leave: no barrier below
    const uint16_t* wr = W + (size_t) e * a.d;
    const bool vec = a.d % 8 == 0 && (((uintptr_t) W | (uintptr_t) x) & 15u) == 0;
    const float be = bf(bias[e]);
    for (int t0 = 0; t0 < T; t0 += RL_TOK) {
        const int nt = min(RL_TOK, T - t0);
        float lo[RL_TOK], hi[RL_TOK];
#pragma unroll
        for (int u = 0; u < RL_TOK; ++u) lo[u] = hi[u] = 0.0f;
        if (vec) {
            for (int c = lane * 8; c < a.d; c += 512) {
                const uint4 q = *(const uint4*) (wr + c);
                const float w[8] = {bf(q.x & 0xFFFFu), bf(q.x >> 16), bf(q.y & 0xFFFFu), bf(q.y >> 16),
                                    bf(q.z & 0xFFFFu), bf(q.z >> 16), bf(q.w & 0xFFFFu), bf(q.w >> 16)};
#pragma unroll
                for (int u = 0; u < RL_TOK; ++u) {
                    const float* xr = x + (size_t) (t0 + min(u, nt - 1)) * a.d + c;   // clamped: the loads stay unconditional
                    const float4 x0 = *(const float4*) xr, x1 = *(const float4*) (xr + 4);
                    const float xv[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        if (c + i < a.hw) lo[u] = fmaf(w[i], xv[i], lo[u]);
                        else hi[u] = fmaf(w[i], xv[i], hi[u]);
                    }
                }
            }
        } else {
            for (int c = lane; c < a.d; c += 64) {
                const float w = bf(wr[c]);
#pragma unroll
                for (int u = 0; u < RL_TOK; ++u) {
                    const float xv = x[(size_t) (t0 + min(u, nt - 1)) * a.d + c];
                    if (c < a.hw) lo[u] = fmaf(w, xv, lo[u]);
                    else hi[u] = fmaf(w, xv, hi[u]);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < RL_TOK; ++u) {
            const float s0 = wave_sum(lo[u]), s1 = wave_sum(hi[u]);
            if (lane == 0 && u < nt) {
                const float sg = 1.0f / (1.0f + expf(-(bfr(s0) + bfr(s1))));
                score[(size_t) (t0 + u) * a.n + e] = sg;
                selout[(size_t) (t0 + u) * a.n + e] = sg + be;
            }
        }
    }
}

// ---- top-k of a row of E <= 1024 values by counting, k <= 32 ----------------------------------------------------------------
// Every value gets a 64-bit key whose integer order is the selection order: the float's order-preserving image above, the
// tie word below (the index itself where the higher index wins a tie, its complement where the lower one does), so no two
// keys are equal and rank(e) = the number of larger keys.  Counting all pairs would be E^2 compares; instead
//   level 1: a wave ranks each group of 64 consecutive values among themselves (64 compares a lane against keys read as
//            LDS broadcasts); a value with k or more larger values in its own group cannot be among the k best of the row,
//   level 2: the survivors (at most k a group) are ranked among themselves; rank r < k is the r-th pick.
// No serial arg-max rounds: the depth of the computation does not grow with k.  One workgroup of 256 threads a row.
// MODE 0, the softmax router (engine/kernels_qwen4.cu:385-416 semantics: ties to the higher index, weights = softmax over
// the k picked, summed in pick order); MODE 1, the sigmoid router's selection (ties to the lowest index, weights =
// score / sum of the picked scores * scale, engine/kernels_moe.cu:742-772 semantics).
#define TK_MAXE 1024
#define TK_MAXK 32
__device__ __forceinline__ uint32_t float_order(float v) {
    const uint32_t b = __float_as_uint(v + 0.0f);   // -0 ranks as +0
    return b ^ ((uint32_t) ((int32_t) b >> 31) | 0x80000000u);
}
// row t of the launch, by a workgroup of NTHR threads (every thread reaches the end: callers may go on with a barrier)
// COH: the selection is stored past the L2 of this workgroup's XCD (agent-scope atomic stores), for a reader in the same launch
template <int MODE, int NTHR, bool COH = false>
__device__ __forceinline__ void topk_row(int t, int E, int k, const float* vals, int ld, const float* score, float scale, int32_t* ind, float* wt) {
    __shared__ __attribute__((aligned(16))) unsigned long long key[TK_MAXE];   // 0 = no value: below every real key
    __shared__ unsigned long long skey[TK_MAXE / 2];                           // survivors of level 1 (at most 32 of every 64)
    __shared__ float pv[TK_MAXK], pw[TK_MAXK];
    __shared__ int pi[TK_MAXK];
    __shared__ int nsurv;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const float* row = vals + (size_t) t * ld;
    const int E64 = (E + 63) & ~63;
    for (int e = tid; e < E64; e += NTHR)
        key[e] = e < E ? (unsigned long long) float_order(row[e]) << 32 | (uint32_t) (MODE == 0 ? e : ~e) : 0ull;
    if (tid == 0) nsurv = 0;
    __syncthreads();
    for (int g = wv; g < E64 / 64; g += NTHR / 64) {
        const unsigned long long mine = key[64 * g + lane];
        int larger = 0;
#pragma unroll 8
        for (int o = 0; o < 64; o += 2) {   // two keys a 16-byte LDS broadcast
            const ulonglong2 q = *(const ulonglong2*) &key[64 * g + o];
            larger += (q.x > mine ? 1 : 0) + (q.y > mine ? 1 : 0);
        }
        const bool keep = mine != 0ull && larger < k;
        const unsigned long long m = __ballot(keep);
        int base = 0;
        if (lane == 0 && m) base = atomicAdd(&nsurv, __popcll(m));
        base = __shfl(base, 0);
        if (keep) skey[base + __popcll(m & ((1ull << lane) - 1ull))] = mine;
    }
    __syncthreads();
    const int S = nsurv;
    for (int j = tid; j < S; j += NTHR) {
        const unsigned long long mine = skey[j];
        int rank = 0;
        for (int o = 0; o < S; ++o) rank += skey[o] > mine ? 1 : 0;
        if (rank < k) {
            const int e = (int) (MODE == 0 ? (uint32_t) mine : ~(uint32_t) mine);
            pi[rank] = e;
            pv[rank] = MODE == 0 ? row[e] : score[(size_t) t * E + e];
        }
    }
    __syncthreads();
    if (wv != 0) return;
    if (lane < k) pw[lane] = MODE == 0 ? expf(pv[lane] - pv[0]) : pv[lane];
    if (lane < k) {   // a wave's LDS accesses stay in order: every lane's pw is written before any lane sums
        float sum = 0.0f;
        for (int r = 0; r < k; ++r) sum += pw[r];
        if (COH) __hip_atomic_store(ind + (size_t) t * k + lane, pi[lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else ind[(size_t) t * k + lane] = pi[lane];
        wt[(size_t) t * k + lane] = MODE == 0 ? pw[lane] / sum : pw[lane] / sum * scale;
    }
}
template <int MODE>
__global__ void __launch_bounds__(256) k_topk_rank(int E, int k, const float* vals, int ld, const float* score, float scale, int32_t* ind,
                                                   float* wt) {
    topk_row<MODE, 256>((int) blockIdx.x, E, k, vals, ld, score, scale, ind, wt);
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

// ---- grouping: selections -> pair ids by expert (ascending inside an expert), tiles of <= MMT_BN pairs, ONE launch ------
// work (= the ntiles buffer, 2n + 3 ints): [0] tile count, [1 .. n+1] pair offsets, [n+2 .. 2n+2] tile offsets.
// A stable counting sort by one workgroup of 16 waves.  Wave w owns the w-th contiguous run of pairs and a histogram row
// hist[w][.] of its own in LDS, so nothing is contended and the order inside an expert is the pair order by construction:
//   count   64 pairs a step; the lanes that hold the same expert find each other with one ballot per index bit (the
//           intersection of the ballots a lane agrees with is the set of its equals), the first of them adds their number,
//   scan    thread x turns column x into running sums over the waves and the workgroup scans the experts' totals
//           (pairs and tiles); thread x writes expert x's tiles,
//   place   the count loop again: hist[w][x] now says where wave w's next pair of expert x goes.
// The reference spends two launches on this (a counting kernel and a one-workgroup-per-expert compaction,
// engine/kernels_moe.cu:527-573); a launch costs more than the work here.
#define BK_WAVES 16
__device__ __forceinline__ unsigned long long equal_lanes(int e, int nbits) {
    unsigned long long m = ~0ull;
    for (int b = 0; b < nbits; ++b) {
        const bool one = (e >> b) & 1;
        const unsigned long long bal = __ballot(one);
        m &= one ? bal : ~bal;
    }
    return m;
}
// COH: the selections were stored by other workgroups of this launch (agent-scope atomic loads)
template <bool COH = false>
__device__ __forceinline__ void bucket_all(const int32_t* inds, int count, int n, int32_t* work, int32_t* perm, MmTile* tiles) {
    auto sel_at = [&](int i) { return COH ? __hip_atomic_load(inds + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : inds[i]; };
    extern __shared__ uint32_t hist[];   // [BK_WAVES][n]
    __shared__ int wsum[2][BK_WAVES];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    int nbits = 1;
    while ((1 << nbits) < n) ++nbits;
    ++nbits;   // one more bit: lanes past the end of the run hold the value n-or-above 1 << (nbits - 1) and only equal each other
    const int run = ((count + BK_WAVES - 1) / BK_WAVES + 63) & ~63, i0 = wv * run, i1 = min(count, i0 + run);
    uint32_t* mine = hist + (size_t) wv * n;
    for (int i = tid; i < BK_WAVES * n; i += 64 * BK_WAVES) hist[i] = 0;
    __syncthreads();
    for (int i = i0; i < i1; i += 64) {
        int e = i + lane < i1 ? sel_at(i + lane) : -1;
        const bool live = (unsigned) e < (unsigned) n;   // an index outside the table is left out
        if (!live) e = 1 << (nbits - 1);
        const unsigned long long eq = equal_lanes(e, nbits);
        if (live && (eq & ((1ull << lane) - 1ull)) == 0) mine[e] += (uint32_t) __popcll(eq);
    }
    __syncthreads();
    int cnt = 0;
    if (tid < n)
        for (int w = 0; w < BK_WAVES; ++w) {
            const uint32_t c = hist[(size_t) w * n + tid];
            hist[(size_t) w * n + tid] = (uint32_t) cnt;
            cnt += (int) c;
        }
    const int ntl = (cnt + MMT_BN - 1) / MMT_BN;
    int pin = cnt, tin = ntl;   // inclusive sums over the experts: across the wave, then across the waves
    for (int o = 1; o < 64; o <<= 1) {
        const int a = __shfl_up(pin, o), b = __shfl_up(tin, o);
        if (lane >= o) { pin += a; tin += b; }
    }
    if (lane == 63) { wsum[0][wv] = pin; wsum[1][wv] = tin; }
    __syncthreads();
    int pofs = pin - cnt, tofs = tin - ntl;
    for (int w = 0; w < wv; ++w) { pofs += wsum[0][w]; tofs += wsum[1][w]; }
    if (tid < n) {
        work[1 + tid] = pofs;
        work[2 + n + tid] = tofs;
        for (int w = 0; w < BK_WAVES; ++w) hist[(size_t) w * n + tid] += (uint32_t) pofs;
        for (int j = 0; j < ntl; ++j) {
            MmTile tl;
            tl.slice = tid;
            tl.start = pofs + j * MMT_BN;
            tl.count = min(MMT_BN, cnt - j * MMT_BN);
            tl.pad = 0;
            tiles[tofs + j] = tl;
        }
        if (tid == n - 1) {
            work[1 + n] = pofs + cnt;
            work[2 + 2 * n] = tofs + ntl;
            work[0] = tofs + ntl;
        }
    }
    __syncthreads();
    for (int i = i0; i < i1; i += 64) {
        int e = i + lane < i1 ? sel_at(i + lane) : -1;
        const bool live = (unsigned) e < (unsigned) n;
        if (!live) e = 1 << (nbits - 1);
        const unsigned long long eq = equal_lanes(e, nbits), before = eq & ((1ull << lane) - 1ull);
        if (live) {
            const uint32_t at = mine[e];   // every lane of the group reads before its first lane moves the mark (LDS in wave order)
            perm[at + (uint32_t) __popcll(before)] = i + lane;
            if (before == 0) mine[e] = at + (uint32_t) __popcll(eq);
        }
    }
}
__global__ void __launch_bounds__(64 * BK_WAVES) k_bucket(const int32_t* inds, int count, int n, int32_t* work, int32_t* perm, MmTile* tiles) {
    bucket_all<false>(inds, count, n, work, perm, tiles);
}
// The batched softmax step's routing and grouping in one launch: workgroup t ranks row t (k_topk_rank<0>'s arithmetic), and the
// workgroup that finishes last - a ticket in the word behind the bucket's work area, back at zero when the launch ends -
// groups the launch's pairs (k_bucket's).  Nobody waits for anybody.
__global__ void __launch_bounds__(64 * BK_WAVES) k_route_bucket(int E, int k, const float* logits, int ld, int32_t* ind, float* wt, int T, int32_t* work,
                                                                int32_t* perm, MmTile* tiles) {
    __shared__ int last;
    topk_row<0, 64 * BK_WAVES, true>((int) blockIdx.x, E, k, logits, ld, (const float*) 0, 1.0f, ind, wt);
    if (threadIdx.x == 0) {   // wave 0 stored the row's selection: those stores have left the wave before the ticket is taken
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        last = atomicAdd((unsigned*) &work[2 * E + 3], 1u) == (unsigned) (T - 1);
    }
    __syncthreads();
    if (!last) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    if (threadIdx.x == 0) __hip_atomic_store((unsigned*) &work[2 * E + 3], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    bucket_all<true>(ind, T * k, E, work, perm, tiles);
}

// ---- expert slot table --------------------------------------------------------------------------------------------------
// One workgroup, thread x = expert x of the layer.  Selected experts that are resident take the new tick.  The others
// (misses, in expert order) take the least recently used slots this call (and, with CACHE_PROTECT_PREV, the previous one)
// did not touch, oldest first, ties to the lowest slot - which is to say: miss number m gets the slot with the m-th
// smallest key (tick, slot index) among the replaceable slots.  So the victims are found all at once instead of one
// arg-min round per miss (engine/kernels_moe.cu:2025-2102 does the rounds): the key that has exactly `admitted` keys at or
// below it is found by bisection on the key's value (one count over the slots per step), the keys at or below it are
// collected, and each victim's place among them is again a count.  Bit sets in LDS stand for "selected" and "miss", so a
// miss's number is a population count.  On a GPU that holds every expert (slots == units) nothing misses and the kernel
// ends after the ticks; hosts skip the launch altogether then.
#define SL_KEEP 8   // keys a thread keeps in registers (8192 slots); slots beyond are read again in every step
__device__ __forceinline__ int block_sum_1024(int v, int* red) {   // red: 16 ints, not in use by a previous call's readers
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    int s = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) s += red[w];
    return s;
}
__global__ void __launch_bounds__(CACHE_MAX_PER_LAYER) k_slots_admit(CachePool p, int sl, const int32_t* inds, int count, int flags) {
    __shared__ uint32_t needw[CACHE_MAX_PER_LAYER / 32], missw[CACHE_MAX_PER_LAYER / 32];
    __shared__ uint16_t missx[CACHE_MAX_PER_LAYER];
    __shared__ unsigned long long vkey[CACHE_MAX_PER_LAYER];
    __shared__ int vslot[CACHE_MAX_PER_LAYER];
    __shared__ int red[2][16];
    __shared__ unsigned long long redk[2][16];
    __shared__ int nvict;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const uint32_t prev = p.tick[0], now = prev + 1;
    const bool protect = (flags & CACHE_PROTECT_PREV) != 0;
    if (tid < CACHE_MAX_PER_LAYER / 32) needw[tid] = missw[tid] = 0;
    if (tid == 0) nvict = 0;
    __syncthreads();
    for (int i = tid; i < count; i += CACHE_MAX_PER_LAYER) atomicOr(&needw[inds[i] >> 5], 1u << (inds[i] & 31));
    __syncthreads();
    const bool sel = tid < p.per_layer && ((needw[tid >> 5] >> (tid & 31)) & 1u);
    const int home = sel ? p.unit_slot[sl * p.per_layer + tid] : -1;
    if (sel && home >= 0) p.slot_last[home] = now;
    if (sel && home < 0) atomicOr(&missw[tid >> 5], 1u << (tid & 31));
    __syncthreads();
    int nsel = 0, nmiss = 0, mine = 0;   // population counts: selected, misses, misses before this expert
#pragma unroll
    for (int w = 0; w < CACHE_MAX_PER_LAYER / 32; ++w) {
        nsel += __popc(needw[w]);
        const int c = __popc(missw[w]);
        nmiss += c;
        if (w < (tid >> 5)) mine += c;
    }
    if (sel && home < 0) missx[mine + __popc(missw[tid >> 5] & ((1u << (tid & 31)) - 1u))] = (uint16_t) tid;
    if (tid == 0) {
        p.tick[0] = now;
        p.stats[0] += (uint32_t) (nsel - nmiss);
        p.stats[1] += (uint32_t) nmiss;
    }
    if (nmiss == 0) {   // uniform
        if (tid == 0) *p.njobs = 0;
        return;
    }
    // a slot's key: (tick of its last use, index); ~0 when it may not be replaced.  Whether this call touched a slot is read
    // off the unit it holds (an expert of this layer that is selected), not off the tick stored a moment ago.
    auto key_of = [&](int s) -> unsigned long long {
        if (s >= p.slots) return ~0ull;
        const int u = p.slot_unit[s];
        const uint32_t last = p.slot_last[s];
        const int x = u - sl * p.per_layer;
        const bool touched = u >= 0 && x >= 0 && x < p.per_layer && ((needw[x >> 5] >> (x & 31)) & 1u);
        if (touched || (protect && last == prev)) return ~0ull;
        return (unsigned long long) last << 20 | (unsigned long long) s;
    };
    unsigned long long kept[SL_KEEP];
#pragma unroll
    for (int j = 0; j < SL_KEEP; ++j) kept[j] = key_of(tid + j * CACHE_MAX_PER_LAYER);
    auto count_le = [&](unsigned long long lim, int* scratch) {   // replaceable slots whose key is <= lim
        int c = 0;
#pragma unroll
        for (int j = 0; j < SL_KEEP; ++j) c += kept[j] <= lim ? 1 : 0;
        for (int s = tid + SL_KEEP * CACHE_MAX_PER_LAYER; s < p.slots; s += CACHE_MAX_PER_LAYER) c += key_of(s) <= lim ? 1 : 0;
        return block_sum_1024(c, scratch);
    };
    unsigned long long lo = ~0ull, hi = 0ull;   // the smallest and the largest replaceable key
#pragma unroll
    for (int j = 0; j < SL_KEEP; ++j)
        if (kept[j] != ~0ull) { lo = kept[j] < lo ? kept[j] : lo; hi = kept[j] > hi ? kept[j] : hi; }
    for (int s = tid + SL_KEEP * CACHE_MAX_PER_LAYER; s < p.slots; s += CACHE_MAX_PER_LAYER) {
        const unsigned long long kk = key_of(s);
        if (kk != ~0ull) { lo = kk < lo ? kk : lo; hi = kk > hi ? kk : hi; }
    }
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long a = __shfl_xor(lo, o), b = __shfl_xor(hi, o);
        lo = a < lo ? a : lo;
        hi = b > hi ? b : hi;
    }
    if (lane == 0) { redk[0][wv] = lo; redk[1][wv] = hi; }
    __syncthreads();
#pragma unroll
    for (int w = 0; w < 16; ++w) { lo = redk[0][w] < lo ? redk[0][w] : lo; hi = redk[1][w] > hi ? redk[1][w] : hi; }
    const int avail = lo == ~0ull ? 0 : count_le(hi, red[0]);
    const int admitted = min(nmiss, avail);   // nothing replaceable left (a pool smaller than two layers' picks): the rest stay out
    if (tid == 0) *p.njobs = admitted;
    if (admitted == 0) return;   // uniform
    int par = 1;
    while (lo < hi) {   // uniform: every thread holds the same bounds
        const unsigned long long mid = lo + ((hi - lo) >> 1);
        if (count_le(mid, red[par]) >= admitted) hi = mid;
        else lo = mid + 1;
        par ^= 1;
    }
    auto collect = [&](unsigned long long kk) {
        if (kk <= hi) vkey[atomicAdd(&nvict, 1)] = kk;
    };
#pragma unroll
    for (int j = 0; j < SL_KEEP; ++j) collect(kept[j]);
    for (int s = tid + SL_KEEP * CACHE_MAX_PER_LAYER; s < p.slots; s += CACHE_MAX_PER_LAYER) collect(key_of(s));
    __syncthreads();
    if (tid < admitted) {
        const unsigned long long kk = vkey[tid];
        int place = 0;
        for (int o = 0; o < admitted; ++o) place += vkey[o] < kk ? 1 : 0;
        vslot[place] = (int) (kk & 0xFFFFFu);
    }
    __syncthreads();
    if (tid < admitted) {   // miss number tid moves into victim number tid; the units and slots of different threads are distinct
        const int x = missx[tid], u = sl * p.per_layer + x, s = vslot[tid], old = p.slot_unit[s];
        if (old >= 0) p.unit_slot[old] = -1;
        p.slot_unit[s] = u;
        p.unit_slot[u] = s;
        p.slot_last[s] = now;
        p.jobs[2 * tid] = u;
        p.jobs[2 * tid + 1] = s;
    }
    for (int i = tid; i < admitted * p.ntens * 4; i += CACHE_MAX_PER_LAYER) {   // the moved units' slice tables point at their slots
        const int m = i / (p.ntens * 4), tn = i / 4 % p.ntens, st = i & 3;
        if (p.off[tn][st] == 0xFFFFFFFFu) continue;
        WSlice* w = p.tab + ((size_t) sl * p.ntens + tn) * p.per_layer + missx[m];
        w->p[st] = p.vram + (uint64_t) vslot[m] * p.unit_bytes + p.off[tn][st];
    }
}
// the queued units, arena -> pool slots: the jobs' 8 KiB pieces dealt round the workgroups, 16 bytes a thread
__global__ void __launch_bounds__(512) k_slots_copy(CachePool p) {
    const uint64_t words = p.unit_bytes / 16, pieces = (words + 511) / 512, total = (uint64_t) *p.njobs * pieces;
    for (uint64_t c = blockIdx.x; c < total; c += gridDim.x) {
        const uint64_t j = c / pieces, w = (c - j * pieces) * 512 + threadIdx.x;
        if (w < words)
            ((uint4*) (p.vram + (uint64_t) p.jobs[2 * j + 1] * p.unit_bytes))[w] = ((const uint4*) (p.host + (uint64_t) p.jobs[2 * j] * p.unit_bytes))[w];
    }
}

// ---- weights to BF16 bits: one thread per 8-weight block ---------------------------------------------------------------
// heads: W.p[2] holds an int32 exponent bias per head (SEED4P4 per-head maps); otherwise the slice's own eb.
#define DEQ_NB 8   // blocks a thread of the seed formats' path takes
__device__ __forceinline__ uint32_t deq_pk_bf16(float lo, float hi) {   // v_cvt_pk_bf16_f32: both round to nearest even
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
// The seed formats, 16-byte aligned output: a thread takes DEQ_NB blocks (block wg * 256 * DEQ_NB + k * 256 + tid, so a wave's
// accesses are consecutive), all their records requested before the first is expanded, a block's eight BF16 values leaving as one
// 16-byte store.  (A block a thread with the tables loaded for every 256 blocks and eight 2-byte stores: 164 instructions a block.)
template <int P>
__global__ void __launch_bounds__(256) k_deq_seed(WSlice W, int rows_per_head, int K, int nblocks, int heads, uint16_t* out) {
    __shared__ uint32_t tab[NSLM_TAB_WORDS];
    load_tables(tab);
    const int nbk = K / 8, b0 = (int) blockIdx.x * 256 * DEQ_NB + (int) threadIdx.x;
    uint32_t seed[DEQ_NB], word[DEQ_NB], cb[DEQ_NB];
    int eb[DEQ_NB];
#pragma unroll
    for (int k = 0; k < DEQ_NB; ++k) {   // (clamped: the loads stay unconditional)
        const int b = min(b0 + 256 * k, nblocks - 1);
        seed[k] = gp<uint16_t>(W.p[0])[b];
        word[k] = gp<uint16_t>(W.p[1])[b];
        cb[k] = P == 4 ? gp<uint8_t>(W.p[3])[b >> 1] : 0u;
        eb[k] = heads ? gp<int32_t>(W.p[2])[(b / nbk) / rows_per_head] : W.eb;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < DEQ_NB; ++k) {
        const int b = b0 + 256 * k;
        if (b >= nblocks) break;
        int is[8];
        block_isum<P>(tab, seed[k], word[k], is);
        const int code = P == 4 ? (int) ((cb[k] >> ((b & 1) * 4)) & 15u) : (int) (word[k] & 15u);
        const float sc = pow2f(eb[k] + code) * NSLM_R32;   // exact: a power-of-two scaling of R32
        float o[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) o[c] = (float) is[c] * sc;
        *(uint4*) (out + (size_t) b * 8) = make_uint4(deq_pk_bf16(o[0], o[1]), deq_pk_bf16(o[2], o[3]), deq_pk_bf16(o[4], o[5]), deq_pk_bf16(o[6], o[7]));
    }
}
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

void launch_deq(hipStream_t st, int fmt, WSlice W, int rows_per_head, int K, int nb, int heads, uint16_t* out) {
    const bool seed = fmt == MF_SEED4P4 || fmt == MF_SEED4;
    if (seed && ((uintptr_t) out & 15u) == 0) {
        const dim3 grid((unsigned) ((nb + 256 * DEQ_NB - 1) / (256 * DEQ_NB)));
        if (fmt == MF_SEED4P4) hipLaunchKernelGGL(k_deq_seed<4>, grid, dim3(256), 0, st, W, rows_per_head, K, nb, heads, out);
        else hipLaunchKernelGGL(k_deq_seed<3>, grid, dim3(256), 0, st, W, rows_per_head, K, nb, heads, out);
        return;
    }
    hipLaunchKernelGGL(k_deq, dim3((unsigned) (nb + 255) / 256), dim3(256), 0, st, fmt, W, rows_per_head, K, nb, heads, out);
}

}   // namespace

extern "C" {

void kc_router_topk(kc_stream_t s, RouterArgs a, const float* score, const float* sel, int32_t* inds, float* wts, int T) {
    if (T < 1) return;
    if (a.n < a.top_k || a.n > TK_MAXE || a.top_k < 1 || a.top_k > TK_MAXK) { host_note_unsupported(); return; }
    hipLaunchKernelGGL(k_topk_rank<1>, dim3((unsigned) T), dim3(256), 0, (hipStream_t) s, a.n, a.top_k, sel, a.n, score, a.scale, inds, wts);
    host_note_launch();
}
void kc_router(kc_stream_t s, RouterArgs a, const uint16_t* W, const uint16_t* bias, const float* x, float* score,
               float* sel, int32_t* inds, float* wts, int T) {
    if (T < 1) return;
    hipLaunchKernelGGL(k_router_logits, dim3((unsigned) (a.n + 3) / 4), dim3(256), 0, (hipStream_t) s, a, W, bias, x, T, score, sel);
    kc_router_topk(s, a, score, sel, inds, wts, T);
}
void kq4_route_ld(kc_stream_t s, const Qwen4Cfg* c, const float* logits, int ld, int32_t* ind, float* wt, int T) {
    if (T < 1) return;
    if (c->n_exp < c->top_k || c->n_exp > TK_MAXE || c->top_k < 1 || c->top_k > TK_MAXK) { host_note_unsupported(); return; }
    hipLaunchKernelGGL(k_topk_rank<0>, dim3((unsigned) T), dim3(256), 0, (hipStream_t) s, c->n_exp, c->top_k, logits, ld, (const float*) 0, 1.0f, ind, wt);
    host_note_launch();
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
    if (n < 1 || n > BUCKET_MAX_EXPERTS || count < 0) { host_note_unsupported(); return; }
    const size_t lds = sizeof(uint32_t) * BK_WAVES * (size_t) n;
    static const hipError_t once = hipFuncSetAttribute((const void*) k_bucket, hipFuncAttributeMaxDynamicSharedMemorySize,
                                                       (int) (sizeof(uint32_t) * BK_WAVES * BUCKET_MAX_EXPERTS));
    (void) once;
    hipLaunchKernelGGL(k_bucket, dim3(1), dim3(64 * BK_WAVES), lds, (hipStream_t) s, inds, count, n, ntiles, perm, tiles);
    host_note_launch();
}
void kq4_route_bucket(kc_stream_t s, const Qwen4Cfg* c, const float* logits, int32_t* ind, float* wt, int T, int32_t* perm, MmTile* tiles,
                      int32_t* ntiles) {
    if (T < 1) return;
    if (c->n_exp < c->top_k || c->n_exp > TK_MAXE || c->top_k < 1 || c->top_k > TK_MAXK || c->n_exp > BUCKET_MAX_EXPERTS) { host_note_unsupported(); return; }
    const size_t lds = sizeof(uint32_t) * BK_WAVES * (size_t) c->n_exp;
    static const hipError_t once = hipFuncSetAttribute((const void*) k_route_bucket, hipFuncAttributeMaxDynamicSharedMemorySize,
                                                       (int) (sizeof(uint32_t) * BK_WAVES * BUCKET_MAX_EXPERTS));
    (void) once;
    hipLaunchKernelGGL(k_route_bucket, dim3((unsigned) T), dim3(64 * BK_WAVES), lds, (hipStream_t) s, c->n_exp, c->top_k, logits, c->n_exp, ind, wt, T,
                       ntiles, perm, tiles);
    host_note_launch();
}
void kc_cache_admit(kc_stream_t s, const CachePool* p, int sl, const int32_t* inds, int count, int flags) {
    if (p->per_layer > CACHE_MAX_PER_LAYER || p->slots > (1 << 20) || p->ntens > 3) { host_note_unsupported(); return; }
    hipLaunchKernelGGL(k_slots_admit, dim3(1), dim3(CACHE_MAX_PER_LAYER), 0, (hipStream_t) s, *p, sl, inds, count, flags);
    host_note_launch();
}
void kc_cache_copy(kc_stream_t s, const CachePool* p, int blocks) {
    hipLaunchKernelGGL(k_slots_copy, dim3((unsigned) (blocks > 0 ? blocks : 1)), dim3(512), 0, (hipStream_t) s, *p);
    host_note_launch();
}
void kc_heads_deq(kc_stream_t s, int fmt, WSlice W, const uint32_t* G, int H, int O, int I, uint16_t* out) {
    (void) G;
    const int nb = H * O * (I / 8);
    if (nb < 1) return;
    launch_deq((hipStream_t) s, fmt, W, O, I, nb, fmt == MF_SEED4P4 ? 1 : 0, out);
}
void kc_slice_deq(kc_stream_t s, int fmt, WSlice w, int K, int R, uint16_t* out) {
    const int nb = R * (K / 8);
    if (nb < 1) return;
    launch_deq((hipStream_t) s, fmt, w, R, K, nb, 0, out);
}

}   // extern "C"
