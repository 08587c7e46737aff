// nslm_fused.hip - one persistent kernel for a whole routed-expert decode step at T <= 8 tokens (k_moe_decode; 9 to 24
// tokens: k_moe_decode_grouped further down): router logits, softmax top-k, fused gate + up + SwiGLU gather, down gather,
// weighted combine.  No counterpart in the reference, which launches
// these as five kernels (engine/qwen4_cuda.c:1023-1083); on MI355X each launch and each dependent global read costs
// microseconds that a ~20 us step cannot afford, so the phases run inside one grid: the data that crosses workgroups says
// itself when it is there (router logits, published routing, ready words and finished-item words, all tagged with the
// launch's generation), so no phase needs a grid-wide barrier.
//
// Arithmetic is the stand-alone kernels', instruction for instruction (k_mv_any's BF16 row dot, k_q4_route's selection
// and weights, k_mv_seed's chunk products and row-sum order, k_q4_moe_combine's sum), so the fused step returns the same
// bits as the five launches.
//
// Data that one workgroup writes and another reads inside the launch (logits, A, D) moves with agent-scope relaxed
// atomic stores and loads: on this GPU every XCD has its own L2, and those accesses go through to the coherent level, so
// no device-scope fence (an L2 write-back / invalidate per workgroup, which costs far more than the step) is needed;
// ordering against the counters and tagged words: every wave waits for its own stores to be acknowledged (an explicit
// s_waitcnt vmcnt(0), see wg_release) before the workgroup barrier that precedes the flag store.
//
// Waiting: the grid is sized to the number of workgroups the device can hold at once (occupancy query), because
// workgroups wait for each other's data; every wait is a bounded poll, and a workgroup that gives up sets an error word
// and runs on to the end, so every wave always exits.
#include <math.h>
#include <stdlib.h>

#include <atomic>

#include "nslm_fused_dev.h"

using namespace nslm;

namespace {

// The first chunk of a pass over rows [v0, v1): issued as early as the slices are known, so its latency hides behind
// whatever comes before the pass (a wait for other workgroups, the staging of the activations).
template <int P, bool GATEUP>
__device__ __forceinline__ Chunk first_chunk(const WSlice& wA, const WSlice& wB, int L, int rpi, int v0, int v1) {
    (void) rpi;
    const int tid = threadIdx.x, lr = tid / L, ch = tid - lr * L, vv = min(v0 + lr, v1 - 1);   // (rows past the last: the last row's records)
    const WSlice& w = (GATEUP && (vv & 1)) ? wB : wA;
    return load_chunk<P>(w, (uint32_t) (GATEUP ? vv >> 1 : vv) * (uint32_t) L + (uint32_t) ch);
}

// rows [v0, v1) of one pair: the k_mv_seed loop with the activations in LDS (xl, chunk-padded).  emit(row, sum, other)
// is called by the thread that owns a finished row sum.
template <int P, bool GATEUP, bool SHFL, typename Emit>
__device__ __forceinline__ void rows_pass(Chunk cur, const WSlice& wA, const WSlice& wB, int L, int rpi, int v0, int v1,
                                          const uint32_t* tab, const float* xl, float (*part)[256], float2* gu, Emit emit) {
    const int tid = threadIdx.x, lr = tid / L, ch = tid - lr * L;
    const bool active = lr < rpi;
    auto fetch = [&](int vv) {   // (rows past the last: the last row's records once more)
        const int vc = min(vv, v1 - 1), r = GATEUP ? vc >> 1 : vc;
        const WSlice& w = (GATEUP && (vc & 1)) ? wB : wA;
        return load_chunk<P>(w, (uint32_t) r * (uint32_t) L + (uint32_t) ch);
    };
    int par = 0;
    for (int vb = v0; vb < v1; vb += rpi, par ^= 1) {
        const int v = vb + lr;
        const Chunk nxt = fetch(v + rpi);
        float acc[1] = {0.0f};
        const int eb = (GATEUP && (v & 1)) ? wB.eb : wA.eb;
        // (two blocks at a time in phase order where three workgroups a CU compute at once; the down pass, whose waves mostly
        // run alone behind their pair's readiness, keeps the compiler's order)
        if (active && v < v1) chunk_dot<P, 1, GATEUP>(cur, eb, tab, xl + ch * xpad<P>(), 0, 1, acc);
        if (SHFL) {
            float s = acc[0];
            for (int o = L >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o);
            if (GATEUP) {
                // (the two row sums wait in LDS: what emit does with them - SwiGLU, a store - is then executed once behind the loop
                // by the threads of a row each, not in every iteration by every wave that holds a row)
                const float other = __shfl_xor(s, L);
                if (active && ch == 0 && !(v & 1) && v < v1) {
                    if (gu) gu[(v - v0) >> 1] = make_float2(s, other);
                    else emit(v >> 1, s * NSLM_R32, other * NSLM_R32);
                }
            } else if (active && ch == 0 && v < v1) emit(v, s * NSLM_R32, 0.0f);
        } else {
            part[par][tid] = acc[0];
            __syncthreads();
            const int nrow = min(rpi, v1 - vb);
            if (GATEUP) {
                if (tid < nrow / 2) {
                    float gs = 0.0f, us = 0.0f;
                    for (int j = 0; j < L; ++j) gs += part[par][(2 * tid) * L + j];
                    for (int j = 0; j < L; ++j) us += part[par][(2 * tid + 1) * L + j];
                    emit((vb >> 1) + tid, gs * NSLM_R32, us * NSLM_R32);
                }
            } else if (tid < nrow) {
                float s = 0.0f;
                for (int j = 0; j < L; ++j) s += part[par][tid * L + j];
                emit(vb + tid, s * NSLM_R32, 0.0f);
            }
        }
        cur = nxt;
    }
    if (!SHFL) __syncthreads();   // part may be reused by the next pass
    if (GATEUP && SHFL && gu) {
        __syncthreads();
        for (int i = tid; i < (v1 - v0) >> 1; i += 256) {
            const float2 q = gu[i];
            emit((v0 >> 1) + i, q.x * NSLM_R32, q.y * NSLM_R32);
        }
    }
}

// n floats of a row staged into LDS in the form the format's matvec reads (store_block: chunk-padded, P = 4 as its 12 column
// values a block) by the whole workgroup; coherent: agent-scope loads (the row was written by other workgroups of this
// launch).  A thread takes whole blocks, four a round, and requests their 32 words before the first is used (clamped
// indices, so the loads are unconditional): one load and one LDS store a round is one memory round trip a round.
template <int P>
__device__ __forceinline__ void stage_row(const float* src, int n, float* xl, bool coherent) {
    const int nb = n / 8;
    for (int b0 = threadIdx.x; b0 < nb; b0 += 256 * 4) {
        float v[4][8];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const float* p = src + (size_t) min(b0 + 256 * u, nb - 1) * 8;
            if (coherent) {
#pragma unroll
                for (int c = 0; c < 8; ++c) v[u][c] = ld_agent(p + c);
            } else {
                const float4 q0 = *(const float4*) p, q1 = *(const float4*) (p + 4);
                v[u][0] = q0.x; v[u][1] = q0.y; v[u][2] = q0.z; v[u][3] = q0.w; v[u][4] = q1.x; v[u][5] = q1.y; v[u][6] = q1.z; v[u][7] = q1.w;
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (b0 + 256 * u < nb) store_block<P>(xl, b0 + 256 * u, v[u]);
    }
}
// an input row, normalised on the way when nw is given: the values kq4_norm1p would have stored
template <int P>
__device__ __forceinline__ void stage_input(const float* src, int n, float* xl, const float* nw, float rn) {
    if (!nw) { stage_row<P>(src, n, xl, false); return; }
    const int nb = n / 8;
    for (int b0 = threadIdx.x; b0 < nb; b0 += 256 * 4) {
        float v[4][8], w[4][8];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const size_t o = (size_t) min(b0 + 256 * u, nb - 1) * 8;
            const float4 q0 = *(const float4*) (src + o), q1 = *(const float4*) (src + o + 4);
            const float4 w0 = *(const float4*) (nw + o), w1 = *(const float4*) (nw + o + 4);
            v[u][0] = q0.x; v[u][1] = q0.y; v[u][2] = q0.z; v[u][3] = q0.w; v[u][4] = q1.x; v[u][5] = q1.y; v[u][6] = q1.z; v[u][7] = q1.w;
            w[u][0] = w0.x; w[u][1] = w0.y; w[u][2] = w0.z; w[u][3] = w0.w; w[u][4] = w1.x; w[u][5] = w1.y; w[u][6] = w1.z; w[u][7] = w1.w;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (b0 + 256 * u < nb) {
#pragma unroll
                for (int c = 0; c < 8; ++c) v[u][c] = v[u][c] * rn * (1.0f + w[u][c]);
                store_block<P>(xl, b0 + 256 * u, v[u]);
            }
    }
}

// The k best of E logits already in LDS (rv, padded to a multiple of four with -inf): ri[r] = the expert of rank r, where
// rank(e) = how many experts come before e (larger logit, or equal logit and higher index): k_q4_route's order.  Called by
// the whole workgroup after a barrier; the caller's next barrier publishes ri.  scratch: 512 words of LDS.
// The logits are BF16 values (phase 1 rounds them), so the upper half of a float's order-preserving integer image holds
// all of a logit and the lower half is free for the expert's index: one 32-bit key whose integer order is the routing
// order, and no two keys are equal.  rank(e) = number of larger keys.  Up to 256 experts: thread (e, part) counts over its
// part of the experts (keys read four at a time as LDS broadcasts: two instructions a compare) and the parts' counts are
// added.  Every instruction counts here, scalar ones too: the workgroups of a CU rank at the same moment, and wave-wide
// compares with scalar population counts took 3 to 6 us of every workgroup's time.
__device__ __forceinline__ void rank_logits(const float* rv, int E, int k, uint32_t* scratch, int* ri) {
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, E4 = (E + 3) & ~3;
    auto key_of = [&](int o) {
        const uint32_t b = __float_as_uint(rv[o] + 0.0f);   // -0 counts as +0, as in a float compare
        return ((b ^ ((uint32_t) ((int32_t) b >> 31) | 0x80000000u)) & 0xFFFF0000u) | (uint32_t) o;
    };
    if (E <= 256) {
        uint32_t* pk = scratch;              // keys (0 = absent, below every real key)
        int* gp = (int*) scratch + 256;      // the parts' counts, [part][expert]
        pk[tid] = tid < E ? key_of(tid) : 0u;
        __syncthreads();
        const int epad = E <= 64 ? 64 : E <= 128 ? 128 : 256, len = epad * epad / 256;
        const int e = tid & (epad - 1), o0 = tid / epad * len;
        const uint32_t ke = pk[e];
        int g = 0;
#pragma unroll 4
        for (int o = o0; o < o0 + len; o += 4) {
            const uint4 q = *(const uint4*) &pk[o];
            g += (q.x > ke ? 1 : 0) + (q.y > ke ? 1 : 0) + (q.z > ke ? 1 : 0) + (q.w > ke ? 1 : 0);
        }
        gp[tid] = g;
        __syncthreads();
        if (tid < E) {
            int rank = 0;
            for (int q = tid; q < 256; q += epad) rank += gp[q];
            if (rank < k) ri[rank] = tid;
        }
    } else {   // a wave takes the experts one at a time
        for (int e = wv; e < E; e += 4) {
            const uint32_t ke = __builtin_amdgcn_readfirstlane(key_of(e));
            int rank = 0;
            for (int o = lane; o < E4 + 63; o += 64) rank += __popcll(__ballot(o < E && key_of(o < 1024 ? o : 1023) > ke));
            if (rank < k && lane == 0) ri[rank] = e;
        }
    }
}

template <int P, bool SHFL_G, bool SHFL_D, int WAVES>
__global__ void __launch_bounds__(256, WAVES) k_moe_decode(FusedArgs a) {   // WAVES waves a SIMD: five = at most 96 registers
    extern __shared__ float xl[];   // activations of the current pair: max(d, ff) floats, chunk-padded
    float2* const gu_s = (float2*) (xl + a.gu_off);   // behind them: the gate and up row sums of the item in hand
    __shared__ uint32_t tab[NSLM_TAB_WORDS];
    __shared__ float part[2][256];
    __shared__ __attribute__((aligned(16))) float rv[1024];   // route: the token's logits
    __shared__ float rw_s[33];      // route: weight by rank (+ the shared expert's 1)
    __shared__ int ri_s[33];        // route: expert by rank
    __shared__ WSlice sl_s[3][33];  // route: the chosen experts' gate / up / down slices (+ the shared expert's)
    // (no workgroup-wide flag: every wait of this kernel is a poll of its own threads)
    __shared__ uint32_t s_tag;
    __shared__ float rn_s[MV_MAXT], nred[4];   // the rows' RMSNorm scales when the kernel normalises its input
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const uint32_t G = (uint32_t) a.grid;
    const int P_ = a.T * a.kk;
    // the generation: lane 0 of every wave reads it (all sense words are equal); the workgroup arrives further down
    const uint32_t my_gen = ld_agent(a.sync + 32 * (BAR_GROUPS + 1 + blockIdx.x % BAR_GROUPS));
    unsigned long long* lg64 = (unsigned long long*) (a.sync + FUSED_LOGIT_WORDS);
    const int items_g = P_ * a.ntile_g, items_d = P_ * a.ntile_d;
    int staged = -1;
    uint32_t* pairw = a.sync + FUSED_PAIR_WORDS;    // [pair][64]: arrivals, ready word
    uint32_t* dflag = a.sync + FUSED_DFLAG_WORDS;   // [token][FUSED_TILES][33]
    if (a.nw) {   // uniform: every workgroup forms every row's scale (T rows of d values from L2)
        for (int t = 0; t < a.T; ++t) {
            const float r = row_rnorm(a.x + (size_t) t * a.xs, a.d, a.neps, nred);
            if (tid == 0) rn_s[t] = r;
        }
        __syncthreads();
    }

    // ---- phase 1: router logits, one wave per (token, expert): k_mv_any's BF16 row dot and BF16 store ----------------
    for (int item = (int) blockIdx.x * 4 + wv; item < a.T * a.E; item += (int) G * 4) {
        const int t = item / a.E, e = item - t * a.E;
        const float lv = router_logit(a.rw + (size_t) e * a.d, a.x + (size_t) t * a.xs, a.d, a.nw, a.nw ? rn_s[t] : 1.0f);
        if (lane == 0) {
            st_agent(a.logits + item, lv);
            st_agent(lg64 + item, (unsigned long long) __float_as_uint(lv) | (unsigned long long) (my_gen + 1u) << 32);
        }
        if (t == 0 && lane >= a.T && lane < FG_MAXT) st_agent(lg64 + (size_t) lane * a.E + e, 0ull);   // rows this launch does not use
    }
    // The decode tables are first needed in phase 2: loaded here, behind the logits (everybody waits for the workgroups
    // that form logits; tables first was one more memory round trip on their way).
    load_tables(tab);
    // the first gate+up item's activations are an input of the launch: staged while the other workgroups' logits arrive
    if ((int) blockIdx.x < items_g) {
        staged = ((int) blockIdx.x / a.ntile_g) / a.kk;
        stage_input<P>(a.x + (size_t) staged * a.xs, a.d, xl, a.nw, a.nw ? rn_s[staged] : 1.0f);
    }
    // No grid barrier: what the other workgroups produce here are the logits, and those say themselves when they are there.
    __syncthreads();   // every wave has used its copy of the generation
    uint32_t arrived = 0;
    if (tid == 0) {
        s_tag = my_gen + 1u;
        arrived = arrive_issue(a.sync, my_gen);
    }

    // ---- route: every workgroup ranks the logits of the token it needs itself (cheap, and nobody waits for a router) ----
    // rank(e) = how many experts come before e (larger logit, or equal logit and higher index): k_q4_route's order
    int routed = -1;
    bool weighted = true;
    auto route = [&](int t) {
        if (routed == t) return;
        routed = t;
        __syncthreads();
        const int E4 = (a.E + 3) & ~3;
        const uint32_t tag = s_tag;
        for (int e = tid; e < E4; e += 256) {
            float v = __uint_as_float(0xFF800000u);
            if (e < a.E) {   // the logit's word carries this launch's tag once its wave has stored it (bounded wait)
                unsigned long long w = ld_agent(lg64 + (size_t) t * a.E + e);
                for (uint32_t spins = 0; (uint32_t) (w >> 32) != tag; w = ld_agent(lg64 + (size_t) t * a.E + e)) {
                    __builtin_amdgcn_s_sleep(2);
                    if (++spins > a.spin) {
                        atomicExch(&a.sync[FUSED_ERR_WORD], 1u);
                        break;
                    }
                }
                v = __uint_as_float((uint32_t) w);
            }
            rv[e] = v;
        }
        __syncthreads();
        rank_logits(rv, a.E, a.k, (uint32_t*) &part[0][0], ri_s);
        __syncthreads();
        if (tid < 3 * a.k) {   // the chosen experts' slices, fetched side by side
            const int which = tid / a.k, j = tid - which * a.k;
            sl_s[which][j] = (which == 0 ? a.gate : which == 1 ? a.up : a.down)[ri_s[j]];
        }
        if (a.ns && tid >= 253) sl_s[tid - 253][a.k] = a.sh[tid - 253];
        __syncthreads();
        weighted = false;
    };
    // The routing weights of the token last routed: softmax over the k chosen logits.  Only the combine needs them, so this
    // runs after the item's first records are requested, on the first wave alone (a wave's LDS accesses stay in order, and a
    // workgroup barrier separates this from every reader and from the next route()).
    auto route_weights = [&](int t) {
        if (weighted) return;
        weighted = true;
        if (wv != 0) return;
        if (lane < a.k) rw_s[lane] = expf(rv[ri_s[lane]] - rv[ri_s[0]]);
        if (lane < a.k) {
            float top = 0.0f;
            for (int r = 0; r < a.k; ++r) top += rw_s[r];
            rw_s[lane] = rw_s[lane] / top;   // every lane has read all k values before any lane writes
        }
        if (a.ns && lane == a.k) rw_s[a.k] = 1.0f;
        if (blockIdx.x == (unsigned) t % G && lane < a.k) {   // one writer per token publishes the routing
            a.ind[(size_t) t * a.k + lane] = ri_s[lane];
            a.wt[(size_t) t * a.k + lane] = rw_s[lane];
        }
    };

    // ---- phase 2: gate + up + SwiGLU, items (pair, row tile) -------------------------------------------------------------
    __builtin_amdgcn_s_setprio(2);   // (gate + up items go before the down items of the workgroups that share the CU: every down item waits for them)
    for (int item = (int) blockIdx.x; item < items_g; item += (int) G) {
        const int p = item / a.ntile_g, tile = item - p * a.ntile_g, t = p / a.kk, j = p - t * a.kk;
        route(t);
        const int v0 = tile * a.it_g / a.ntile_g * a.rpig, v1 = min((tile + 1) * a.it_g / a.ntile_g * a.rpig, 2 * a.ff);
        const Chunk c0 = first_chunk<P, true>(sl_s[0][j], sl_s[1][j], a.Lg, a.rpig, v0, v1);
        route_weights(t);
        if (staged != t) {
            __syncthreads();
            stage_input<P>(a.x + (size_t) t * a.xs, a.d, xl, a.nw, a.nw ? rn_s[t] : 1.0f);
            staged = t;
            __syncthreads();
        }
        float* Ap = a.A + (size_t) p * a.ff;
        rows_pass<P, true, SHFL_G>(c0, sl_s[0][j], sl_s[1][j], a.Lg, a.rpig, v0, v1, tab, xl, part, gu_s,
                                   [&](int r, float gs, float us) { st_agent(Ap + r, bfr(silu_bf(bfr(gs)) * bfr(us))); });
        wg_release();   // this item's rows of A are written: one more of the pair's gate+up items is done
        __syncthreads();
        if (tid == 0 && atomicAdd(&pairw[p * 64], 1u) == (uint32_t) (a.ntile_g - 1)) {
            st_agent(&pairw[p * 64], 0u);
            st_agent(&pairw[p * 64 + 32], s_tag);   // the pair's A is complete
        }
    }
    // tokens whose routing nobody needed here still get published by their designated workgroup
    for (int t = (int) blockIdx.x; t < a.T; t += (int) G) {
        route(t);
        route_weights(t);
    }
    if (tid == 0) arrive_finish(a.sync, G, my_gen, arrived);   // here most workgroups are about to wait for their pair anyway
    __builtin_amdgcn_s_setprio(0);

    // ---- phase 3: down, then the last workgroup of a (token, row tile) sums the k experts --------------------------------
    // the first down item's records do not depend on phase 2: they are requested before the wait for the pair
    Chunk d0;
    if ((int) blockIdx.x < items_d) {
        const int p = (int) blockIdx.x / a.ntile_d, tile = (int) blockIdx.x - p * a.ntile_d, t = p / a.kk, j = p - t * a.kk;
        route(t);
        d0 = first_chunk<P, false>(sl_s[2][j], sl_s[2][j], a.Ld, a.rpid, tile * a.it_d / a.ntile_d * a.rpid, min((tile + 1) * a.it_d / a.ntile_d * a.rpid, a.d));
        route_weights(t);
    }
    // No grid barrier here: a down item needs its own pair's A only, so it waits for that pair's gate+up items (every
    // workgroup finishes its gate+up items before it waits, and the whole grid is resident, so the wait ends; bounded anyway).
    for (int item = (int) blockIdx.x; item < items_d; item += (int) G) {
        const int p = item / a.ntile_d, tile = item - p * a.ntile_d, t = p / a.kk, j = p - t * a.kk;
        route(t);
        const int v0 = tile * a.it_d / a.ntile_d * a.rpid, v1 = min((tile + 1) * a.it_d / a.ntile_d * a.rpid, a.d);
        if (item != (int) blockIdx.x) d0 = first_chunk<P, false>(sl_s[2][j], sl_s[2][j], a.Ld, a.rpid, v0, v1);
        route_weights(t);
        if (tid == 0) {   // the pair's A is complete when its last gate+up item has said so (bounded wait)
            const uint32_t tag = s_tag;
            uint32_t spins = 0;
            while (ld_agent(&pairw[p * 64 + 32]) != tag) {
                __builtin_amdgcn_s_sleep(2);
                if (++spins > a.spin) {
                    atomicExch(&a.sync[FUSED_ERR_WORD], 1u);
                    break;
                }
            }
        }
        __syncthreads();
        wg_acquire();
        stage_row<P>(a.A + (size_t) p * a.ff, a.ff, xl, true);
        staged = -1;
        __syncthreads();
        float* Dp = a.D + (size_t) p * a.d;
        rows_pass<P, false, SHFL_D>(d0, sl_s[2][j], sl_s[2][j], a.Ld, a.rpid, v0, v1, tab, xl, part, nullptr,
                                    [&](int r, float s, float) { st_agent(Dp + r, bfr(s)); });
        wg_release();
        __syncthreads();
        if (j != a.kk - 1) {
            if (tid == 0) st_agent(&dflag[((size_t) t * FUSED_TILES + tile) * 33 + j], s_tag);
        } else {   // the token's last expert sums: out = 0.5 * 0 + sum_j wt_j D_j, in j order, once the others' rows are there
            if (tid < a.kk - 1) {
                const uint32_t tag = s_tag;
                uint32_t spins = 0;
                while (ld_agent(&dflag[((size_t) t * FUSED_TILES + tile) * 33 + tid]) != tag) {
                    __builtin_amdgcn_s_sleep(2);
                    if (++spins > a.spin) {
                        atomicExch(&a.sync[FUSED_ERR_WORD], 1u);
                        break;
                    }
                }
            }
            __syncthreads();
            wg_acquire();
            for (int r = v0 + tid; r < v1; r += 256) {
                float acc = 0.0f;
                for (int jj = 0; jj < a.kk; ++jj) acc = fmaf(rw_s[jj], ld_agent(a.D + ((size_t) t * a.kk + jj) * a.d + r), acc);
                a.out[(size_t) t * a.os + r] = a.res ? bfr(a.res[(size_t) t * a.os + r] + bfr(acc)) : acc;
            }
        }
    }
}

// ---- 9 to 24 tokens: the pairs of one expert share its decoded blocks ---------------------------------------------------
// With more tokens than experts-per-token slots, several (token, expert) pairs meet on the same expert, and the decode of
// a block (nine tenths of the work) can serve them all.  Pairs are grouped by expert in runs of at most NT; an item is a
// (group, row tile); a thread decodes its chunk once and multiplies it with the NT rows of activations staged side by side
// in LDS (chunk_dot<P, NT>: per token the same chain of operations as the one-token kernel, hence the same bits).  The
// groups must be the same in every workgroup, so the routing is done once (workgroup t routes token t) and published;
// every workgroup polls the published selection (tagged with the generation) and builds the same table from it: position
// of a pair among the pairs of its expert in pair order, groups numbered in expert order.  Pair p = (token p / kk, slot p % kk),
// slots >= k are the always-on experts (expert ids E, E + 1, ...).
#define FG_MAXP 512    // pairs a launch: T * kk
#define FG_RN_WORDS 64   // the rows' RMSNorm scales behind the pairs' words of the sync area
#define FG_PRE_BYTES (1024 * 4 + FG_MAXP * 2 + 2 * (1024 + 32) * 2)   // dynamic LDS the phases before the passes use

template <int P, bool GATEUP, bool SHFL, int NT, typename Emit>
__device__ __forceinline__ void rows_pass_n(Chunk cur, const WSlice& wA, const WSlice& wB, int L, int rpi, int v0, int v1,
                                            const uint32_t* tab, const float* xl, int xstride, int nt, float* part, float2* gu, Emit emit) {
    const int tid = threadIdx.x, lr = tid / L, ch = tid - lr * L;
    const bool active = lr < rpi;
    auto fetch = [&](int vv) {   // (rows past the last: the last row's records once more)
        const int vc = min(vv, v1 - 1), r = GATEUP ? vc >> 1 : vc;
        const WSlice& w = (GATEUP && (vc & 1)) ? wB : wA;
        return load_chunk<P>(w, (uint32_t) r * (uint32_t) L + (uint32_t) ch);
    };
    int par = 0;
    for (int vb = v0; vb < v1; vb += rpi, par ^= 1) {
        const int v = vb + lr;
        const Chunk nxt = fetch(v + rpi);
        float acc[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = 0.0f;
        const int eb = (GATEUP && (v & 1)) ? wB.eb : wA.eb;
        if (active && v < v1) chunk_dot<P, NT, true>(cur, eb, tab, xl + ch * xpad<P>(), xstride, nt, acc);
        if (SHFL) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                float s = acc[t];
                for (int o = L >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o);
                if (GATEUP) {
                    const float other = __shfl_xor(s, L);
                    if (t < nt && active && ch == 0 && !(v & 1) && v < v1) {
                        if (gu) gu[t * ((v1 - v0) >> 1) + ((v - v0) >> 1)] = make_float2(s, other);   // (as in rows_pass)
                        else emit(t, v >> 1, s * NSLM_R32, other * NSLM_R32);
                    }
                } else if (t < nt && active && ch == 0 && v < v1) emit(t, v, s * NSLM_R32, 0.0f);
            }
        } else {
            float* pp = part + par * NT * 256;
#pragma unroll
            for (int t = 0; t < NT; ++t) pp[t * 256 + tid] = acc[t];
            __syncthreads();   // one barrier per iteration: part is double-buffered by iteration parity
            const int nrow = min(rpi, v1 - vb);
            if (GATEUP) {
                const int nr2 = nrow / 2;
                for (int w = tid; w < nr2 * nt; w += 256) {   // (token, row) sums: more than 256 when rows are short
                    const int t = w / nr2, r = w - t * nr2;
                    float gs = 0.0f, us = 0.0f;
                    for (int j = 0; j < L; ++j) gs += pp[t * 256 + (2 * r) * L + j];
                    for (int j = 0; j < L; ++j) us += pp[t * 256 + (2 * r + 1) * L + j];
                    emit(t, (vb >> 1) + r, gs * NSLM_R32, us * NSLM_R32);
                }
            } else {
                for (int w = tid; w < nrow * nt; w += 256) {
                    const int t = w / nrow, r = w - t * nrow;
                    float sm = 0.0f;
                    for (int j = 0; j < L; ++j) sm += pp[t * 256 + r * L + j];
                    emit(t, vb + r, sm * NSLM_R32, 0.0f);
                }
            }
        }
        cur = nxt;
    }
    if (!SHFL) __syncthreads();   // part may be reused by the next pass
    if (GATEUP && SHFL && gu) {
        __syncthreads();
        const int nr = (v1 - v0) >> 1;
        for (int i = tid; i < nr * nt; i += 256) {
            const int t = i / nr, r = i - t * nr;
            const float2 q = gu[i];
            emit(t, (v0 >> 1) + r, q.x * NSLM_R32, q.y * NSLM_R32);
        }
    }
}

template <int P, int NT, bool SHFL_G, bool SHFL_D>
__global__ void __launch_bounds__(256) k_moe_decode_grouped(FusedArgs a) {
    extern __shared__ __attribute__((aligned(16))) float xl[];   // NT rows of max(d, ff) activations, chunk-padded, side by side
    // behind them, where the launcher found room without giving up a resident workgroup: the gate and up row sums of the item in hand
    float2* const gu_s = a.gu_off > 0 ? (float2*) (xl + a.gu_off) : nullptr;
    // What only the routing and the building of the groups need lives in the same area, which the passes overwrite (the launch
    // asks for FG_PRE_BYTES at least): a kilobyte of static LDS less is a resident workgroup more at some widths.
    float* const rv = xl;                                          // [1024] a token's logits
    uint16_t* const gof = (uint16_t*) (xl + 1024);                 // [FG_MAXP] a pair's position among its expert's pairs
    uint16_t* const cnt_s = gof + FG_MAXP;                         // [1024 + 32] per expert: pairs
    uint16_t* const base_s = cnt_s + 1024 + 32;                    // [1024 + 32] per expert: first group
    __shared__ uint32_t tab[NSLM_TAB_WORDS];
    __shared__ float part[2 * NT * 256];
    __shared__ float rw_s[33];
    __shared__ int ri_s[33];
    __shared__ WSlice sl_s[3];
    __shared__ int s_flag, s_ng;
    __shared__ float rn_s[FG_MAXT], nred[4];
    __shared__ __attribute__((aligned(16))) uint16_t pe[FG_MAXP + 8];   // a pair's expert
    __shared__ uint16_t gm[FG_MAXP * NT];   // a group's members
    __shared__ uint8_t gn[FG_MAXP];   // a group's number of members
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const uint32_t G = (uint32_t) a.grid;
    const int P_ = a.T * a.kk, NE = a.E + a.ns;
    const int xsg = a.Lg * xpad<P>(), xsd = a.Ld * xpad<P>();   // LDS floats between two rows of activations
    // (fixed places, whatever the launch's rows and widths: launches of different sizes share the area, and every word
    // but the scales is back at zero when a launch ends)
    float* rnpub = (float*) (a.sync + FUSED_SYNC_WORDS);
    uint32_t* grpc = a.sync + FUSED_SYNC_WORDS + FG_RN_WORDS;                     // [group][3][32]: arrivals, ready, done
    uint32_t* tick = grpc + (size_t) FG_MAXP * 96;                                // [token][down row tile]
    // the generation (all sense words are equal); the workgroup arrives, without waiting, further down
    const uint32_t my_gen = ld_agent(a.sync + 32 * (BAR_GROUPS + 1 + blockIdx.x % BAR_GROUPS));
    const uint32_t tag = my_gen + 1u;
    unsigned long long* lg64 = (unsigned long long*) (a.sync + FUSED_LOGIT_WORDS);
    unsigned long long* ind64 = (unsigned long long*) (a.sync + FUSED_IND_WORDS);
    load_tables(tab);

    // ---- phase 1: router logits, one wave per (token, expert) -------------------------------------------------------------
    if (a.nw) {   // the scales of the rows whose logits this workgroup forms (uniform over the workgroup)
        for (int base = (int) blockIdx.x * 4; base < a.T * a.E; base += (int) G * 4) {
            const int t0 = base / a.E, t1 = min(base + 3, a.T * a.E - 1) / a.E;
            for (int t = t0; t <= t1; ++t) {
                const float r = row_rnorm(a.x + (size_t) t * a.xs, a.d, a.neps, nred);
                if (tid == 0) rn_s[t] = r;
            }
        }
        __syncthreads();
    }
    for (int item = (int) blockIdx.x * 4 + wv; item < a.T * a.E; item += (int) G * 4) {
        const int t = item / a.E, e = item - t * a.E;
        const float lv = router_logit(a.rw + (size_t) e * a.d, a.x + (size_t) t * a.xs, a.d, a.nw, a.nw ? rn_s[t] : 1.0f);
        if (lane == 0) {
            st_agent(a.logits + item, lv);
            st_agent(lg64 + item, (unsigned long long) __float_as_uint(lv) | (unsigned long long) tag << 32);
        }
        if (t == 0 && lane >= a.T && lane < FG_MAXT) st_agent(lg64 + (size_t) lane * a.E + e, 0ull);   // rows this launch does not use
    }
    // No grid barriers: the logits and the published routing carry the launch's generation and are polled where they are
    // needed.  The generation moves on with the workgroups' arrivals, which nobody waits for.
    __syncthreads();   // every wave has its copy of the generation
    uint32_t arrived = 0;
    if (tid == 0) arrived = arrive_issue(a.sync, my_gen);

    // ---- routing, once per token: workgroup t % G ranks token t and publishes selection, weights and the row's scale ----
    for (int t = (int) blockIdx.x; t < a.T; t += (int) G) {
        __syncthreads();
        const int E4 = (a.E + 3) & ~3;
        for (int e = tid; e < E4; e += 256) {
            float v = __uint_as_float(0xFF800000u);
            if (e < a.E) {   // bounded wait for the logit's wave
                unsigned long long w = ld_agent(lg64 + (size_t) t * a.E + e);
                for (uint32_t spins = 0; (uint32_t) (w >> 32) != tag; w = ld_agent(lg64 + (size_t) t * a.E + e)) {
                    __builtin_amdgcn_s_sleep(2);
                    if (++spins > a.spin) {
                        atomicExch(&a.sync[FUSED_ERR_WORD], 1u);
                        break;
                    }
                }
                v = __uint_as_float((uint32_t) w);
            }
            rv[e] = v;
        }
        __syncthreads();
        rank_logits(rv, a.E, a.k, (uint32_t*) part, ri_s);
        __syncthreads();
        if (a.nw) {
            const float r = row_rnorm(a.x + (size_t) t * a.xs, a.d, a.neps, nred);
            if (tid == 0) st_agent(rnpub + t, r);
        }
        wg_release();   // the scale is stored before the selection that announces it
        __syncthreads();
        if (wv == 0) {
            if (lane < a.k) rw_s[lane] = expf(rv[ri_s[lane]] - rv[ri_s[0]]);
            if (lane < a.k) {
                float top = 0.0f;
                for (int r = 0; r < a.k; ++r) top += rw_s[r];
                st_agent((uint32_t*) a.ind + (size_t) t * a.k + lane, (uint32_t) ri_s[lane]);
                st_agent(a.wt + (size_t) t * a.k + lane, rw_s[lane] / top);
            }
            wg_release();   // weights before the tagged selection
            if (lane < a.k) st_agent(ind64 + (size_t) t * 32 + lane, (unsigned long long) (uint32_t) ri_s[lane] | (unsigned long long) tag << 32);
        }
    }

    // ---- the groups: the same table in every workgroup ----------------------------------------------------------------------
    for (int i = tid; i < NE; i += 256) cnt_s[i] = 0;
    for (int p = tid; p < P_ + 8; p += 256) {
        const int pc = min(p, P_ - 1), t = pc / a.kk, j = pc - t * a.kk;
        int e = a.E + (j - a.k);
        if (j < a.k) {   // bounded wait for the token's routing
            unsigned long long w = ld_agent(ind64 + (size_t) t * 32 + j);
            for (uint32_t spins = 0; (uint32_t) (w >> 32) != tag; w = ld_agent(ind64 + (size_t) t * 32 + j)) {
                __builtin_amdgcn_s_sleep(2);
                if (++spins > a.spin) {
                    atomicExch(&a.sync[FUSED_ERR_WORD], 1u);
                    w = 0;   // expert 0: the results are void, the indices stay in range
                    break;
                }
            }
            e = (int) (uint32_t) w;
        }
        if (p < FG_MAXP + 8) pe[p] = (uint16_t) (p < P_ ? e : 0xFFFF);   // the table is read eight at a time: pad with "no expert"
    }
    __syncthreads();
    wg_acquire();   // the selections have been seen: the scales and weights stored before them are there
    if (a.nw && tid < a.T) rn_s[tid] = ld_agent(rnpub + tid);
    __syncthreads();
    for (int p = tid; p < P_; p += 256) {   // position among the pairs of the same expert (in pair order), and their number
        const uint32_t e = pe[p];
        int before = 0, all = 0;
        for (int q0 = 0; q0 < P_; q0 += 8) {
            const uint4 w = *(const uint4*) &pe[q0];
            const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int m0 = (ww[u] & 0xFFFFu) == e ? 1 : 0, m1 = (ww[u] >> 16) == e ? 1 : 0;
                all += m0 + m1;
                before += (q0 + 2 * u < p ? m0 : 0) + (q0 + 2 * u + 1 < p ? m1 : 0);
            }
        }
        gof[p] = (uint16_t) before;
        cnt_s[e] = (uint16_t) all;   // every pair of the expert writes the same number
    }
    __syncthreads();
    {   // groups before expert e: exclusive sums of ceil(cnt / NT), five experts a thread
        int own[5], sum = 0;
#pragma unroll
        for (int u = 0; u < 5; ++u) {
            const int e = tid * 5 + u;
            own[u] = e < NE ? (cnt_s[e] + NT - 1) / NT : 0;
            sum += own[u];
        }
        int inc = sum;
        for (int o = 1; o < 64; o <<= 1) {
            const int v = __shfl_up(inc, o);
            if (lane >= o) inc += v;
        }
        if (lane == 63) ri_s[wv] = inc;   // the waves' totals (ri_s is free after the routing)
        __syncthreads();
        int off = inc - sum;
        for (int w = 0; w < wv; ++w) off += ri_s[w];
#pragma unroll
        for (int u = 0; u < 5; ++u) {
            const int e = tid * 5 + u;
            if (e < NE) base_s[e] = (uint16_t) off;
            off += own[u];
        }
        if (tid == 255) s_ng = off;
    }
    __syncthreads();
    for (int p = tid; p < P_; p += 256) {
        const int e = pe[p], pos = gof[p], g = base_s[e] + pos / NT;
        gm[g * NT + pos % NT] = (uint16_t) p;
        if (pos % NT == 0) gn[g] = (uint8_t) min(NT, (int) cnt_s[e] - pos);
    }
    __syncthreads();
    const int NG = s_ng, items_g = NG * a.ntile_g, items_d = NG * a.ntile_d;

    // ---- gate + up + SwiGLU: items (group, row tile) ---------------------------------------------------------------------------
    int staged_g = -1;
    __builtin_amdgcn_s_setprio(2);   // (as in k_moe_decode: gate + up items before the down items that wait for them)
    for (int item = (int) blockIdx.x; item < items_g; item += (int) G) {
        const int g = item / a.ntile_g, tile = item - g * a.ntile_g, nt = gn[g], e = pe[gm[g * NT]];
        const int v0 = tile * a.it_g / a.ntile_g * a.rpig, v1 = min((tile + 1) * a.it_g / a.ntile_g * a.rpig, 2 * a.ff);
        __syncthreads();
        if (tid < 2) sl_s[tid] = e < a.E ? (tid == 0 ? a.gate : a.up)[e] : a.sh[tid];
        __syncthreads();
        const Chunk c0 = first_chunk<P, true>(sl_s[0], sl_s[1], a.Lg, a.rpig, v0, v1);
        if (staged_g != g) {
            for (int m = 0; m < nt; ++m) {
                const int t = gm[g * NT + m] / a.kk;
                stage_input<P>(a.x + (size_t) t * a.xs, a.d, xl + m * xsg, a.nw, a.nw ? rn_s[t] : 1.0f);
            }
            staged_g = g;
            __syncthreads();
        }
        auto put_a = [&](int m, int r, float gs, float us) {
            st_agent(a.A + (size_t) gm[g * NT + m] * a.ff + r, bfr(silu_bf(bfr(gs)) * bfr(us)));
        };
        if (nt == 1)   // a group of one: the one-token loop, no second row of multiply-adds
            rows_pass<P, true, SHFL_G>(c0, sl_s[0], sl_s[1], a.Lg, a.rpig, v0, v1, tab, xl, (float (*)[256]) part, gu_s,
                                       [&](int r, float gs, float us) { put_a(0, r, gs, us); });
        else
            rows_pass_n<P, true, SHFL_G, NT>(c0, sl_s[0], sl_s[1], a.Lg, a.rpig, v0, v1, tab, xl, xsg, nt, part, gu_s, put_a);
        wg_release();   // this item's rows of A are written: one more of the group's gate+up items is done
        __syncthreads();
        if (tid == 0 && atomicAdd(&grpc[g * 96], 1u) == (uint32_t) (a.ntile_g - 1)) st_agent(&grpc[g * 96 + 32], 1u);
    }

    if (tid == 0) arrive_finish(a.sync, G, my_gen, arrived);
    __builtin_amdgcn_s_setprio(0);

    // ---- down, then the last workgroup of a (token, row tile) sums the token's experts ------------------------------------
    for (int item = (int) blockIdx.x; item < items_d; item += (int) G) {
        const int g = item / a.ntile_d, tile = item - g * a.ntile_d, nt = gn[g], e = pe[gm[g * NT]];
        const int v0 = tile * a.it_d / a.ntile_d * a.rpid, v1 = min((tile + 1) * a.it_d / a.ntile_d * a.rpid, a.d);
        __syncthreads();
        if (tid == 0) sl_s[2] = e < a.E ? a.down[e] : a.sh[2];
        __syncthreads();
        const Chunk d0 = first_chunk<P, false>(sl_s[2], sl_s[2], a.Ld, a.rpid, v0, v1);
        if (tid == 0) {   // the group's A is complete when its last gate+up item has said so (bounded wait)
            uint32_t spins = 0;
            while (ld_agent(&grpc[g * 96 + 32]) == 0u) {
                __builtin_amdgcn_s_sleep(2);
                if (++spins > a.spin) {
                    atomicExch(&a.sync[FUSED_ERR_WORD], 1u);
                    break;
                }
            }
        }
        __syncthreads();
        wg_acquire();
        for (int m = 0; m < nt; ++m) stage_row<P>(a.A + (size_t) gm[g * NT + m] * a.ff, a.ff, xl + m * xsd, true);
        staged_g = -1;
        __syncthreads();
        auto put_d = [&](int m, int r, float sm, float) { st_agent(a.D + (size_t) gm[g * NT + m] * a.d + r, bfr(sm)); };
        if (nt == 1)
            rows_pass<P, false, SHFL_D>(d0, sl_s[2], sl_s[2], a.Ld, a.rpid, v0, v1, tab, xl, (float (*)[256]) part, nullptr,
                                        [&](int r, float sm, float) { put_d(0, r, sm, 0.0f); });
        else
            rows_pass_n<P, false, SHFL_D, NT>(d0, sl_s[2], sl_s[2], a.Ld, a.rpid, v0, v1, tab, xl, xsd, nt, part, nullptr, put_d);
        wg_release();
        for (int m = 0; m < nt; ++m) {   // one ticket per member's (token, row tile); the token's last arrival sums its experts
            const int t = gm[g * NT + m] / a.kk;
            __syncthreads();
            if (tid == 0) s_flag = atomicAdd(&tick[t * a.ntile_d + tile], 1u) == (uint32_t) (a.kk - 1);
            if (tid < a.kk) rw_s[tid] = tid < a.k ? ld_agent(a.wt + (size_t) t * a.k + tid) : 1.0f;
            __syncthreads();
            if (s_flag) {
                wg_acquire();
                for (int r = v0 + tid; r < v1; r += 256) {
                    float acc = 0.0f;
                    for (int jj = 0; jj < a.kk; ++jj) acc = fmaf(rw_s[jj], ld_agent(a.D + ((size_t) t * a.kk + jj) * a.d + r), acc);
                    a.out[(size_t) t * a.os + r] = a.res ? bfr(a.res[(size_t) t * a.os + r] + bfr(acc)) : acc;
                }
                if (tid == 0) st_agent(&tick[t * a.ntile_d + tile], 0u);
            }
        }
        // the group's last down item leaves its three words at zero for the next launch
        if (tid == 0 && atomicAdd(&grpc[g * 96 + 64], 1u) == (uint32_t) (a.ntile_d - 1)) {
            st_agent(&grpc[g * 96], 0u);
            st_agent(&grpc[g * 96 + 32], 0u);
            st_agent(&grpc[g * 96 + 64], 0u);
        }
    }
}

std::atomic<uint32_t> g_spin_limit{SPIN_LIMIT};   // (any thread may set it while another launches)

int g_kernel_choice = 0;   // kc_moe_decode_kernel: 0 the faster kernel for the shape, 1 a workgroup an item, 2 a workgroup a CU where it fits

int cu_count() { return fused_cu_count(); }

bool shape_of(int K, bool gateup, int* L, int* rpi, bool* shfl) {
    if (K % 64 || K / 64 > 128) return false;
    const int l = K / 64;
    int r = 256 / l;
    if (gateup) r &= ~1;
    if (r < 1) return false;
    *L = l;
    *rpi = r;
    *shfl = (l & (l - 1)) == 0 && l <= (gateup ? 32 : 64);
    return true;
}

// Items per pair (or group) of a phase of `iters` iterations, `units` pairs, at most gmax workgroups.
// one_round: the count that gives the busiest workgroup the least to do when every workgroup takes its items one after the
// other (an item's set-up priced at a third of an iteration, unequal items at half an iteration: workgroups i, i + 256, ...
// share a CU, so the long items of a regular pattern meet on the same CUs); up to `slack` items more than the workgroups still
// count as one round.
int pick_one_round(int units, int iters, int gmax, int nmax, int slack = 0, int setup = 2) {
    int best = 1;
    long best_cost = -1;
    for (int n = 1; n <= iters && n <= nmax; ++n) {
        const long over = (long) units * n - slack, rounds = over <= gmax ? 1 : (over + gmax - 1) / gmax, per = (iters + n - 1) / n;
        const long cost = rounds * (6 * per + (iters % n ? 3 : 0) + setup);
        if (best_cost < 0 || cost <= best_cost) { best = n; best_cost = cost; }   // ties: more, shorter items
    }
    return best;
}
// by_cu_load: the count that gives the busiest CU the least to do (items go round the workgroups, the workgroups round the
// CUs, and a CU's waves share its issue slots, so a CU is as late as the sum of its items, plus one item for the end of
// the phase, when the CU is no longer full), with fewer than five workgroups a CU priced for the latencies they no longer hide.
int pick_by_cu_load(int units, int iters, int cus, int nmax) {
    static const int thin[6] = {200, 160, 130, 115, 103, 100};
    int best = 1;
    long best_cost = -1;
    for (int n = 1; n <= iters && n <= nmax; ++n) {
        const long items = (long) units * n, per = (iters + n - 1) / n, on_cu = (items + cus - 1) / cus;
        const long cost = (on_cu * (6 * per + (iters % n ? 3 : 0) + 2) + 2 * per) * thin[items / cus < 5 ? items / cus : 5];
        if (best_cost < 0 || cost <= best_cost) { best = n; best_cost = cost; }
    }
    return best;
}

#define GU_ROWS 128   // SwiGLU rows of an item whose two sums wait in LDS for the end of the item's row loop (per-item kernel)
// the fewest items a pair at which an item's rows fit that area
int gu_min_tiles(const FusedArgs& a) {
    int n = 1;
    while (n < FUSED_TILES && (long) ((a.it_g + n - 1) / n) * a.rpig / 2 > GU_ROWS) ++n;
    return n;
}

template <int P>
int launch_fused(hipStream_t st, FusedArgs& a, bool sg, bool sd, size_t lds) {
    a.gu_off = (int) (lds / sizeof(float));
    lds += GU_ROWS * sizeof(float2);
    // One token is at most a few hundred items more than three workgroups a CU hold (C2: 784): that launch may use the
    // registers of four waves a SIMD instead of five (107 instead of 96, no spills: 35.0 -> 34.5 us).  With the P = 4 column form the
    // same holds up to four tokens (C2, four / five waves, us: 2 tokens 41.4 / 45.8, 3: 55.6 / 56.3, 4: 66.4 / 69.8, 5: 85.9 / 80.3,
    // 8: 115.1 / 110.8; P = 3, C3: 2 tokens 166.5 / 157.7, 4: 272.6 / 263.7).
    const bool few = a.T == 1 || (P == 4 && a.T <= 4);
    void (*kern)(FusedArgs) = few ? (sg ? (sd ? k_moe_decode<P, true, true, 4> : k_moe_decode<P, true, false, 4>)
                                        : (sd ? k_moe_decode<P, false, true, 4> : k_moe_decode<P, false, false, 4>))
                                  : (sg ? (sd ? k_moe_decode<P, true, true, 5> : k_moe_decode<P, true, false, 5>)
                                        : (sd ? k_moe_decode<P, false, true, 5> : k_moe_decode<P, false, false, 5>));
    // resident workgroups per CU, by kernel variant, for the largest LDS request seen (the request grows with max(d, ff): a launch
    // that asks for more than the cached answer covered asks the occupancy calculator again, and raises the kernel's limit above 48 KB)
    static int cached[2][2][2] = {};
    static size_t cached_lds[2][2][2] = {};
    int& per_cu = cached[few][sg][sd];
    if (!per_cu || lds > cached_lds[few][sg][sd]) {
        if (lds > 48 * 1024 && hipFuncSetAttribute((const void*) kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds) != hipSuccess) return -1;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, 256, lds) != hipSuccess || per_cu < 1) {
            per_cu = 0;
            return -1;
        }
        cached_lds[few][sg][sd] = lds;
    }
    // The grid must be resident at once (workgroups wait for each other's data): at most what the device holds, and no more than
    // five workgroups a CU (the most that was tried).  Items per pair (an item = a run of a pair's iterations, as
    // equal as whole iterations allow).  Down items, and every item of one token: one round (measured on C2, one token: 96 x 2
    // gate+up iterations and 98 x 1 down iterations a pair on 784 workgroups, 40.1 us; 96 unequal down items on 768
    // workgroups: 42.9; 8 tokens with 32 instead of 20 down items a pair: 144 against 131 us - a down item waits for its
    // pair, and a second round of them waits behind the first).  Gate+up items of several tokens: by the CUs' load, which
    // takes more, shorter items than one round holds (C2, items a pair -> us; 4 tokens: 24 -> 82.2, 40 -> 79.6, 64 -> 78.0;
    // 6 tokens: 24 -> 120.2, 32 -> 111.4, 48 -> 115.2; 8 tokens: 20 -> 135.4, 32 -> 131.2, 48 -> 138.9); where the row sums go
    // through LDS (C3) one round stayed ahead.
    const int gmax = (per_cu < 5 ? per_cu : 5) * cu_count(), P_ = a.T * a.kk;
    a.ntile_g = few || !sg ? pick_one_round(P_, a.it_g, gmax, FUSED_TILES) : pick_by_cu_load(P_, a.it_g, cu_count(), FUSED_TILES);
    // (a down item's set-up - the wait for its pair, the staging of A - priced at two thirds of an iteration: at a third, six
    // tokens of C2 took two rounds of 49 two-iteration items a pair, 81.6 us, where one round of 26 takes 76.5)
    a.ntile_d = pick_one_round(P_, a.it_d, gmax, FUSED_TILES, 0, 4);
    if (a.ntile_g < gu_min_tiles(a)) a.ntile_g = gu_min_tiles(a);
    if ((long) ((a.it_g + a.ntile_g - 1) / a.ntile_g) * a.rpig / 2 > GU_ROWS) return -1;
    const long items = (long) P_ * (a.ntile_g > a.ntile_d ? a.ntile_g : a.ntile_d);
    int grid = items < gmax ? (int) items : gmax;
    if (grid < 1) grid = 1;
    a.grid = grid;
    hipLaunchKernelGGL(kern, dim3((unsigned) grid), dim3(256), lds, st, a);
    host_note_launch();
    return 0;
}


template <int P, int NT>
int launch_grouped(hipStream_t st, FusedArgs& a, bool sg, bool sd) {
    void (*kern)(FusedArgs) = sg ? (sd ? k_moe_decode_grouped<P, NT, true, true> : k_moe_decode_grouped<P, NT, true, false>)
                                 : (sd ? k_moe_decode_grouped<P, NT, false, true> : k_moe_decode_grouped<P, NT, false, false>);
    const int lmax = a.Lg > a.Ld ? a.Lg : a.Ld;
    size_t lds = (size_t) NT * lmax * xpad<P>() * sizeof(float);
    if (lds < FG_PRE_BYTES) lds = FG_PRE_BYTES;

    static int cached[2][2] = {{0, 0}, {0, 0}};   // resident workgroups per CU, by kernel variant, for the largest request seen
    static size_t cached_lds[2][2] = {{0, 0}, {0, 0}};
    int& per_cu = cached[sg][sd];
    if (!per_cu || lds > cached_lds[sg][sd]) {
        if (lds > 48 * 1024 && hipFuncSetAttribute((const void*) kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds) != hipSuccess) return -1;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, 256, lds) != hipSuccess || per_cu < 1) {
            per_cu = 0;
            return -1;
        }
        cached_lds[sg][sd] = lds;
    }
    // The groups are formed on the device; the host sizes the items for the number it expects from a uniform routing:
    // the experts that receive a pair at all, plus the always-on experts' runs of NT tokens.  Four workgroups a CU are
    // resident, and items for about five were fastest (C2, 16 rows, 81 groups on 1024 workgroups, gate+up items a group
    // -> us: 12 -> 228, 14 -> 223, 16 -> 212, 18 -> 216, 20 -> 230; down items: 10 -> 207, 14 -> 202, 24 -> 208, 49 -> 214):
    // one round that may run over by three eighths.
    const double pairs = (double) a.T * a.k;
    int groups = (int) (a.E * (1.0 - pow(1.0 - 1.0 / a.E, pairs)) + 0.5) + a.ns * ((a.T + NT - 1) / NT);
    if (groups < 1) groups = 1;
    const int gmax = (per_cu < 5 ? per_cu : 5) * cu_count();
    a.ntile_g = pick_one_round(groups, a.it_g, gmax, a.it_g, 3 * gmax / 8);
    a.ntile_d = pick_one_round(groups, a.it_d, gmax, a.it_d, 3 * gmax / 8);
    const long items = (long) groups * (a.ntile_g > a.ntile_d ? a.ntile_g : a.ntile_d);
    int grid = items < gmax ? (int) items : gmax;
    if (grid < a.T) grid = a.T < gmax ? a.T : gmax;
    a.grid = grid;
    // Room behind the staged rows for the row sums of a gate + up item (so that SwiGLU and the store run once behind the item's
    // row loop), taken only where it costs no resident workgroup: with 4 KB for it C2's 16-row step lost one of four and 6 %.
    a.gu_off = 0;
    if (sg) {
        const size_t base = (lds + 15) & ~(size_t) 15;
        const size_t want = base + (size_t) NT * ((a.it_g + a.ntile_g - 1) / a.ntile_g) * (a.rpig / 2) * sizeof(float2);
        static size_t ok_lds[2] = {0, 0}, bad_lds[2] = {~(size_t) 0, ~(size_t) 0};   // by sd: the largest request known to keep per_cu, the smallest known not to
        bool fits = want <= ok_lds[sd];
        if (!fits && want < bad_lds[sd] && want <= 48 * 1024) {
            int n = 0;
            fits = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, 256, want) == hipSuccess && n >= per_cu;
            if (fits) ok_lds[sd] = want;
            else bad_lds[sd] = want;
        }
        if (fits) {
            a.gu_off = (int) (base / sizeof(float));
            lds = want;
        }
    }
    hipLaunchKernelGGL(kern, dim3((unsigned) grid), dim3(256), lds, st, a);
    host_note_launch();
    return 0;
}

// ---- the step without a workspace argument -------------------------------------------------------------------------------
// kc_moe_decode_static keeps what kc_moe_decode's caller brings along (logits, A, D, the sync words) in one array in device
// memory that the library's code object itself holds, so the call allocates nothing: for callers that cannot call
// hipMalloc (stream capture, tight serving loops, harnesses that forbid it).  Every GPU has its own copy of the array at
// its own address; host code may not use the array's name as an address (that name is a host-side stand-in), so the address
// on the current device is asked for once per device with hipGetSymbolAddress and kept.
// Layout (uint32 words): [0, NA_SYNC_WORDS) the sync words, laid out as kc_moe_decode's with the ticket area sized
// NA_TICK_WORDS - zero when the code object is loaded, and kept consistent by the kernels from launch to launch;
// [NA_SYNC_WORDS, + NA_DATA_WORDS) logits [T][n_exp], A [T kk][ff], D [T kk][d], each starting on a 256-byte boundary,
// overwritten by every call before it is read.
#define NA_TICK_WORDS (FG_MAXT * 1024)
#define NA_SYNC_WORDS (((FUSED_SYNC_WORDS + FG_RN_WORDS + FG_MAXP * 96 + NA_TICK_WORDS) + 63) & ~63)
#define NA_DATA_WORDS (1 << 20)   // 4 MiB
#define NA_MAX_DEVICES 64
static __device__ __align__(256) uint32_t scratch[NA_SYNC_WORDS + NA_DATA_WORDS];

uint32_t* scratch_on_this_device() {
    static uint32_t* at[NA_MAX_DEVICES] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= NA_MAX_DEVICES) return nullptr;
    if (!at[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
        at[dev] = (uint32_t*) p;   // (two threads racing here store the same address)
    }
    return at[dev];
}
__global__ void __launch_bounds__(256) k_words_zero(uint32_t* p, size_t n) {
    for (size_t i = (size_t) blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t) gridDim.x * 256) p[i] = 0u;
}
__global__ void k_word_copy(uint32_t* dst, const uint32_t* src) { *dst = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

}   // namespace

extern "C" {

size_t kc_moe_decode_sync_words(int T, int d) { return FUSED_SYNC_WORDS + FG_RN_WORDS + (size_t) FG_MAXP * 96 + (size_t) T * (size_t) (d + 1); }
int kc_moe_decode_max_rows(void) { return FG_MAXT; }
int kc_moe_decode_error_word(void) { return FUSED_ERR_WORD; }

int kc_moe_decode(kc_stream_t s, int fmt, const uint16_t* router_w, const WSlice* gate, const WSlice* up, const WSlice* down,
                  int n_exp, int top_k, int d, int ff, const float* x, int xs, int T, float* out, int os, float* logits,
                  int32_t* ind, float* wt, float* A, float* D, uint32_t* sync) {
    return kc_moe_decode_layer(s, fmt, router_w, gate, up, down, n_exp, top_k, d, ff, x, xs, T, out, os, logits, ind, wt, A, D, sync, NULL, NULL, NULL, 0.0f);
}

int kc_moe_decode_layer(kc_stream_t s, int fmt, const uint16_t* router_w, const WSlice* gate, const WSlice* up, const WSlice* down,
                        int n_exp, int top_k, int d, int ff, const float* x, int xs, int T, float* out, int os, float* logits,
                        int32_t* ind, float* wt, float* A, float* D, uint32_t* sync, const WSlice* shared, const float* res, const float* norm_w,
                        float norm_eps) {
    if (T < 1 || T > FG_MAXT || top_k < 1 || top_k > 32 || n_exp > 1024 || n_exp < top_k) return -1;
    if (T > MV_MAXT && T * (top_k + (shared ? 1 : 0)) > FG_MAXP) return -1;
    if (fmt != MF_SEED4P4 && fmt != MF_SEED4) return -1;
    if (host_store_f32() || d % 8 || ((uintptr_t) x & 15u) || xs % 4 || ((uintptr_t) router_w & 15u)) return -1;
    FusedArgs a = {};
    a.spin = g_spin_limit;
    bool sg, sd;
    if (!shape_of(d, true, &a.Lg, &a.rpig, &sg) || !shape_of(ff, false, &a.Ld, &a.rpid, &sd)) return -1;
    a.rw = router_w; a.gate = gate; a.up = up; a.down = down; a.x = x; a.out = out; a.logits = logits; a.wt = wt; a.A = A;
    a.D = D; a.ind = ind; a.sync = sync; a.E = n_exp; a.k = top_k; a.d = d; a.ff = ff; a.T = T; a.xs = xs; a.os = os;
    a.ns = shared ? 1 : 0; a.kk = top_k + a.ns; a.res = res; a.nw = norm_w; a.neps = norm_eps;
    if (norm_w && (d > 256 * 16 || ((uintptr_t) norm_w & 15u))) return -1;
    for (int i = 0; i < 3 && shared; ++i) a.sh[i] = shared[i];
    a.it_g = (2 * ff + a.rpig - 1) / a.rpig;
    a.it_d = (d + a.rpid - 1) / a.rpid;
    if (T > MV_MAXT || (shared && T >= FG_MINT_SHARED && sg && T * a.kk <= FG_MAXP)) {
        // More rows than the per-pair kernel takes: pairs grouped by expert, two to a decode.  Measured against the grouped
        // GEMMs of the separate launches (C2, 16 rows: 199 against 268 us; 20 rows: 242 against 295; 24 rows: 278 against 305;
        // 28 rows: 335 against 327, so the limit is 24); with four to a decode (402 against 338 us at 32 rows) and where the gate+up row sums go through LDS (C3's 45 chunks a row: 1129 against 753 us) the GEMMs
        // win, so those shapes are left to them.  With an always-on expert every row brings a pair on the same expert, and
        // the grouped kernel is already ahead of the per-pair one at 5 rows (whole model, 5 rows: 4.05 against 4.18 ms, 8 rows:
        // 5.37 against 5.70; 4 rows: 3.85 against 3.68); without
        // one the two are level at 8 rows (130 us) and the per-pair kernel is ahead below.
        if (!sg) return -1;
        return fmt == MF_SEED4P4 ? launch_grouped<4, 2>((hipStream_t) s, a, sg, sd) : launch_grouped<3, 2>((hipStream_t) s, a, sg, sd);
    }
    // one workgroup per CU: ahead at one token everywhere, at two where the step is large or P = 3 (us, a workgroup per CU / per
    // item, records from HBM.  C2: 1 token 19.9 / 25.2, 2: 36.6 / 35.5, 3: 48.4 / 45.5; C2's shape in P = 3: 24.6 / 26.3,
    // 39.4 / 43.5, 54.7 / 50.9, 4: 70.0 / 63.8; 256 experts of 4096 x 1024: 45.8 / 54.9, 80.7 / 90.6, 168.8 / 168.9; C3, whose rows
    // of 45 chunks make that kernel's passes go by iterations of the workgroup: 55.0 / 67.3, 100.9 / 104.7, 146.9 / 147.6,
    // 192.6 / 186.2)
    const bool cu_two = fmt != MF_SEED4P4 || (sg && (long) top_k * d * ff >= 24L << 20);
    if ((g_kernel_choice == 2 || (g_kernel_choice == 0 && T <= (cu_two ? 2 : 1))) && launch_moe_decode_cu((hipStream_t) s, a, fmt == MF_SEED4P4 ? 4 : 3, sd) == 0) return 0;
    const int kmax = d > ff ? d : ff;
    size_t lds = (size_t) (kmax / 64) * (fmt == MF_SEED4P4 ? xpad<4>() : xpad<3>()) * sizeof(float);
    return fmt == MF_SEED4P4 ? launch_fused<4>((hipStream_t) s, a, sg, sd, lds) : launch_fused<3>((hipStream_t) s, a, sg, sd, lds);
}

void kc_moe_decode_spin_limit(unsigned polls) { g_spin_limit = polls ? polls : SPIN_LIMIT; }
void kc_moe_decode_kernel(int which) { g_kernel_choice = which >= 0 && which <= 2 ? which : 0; }

int kc_moe_decode_static(kc_stream_t s, int fmt, const uint16_t* router_w, const WSlice* gate, const WSlice* up, const WSlice* down,
                         int n_exp, int top_k, int d, int ff, const float* x, int xs, int T, float* out, int os, int32_t* ind, float* wt,
                         uint32_t* status, int clear) {
    if (T < 1 || T > FG_MAXT || n_exp < 1 || n_exp > 1024 || top_k < 1 || top_k > 32 || d < 8 || ff < 8) return -1;
    // what the call needs of the array: the ticket words of the grouped kernel (rows x down iterations at most) and the data
    int Ld, rpid;
    bool sd;
    if (!shape_of(ff, false, &Ld, &rpid, &sd)) return -1;
    const size_t it_d = ((size_t) d + rpid - 1) / rpid, pairs = (size_t) T * top_k;
    const size_t wl = ((size_t) T * n_exp + 63) & ~(size_t) 63, wa = (pairs * ff + 63) & ~(size_t) 63, wd = (pairs * d + 63) & ~(size_t) 63;
    if ((size_t) T * it_d > NA_TICK_WORDS || wl + wa + wd > NA_DATA_WORDS) {
        host_note_unsupported();
        return -2;
    }
    uint32_t* base = scratch_on_this_device();
    if (!base) {
        host_note_unsupported();
        return -3;
    }
    // what kc_moe_decode_layer would refuse is refused here, before anything is launched (the clear included)
    {
        int L1, r1;
        bool s1;
        if ((fmt != MF_SEED4P4 && fmt != MF_SEED4) || n_exp < top_k || host_store_f32() || d % 8 || ((uintptr_t) x & 15u) || xs % 4 || ((uintptr_t) router_w & 15u) ||
            !shape_of(d, true, &L1, &r1, &s1) || (T > MV_MAXT && (!s1 || T * top_k > FG_MAXP)))
            return -1;
    }
    if (clear) {   // by a kernel, not a memset node: callers may be capturing
        hipLaunchKernelGGL(k_words_zero, dim3(64), dim3(256), 0, (hipStream_t) s, base, (size_t) NA_SYNC_WORDS);
        host_note_launch();
    }
    float* logits = (float*) (base + NA_SYNC_WORDS);
    float* A = logits + wl;
    float* D = A + wa;
    const int rc = kc_moe_decode_layer(s, fmt, router_w, gate, up, down, n_exp, top_k, d, ff, x, xs, T, out, os, logits, ind, wt, A, D, base, NULL, NULL, NULL,
                                       0.0f);
    if (rc == 0 && status) {
        hipLaunchKernelGGL(k_word_copy, dim3(1), dim3(1), 0, (hipStream_t) s, status, (const uint32_t*) base + FUSED_ERR_WORD);
        host_note_launch();
    }
    return rc;
}

}   // extern "C"

