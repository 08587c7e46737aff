// nslm_fused_cu.hip - the routed-expert decode step of up to MV_MAXT tokens as one persistent kernel with ONE workgroup per CU
// (k_moe_decode_cu).  Same arithmetic, instruction for instruction, as the kernel of nslm_fused.hip (and so as the five
// separate launches, engine/qwen4_cuda.c:1023-1083): what differs is who computes what, and how the results travel.
//
//   - A workgroup is 16 waves and owns its CU.  What every workgroup of the other kernel does for itself - polling and
//     ranking the logits, caching the chosen experts' slices, staging the input in the form the matvec reads - happens once a
//     CU, and the waves of a CU go through the phases together: no wave is left alone on its SIMD in a phase's tail.
//   - Gate + up: a token's (pair, row) tasks are dealt evenly, a contiguous run to each CU; inside the CU a wave takes the next
//     task when it is ready for one (the row's chunks over the wave's lanes, row sums by xor-shuffles), no workgroup barrier
//     inside the pass.
//   - The SwiGLU outputs A are the only data that crosses CUs.  A CU's waves count their tasks off in LDS as their stores of a
//     token's values are acknowledged; the wave that completes the count arrives for the CU on a two-level counter (groups of
//     CUs, then the groups), and the last arrival of all raises the token's ready words, one per group of CUs, which one lane
//     per CU polls.  Then every CU reads the token's A once, as BF16.  (Values that carried the generation themselves, polled
//     in place by every thread that needs them, were a round trip shorter on paper; in practice 256 CUs polling 48 KB starved
//     the very stores they were waiting for, and so did 256 CUs polling one word per CU.)
//   - Down: CU c owns output rows [c rpc, (c + 1) rpc) of EVERY pair of the token, so the weighted sum of the experts is a
//     sum inside the workgroup - no second exchange and no waiting for another CU behind the down rows.
//   - Several tokens: gate + up of all tokens first, then the down passes; a token's A has been on its way for a whole pass
//     when its down pass needs it, so only a one-token launch waits for the exchange.
//   - Every instruction outside the row loops counts (a CU's waves all execute it at the same moment): what can be computed
//     on the host arrives in the arguments, and no index is formed by an integer division.
//   - Rows whose chunks do not fit a wave as a power of two (45 chunks, say) take both passes by iterations of the whole
//     workgroup instead - the token's chunks dealt to the threads as one list, the row sums through LDS in chunk order, one barrier
//     an iteration - with 1012 of 1024 threads busy where a 256-thread workgroup fills 4 of 5.7 possible rows.
// Shapes: a row of at most 256 chunks, T * pairs * ff <= FUSED_XA_MAX, the workgroup's LDS <= 160 KB less the table.  Other
// shapes stay with the kernel of nslm_fused.hip.
#include "nslm_fused_dev.h"

using namespace nslm;

namespace {

#define CU_LDS_MAX (160 * 1024 - NSLM_TAB_WORDS * 4)   // dynamic LDS: what the kernel's own table leaves of a CU's 160 KB
#define CU_LDS_MIN (82 * 1024)   // more than half a CU's LDS: two of these workgroups never share a CU
#define CU_LG 4                  // router logits a CU forms
#define CU_PRE_MAXE 256          // experts whose slice tables are copied to LDS while the logits are on their way

// x / d for x < 2^32 / d', d' = the power of two >= d: one multiply (m = ceil(2^32 / d); d = 1: m = 0 stands for x itself)
struct FastDiv {
    uint32_t m;
};
inline FastDiv fastdiv_of(uint32_t d) { return FastDiv{d <= 1 ? 0u : (uint32_t) ((0x100000000ull + d - 1) / d)}; }
__device__ __forceinline__ uint32_t operator/(uint32_t x, FastDiv f) { return f.m ? __umulhi(x, f.m) : x; }

// What the host works out once per launch (offsets into the workgroup's dynamic LDS in 4-byte words, each a multiple of 4)
struct CuParams {
    int xg;      // [T][Lg * xpad] the tokens' inputs in the form the gate + up matvec reads
    int xd;      // [kk][Ld * xpad] one token's A, all pairs, in the form the down matvec reads
    int scr;     // [4 NTHR] passes by iterations: the chunks' sums of three iterations, the first iteration's slots twice
    int pk;      // [T][KP] ranking: the logits' keys
    int rv;      // [T][E4] the logits
    int dsum;    // [kk][rpc] the down rows of the token in hand, rounded to BF16
    int ri;      // [T][32] expert by rank
    int rw;      // [T][36] weight by rank (+ the shared expert's 1)
    int rn;      // [MV_MAXT + 16] the rows' RMSNorm scales, the waves' partial sums of a norm
    int cnt;     // [2][MV_MAXT] per token: this CU's gate + up tasks handed out / finished
    int av;      // [T][n_c * vpt][2] this CU's gate and up row sums until the token's last task is done
    int lgs;     // [16] the logits this CU forms, until one wave stores them
    int sel;     // [3 + T * kk * 3] WSlice: the shared expert's slices; with more than CU_PRE_MAXE experts the pairs' slices
    int pre;     // [3][E] WSlice: the layer's slice tables (E <= CU_PRE_MAXE)
    int total;
    int G;                // CUs = workgroups
    int lgL;              // log2 of the chunks in a gate / up row (Lg)
    int rpw, tpp, Wt;     // gate + up: virtual rows a wave-task, tasks a pair, tasks a token
    int n_c, ncu_act;     // tasks a CU and token; CUs that have tasks
    int nit_g;            // gate + up where a row's chunks do not fit a wave: iterations of the workgroup a token
    int ltail_g, ltail_d; // P = 3, passes by iterations: log2 of the lanes that share a chunk in the pass's last iteration (0: a thread a chunk there too)
    int rpc;              // down: output rows a CU owns
    int rpi, rows_t, nit; // down: (pair, row)s an iteration of the workgroup, (pair, row)s a token and CU, iterations a token
    int nbp;              // blocks of 8 in a row of A
    int vpt, lgV;         // SwiGLU outputs a task (rpw / 2) and its log2
    int E4, KP;           // E padded to 4; keys a token (E padded to 16)
    FastDiv by_tpp, by_rpc, by_Ld, by_Lg, by_nbp, by_kk, by_E, by_ring;
};

// NORM: the launch normalises its input (a.nw); launches that do not are compiled without what that path adds.
template <int P, bool SHFL_G, bool SHFL_D, int NTHR, bool NORM>
__global__ void __launch_bounds__(NTHR) k_moe_decode_cu(FusedArgs a, CuParams c) {
    constexpr int NW = NTHR / 64, XP = xpad<P>();
    extern __shared__ __attribute__((aligned(16))) float dyn[];
    __shared__ uint32_t tab[NSLM_TAB_WORDS];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int G = c.G, T = a.T, E = a.E, kk = a.kk, Lg = a.Lg, Ld = a.Ld, E4 = c.E4, rpc = c.rpc;
    float* const xg = dyn + c.xg;
    float* const xd = dyn + c.xd;
    uint32_t* const scr = (uint32_t*) (dyn + c.scr);
    float* const rv = dyn + c.rv;
    float* const dsum = dyn + c.dsum;
    int* const ri_s = (int*) (dyn + c.ri);
    float* const rw_s = dyn + c.rw;
    float* const rn_s = dyn + c.rn;
    uint32_t* const cnt_s = (uint32_t*) (dyn + c.cnt);
    WSlice* const sel = (WSlice*) (dyn + c.sel);
    uint4* const pre = (uint4*) (dyn + c.pre);
    uint32_t* const pk = (uint32_t*) (dyn + c.pk);
    float* const avs = dyn + c.av;
    float* const lgs = dyn + c.lgs;
    const bool preload = E <= CU_PRE_MAXE;

    // ---- what does not depend on the routing: generation, tables, slice tables, norm scales, the staged input, the logits ----
    const uint32_t gen = ld_agent(a.sync + 32 * (BAR_GROUPS + 1 + blockIdx.x % BAR_GROUPS));
    const TableWords<NTHR> tw = tables_fetch<NTHR>();
    // the layer's three slice tables, 16 bytes of each a thread (unconditional: with more experts than the LDS copy takes,
    // pieces that are not kept)
    static_assert(CU_PRE_MAXE * sizeof(WSlice) / 16 <= NTHR, "a thread a piece covers a slice table");
    const int per = E * (int) (sizeof(WSlice) / 16);   // 16-byte pieces of a table
    const int piece = min(tid, per - 1);
    const uint4 pw0 = ((const uint4*) a.gate)[piece], pw1 = ((const uint4*) a.up)[piece], pw2 = ((const uint4*) a.down)[piece];
    loads_issued();
    // With a norm, this CU's router rows - the operand of a logit that comes from HBM - are requested before the rows' scales are
    // formed, not behind their two barriers (the inputs and the norm weights, which the CU has read by then, follow there).
    const int lg0 = CU_LG * (int) blockIdx.x, lgn = max(0, min(CU_LG, T * E - lg0));
    const int nb_x = a.d >> 3;
    const bool early = NORM && nb_x <= 256;   // (a logit's operands in one request a lane)
    RouterRegs rr;
    if (early && wv >= NW - lgn) {
        const int item = lg0 + NW - 1 - wv, e = item - (int) ((uint32_t) item / c.by_E) * E;
        router_fetch_row(rr, a.rw + (size_t) e * a.d, nb_x, lane);
    }
    if (a.nw) {   // the rows' scales, as the norm kernel sums them: 256 threads, thread i takes x[i], x[i + 256], ..
        for (int t = 0; t < T; ++t) {
            float ss = 0.0f;
            if (tid < 256) {
                const float* xi = a.x + (size_t) t * a.xs;
#pragma unroll
                for (int j = 0; j < NSLM_NORM_NR; ++j) {
                    const int k = tid + j * 256;
                    const float xv = xi[min(k, a.d - 1)];
                    const float v = k < a.d ? xv : 0.0f;
                    ss = fmaf(v, v, ss);
                }
                for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
                if (lane == 0) rn_s[MV_MAXT + wv] = ss;
            }
            __syncthreads();
            if (tid == 0) rn_s[t] = rsqrtf(((rn_s[MV_MAXT] + rn_s[MV_MAXT + 1]) + (rn_s[MV_MAXT + 2] + rn_s[MV_MAXT + 3])) / (float) a.d + a.neps);
            __syncthreads();
        }
    }
    const uint32_t tag = gen + 1u;
    unsigned long long* lg64 = (unsigned long long*) (a.sync + FUSED_CULG_WORDS);   // [FUSED_CULG_LINES][16]: a line a CU's logits
    uint16_t* const xa16 = (uint16_t*) (a.sync + FUSED_XA_WORDS);   // [token][pair][ff]: the SwiGLU outputs as BF16 bits
    if (tid < 2 * MV_MAXT) cnt_s[tid] = 0u;
    // Router logits: CU c forms items [CU_LG c, CU_LG c + CU_LG) of the [token][expert] table, a wave an item (the last waves:
    // the first ones stage the input meanwhile), and gathers them in LDS; one wave then stores them into the CU's own 128-byte
    // line (item i at word 16 (i / CU_LG) + i % CU_LG), which is written once, by one instruction.  (A line that 16 CUs each
    // wrote a word of, while every CU polled it, took 1.7 us from the last store to the first CU that saw all of it; a line
    // written once is seen 0.4 us later.  Few items a CU: a CU's vector-memory path takes 1.5 us to load twelve router rows.)
    if (wv >= NW - lgn) {
        const int u = NW - 1 - wv, item = lg0 + u, t = (int) ((uint32_t) item / c.by_E), e = item - t * E;
        if (early) router_fetch_input(rr, a.x + (size_t) t * a.xs, nb_x, a.nw, lane);
        const float lv = early ? router_sum(router_add(rr, nb_x, true, rn_s[t], lane, 0.0f))
                               : router_logit(a.rw + (size_t) e * a.d, a.x + (size_t) t * a.xs, a.d, a.nw, a.nw ? rn_s[t] : 1.0f);
        if (lane == 0) lgs[u] = lv;
    }
    tables_store<NTHR>(tab, tw);
    if (preload && tid < per) {
        pre[tid] = pw0;
        pre[per + tid] = pw1;
        pre[2 * per + tid] = pw2;
    }
    {   // the tokens' inputs, normalised on the way when nw is given (the values kq4_norm1p would have stored)
        const int nb = a.d >> 3;
        for (int t = 0; t < T; ++t)
            for (int b = tid; b < nb; b += NTHR) {
                const float* src = a.x + (size_t) t * a.xs + (size_t) b * 8;
                const float4 q0 = *(const float4*) src, q1 = *(const float4*) (src + 4);
                float v[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
                if (a.nw) {
                    const float4 w0 = *(const float4*) (a.nw + (size_t) b * 8), w1 = *(const float4*) (a.nw + (size_t) b * 8 + 4);
                    const float w[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
                    const float rn = rn_s[t];
#pragma unroll
                    for (int cc = 0; cc < 8; ++cc) v[cc] = v[cc] * rn * (1.0f + w[cc]);
                }
                store_block<P>(xg + t * (Lg * XP), b, v);
            }
    }
    if (a.ns && tid < 3) {   // the shared expert's slices (field by field: a struct copy of a kernel argument goes through scratch memory)
#define PUT_SH(i) do { WSlice* q = &sel[i]; q->p[0] = a.sh[i].p[0]; q->p[1] = a.sh[i].p[1]; q->p[2] = a.sh[i].p[2]; q->p[3] = a.sh[i].p[3]; q->eb = a.sh[i].eb; q->gs = a.sh[i].gs; } while (0)
        if (tid == 0) PUT_SH(0);
        if (tid == 1) PUT_SH(1);
        if (tid == 2) PUT_SH(2);
#undef PUT_SH
    }
    __syncthreads();   // every wave has used its copy of the generation; tables, slice tables, inputs and this CU's logits are in LDS
    if (tid < lgn) {
        const float lv = lgs[tid];
        st_agent(lg64 + 16 * (int) blockIdx.x + tid, (unsigned long long) __float_as_uint(lv) | (unsigned long long) tag << 32);
        a.logits[lg0 + tid] = lv;
    }
    uint32_t arrived = 0;
    if (tid == 0) arrived = arrive_issue(a.sync, gen);

    // Every wait of this kernel is a bounded poll; a thread that has once given up (error word set, results void) waits for
    // nothing any more, so the grid drains quickly.
    uint32_t polls_left = a.spin;
    // ---- the logits of every token, polled until they carry this launch's generation (bounded) -----------------------------
    // rank(e) = how many experts come before e (larger logit, or equal logit and higher index): k_q4_route's order.  The
    // logits are BF16 values, so (order-preserving upper half of the float | index) is a unique 32-bit key and rank = number of
    // larger keys; the thread that has polled a logit leaves its key.
    for (int t = 0; t < T; ++t)
        for (int e = tid; e < c.KP; e += NTHR) {
            float v = __uint_as_float(0xFF800000u);
            uint32_t key = 0u;   // absent: below every real key
            if (e < E) {
                const int item = t * E + e;
                const unsigned long long* lw = lg64 + 16 * (item / CU_LG) + item % CU_LG;
                unsigned long long w = ld_agent(lw);
                for (; (uint32_t) (w >> 32) != tag; w = ld_agent(lw)) {
                    __builtin_amdgcn_s_sleep(2);
                    if (polls_left == 0 || --polls_left == 0) {
                        atomicExch(&a.sync[FUSED_ERR_WORD], 1u);
                        a.sync[FUSED_ERR_WORD + 1] = 0x10000000u | (uint32_t) (t * E + e);
                        break;
                    }
                }
                v = __uint_as_float((uint32_t) w);
                const uint32_t b = __float_as_uint(v + 0.0f);   // -0 counts as +0, as in a float compare
                key = ((b ^ ((uint32_t) ((int32_t) b >> 31) | 0x80000000u)) & 0xFFFF0000u) | (uint32_t) e;
            }
            if (e < E4) rv[t * E4 + e] = v;
            pk[t * c.KP + e] = key;
        }
    __syncthreads();
    // four lanes an expert, each counts over a quarter of the token's keys (read four at a time as LDS broadcasts); the quarters
    // meet by two shuffles, so a rank needs no second pass through LDS
    {
        const int part = lane & 3, q4 = c.KP >> 2;
        for (int t = 0; t < T; ++t)
            for (int e0 = 16 * wv; e0 < E; e0 += NTHR / 4) {   // (a wave 16 experts: uniform over the wave, whose shuffles these are)
                const int e = e0 + (lane >> 2);
                const uint32_t* kt = pk + t * c.KP;
                const uint32_t ke = kt[min(e, c.KP - 1)];
                int g = 0;
#pragma unroll 2
                for (int o = part * q4; o < (part + 1) * q4; o += 4) {
                    const uint4 q = *(const uint4*) &kt[o];
                    g += (q.x > ke ? 1 : 0) + (q.y > ke ? 1 : 0) + (q.z > ke ? 1 : 0) + (q.w > ke ? 1 : 0);
                }
                g += __shfl_xor(g, 1);
                g += __shfl_xor(g, 2);
                if (part == 0 && e < E && g < a.k) ri_s[t * 32 + g] = e;
            }
    }
    __syncthreads();
    // the routing weights (softmax over the k chosen logits): wave t for token t (the combine reads them, barriers later)
    if (wv < T) {
        const int t = wv;
        float* rw = rw_s + t * 36;
        const int* ri = ri_s + t * 32;
        if (lane < a.k) rw[lane] = expf(rv[t * E4 + ri[lane]] - rv[t * E4 + ri[0]]);
        if (lane < a.k) {
            float top = 0.0f;
            for (int r = 0; r < a.k; ++r) top += rw[r];
            rw[lane] = rw[lane] / top;   // every lane has read all k values before any lane writes
        }
        if (a.ns && lane == a.k) rw[a.k] = 1.0f;
        if ((int) blockIdx.x == t % G && lane < a.k) {   // one writer per token publishes the routing
            a.ind[(size_t) t * a.k + lane] = ri[lane];
            a.wt[(size_t) t * a.k + lane] = rw[lane];
        }
    }
    if (!preload) {   // more experts than the LDS copy of the slice tables takes: the pairs' slices from memory
        for (int p = tid; p < T * kk; p += NTHR) {
            const int t = (int) ((uint32_t) p / c.by_kk), j = p - t * kk;
            if (j < a.k) {
                const int e = ri_s[t * 32 + j];
                sel[3 + p * 3] = a.gate[e];
                sel[3 + p * 3 + 1] = a.up[e];
                sel[3 + p * 3 + 2] = a.down[e];
            }
        }
        __syncthreads();
    }
    // slice `which` (0 gate, 1 up, 2 down) of pair (t, j), in LDS
    auto slice = [&](int t, int j, int which) -> const WSlice& {
        if (j >= a.k) return sel[which];
        if (preload) return ((const WSlice*) pre)[which * E + ri_s[t * 32 + j]];
        return sel[3 + (t * kk + j) * 3 + which];
    };

    // (the down pass's threads and records, here already: a wave that has run out of gate + up tasks requests its first down records
    // in the slot where its next task's records would have been requested, a whole task ahead of their use)
    const int r0 = (int) blockIdx.x * rpc, nr = max(0, min(rpc, a.d - r0));
    const int dl = (int) ((uint32_t) tid / c.by_Ld), dch = tid - dl * Ld;
    // Passes by iterations (rows whose chunks are no power of two inside a wave) deal a token's chunks to the threads as one
    // list - thread i of iteration it takes chunk it NTHR + i, rows end where they end - so only the pass's last iteration can
    // be short.  A thread a chunk would make that one as long as a full one; where its chunks fit the workgroup 2, 4 or 8 times
    // over (P = 3), as many adjacent lanes share a chunk there (chunk_dot_split: the same bits).  The chunk sums wait for their
    // row's last in a ring of three iterations: a row's chunks lie in at most two, and the third is being written.  The ring's first
    // NTHR slots are kept twice, the copy behind its end, so that a row's sums are read from consecutive words wherever it starts.
    constexpr int RING = 3 * NTHR;
    const int ltg = P == 3 ? c.ltail_g : 0, ltd = P == 3 ? c.ltail_d : 0;
    struct Deal {
        int f, row, ch, sub;   // chunk of the token's list, its row and place in the row, the thread's place among the chunk's lanes
        bool tail;
    };
    auto deal = [&](int it, int nit, int lt, int L, FastDiv by_L) {
        Deal q;
        q.tail = lt && it == nit - 1;
        q.f = it * NTHR + (q.tail ? tid >> lt : tid);
        q.row = (int) ((uint32_t) q.f / by_L);
        q.ch = q.f - q.row * L;
        q.sub = q.tail ? tid & ((1 << lt) - 1) : 0;
        return q;
    };
    auto ring_slot = [&](int f) { return f - (int) ((uint32_t) f / c.by_ring) * RING; };
    auto ring_put = [&](float* ring, int f, float v) {
        const int sl = ring_slot(f);
        ring[sl] = v;
        if (sl < NTHR) ring[sl + RING] = v;
    };
    // (down rows whose chunks are a power of two inside a wave: whole rows an iteration, the thread's place in them fixed)
    auto deal_d = [&](int it) {
        if constexpr (SHFL_D) return Deal{it * NTHR + tid, it * c.rpi + dl, dch, 0, false};
        else return deal(it, c.nit, ltd, Ld, c.by_Ld);
    };
    auto fetch_d = [&](int t, int it) {   // (unconditional too: rows and pairs past the end are clamped)
        const Deal q = deal_d(it);
        const int g = min(q.row, c.rows_t - 1), jj = (int) ((uint32_t) g / c.by_rpc), rr = g - jj * rpc;
        const WSlice& w = slice(min(t, T - 1), jj, 2);
        return load_chunk<P>(w, (uint32_t) min(r0 + rr, a.d - 1) * (uint32_t) Ld + (uint32_t) q.ch);
    };
    Chunk dcur;
    // ---- gate + up + SwiGLU: a wave a task = 64 / Lg virtual rows (2r = gate row r, 2r + 1 = up row r) of one pair -------------
    const int q_lo = (int) blockIdx.x * c.n_c, n_loc = max(0, min(c.n_c, c.Wt - q_lo));   // this CU's tasks a token
    const int lr = lane >> c.lgL, ch = lane & (Lg - 1);
    // a lane's share of a task's addresses, formed once: gate or up (a task's rows come in pairs: Lg <= 32), and where in the
    // task's records the lane reads
    const int wsel = lr & 1;
    const uint32_t lane_unit = (uint32_t) (lr >> 1) * (uint32_t) Lg + (uint32_t) ch;
    const WSlice* const lane_pre = (const WSlice*) pre + wsel * E;
    auto slice_gu = [&](int t, int j) -> const WSlice& {   // slice(t, j, wsel) with the lane's part taken out
        if (j >= a.k) return sel[wsel];
        if (preload) return lane_pre[__builtin_amdgcn_readfirstlane(ri_s[t * 32 + j])];
        return sel[3 + (t * kk + j) * 3 + wsel];
    };
    const int nav = c.n_c << c.lgV;   // SwiGLU outputs a CU and token at most
    // One wave stores the CU's values of a token - SwiGLU of the two row sums, as BF16 for the other CUs and as f32 for the caller -
    // and, once the stores are acknowledged, arrives for the CU; the last CU of all raises the token's ready words.
    auto publish = [&](int t) {
        for (int u = lane; u < (n_loc << c.lgV); u += 64) {
            const int qq = q_lo + (u >> c.lgV), jj = (int) ((uint32_t) qq / c.by_tpp);
            const size_t at = (size_t) (t * kk + jj) * a.ff + (size_t) (((qq - jj * c.tpp) << c.lgV) + (u & (c.vpt - 1)));
            const float2 gu = *(const float2*) &avs[2 * (t * nav + u)];
            const float av = bfr(silu_bf(bfr(gu.x * NSLM_R32)) * bfr(gu.y * NSLM_R32));
            st_agent(xa16 + at, (uint16_t) (__float_as_uint(av) >> 16));
            a.A[at] = av;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (lane == 0) {
            uint32_t* bar = a.sync + FUSED_CU_WORDS + t * FUSED_CU_TOKEN_WORDS;   // [32 group lines][root line][32 ready lines]
            const uint32_t g = blockIdx.x % BAR_GROUPS, ncu = (uint32_t) c.ncu_act, ng = ncu < BAR_GROUPS ? ncu : BAR_GROUPS;
            const uint32_t in_group = (ncu - g + BAR_GROUPS - 1) / BAR_GROUPS;
            if (atomicAdd(bar + 32 * g, 1u) == in_group - 1) {
                st_agent(bar + 32 * g, 0u);
                if (atomicAdd(bar + 32 * BAR_GROUPS, 1u) == ng - 1) {
                    st_agent(bar + 32 * BAR_GROUPS, 0u);
#pragma unroll
                    for (uint32_t r = 0; r < BAR_GROUPS; ++r) st_agent(bar + 32 * (BAR_GROUPS + 1 + r), tag);
                }
            }
        }
    };
    if constexpr (SHFL_G) {
        // One token: wave w takes the CU's tasks w, w + 16, ..  Waves w, w + 4, w + 8, w + 12 share a SIMD, so the SIMDs' task counts
        // differ by one at most, and the first records are requested without a counter's round trip.  (Handed out in the order
        // of asking, the second round's tasks went to the waves that happened to finish first - on 28 % of the CUs three of them
        // on one SIMD, whose last task then ended 0.8 us after the other CUs' - and some such CU is always the step's last.)
        // More tokens: a token's tasks go to whichever wave asks next, because the wave that stores a token's values is busy for
        // most of a task's time and falls behind a fixed schedule (3 tokens: 51.5 against 48.7 us).
        // A wave asks for its next task before it computes the current one, so that task's records travel meanwhile.
        // Task = (token, index in the CU's run); token T = none left.
        int ct = 0, ci = wv - NW;   // the token this wave draws from; one token: the wave's last task
        auto claim = [&](int& t, int& i) {
            if (T == 1) {
                ci += NW;
                if (ci < n_loc) { t = 0; i = ci; }
                else { t = T; i = 0; }
                return;
            }
            for (;;) {
                if (ct >= T || n_loc == 0) { t = T; i = 0; return; }
                uint32_t got = 0;
                if (lane == 0) got = atomicAdd(&cnt_s[ct], 1u);
                got = __builtin_amdgcn_readfirstlane(got);
                if ((int) got < n_loc) { t = ct; i = (int) got; return; }
                ++ct;
            }
        };
        // (the loads are unconditional: a load under a condition keeps the compiler from counting the loads in flight, and it
        // then waits for the next task's records before it computes the current one.  Past the last task the slot requests
        // the thread's first down records instead.)
        const Deal q_d = deal_d(0);   // (fetch_d(0, 0)'s records)
        const int g_d = min(q_d.row, c.rows_t - 1), jj_d = (int) ((uint32_t) g_d / c.by_rpc);
        const uint32_t unit_d = (uint32_t) min(r0 + g_d - jj_d * rpc, a.d - 1) * (uint32_t) Ld + (uint32_t) q_d.ch;
        auto fetch = [&](int t, int i) {
            const bool ok = t < T;
            const int q = ok ? q_lo + i : 0, j = (int) ((uint32_t) q / c.by_tpp), r = (q - j * c.tpp) << c.lgV;   // the task's first SwiGLU row
            const WSlice& w = ok ? slice_gu(t, j) : slice(0, jj_d, 2);
            return load_chunk<P>(w, ok ? (uint32_t) r * (uint32_t) Lg + lane_unit : unit_d);
        };
        int t, i;
        claim(t, i);
        Chunk cur = fetch(t, i);
        __builtin_amdgcn_s_setprio(2);   // (tasks, and the store of the CU's values, go before the waves that have run out of tasks)
        uint32_t mine = 0;   // tasks of the token in hand this wave has finished
        while (t < T) {
            int tn, inx;
            claim(tn, inx);
            const Chunk nxt = fetch(tn, inx);
            const int q = q_lo + i, j = (int) ((uint32_t) q / c.by_tpp);
            float acc[1] = {0.0f};
            chunk_dot<P, 1, true>(cur, slice_gu(t, j).eb, tab, xg + t * (Lg * XP) + ch * XP, 0, 1, acc);
            float s = acc[0];
            for (int o = Lg >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o);
            const float other = __shfl_xor(s, Lg);
            // (results leave after the loop: a store here would sit in front of the wait for the next task's records)
            // (the two row sums; SwiGLU is left to the wave that stores the CU's values: one wave's instructions instead of every task's)
            if (ch == 0 && !wsel) *(float2*) &avs[2 * (t * nav + (i << c.lgV) + (lr >> 1))] = make_float2(s, other);
            ++mine;
            if (tn != t) {   // The wave's last task of token t: it adds its tasks to the CU's count.  The wave that completes the
                             // count stores the CU's values of the token (as BF16 for the other CUs, as f32 for the caller), and once
                             // they are acknowledged arrives for the CU; the last CU of all raises the token's ready words.
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                uint32_t before = 0;
                if (lane == 0) before = atomicAdd(&cnt_s[MV_MAXT + t], mine);
                before = __builtin_amdgcn_readfirstlane(before);
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                if (before + mine == (uint32_t) n_loc) publish(t);
                mine = 0;
            }
            cur = nxt;
            t = tn;
            i = inx;
        }
        dcur = cur;   // (the last request of the loop, or of the first claim: the down records)
        __builtin_amdgcn_s_setprio(0);
    }
    else if (n_loc > 0) {
        // Rows whose chunks do not fit a wave (a row of 45 chunks, say): the pass goes by iterations of the whole workgroup over the
        // chunks of the CU's virtual rows (2r = gate row r, 2r + 1 = up row r of its run of SwiGLU rows, a "task" being one such
        // pair of rows), the row sums through LDS in chunk order (the separate launches' order), one workgroup barrier an iteration.
        float* const partg = (float*) scr;   // [RING + NTHR]
        const int nch = 2 * n_loc * Lg;      // this CU's chunks a token
        auto fetch_g = [&](int t, int it) {   // (unconditional: rows past the CU's last are clamped)
            const Deal q = deal(it, c.nit_g, ltg, Lg, c.by_Lg);
            const int v = min(q.row, 2 * n_loc - 1), u = q_lo + (v >> 1), j = (int) ((uint32_t) u / c.by_tpp);
            return load_chunk<P>(slice(min(t, T - 1), j, v & 1), (uint32_t) (u - j * c.tpp) * (uint32_t) Lg + (uint32_t) q.ch);
        };
        Chunk cur = fetch_g(0, 0);
        for (int t = 0; t < T; ++t) {
            int pd = 0;   // SwiGLU rows of the token whose two sums are formed
            for (int it = 0; it < c.nit_g; ++it) {
                const bool last = it + 1 == c.nit_g;
                const Chunk nxt = fetch_g(last ? t + 1 : t, last ? 0 : it + 1);
                const Deal q = deal(it, c.nit_g, ltg, Lg, c.by_Lg);
                const int vc = min(q.row, 2 * n_loc - 1), u = q_lo + (vc >> 1), j = (int) ((uint32_t) u / c.by_tpp);
                const float* xq = xg + t * (Lg * XP) + q.ch * XP;
                if (!q.tail) {
                    float acc[1] = {0.0f};
                    if (q.f < nch) chunk_dot<P, 1, true>(cur, slice(t, j, vc & 1).eb, tab, xq, 0, 1, acc);
                    ring_put(partg, q.f, acc[0]);
                } else if constexpr (P == 3) {
                    if (q.f < nch) {   // (the lanes of a shared chunk take this branch together)
                        const float sum = chunk_dot_split(cur, slice(t, j, vc & 1).eb, tab, xq, q.sub, ltg);
                        if (q.sub == (1 << ltg) - 1) ring_put(partg, q.f, sum);
                    }
                }
                __syncthreads();
                // the SwiGLU rows whose last chunk this iteration held, a thread each
                const int pe = last ? n_loc : min(n_loc, (int) ((uint32_t) ((it + 1) * NTHR) / c.by_Lg) >> 1);
                if (tid < pe - pd) {
                    // the two rows' partial sums in chunk order; sixteen of each are read before the first is added (a chunk past the row's
                    // last counts +0, which leaves the sum's bits alone)
                    const float* const pg = partg + ring_slot(2 * (pd + tid) * Lg);   // (2 Lg <= NTHR: the copy covers the two rows)
                    auto at = [&](int o) { return pg[o]; };
                    float gs = 0.0f, us = 0.0f;
                    for (int c0 = 0; c0 < Lg; c0 += 16) {
                        float pv[16], pu[16];
#pragma unroll
                        for (int cc = 0; cc < 16; ++cc) {
                            pv[cc] = at(min(c0 + cc, Lg - 1));
                            pu[cc] = at(Lg + min(c0 + cc, Lg - 1));
                        }
#pragma unroll
                        for (int cc = 0; cc < 16; ++cc) {
                            gs += c0 + cc < Lg ? pv[cc] : 0.0f;
                            us += c0 + cc < Lg ? pu[cc] : 0.0f;
                        }
                    }
                    *(float2*) &avs[2 * (t * nav + pd + tid)] = make_float2(gs, us);
                }
                pd = pe;
                cur = nxt;
            }
            __syncthreads();   // the token's row sums are all in LDS (and the ring is free for the next token's chunks)
            if (wv == NW - 1) publish(t);
        }
    }
    if constexpr (!SHFL_G) dcur = fetch_d(0, 0);
    // Housekeeping, off the critical path: the lines of this kernel's logits table that this launch did not write, and the
    // other step kernels' table (every launch of theirs rewrites all of it, the rows it does not use with zero: a word that
    // does not carry the current generation is then never older than one launch), are left at zero.
    {
        unsigned long long* lgo = (unsigned long long*) (a.sync + FUSED_LOGIT_WORDS);
        const int used = (T * E + CU_LG - 1) / CU_LG;
        for (int w = (int) blockIdx.x * NTHR + tid; w < FG_MAXT * E; w += G * NTHR) st_agent(lgo + w, 0ull);
        for (int w = (int) blockIdx.x * NTHR + tid; w < (FUSED_CULG_LINES - used) * 16; w += G * NTHR) st_agent(lg64 + 16 * used + w, 0ull);
    }
    if (tid == 0) arrive_finish(a.sync, (uint32_t) G, gen, arrived);

    // ---- down: CU c owns rows [c rpc, (c + 1) rpc) of every pair; a thread a chunk of a (pair, row); then the experts' sum --------
    float* part = (float*) scr;
    // the token's A is complete when the last CU has raised the ready words (lane 0 polls the word of this CU's group, bounded);
    // then all pairs' A of the token, 16 bytes (a block of 8 values) a thread, staged as the down matvec reads it
    // (block b of the token = block b % nbp of pair b / nbp: a pair's row is whole chunks, so the token's pairs lie in xd as one row)
    auto wait_stage = [&](int t) {
        if (tid == 0) {
            const uint32_t* rdy = a.sync + FUSED_CU_WORDS + t * FUSED_CU_TOKEN_WORDS + 32 * (BAR_GROUPS + 1 + blockIdx.x % BAR_GROUPS);
            while (ld_agent(rdy) != tag) {
                __builtin_amdgcn_s_sleep(2);
                if (polls_left == 0 || --polls_left == 0) {
                    atomicExch(&a.sync[FUSED_ERR_WORD], 1u);
                    a.sync[FUSED_ERR_WORD + 1] = 0x20000000u | (uint32_t) t;
                    break;
                }
            }
        }
        __syncthreads();
        for (int b = tid; b < kk * c.nbp; b += NTHR) {
            const unsigned long long* src = (const unsigned long long*) (xa16 + (size_t) t * kk * a.ff + (size_t) b * 8);
            const unsigned long long lo = ld_agent(src), hi = ld_agent(src + 1);
            const float v[8] = {bf((uint32_t) lo & 0xFFFFu), bf((uint32_t) (lo >> 16) & 0xFFFFu), bf((uint32_t) (lo >> 32) & 0xFFFFu), bf((uint32_t) (lo >> 48)),
                                bf((uint32_t) hi & 0xFFFFu), bf((uint32_t) (hi >> 16) & 0xFFFFu), bf((uint32_t) (hi >> 32) & 0xFFFFu), bf((uint32_t) (hi >> 48))};
            store_block<P>(xd, b, v);
        }
        __syncthreads();
    };
    // the rows' sums of one iteration from the threads' chunk sums, rounded as the separate launches round them
    int ud = 0;   // (pair, row)s of the token in hand whose sums are formed
    auto rows_out = [&](int t, int it, float acc0, bool ok, int g, int j, int rr, bool last, int slot) {   // slot: the thread's chunk in the token's list (< 0: it has none to store)
        if (SHFL_D) {
            float s = acc0;
            for (int o = Ld >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o);
            if (ok && dch == 0) {
                const float dv = bfr(s * NSLM_R32);
                dsum[g] = dv;
                a.D[((size_t) t * kk + j) * a.d + r0 + rr] = dv;
            }
        } else {
            // (the chunk sums wait in the ring, as the gate + up pass's: the next iteration's chunks are decoded while this one's
            // rows are summed)
            if (slot >= 0) ring_put(part, slot, acc0);
            __syncthreads();
            // the (pair, row)s whose last chunk this iteration held, a thread each
            const int ue = last ? c.rows_t : min(c.rows_t, (int) ((uint32_t) ((it + 1) * NTHR) / c.by_Ld));
            const int gs = ud + tid, js = min((int) ((uint32_t) gs / c.by_rpc), kk - 1), rs = gs - (int) ((uint32_t) gs / c.by_rpc) * rpc;
            if (tid < ue - ud && rs < nr) {
                // the row's partial sums in chunk order; sixteen are read before the first is added (a chunk past the row's
                // last counts +0, which leaves the sum's bits alone)
                const float* const pg = part + ring_slot(gs * Ld);   // (Ld <= NTHR: the copy covers the row)
                float s = 0.0f;
                for (int c0 = 0; c0 < Ld; c0 += 16) {
                    float pv[16];
#pragma unroll
                    for (int cc = 0; cc < 16; ++cc) pv[cc] = pg[min(c0 + cc, Ld - 1)];
#pragma unroll
                    for (int cc = 0; cc < 16; ++cc) s += c0 + cc < Ld ? pv[cc] : 0.0f;
                }
                const float dv = bfr(s * NSLM_R32);
                dsum[gs] = dv;
                a.D[((size_t) t * kk + js) * a.d + r0 + rs] = dv;
            }
            ud = ue;
        }
    };
    // out = sum_j wt_j D_j in j order (kq4_moe_combine's FMA chain), the shared expert's pair with weight 1 last
    auto combine = [&](int t) {
        if (tid < nr) {
            const float* rw = rw_s + t * 36;
            float acc = 0.0f;
            for (int j0 = 0; j0 < kk; j0 += 8) {   // (eight experts' values read before the first is used; the chain's order is j's)
                float wv8[8], dv8[8];
#pragma unroll
                for (int jj = 0; jj < 8; ++jj) {
                    wv8[jj] = rw[min(j0 + jj, kk - 1)];
                    dv8[jj] = dsum[min(j0 + jj, kk - 1) * rpc + tid];
                }
#pragma unroll
                for (int jj = 0; jj < 8; ++jj)
                    if (j0 + jj < kk) acc = fmaf(wv8[jj], dv8[jj], acc);
            }
            const size_t at = (size_t) t * a.os + r0 + tid;
            a.out[at] = a.res ? bfr(a.res[at] + bfr(acc)) : acc;
        }
    };
    if (P == 4 && T == 1 && c.nit == 1) {
        // One token whose down rows take one iteration: what the chunk can do without A - the streams, the byte transposition,
        // the twelve exact column sums of every block - is done now, while A is still on its way between the CUs; what remains
        // behind the exchange is a convert and a multiply-add a column (cols_pre / cols_post: chunk_dot's bits).
        if constexpr (P == 4) {
            const int g = dl, j = min((int) ((uint32_t) g / c.by_rpc), kk - 1), rr = g - (int) ((uint32_t) g / c.by_rpc) * rpc;
            const bool ok = dl < c.rpi && g < c.rows_t && rr < nr;
            uint32_t zp[8][6];
            if (ok) cols_pre(dcur, tab, zp);
            wait_stage(0);
            float acc0 = 0.0f;
            if (ok) cols_post(zp, dcur.codes, slice(0, j, 2).eb, xd + j * (Ld * XP) + dch * XP, acc0);
            if constexpr (SHFL_D) rows_out(0, 0, acc0, ok, g, j, rr, true, tid);
            else {
                // (one iteration: the threads' sums side by side, no ring - this path is the C2 step's, and every instruction of it counts)
                part[tid] = acc0;
                __syncthreads();
                const int js = min((int) ((uint32_t) tid / c.by_rpc), kk - 1), rs = tid - (int) ((uint32_t) tid / c.by_rpc) * rpc;
                if (tid < c.rows_t && rs < nr) {
                    float sm = 0.0f;
                    for (int c0 = 0; c0 < Ld; c0 += 8) {
                        float pv[8];
#pragma unroll
                        for (int cc = 0; cc < 8; ++cc) pv[cc] = part[tid * Ld + min(c0 + cc, Ld - 1)];
#pragma unroll
                        for (int cc = 0; cc < 8; ++cc) sm += c0 + cc < Ld ? pv[cc] : 0.0f;
                    }
                    const float dv = bfr(sm * NSLM_R32);
                    dsum[tid] = dv;
                    a.D[(size_t) js * a.d + r0 + rs] = dv;
                }
            }
            __syncthreads();
            combine(0);
        }
        return;
    }
    for (int t = 0; t < T; ++t) {
        wait_stage(t);
        ud = 0;
        for (int it = 0; it < c.nit; ++it) {
            const bool last = it + 1 == c.nit;
            const Chunk dnxt = fetch_d(last ? t + 1 : t, last ? 0 : it + 1);
            const Deal q = deal_d(it);
            const int g = q.row, j = min((int) ((uint32_t) g / c.by_rpc), kk - 1), rr = g - (int) ((uint32_t) g / c.by_rpc) * rpc;
            const bool ok = g < c.rows_t && rr < nr;
            float acc[1] = {0.0f};
            int slot = ok ? q.f : -1;
            if (!q.tail) {
                if (ok) chunk_dot<P, 1, false>(dcur, slice(t, j, 2).eb, tab, xd + j * (Ld * XP) + q.ch * XP, 0, 1, acc);
            } else if constexpr (P == 3) {
                if (ok) acc[0] = chunk_dot_split(dcur, slice(t, j, 2).eb, tab, xd + j * (Ld * XP) + q.ch * XP, q.sub, ltd);   // (a chunk's lanes together)
                if (q.sub != (1 << ltd) - 1) slot = -1;
            }
            rows_out(t, it, acc[0], ok, g, j, rr, last, slot);
            dcur = dnxt;
        }
        __syncthreads();
        combine(t);
        // (the next token's staging writes xd, which every thread has finished reading before the barrier above; dsum and part
        // are next written behind the next token's first barrier)
    }
}

template <int P, bool SG, bool SD, int NTHR, bool NORM>
int launch_one_n(hipStream_t st, const FusedArgs& a, const CuParams& c, size_t lds) {
    void (*kern)(FusedArgs, CuParams) = k_moe_decode_cu<P, SG, SD, NTHR, NORM>;
    static size_t lds_set = 0;   // the largest dynamic-LDS request this kernel has been prepared for
    static int resident = 0;
    if (lds > lds_set) {
        // (a refusal is this launcher's answer "not my shape", not an error of the step: the runtime's error state is cleared)
        if (hipFuncSetAttribute((const void*) kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds) != hipSuccess) {
            (void) hipGetLastError();
            return -1;
        }
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, NTHR, lds) != hipSuccess || per_cu < 1) {
            (void) hipGetLastError();
            return -1;
        }
        resident = per_cu;
        lds_set = lds;
    }
    if (resident < 1) return -1;
    hipLaunchKernelGGL(kern, dim3((unsigned) c.G), dim3(NTHR), lds, st, a, c);
    host_note_launch();
    return 0;
}

int log2_of(int v) {
    int l = 0;
    while ((1 << l) < v) ++l;
    return l;
}

}   // namespace

namespace nslm {

template <int P, bool SG, bool SD, int NTHR>
int launch_one(hipStream_t st, const FusedArgs& a, const CuParams& c, size_t lds) {
    return a.nw ? launch_one_n<P, SG, SD, NTHR, true>(st, a, c, lds) : launch_one_n<P, SG, SD, NTHR, false>(st, a, c, lds);
}

// 0 launched; -1 the shape is not this kernel's (nothing launched)
int launch_moe_decode_cu(hipStream_t st, FusedArgs& a, int P, bool sd) {
    if (a.T < 1 || a.T > MV_MAXT) return -1;
    const bool sg = a.Lg <= 32 && !(a.Lg & (a.Lg - 1));   // a gate / up row's chunks are a power of two inside a wave: row sums by shuffles
    if (a.Lg > 256 || a.Ld > 1024) return -1;   // (a SwiGLU row's two rows of chunks, a down row's chunks: inside one iteration's threads)
    if ((long) a.T * a.kk * a.ff > FUSED_XA_MAX || a.ff % 64 || a.kk > 33) return -1;
    const int G = fused_cu_count();
    if (G < 1 || a.E > 1024 || (long) a.T * a.E > (long) CU_LG * (G < FUSED_CULG_LINES ? G : FUSED_CULG_LINES)) return -1;   // (a CU forms CU_LG logits)
    a.grid = G;
    CuParams c = {};
    c.G = G;
    const int nthr = 1024;
    if (sg) {
        c.lgL = log2_of(a.Lg);
        c.rpw = 64 / a.Lg;
        c.tpp = 2 * a.ff / c.rpw;
    } else {   // a task is one SwiGLU row (two virtual rows), dealt to the workgroup's threads by iterations
        c.lgL = 0;
        c.rpw = 2;
        c.tpp = a.ff;
    }
    c.Wt = a.kk * c.tpp;
    c.n_c = (c.Wt + G - 1) / G;
    c.ncu_act = (c.Wt + c.n_c - 1) / c.n_c;
    c.rpc = (a.d + G - 1) / G;
    c.rows_t = a.kk * c.rpc;
    c.nbp = a.ff / 8;
    c.E4 = (a.E + 3) & ~3;
    // 16 waves: four a SIMD get through a block's dependent instruction chains faster than three (C2, one token: 22.6 against
    // 23.3 us with 12 waves, whose tasks divide evenly among them; 4 tokens 62.5 against 64.2)
    c.rpi = nthr / a.Ld;
    c.nit = (c.rows_t * a.Ld + nthr - 1) / nthr;   // (rows whose chunks are a power of two inside a wave: whole rows an iteration)
    c.KP = (a.E + 15) & ~15;
    c.vpt = c.rpw / 2;
    c.lgV = log2_of(c.vpt);
    c.nit_g = sg ? 0 : (2 * c.n_c * a.Lg + nthr - 1) / nthr;
    if (P == 3) {   // the last iteration's chunks over 2, 4 or 8 lanes each where they fit
        auto lanes_log2 = [&](int chunks) {
            for (int l = 3; l >= 1; --l)
                if (((long) chunks << l) <= nthr) return l;
            return 0;
        };
        if (!sg) c.ltail_g = lanes_log2(2 * c.n_c * a.Lg - (c.nit_g - 1) * nthr);
        if (!sd) c.ltail_d = lanes_log2(c.rows_t * a.Ld - (c.nit - 1) * nthr);
    }
    c.by_ring = fastdiv_of((uint32_t) (3 * nthr));
    c.by_Lg = fastdiv_of((uint32_t) a.Lg);
    c.by_E = fastdiv_of((uint32_t) a.E);
    c.by_tpp = fastdiv_of((uint32_t) c.tpp);
    c.by_rpc = fastdiv_of((uint32_t) c.rpc);
    c.by_Ld = fastdiv_of((uint32_t) a.Ld);
    c.by_nbp = fastdiv_of((uint32_t) c.nbp);
    c.by_kk = fastdiv_of((uint32_t) a.kk);
    const int xp = P == 4 ? xpad<4>() : xpad<3>(), ws = (int) (sizeof(WSlice) / 4);
    int o = 0;
    auto take = [&](int words) { const int at = o; o += (words + 3) & ~3; return at; };
    c.xg = take(a.T * a.Lg * xp);
    c.xd = take(a.kk * a.Ld * xp);
    c.scr = take(sg && sd ? 2 * nthr : 4 * nthr);   // (both passes by shuffles: unused)
    c.pk = take(a.T * c.KP);
    c.rv = take(a.T * c.E4);
    c.dsum = take(a.kk * c.rpc);
    c.ri = take(a.T * 32);
    c.rw = take(a.T * 36);
    c.rn = take(MV_MAXT + 16);
    c.cnt = take(2 * MV_MAXT);
    c.av = take(2 * a.T * c.n_c * c.vpt);
    c.lgs = take(16);
    c.sel = take((3 + (a.E <= CU_PRE_MAXE ? 0 : a.T * a.kk * 3)) * ws);
    c.pre = take(a.E <= CU_PRE_MAXE ? 3 * a.E * ws : 0);
    c.total = o;
    size_t lds = (size_t) c.total * 4;
    if (lds > CU_LDS_MAX) return -1;
    if (lds < CU_LDS_MIN) lds = CU_LDS_MIN;
    if (P == 4) {
        if (sg) return sd ? launch_one<4, true, true, 1024>(st, a, c, lds) : launch_one<4, true, false, 1024>(st, a, c, lds);
        return sd ? launch_one<4, false, true, 1024>(st, a, c, lds) : launch_one<4, false, false, 1024>(st, a, c, lds);
    }
    if (sg) return sd ? launch_one<3, true, true, 1024>(st, a, c, lds) : launch_one<3, true, false, 1024>(st, a, c, lds);
    return sd ? launch_one<3, false, true, 1024>(st, a, c, lds) : launch_one<3, false, false, 1024>(st, a, c, lds);
}

}   // namespace nslm

