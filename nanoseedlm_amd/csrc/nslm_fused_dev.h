// nslm_fused_dev.h - what the persistent decode-step kernels (nslm_fused.hip: a workgroup an item; nslm_fused_cu.hip: a workgroup
// a CU) share: the launch's arguments, the layout of the sync words, the agent-scope loads and stores that carry data between
// workgroups, the generation that moves on once per launch, and the router's BF16 row dot.
#pragma once
#include "nslm_mv_dev.h"

namespace nslm {

struct FusedArgs {
    const uint16_t* rw;                 // router weight BF16 [E][d]
    const WSlice *gate, *up, *down;     // device slice tables [E]
    const float* x;                     // [T][xs]
    float* out;                         // [T][os]
    float *logits, *wt, *A, *D;         // scratch: [T][E], [T][k], [T*k][ff], [T*k][d]
    int32_t* ind;                       // [T][k]
    uint32_t* sync;                     // [FUSED_SYNC_WORDS + T * ntile_d], see below
    int E, k, d, ff, T, xs, os;
    int kk;                             // pairs a token: k routed experts + ns always-on (shared) experts
    int ns;
    WSlice sh[3];                       // ns = 1: the shared expert's gate / up / down slices (pair k of every token, weight 1)
    const float* res;                   // non-null: out = bf16(res + bf16(sum)) (the residual stream; may alias out)
    const float* nw;                    // non-null: x is normalised first, xn_k = x_k r (1 + nw_k), r = rsqrt(mean(x^2) + neps)
    float neps;
    int Lg, rpig, it_g, ntile_g;        // gate+up pass: chunks per row, virtual rows per iteration, iterations and items per pair
    int Ld, rpid, it_d, ntile_d;        // down pass (item i of a pair owns iterations i it / ntile .. (i + 1) it / ntile)
    int grid;
    int gu_off;                         // per-item and grouped kernels: where, in floats of dynamic LDS, an item's gate / up row sums wait
    uint32_t spin;                      // polls a bounded wait makes before it gives up and sets the error word
};

// Words of the sync area (uint32; every counter sits alone on a 128-byte line = 32 words):
//   [32 g], [32 g + 1]   arrivals of group g = blockIdx.x % BAR_GROUPS, for launches of even / odd generation
//   [32 BAR_GROUPS], [.. + 1] groups that are complete (even / odd generation)
//   [32 (BAR_GROUPS+1+g)] the generation, the same number in all BAR_GROUPS words: a launch reads it at its start and its
//                        last arrival writes the next number to every word
//   [32 (2 BAR_GROUPS+1)] error word
//   [FUSED_LOGIT_WORDS ..] the router logits [FG_MAXT][E], each a 64-bit word: the BF16 value's float bits below, the
//                        launch's generation + 1 above.  A reader polls until the upper half is its own launch's: the
//                        logits need no grid barrier.  Every launch rewrites all FG_MAXT rows (rows it does not use with
//                        zero), so a stale word is always the preceding launch's and never matches.
//   [FUSED_IND_WORDS ..]  the grouped kernel's published selection [FG_MAXT][32], tagged the same way (the weights and the
//                        row's scale are stored before it)
//   [FUSED_PAIR_WORDS ..] the per-pair kernel's two words per pair, each on its own line: finished gate+up items (atomics
//                        only; the last arrival puts it back to zero) and the pair's ready word, set to the launch's
//                        generation + 1 by that last arrival (what the pair's down items poll: polling the counter's
//                        line would slow the arrivals, and a word per item - 96 polls a workgroup - was slower too)
//   [FUSED_DFLAG_WORDS ..] a word per down item, set to the generation + 1 when its rows are stored; the down item of a
//                        token's last expert polls the words of the other experts' items of its row tile and sums (a
//                        ticket per (token, row tile) cost an atomic's round trip more before the sum)
//   [FUSED_CU_WORDS ..]  the workgroup-a-CU kernel's words, FUSED_CU_TOKEN_WORDS per token, every word on a line of its own:
//                        arrivals of the CUs of group g = blockIdx.x % BAR_GROUPS whose part of the token's SwiGLU outputs is
//                        stored [BAR_GROUPS], groups that are complete [1], the token's ready words [BAR_GROUPS] (the
//                        launch's generation + 1, written by the last arrival of all; a CU polls its group's)
//   [FUSED_CULG_WORDS ..] that kernel's router logits, tagged like the ones above: line c (16 words of 64 bits) holds the logits CU
//                        c forms, one per wave, stored by one instruction - a polled line has one writer
//   [FUSED_XA_WORDS ..]  that kernel's copy of the SwiGLU outputs [token][pair][ff] as BF16 bits, which the CUs read from each other
//   [FUSED_SYNC_WORDS ..] the grouped kernel's words: FG_RN_WORDS for the rows' published scales; three words per group
//                        (FG_MAXP groups at most), each on its own line: finished gate+up items (atomics only), the group's
//                        ready flag (what waiters poll), finished down items; then one ticket per (token, down row tile)
// Hundreds of device-scope atomics on ONE address serialise at tens of nanoseconds each, so arrivals go to 32 group
// counters and only each group's last arrival touches the shared one.  Earlier versions of these kernels separated their
// phases by grid barriers on the same words (arrive, then poll the group's generation word): 3.3 us behind the last
// arrival when the opener read and flipped 32 sense words, 1.2 us with generation numbers, and none now that the data
// carries the generation itself.  No clean-up between launches: every counter is reset by the launch that used it.
#define BAR_GROUPS 32
#define FUSED_ERR_WORD (32 * (2 * BAR_GROUPS + 1))
#define FG_MAXT 24      // rows of the grouped kernel
#define FG_MINT_SHARED 5   // with an always-on expert (every row a pair on the same expert) it also takes 5 to 8 rows
#define FUSED_LOGIT_WORDS (32 * (2 * BAR_GROUPS + 2))   // FG_MAXT x 1024 router logits, 64 bits each: value | generation << 32
#define FUSED_IND_WORDS (FUSED_LOGIT_WORDS + 2 * FG_MAXT * 1024)   // FG_MAXT x 32 published selections, tagged the same way
#define FUSED_TILES 256   // most items a pair in a pass of the per-pair kernel
#define FUSED_PAIR_WORDS (FUSED_IND_WORDS + 2 * FG_MAXT * 32)        // per-pair kernel: [MV_MAXT * 33 pairs][64]: arrivals, ready word
#define FUSED_DFLAG_WORDS (FUSED_PAIR_WORDS + MV_MAXT * 33 * 64)     // per-pair kernel: [MV_MAXT][FUSED_TILES][33] finished down items
#define FUSED_CU_WORDS (FUSED_DFLAG_WORDS + MV_MAXT * FUSED_TILES * 33)   // workgroup-a-CU kernel: [MV_MAXT][FUSED_CU_TOKEN_WORDS]
#define FUSED_CU_TOKEN_WORDS (32 * (2 * BAR_GROUPS + 1))
#define FUSED_XA_WORDS (FUSED_CU_WORDS + MV_MAXT * FUSED_CU_TOKEN_WORDS)   // workgroup-a-CU kernel: FUSED_XA_MAX SwiGLU outputs as BF16 bits
#define FUSED_XA_MAX 65536   // T * (top_k + shared) * ff at most for that kernel
#define FUSED_CULG_WORDS (FUSED_XA_WORDS + FUSED_XA_MAX / 2)          // workgroup-a-CU kernel: its logits, [FUSED_CULG_LINES][16] 64-bit words
#define FUSED_CULG_LINES 256
#define FUSED_SYNC_WORDS (FUSED_CULG_WORDS + FUSED_CULG_LINES * 32)
#define SPIN_LIMIT (1u << 21)   // the default of FusedArgs::spin

__device__ __forceinline__ uint32_t ld_agent(const uint32_t* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float ld_agent(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_agent(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_agent(uint32_t* p, uint32_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_agent(uint16_t* p, uint16_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ unsigned long long ld_agent(const unsigned long long* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_agent(unsigned long long* p, unsigned long long v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// Release: every store this wave has issued is acknowledged before the wave goes on to the barrier behind which the
// workgroup's flag (or counter) is written.  The data stores are agent-scope atomics, which write through to the level all
// XCDs share, so "acknowledged" means "readable by an agent-scope load of any workgroup"; the wait for the vector-memory
// counter is spelled out because a workgroup-scope fence alone need not contain one on this target (waves of one workgroup
// share a CU and its cache, so the compiler may leave it out).  The fence keeps the compiler from moving memory operations
// across this point.  Acquire: the readers' loads are agent-scope atomics issued after the poll's value has been used, so
// nothing has to be invalidated; the fence again only pins the compiler's order.
__device__ __forceinline__ void wg_release() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}
__device__ __forceinline__ void wg_acquire() { __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup"); }

// The generation moves on once per launch: every workgroup arrives (nobody waits), the last arrival writes the next number
// to all sense words (two sets of counters, by generation parity: the next launch counts in the other set, so the reset of
// this launch's set needs no wait).  By thread 0, after every wave of the workgroup has read the generation.  In two halves, so
// that the atomic's round trip lies under other work: arrive_issue() returns what the group's counter held, and
// arrive_finish() acts on it later.
__device__ __forceinline__ uint32_t arrive_issue(uint32_t* sync, uint32_t gen) {
    return atomicAdd(sync + 32 * (blockIdx.x % BAR_GROUPS) + (gen & 1u), 1u);
}
__device__ __forceinline__ void arrive_finish(uint32_t* sync, uint32_t G, uint32_t gen, uint32_t old) {
    const uint32_t g = blockIdx.x % BAR_GROUPS, ng = G < BAR_GROUPS ? G : BAR_GROUPS, mine = (G - g + BAR_GROUPS - 1) / BAR_GROUPS;
    const uint32_t set = gen & 1u;
    if (old == mine - 1) {
        st_agent(sync + 32 * g + set, 0u);
        if (atomicAdd(sync + 32 * BAR_GROUPS + set, 1u) == ng - 1) {
            st_agent(sync + 32 * BAR_GROUPS + set, 0u);
#pragma unroll
            for (uint32_t i = 0; i < BAR_GROUPS; ++i) st_agent(sync + 32 * (BAR_GROUPS + 1 + i), gen + 1u);
        }
    }
}

// Router logit of (token t, expert e) by one wave: k_mv_any's BF16 row dot (lanes over blocks of 8, four blocks a round, every
// load of the round requested before the first use; an 8-term FMA chain a block, the blocks added in order, the lanes by
// xor-shuffles) on the input - normalised on the way as kq4_norm1p would have stored it when nw is given (rn: the row's scale) -
// rounded to BF16.  Every lane returns the value.
// router_logit in pieces (the same loads, the same chain of operations), for a kernel that requests a logit's router row before it
// knows the row's scale: router_fetch_row / router_fetch_input ask for the lane's four blocks from j0 on, router_add adds their
// dot products to acc in block order, router_sum is the wave's sum and its rounding.  (router_logit itself stays as it is: built
// from these pieces it was 0.6 us slower inside the step kernels.)
struct RouterRegs {
    uint4 q[4];
    float4 x0[4], x1[4], w0[4], w1[4];
};
// (the router's row alone - the operand that comes from HBM; the input and the norm weights, which the CU has just read, follow)
__device__ __forceinline__ void router_fetch_row(RouterRegs& r, const uint16_t* wr, int nb, int j0) {
#pragma unroll
    for (int u = 0; u < 4; ++u) r.q[u] = *(const uint4*) (wr + (size_t) min(j0 + 64 * u, nb - 1) * 8);   // clamped: the loads stay unconditional
}
__device__ __forceinline__ void router_fetch_input(RouterRegs& r, const float* xr, int nb, const float* nw, int j0) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const size_t j = (size_t) min(j0 + 64 * u, nb - 1);
        r.x0[u] = *(const float4*) (xr + j * 8);
        r.x1[u] = *(const float4*) (xr + j * 8 + 4);
        if (nw) {
            r.w0[u] = *(const float4*) (nw + j * 8);
            r.w1[u] = *(const float4*) (nw + j * 8 + 4);
        }
    }
}
__device__ __forceinline__ void router_fetch(RouterRegs& r, const uint16_t* wr, const float* xr, int nb, const float* nw, int j0) {
    router_fetch_row(r, wr, nb, j0);
    router_fetch_input(r, xr, nb, nw, j0);
}
__device__ __forceinline__ float router_add(const RouterRegs& r, int nb, bool normed, float rn, int j0, float acc) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        if (j0 + 64 * u >= nb) break;
        float4 y0 = r.x0[u], y1 = r.x1[u];
        if (normed) {
            y0.x = y0.x * rn * (1.0f + r.w0[u].x); y0.y = y0.y * rn * (1.0f + r.w0[u].y); y0.z = y0.z * rn * (1.0f + r.w0[u].z); y0.w = y0.w * rn * (1.0f + r.w0[u].w);
            y1.x = y1.x * rn * (1.0f + r.w1[u].x); y1.y = y1.y * rn * (1.0f + r.w1[u].y); y1.z = y1.z * rn * (1.0f + r.w1[u].z); y1.w = y1.w * rn * (1.0f + r.w1[u].w);
        }
        float dd = bf(r.q[u].x & 0xFFFFu) * y0.x;
        dd = fmaf(bf(r.q[u].x >> 16), y0.y, dd);
        dd = fmaf(bf(r.q[u].y & 0xFFFFu), y0.z, dd);
        dd = fmaf(bf(r.q[u].y >> 16), y0.w, dd);
        dd = fmaf(bf(r.q[u].z & 0xFFFFu), y1.x, dd);
        dd = fmaf(bf(r.q[u].z >> 16), y1.y, dd);
        dd = fmaf(bf(r.q[u].w & 0xFFFFu), y1.z, dd);
        dd = fmaf(bf(r.q[u].w >> 16), y1.w, dd);
        acc = fmaf(dd, 1.0f, acc);
    }
    return acc;
}
__device__ __forceinline__ float router_sum(float acc) {
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
    return bfr(acc);
}
__device__ __forceinline__ float router_logit(const uint16_t* wr, const float* xr, int d, const float* nw, float rn) {
    const int lane = threadIdx.x & 63, nb = d / 8;
    float acc = 0.0f;
    for (int j0 = lane; j0 < nb; j0 += 256) {
        uint4 q[4];
        float4 x0[4], x1[4], w0[4], w1[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const size_t j = (size_t) min(j0 + 64 * u, nb - 1);   // clamped: the loads stay unconditional
            q[u] = *(const uint4*) (wr + j * 8);
            x0[u] = *(const float4*) (xr + j * 8);
            x1[u] = *(const float4*) (xr + j * 8 + 4);
            if (nw) {
                w0[u] = *(const float4*) (nw + j * 8);
                w1[u] = *(const float4*) (nw + j * 8 + 4);
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (j0 + 64 * u >= nb) break;
            float4 y0 = x0[u], y1 = x1[u];
            if (nw) {
                y0.x = y0.x * rn * (1.0f + w0[u].x); y0.y = y0.y * rn * (1.0f + w0[u].y); y0.z = y0.z * rn * (1.0f + w0[u].z); y0.w = y0.w * rn * (1.0f + w0[u].w);
                y1.x = y1.x * rn * (1.0f + w1[u].x); y1.y = y1.y * rn * (1.0f + w1[u].y); y1.z = y1.z * rn * (1.0f + w1[u].z); y1.w = y1.w * rn * (1.0f + w1[u].w);
            }
            float dd = bf(q[u].x & 0xFFFFu) * y0.x;
            dd = fmaf(bf(q[u].x >> 16), y0.y, dd);
            dd = fmaf(bf(q[u].y & 0xFFFFu), y0.z, dd);
            dd = fmaf(bf(q[u].y >> 16), y0.w, dd);
            dd = fmaf(bf(q[u].z & 0xFFFFu), y1.x, dd);
            dd = fmaf(bf(q[u].z >> 16), y1.y, dd);
            dd = fmaf(bf(q[u].w & 0xFFFFu), y1.z, dd);
            dd = fmaf(bf(q[u].w >> 16), y1.w, dd);
            acc = fmaf(dd, 1.0f, acc);
        }
    }
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
    return bfr(acc);
}

// CUs of the current device (256 where the properties cannot be read)
inline int fused_cu_count() {
    static int n = 0;
    if (!n) {
        int dev = 0;
        hipDeviceProp_t pr;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&pr, dev) == hipSuccess) n = pr.multiProcessorCount;
        if (n <= 0) n = 256;
    }
    return n;
}
// nslm_fused_cu.hip: the step with one workgroup per CU.  0 launched; -1 the shape is not that kernel's (nothing launched).
// a: as kc_moe_decode_layer fills it (Lg, Ld set); P: 3 or 4; sd: the down rows' chunks fit a shuffle.
int launch_moe_decode_cu(hipStream_t st, FusedArgs& a, int P, bool sd);

}   // namespace nslm
