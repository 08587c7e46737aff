// nslm_mv.hip - the decode matvec family for gfx950: dense (kc_mv), expert gather (kc_mv_sel) and the fused routed
// gate + up + SwiGLU (kc_mv_gu).  Replaces the reference's k_mv_*, k_mv1_*, k_mv_gu_* (engine/kernels_moe.cu:130-348,
// 576-600) behind the same launchers (:2308-2328).
//
// Seed fast path (k_mv_seed).  A row of K weights is K/64 "chunks" of 8 blocks; a chunk's records are one 16-byte load
// of seeds, one of coefficient words and (P = 4) one dword of exponent codes.  A workgroup of 256 threads owns
// rpi = 256 / (K/64) rows per iteration; thread t keeps chunk t % (K/64) for the whole kernel, so at one token its 64
// activations stay in registers and the records of consecutive threads are consecutive 16-byte units of the row-major
// streams: every load instruction of a wave reads one contiguous kilobyte.  The LFSR stream of a seed comes from two
// 256-entry LDS lookups (GF(2) linearity), the 32 states are 16-bit windows cut with v_alignbit, and the 8 integer
// sums of a block are sixteen v_dot2_i32_i16 on packed state pairs: exact integers, one convert and one FMA per weight.
// Row sums are reduced in a fixed order that depends on K and the entry point only, never on the token count, so a
// token's rows are bit-identical whether it is computed alone or with others (the reference's batch invariance,
// engine/kernels_moe.cu:239-240).
//
// Generic path (k_mv_any): one wave per row, lanes over blocks; every format, any K % 8 == 0, any alignment.
#include <stdlib.h>

#include "nslm_mv_dev.h"

using namespace nslm;

namespace {

int g_store_f32 = 0;   // kc_store_f32
thread_local int g_last_error = 0;

struct MvArgs {
    WSlice wd;            // dense: the slice
    const WSlice* ws;     // gather: slices; gu: gate slices
    const WSlice* wu;     // gu: up slices
    const float* x;
    float* y;
    const int32_t* sel;
    int K, R, xdiv, xs, ys, add, nt, f32out;
    int L, rpi, rows_per_wg;   // fast path: chunks per row, rows per iteration, virtual rows per workgroup
    // MULTI: up to MV_MAXJ dense matrices over the same x in one launch; job j owns workgroups [wg0[j], wg0[j + 1])
    WSlice wj[4];
    float* yj[4];
    int Rj[4], ysj[4], addj[4], wg0[5], nj;
    const float* nw;      // non-null (dense modes): x is normalised first, xn_k = x_k r (1 + nw_k), r = rsqrt(mean(x^2) + neps)
    float neps;
    int ttot;             // dense modes with NT > 1: tokens of the launch; workgroup row blockIdx.y takes tokens NT y .. (nt = NT)
    int trun;             // k_mv_wide, dense, ttot > 0: tokens a workgroup row takes (0: MV_MAXT)
                          // (last, so that the one-token kernels read their arguments where they always did: a field
                          // added in the middle cost them a second round of argument loads, 0.3 us a launch)
    uint16_t* px;         // k_mv_wide, dense: non-null = the staged rows also leave as BF16 bits [token][K] (the batched GEMMs' view)
};
#define MV_MAXJ 4
#define MV_YBUF 1024   // virtual rows a workgroup takes at most (rpi <= 256 of them an iteration)

enum { DENSE = 0, GATHER = 1, GATEUP = 2, MULTI = 3 };

// SHFL: L is a power of two <= 64 (<= 32 for GATEUP): row sums by wave shuffles, no barrier.  Otherwise through LDS.
// NTHR: threads a workgroup (256; 512 or 1024 for one-token SHFL launches whose rows fill more than four waves a CU - the
// row and the tables are then fetched once per CU instead of once per four waves).
// COLS: P = 4 blocks in the column form (one- and two-token passes, and every pass of a launch of up to MV_MAXT tokens, whose
// tokens get the bits of a one-token call); false: the weights' form (launches of more tokens, four to a pass).
template <int P, int MODE, int NT, bool SHFL, int NTHR = 256, bool COLS = (P == 4)>
__global__ void __launch_bounds__(NTHR) k_mv_seed(MvArgs a) {
    static_assert(NTHR == 256 || (SHFL && NT == 1), "the LDS row sums and the staged multi-token passes are written for 256 threads");
    extern __shared__ float xl[];                  // activations as the format reads them (xform_block): [token][chunk][xpad<P>()]
    __shared__ uint32_t tab[NSLM_TAB_WORDS];
    __shared__ float part[SHFL ? 1 : 2][SHFL ? 1 : NT][SHFL ? 1 : 256];
    __shared__ float nred[4];
    // The workgroup's results wait here until the loop is over and leave as coalesced stores.  A store inside the loop costs a
    // memory round trip per iteration: the wait for the next records at the end of an iteration is a wait for every
    // outstanding vector memory operation, the store of a moment ago included (C0: 3.5 us for the first of two
    // iterations, 2.35 us - the arithmetic - for the second, which ends the kernel and waits for nothing).
    __shared__ float ybuf[NT][MV_YBUF];
    const int tid = threadIdx.x, L = a.L, rpi = a.rpi;
    const int lr = tid / L, ch = tid - lr * L;
    const bool active = lr < rpi;
    constexpr bool DN = MODE == DENSE || MODE == MULTI;   // all tokens against one matrix
    const int pair = DN ? 0 : (int) blockIdx.y;
    int job = 0, wg = (int) blockIdx.x;
    if (MODE == MULTI) {
        while (job + 1 < a.nj && wg >= a.wg0[job + 1]) ++job;
        wg -= a.wg0[job];
    }
    const int R = MODE == MULTI ? a.Rj[job] : a.R, ys = MODE == MULTI ? a.ysj[job] : a.ys, add = MODE == MULTI ? a.addj[job] : a.add;
    // staged dense passes: the launch's tokens are dealt to grid.y in runs of NT, so a workgroup stages NT rows however
    // many tokens there are (16 rows in one workgroup's LDS left room for one workgroup a CU)
    constexpr bool TGRP = DN && NT > 1;
    const int tg0 = TGRP ? (int) blockIdx.y * NT : 0, nt_ = TGRP ? min(NT, a.ttot - tg0) : a.nt;
    const float* const xbase = a.x + (size_t) tg0 * a.xs;
    float* const yb = (MODE == MULTI ? a.yj[job] : a.y) + (size_t) tg0 * (MODE == MULTI ? a.ysj[job] : a.ys);
    const int V = MODE == GATEUP ? 2 * R : R;   // virtual rows: gate row r = 2r, up row r = 2r + 1
    const int v0 = wg * a.rows_per_wg, v1 = min(v0 + a.rows_per_wg, V);
    const float* xrow = a.x + (size_t) (DN ? 0 : pair / a.xdiv) * a.xs;
    // Request order = return order (a wave's loads come back in the order they went out): the tables and the row, which sit in
    // L2 and are needed first, go out before the records, which come from HBM behind everybody else's.
    const TableWords<NTHR> tw = tables_fetch<NTHR>();
    const bool prenorm = MODE == MULTI && a.nw != nullptr;   // uniform; the other modes compile without it
    constexpr int XW = xw<P, COLS>(), XP = xpad<P, COLS>();
    constexpr bool XREG = NT == 1 && !COLS;   // P = 3 keeps the thread's 64 activations in registers; the 96 column values of
                                               // P = 4 stay in LDS (three 16-byte reads a block), which leaves the registers for eight waves a SIMD
    float xreg[XREG ? 8 * XW : 1];
    constexpr int NXQ = 1024 / NTHR;   // K <= 8192: at most 1024 blocks of a row, a thread takes whole blocks (two 16-byte pieces)
    float4 xq[NT == 1 ? NXQ : 1][2], wq[NT == 1 ? NXQ : 1][2];
    if (NT == 1) {   // clamped, so that the loads stay unconditional
#pragma unroll
        for (int j = 0; j < NXQ; ++j) {
            const int i = min(tid + NTHR * j, a.K / 8 - 1);
            xq[j][0] = ((const float4*) xrow)[2 * i];
            xq[j][1] = ((const float4*) xrow)[2 * i + 1];
            if (MODE == MULTI && prenorm) {
                wq[j][0] = ((const float4*) a.nw)[2 * i];
                wq[j][1] = ((const float4*) a.nw)[2 * i + 1];
            }
        }
    }
    loads_issued();
    WSlice wA = MODE == MULTI ? a.wj[job] : a.wd, wB = wA;
    if (!DN) {
        const int sl = a.sel[pair];
        wA = a.ws[sl];
        if (MODE == GATEUP) wB = a.wu[sl];
    }
    // first records in flight before the first wait
    int v = v0 + lr;
    auto fetch = [&](int vv) {   // (rows past the workgroup's last: its last row's records once more)
        const int vc = min(vv, v1 - 1), r = MODE == GATEUP ? vc >> 1 : vc;
        const WSlice& w = (MODE == GATEUP && (vc & 1)) ? wB : wA;
        return load_chunk<P>(w, (uint32_t) r * (uint32_t) L + (uint32_t) ch);
    };
    // (Half the waves ask a moment later.  With all 9.4 MB of a 4096 x 4096 matrix requested in the same instant - one workgroup of 16
    // waves a CU, every wave one chunk of records - the launch took 8.5 us; with the requests in two waves of arrivals, 64 clocks
    // apart (any split of the waves does, longer pauses do less), the first records are back sooner and the launch takes 7.8.  The
    // smaller workgroups of the other shapes gain a few tenths of a percent.)
    if ((tid >> 6) >= NTHR / 128) __builtin_amdgcn_s_sleep(1);
    Chunk cur = fetch(v);
    loads_issued();
    if (NT == 1) {
        // The row goes through LDS once per workgroup and from there into each thread's registers (the 256 / L threads that
        // share a chunk do not each fetch it).  Every load of the prologue - tables, row, records - is requested before the
        // first wait, so the kernel starts after one memory round trip.
        // (with a norm: the row's scale, bit for bit as the norm kernel forms it - a second pass over the row, from L2)
        const float rn = (MODE == MULTI && prenorm) ? row_rnorm(xrow, a.K, a.neps, nred) : 1.0f;
        tables_store<NTHR>(tab, tw);
#pragma unroll
        for (int j = 0; j < NXQ; ++j) {
            const int i = tid + NTHR * j;
            if (i < a.K / 8) {
                float x8[8] = {xq[j][0].x, xq[j][0].y, xq[j][0].z, xq[j][0].w, xq[j][1].x, xq[j][1].y, xq[j][1].z, xq[j][1].w};
                if (MODE == MULTI && prenorm) {
                    const float w8[8] = {wq[j][0].x, wq[j][0].y, wq[j][0].z, wq[j][0].w, wq[j][1].x, wq[j][1].y, wq[j][1].z, wq[j][1].w};
#pragma unroll
                    for (int c = 0; c < 8; ++c) x8[c] = x8[c] * rn * (1.0f + w8[c]);
                }
                store_block<P, COLS>(xl, i, x8);
            }
        }
    } else {
        // Stage nt rows of K floats: 8 loads in flight a thread before the first store (a loop of load-then-store over a
        // run-time count waits for every load in turn).
        tables_store<NTHR>(tab, tw);
        __shared__ float rn_s[NT];
        if (prenorm) {
            for (int t = 0; t < nt_; ++t) {
                const float rn = row_rnorm(xbase + (size_t) t * a.xs, a.K, a.neps, nred);
                if (tid == 0) rn_s[t] = rn;
            }
            __syncthreads();
        }
        const int nb = a.K / 8, tot = nt_ * nb;   // whole blocks: four a thread and round, their eight loads in flight together
        for (int base = tid; base < tot; base += 256 * 4) {
            float4 q[4][2];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int idx = min(base + 256 * j, tot - 1), t = idx / nb, i = idx - t * nb;
                q[j][0] = ((const float4*) (xbase + (size_t) t * a.xs))[2 * i];
                q[j][1] = ((const float4*) (xbase + (size_t) t * a.xs))[2 * i + 1];
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int idx = base + 256 * j;
                if (idx >= tot) break;
                const int t = idx / nb, i = idx - t * nb;
                float x8[8] = {q[j][0].x, q[j][0].y, q[j][0].z, q[j][0].w, q[j][1].x, q[j][1].y, q[j][1].z, q[j][1].w};
                if (prenorm) {
                    const float4 w0 = ((const float4*) a.nw)[2 * i], w1 = ((const float4*) a.nw)[2 * i + 1];
                    const float w8[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
                    const float rn = rn_s[t];
#pragma unroll
                    for (int c = 0; c < 8; ++c) x8[c] = x8[c] * rn * (1.0f + w8[c]);
                }
                store_block<P, COLS>(xl + (size_t) t * L * XP, i, x8);
            }
        }
    }
    __syncthreads();
    if (XREG && active) {
#pragma unroll
        for (int i = 0; i < 2 * XW; ++i) {
            const float4 q = *(const float4*) &xl[ch * XP + 4 * i];
            xreg[4 * i] = q.x; xreg[4 * i + 1] = q.y; xreg[4 * i + 2] = q.z; xreg[4 * i + 3] = q.w;
        }
    }

    const int eA = wA.eb, eB = wB.eb;
    const bool single = SHFL && MODE != GATEUP && v1 - v0 <= rpi;   // (uniform over the workgroup)
    int par = 0;
    for (int vb = v0; vb < v1; vb += rpi, par ^= 1) {
        v = vb + lr;
        const Chunk nxt = fetch(v + rpi);
        float acc[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = 0.0f;
        const int eb = (MODE == GATEUP && (v & 1)) ? eB : eA;
        if (active && v < v1) {
            if (XREG) chunk_dot<P, NT, false, COLS>(cur, eb, tab, xreg, 0, 1, acc);
            else chunk_dot<P, NT, false, COLS>(cur, eb, tab, xl + ch * XP, L * XP, nt_, acc);
        }
        if (SHFL) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                if (NT > 1 && t >= nt_) break;
                float s = acc[t];
                for (int o = L >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o);
                if (MODE == GATEUP) {
                    const float other = __shfl_xor(s, L);   // rows 2r and 2r+1 sit side by side in the wave
                    if (active && ch == 0 && !(v & 1) && v < v1) {
                        const float gs = s * NSLM_R32, us = other * NSLM_R32;
                        ybuf[t][(v - v0) >> 1] = a.f32out ? (gs / (1.0f + expf(-gs))) * us : bfr(silu_bf(bfr(gs)) * bfr(us));
                    }
                } else if (active && ch == 0 && v < v1) {
                    // a workgroup with one iteration has no later wait that a store could hold up: its sums leave at once
                    if (single) store_y(yb + (size_t) (DN ? t : pair) * ys + v, s * NSLM_R32, add, a.f32out);
                    else ybuf[t][v - v0] = s * NSLM_R32;
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < NT; ++t) part[par][t][tid] = acc[t];
            __syncthreads();   // one barrier per iteration: part is double-buffered by iteration parity
            const int nrow = min(rpi, v1 - vb);
            if (MODE == GATEUP) {
                if (tid < nrow / 2) {
                    float gs = 0.0f, us = 0.0f;
                    for (int j = 0; j < L; ++j) gs += part[par][0][(2 * tid) * L + j];
                    for (int j = 0; j < L; ++j) us += part[par][0][(2 * tid + 1) * L + j];
                    gs *= NSLM_R32;
                    us *= NSLM_R32;
                    ybuf[0][((vb - v0) >> 1) + tid] = a.f32out ? (gs / (1.0f + expf(-gs))) * us : bfr(silu_bf(bfr(gs)) * bfr(us));
                }
            } else {
                for (int w = tid; w < nrow * (NT > 1 ? nt_ : 1); w += 256) {   // (token, row) sums: more than 256 with many tokens of short rows
                    const int t = w / nrow, r = w - t * nrow;
                    float s = 0.0f;
                    for (int j = 0; j < L; ++j) s += part[par][t][r * L + j];
                    ybuf[t][vb - v0 + r] = s * NSLM_R32;
                }
            }
        }
        cur = nxt;
    }
    if (single) return;
    __syncthreads();
    const int nout = MODE == GATEUP ? (v1 - v0) >> 1 : v1 - v0, o0 = MODE == GATEUP ? v0 >> 1 : v0;
    for (int w = tid; w < nout * (NT > 1 ? nt_ : 1); w += NTHR) {
        const int t = w / nout, r = w - t * nout;
        float* yo = yb + (size_t) (DN ? t : pair) * ys + (o0 + r);
        if (MODE == GATEUP) *yo = ybuf[t][r];
        else store_y(yo, ybuf[t][r], add, a.f32out);
    }
}

// ---- generic path: every format, one wave per row --------------------------------------------------------------------
template <int MODE>
__global__ void __launch_bounds__(256) k_mv_any(int fmt, MvArgs a) {
    __shared__ uint32_t tab[NSLM_TAB_WORDS];
    load_tables(tab);
    __syncthreads();
    const int lane = threadIdx.x & 63, r = (int) blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= a.R) return;
    const int pair = MODE == DENSE ? 0 : (int) blockIdx.y;
    WSlice wA = a.wd, wB = a.wd;
    if (MODE != DENSE) {
        const int sl = a.sel[pair];
        wA = a.ws[sl];
        if (MODE == GATEUP) wB = a.wu[sl];
    }
    const float* xrow = a.x + (size_t) (MODE == DENSE ? 0 : pair / a.xdiv) * a.xs;
    const int nbk = a.K / 8, nt = MODE == DENSE ? a.nt : 1;
    float acc[MV_MAXT], accu = 0.0f;
#pragma unroll
    for (int t = 0; t < MV_MAXT; ++t) acc[t] = 0.0f;
    for (int j = lane; j < nbk; j += 64) {
        float w[8], sc;
        block_weights(fmt, wA, tab, r, a.K, j, w, &sc);
#pragma unroll
        for (int t = 0; t < MV_MAXT; ++t) {
            if (t >= nt) break;
            const float* xb = xrow + (size_t) t * a.xs + (size_t) j * 8;
            float d = w[0] * xb[0];
#pragma unroll
            for (int c = 1; c < 8; ++c) d = fmaf(w[c], xb[c], d);
            acc[t] = fmaf(d, sc, acc[t]);
        }
        if (MODE == GATEUP) {
            block_weights(fmt, wB, tab, r, a.K, j, w, &sc);
            const float* xb = xrow + (size_t) j * 8;
            float d = w[0] * xb[0];
#pragma unroll
            for (int c = 1; c < 8; ++c) d = fmaf(w[c], xb[c], d);
            accu = fmaf(d, sc, accu);
        }
    }
#pragma unroll
    for (int t = 0; t < MV_MAXT; ++t) {
        if (t >= nt) break;
        float s = acc[t];
        for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
        if (MODE == GATEUP) {
            float u = accu;
            for (int o = 32; o > 0; o >>= 1) u += __shfl_xor(u, o);
            if (lane == 0) a.y[(size_t) pair * a.ys + r] = a.f32out ? (s / (1.0f + expf(-s))) * u : bfr(silu_bf(bfr(s)) * bfr(u));
        } else if (lane == 0) {
            store_y(a.y + (size_t) (MODE == DENSE ? t : pair) * a.ys + r, s, a.add, a.f32out);
        }
    }
}

// ---- BF16 / Q8 / Q4 rows: HBM-bound, so the point is bytes in flight -------------------------------------------------------
// Same arithmetic and lane assignment as k_mv_any (lane l owns blocks l, l + 64, ...; an FMA chain per block; the wave's
// xor-shuffle sum), hence the same bits - but the activations are staged once per workgroup in LDS instead of being
// re-read from global memory for every row, a block's weights arrive as one 16 / 8 / 4-byte load, a wave walks its rows
// with a grid stride and keeps the loads of four blocks in flight, and many small workgroups share a CU.
#define WIDE_RB 2   // rows a wave of a several-token dense launch takes at a time
template <int FMT>
struct WideRaw {
    uint4 q;         // BF16: 8 weights; Q8: q.xy; Q4: q.x
    uint32_t s, b;   // Q8 / Q4: the group's scale and bias bits
};
// al: the slice's weight words are 16-byte aligned; otherwise the same words by 2- and 4-byte loads
template <int FMT>
__device__ __forceinline__ WideRaw<FMT> wide_load(const WSlice& w, int r, int K, int j, bool al) {
    WideRaw<FMT> v;
    const size_t e0 = (size_t) r * K + (size_t) j * 8;
    if (FMT == MF_BF16) {
        if (al) {
            v.q = ldg16(gp<uint16_t>(w.p[0]) + e0);
        } else {
            const NSLM_GLOBAL uint16_t* p = gp<uint16_t>(w.p[0]) + e0;
            v.q = make_uint4(p[0] | (uint32_t) p[1] << 16, p[2] | (uint32_t) p[3] << 16, p[4] | (uint32_t) p[5] << 16,
                             p[6] | (uint32_t) p[7] << 16);
        }
    } else {
        const size_t gi = e0 >> group_shift(w);
        v.s = gp<uint16_t>(w.p[1])[gi];
        v.b = gp<uint16_t>(w.p[2])[gi];
        if (FMT == MF_Q8) {
            if (al) {
                const uint2 q = ldg8(gp<uint8_t>(w.p[0]) + e0);
                v.q = make_uint4(q.x, q.y, 0, 0);
            } else {
                const NSLM_GLOBAL uint8_t* p = gp<uint8_t>(w.p[0]) + e0;
                v.q = make_uint4(p[0] | (uint32_t) p[1] << 8 | (uint32_t) p[2] << 16 | (uint32_t) p[3] << 24,
                                 p[4] | (uint32_t) p[5] << 8 | (uint32_t) p[6] << 16 | (uint32_t) p[7] << 24, 0, 0);
            }
        } else {
            if (al) {
                v.q = make_uint4(gp<uint32_t>(w.p[0])[e0 / 8], 0, 0, 0);
            } else {
                const NSLM_GLOBAL uint8_t* p = gp<uint8_t>(w.p[0]) + e0 / 2;
                v.q = make_uint4(p[0] | (uint32_t) p[1] << 8 | (uint32_t) p[2] << 16 | (uint32_t) p[3] << 24, 0, 0, 0);
            }
        }
    }
    return v;
}
// BF16 / Q8 as their BF16 values, Q4 in the matvec form s q + b unrounded: block_weights' values
template <int FMT>
__device__ __forceinline__ void wide_weights(const WideRaw<FMT>& v, float (&o)[8]) {
    if (FMT == MF_BF16) {
        const uint32_t u[4] = {v.q.x, v.q.y, v.q.z, v.q.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) { o[2 * i] = __uint_as_float(u[i] << 16); o[2 * i + 1] = __uint_as_float(u[i] & 0xFFFF0000u); }
    } else {
        const float s = bf(v.s), b = bf(v.b);
        if (FMT == MF_Q8) {
#pragma unroll
            for (int c = 0; c < 8; ++c) o[c] = bfr(s * (float) (((c < 4 ? v.q.x : v.q.y) >> (8 * (c & 3))) & 255u) + b);
        } else {
#pragma unroll
            for (int c = 0; c < 8; ++c) o[c] = s * (float) ((v.q.x >> (4 * c)) & 15u) + b;
        }
    }
}
__device__ __forceinline__ float wide_dot(const float (&w)[8], const float* xb) {
    const float4 x0 = *(const float4*) xb, x1 = *(const float4*) (xb + 4);
    float d = w[0] * x0.x;
    d = fmaf(w[1], x0.y, d);
    d = fmaf(w[2], x0.z, d);
    d = fmaf(w[3], x0.w, d);
    d = fmaf(w[4], x1.x, d);
    d = fmaf(w[5], x1.y, d);
    d = fmaf(w[6], x1.z, d);
    return fmaf(w[7], x1.w, d);
}
// ONE: a launch whose workgroups stage one row of activations for the rows of one matrix (gather launches; dense launches of one
// token that do not also write the BF16 view).  Its waves request their pieces of work - 256 blocks of a row, four a lane - one
// piece ahead: the first before the activations are staged, every later one before the piece in hand is multiplied, a row's
// last before its sums are formed and stored.  So a wave's round trips to memory overlap with its other work (a launch of one row
// a wave, 2880 x 2880 in Q4, was two latencies long: 5.9 us for 4.7 MB), and a wave that walks many rows waits for one piece while
// it computes another.  (Launches of several tokens keep the plain loop: their accumulators, carried around the pipelined
// loop, cost 70 registers and half the resident waves.)
template <int FMT, int MODE, bool ONE>
__global__ void __launch_bounds__(256) k_mv_wide(MvArgs a) {
    extern __shared__ __attribute__((aligned(16))) float xw[];   // [nt][K]
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    constexpr bool DNW = MODE == DENSE || MODE == MULTI;   // all tokens against the rows of one matrix (MULTI: of up to MV_MAXJ)
    const int pair = DNW ? 0 : (int) blockIdx.y;
    WSlice wA = a.wd, wB = a.wd;
    if (!DNW) {
        const int sl = a.sel[pair];
        wA = a.ws[sl];
        if (MODE == GATEUP) wB = a.wu[sl];
    }
    // dense launches of more than MV_MAXT tokens (ttot > 0): the tokens are dealt to grid.y in runs of MV_MAXT
    const int trun = a.trun ? a.trun : MV_MAXT;
    const int tg0 = (MODE == DENSE && a.ttot > 0) ? (int) blockIdx.y * trun : 0;
    const float* xrow = a.x + (size_t) (DNW ? tg0 : pair / a.xdiv) * a.xs;
    const int nbk = a.K / 8, nt = !DNW ? 1 : (MODE == DENSE && a.ttot > 0) ? min(trun, a.ttot - tg0) : a.nt;
    bool alA = ((uintptr_t) wA.p[0] & 15u) == 0;
    const bool alB = ((uintptr_t) wB.p[0] & 15u) == 0;
    int total = a.R;
    if (MODE == MULTI) {
        total = 0;
        for (int j = 0; j < a.nj; ++j) total += a.Rj[j];
    }
    if constexpr (ONE) {
        // a wave's row rr: the matrix it belongs to (MULTI: the rows of the matrices follow each other) and its number there
        auto row_of = [&](int rr, int& r, int& job) {
            r = rr;
            job = 0;
            if (MODE == MULTI) {
                while (job + 1 < a.nj && r >= a.Rj[job]) r -= a.Rj[job++];
                wA = a.wj[job];
                alA = ((uintptr_t) wA.p[0] & 15u) == 0;
            }
        };
        auto request = [&](WideRaw<FMT> (&ra)[4], WideRaw<FMT> (&rb)[4], int r, int j0) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int j = j0 + 64 * u;
                if (j < nbk) {
                    ra[u] = wide_load<FMT>(wA, r, a.K, j, alA);
                    if (MODE == GATEUP) rb[u] = wide_load<FMT>(wB, r, a.K, j, alB);
                }
            }
        };
        const int rstep = (int) gridDim.x * 4;
        int rr = (int) blockIdx.x * 4 + wv, jb = 0, r = 0, job = 0;   // the piece in hand: row, first block (the same for all lanes)
        WideRaw<FMT> na[4], nb[4];
        if (rr < total) {
            row_of(rr, r, job);
            request(na, nb, r, lane);
        }
        for (int i = tid; i < a.K / 4; i += 256) ((float4*) xw)[i] = ((const float4*) xrow)[i];
        __syncthreads();
        float acc = 0.0f, accu = 0.0f;
        while (rr < total) {
            WideRaw<FMT> ca[4], cb[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                ca[u] = na[u];
                cb[u] = nb[u];
            }
            const int r_now = r, job_now = job, j_now = jb + lane;
            jb += 256;
            const bool row_done = jb >= nbk;   // (for the wave, not the lane: the sums below are the whole wave's)
            if (row_done) {
                rr += rstep;
                jb = 0;
                if (rr < total) row_of(rr, r, job);
            }
            if (rr < total) request(na, nb, r, jb + lane);
#pragma unroll
            for (int u = 0; u < 4; ++u) {   // the piece's arithmetic, in block order
                const int j = j_now + 64 * u;
                if (j >= nbk) break;
                float w[8];
                wide_weights<FMT>(ca[u], w);
                acc = fmaf(wide_dot(w, xw + (size_t) j * 8), 1.0f, acc);
                if (MODE == GATEUP) {
                    wide_weights<FMT>(cb[u], w);
                    accu = fmaf(wide_dot(w, xw + (size_t) j * 8), 1.0f, accu);
                }
            }
            if (!row_done) continue;
            float s = acc;
            for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
            if (MODE == GATEUP) {
                float u = accu;
                for (int o = 32; o > 0; o >>= 1) u += __shfl_xor(u, o);
                if (lane == 0) a.y[(size_t) pair * a.ys + r_now] = a.f32out ? (s / (1.0f + expf(-s))) * u : bfr(silu_bf(bfr(s)) * bfr(u));
            } else if (lane == 0) {
                if (MODE == MULTI) store_y(a.yj[job_now] + r_now, s, a.addj[job_now], a.f32out);
                else store_y(a.y + (size_t) (MODE == DENSE ? tg0 : pair) * a.ys + r_now, s, a.add, a.f32out);
            }
            acc = 0.0f;
            accu = 0.0f;
        }
        return;
    }
    // staging: with several rows a piece of every row is requested before the first is stored (a loop over the rows with a load
    // and a store each is one memory round trip a row: 8 us of a 14 us launch at 8 rows of 2048)
    if (nt == 1 && !(MODE == DENSE && a.px)) {
        for (int i = tid; i < a.K / 4; i += 256) ((float4*) xw)[i] = ((const float4*) xrow)[i];
    } else {
        for (int i = tid; i < a.K / 4; i += 256) {
            float4 q[MV_MAXT];
#pragma unroll
            for (int t = 0; t < MV_MAXT; ++t) q[t] = ((const float4*) (xrow + (size_t) min(t, nt - 1) * a.xs))[i];   // clamped: unconditional loads
#pragma unroll
            for (int t = 0; t < MV_MAXT; ++t) {
                if (t >= nt) break;
                if (MODE == DENSE && a.px) { q[t].x = bfr(q[t].x); q[t].y = bfr(q[t].y); q[t].z = bfr(q[t].z); q[t].w = bfr(q[t].w); }   // the rows as the GEMMs see them
                ((float4*) xw)[(size_t) t * (a.K / 4) + i] = q[t];
            }
        }
    }
    __syncthreads();
    if (MODE == DENSE && a.px && blockIdx.x == 0) {   // one workgroup of each token run writes the run's BF16 view
        for (int i = tid; i < nt * nbk; i += 256) {
            const int t = i / nbk, j = i - t * nbk;
            const float4 q0 = ((const float4*) xw)[(size_t) t * (a.K / 4) + 2 * j], q1 = ((const float4*) xw)[(size_t) t * (a.K / 4) + 2 * j + 1];
            ((uint4*) (a.px + (size_t) (tg0 + t) * a.K))[j] = make_uint4(pack_bf2(q0.x, q0.y), pack_bf2(q0.z, q0.w), pack_bf2(q1.x, q1.y), pack_bf2(q1.z, q1.w));
        }
    }
    if (MODE == DENSE && nt > 1) {
        // Several tokens: a wave takes WIDE_RB rows at a time, so a block's activations are read from LDS once for the four rows'
        // multiply-adds.  (A row at a time, 16 tokens on 2880 x 2880 in Q4 read 0.5 GB from LDS and took 24 us; the LM head at 8
        // tokens was bound by those reads, not by HBM.)  Per (row, token) the blocks still add up in the one-row order.
        for (int rg = ((int) blockIdx.x * 4 + wv) * WIDE_RB; rg < total; rg += (int) gridDim.x * 4 * WIDE_RB) {
            float acc[WIDE_RB][MV_MAXT];
#pragma unroll
            for (int rb = 0; rb < WIDE_RB; ++rb)
#pragma unroll
                for (int t = 0; t < MV_MAXT; ++t) acc[rb][t] = 0.0f;
            for (int j0 = lane; j0 < nbk; j0 += 128) {   // two blocks of each row in flight, then their arithmetic in block order
                WideRaw<FMT> ra[WIDE_RB][2];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const int j = j0 + 64 * u;
                    if (j < nbk) {
#pragma unroll
                        for (int rb = 0; rb < WIDE_RB; ++rb) ra[rb][u] = wide_load<FMT>(wA, min(rg + rb, total - 1), a.K, j, alA);
                    }
                }
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const int j = j0 + 64 * u;
                    if (j >= nbk) break;
                    float w[WIDE_RB][8];
#pragma unroll
                    for (int rb = 0; rb < WIDE_RB; ++rb) wide_weights<FMT>(ra[rb][u], w[rb]);
#pragma unroll
                    for (int t = 0; t < MV_MAXT; ++t) {
                        if (t >= nt) break;
                        const float* xb = xw + (size_t) t * a.K + (size_t) j * 8;
                        const float4 x0 = *(const float4*) xb, x1 = *(const float4*) (xb + 4);
#pragma unroll
                        for (int rb = 0; rb < WIDE_RB; ++rb) {   // (wide_dot's chain of operations)
                            float d = w[rb][0] * x0.x;
                            d = fmaf(w[rb][1], x0.y, d);
                            d = fmaf(w[rb][2], x0.z, d);
                            d = fmaf(w[rb][3], x0.w, d);
                            d = fmaf(w[rb][4], x1.x, d);
                            d = fmaf(w[rb][5], x1.y, d);
                            d = fmaf(w[rb][6], x1.z, d);
                            d = fmaf(w[rb][7], x1.w, d);
                            acc[rb][t] = fmaf(d, 1.0f, acc[rb][t]);
                        }
                    }
                }
            }
#pragma unroll
            for (int rb = 0; rb < WIDE_RB; ++rb)
#pragma unroll
                for (int t = 0; t < MV_MAXT; ++t) {
                    if (t >= nt) break;
                    float sum = acc[rb][t];
                    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
                    if (lane == 0 && rg + rb < total) store_y(a.y + (size_t) (tg0 + t) * a.ys + rg + rb, sum, a.add, a.f32out);
                }
        }
        return;
    }
    for (int rr = (int) blockIdx.x * 4 + wv; rr < total; rr += (int) gridDim.x * 4) {
        int r = rr, job = 0;
        if (MODE == MULTI) {   // the matrix this row belongs to (the rows of the matrices follow each other)
            while (job + 1 < a.nj && r >= a.Rj[job]) r -= a.Rj[job++];
            wA = a.wj[job];
            alA = ((uintptr_t) wA.p[0] & 15u) == 0;
        }
        float acc[MV_MAXT], accu = 0.0f;
#pragma unroll
        for (int t = 0; t < MV_MAXT; ++t) acc[t] = 0.0f;
        for (int j0 = lane; j0 < nbk; j0 += 256) {   // four blocks' loads in flight, then their arithmetic in block order
            WideRaw<FMT> ra[4], rb[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int j = j0 + 64 * u;
                if (j < nbk) {
                    ra[u] = wide_load<FMT>(wA, r, a.K, j, alA);
                    if (MODE == GATEUP) rb[u] = wide_load<FMT>(wB, r, a.K, j, alB);
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int j = j0 + 64 * u;
                if (j >= nbk) break;
                float w[8];
                wide_weights<FMT>(ra[u], w);
#pragma unroll
                for (int t = 0; t < MV_MAXT; ++t) {
                    if (t >= nt) break;
                    acc[t] = fmaf(wide_dot(w, xw + (size_t) t * a.K + (size_t) j * 8), 1.0f, acc[t]);
                }
                if (MODE == GATEUP) {
                    wide_weights<FMT>(rb[u], w);
                    accu = fmaf(wide_dot(w, xw + (size_t) j * 8), 1.0f, accu);
                }
            }
        }
#pragma unroll
        for (int t = 0; t < MV_MAXT; ++t) {
            if (t >= nt) break;
            float s = acc[t];
            for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
            if (MODE == GATEUP) {
                float u = accu;
                for (int o = 32; o > 0; o >>= 1) u += __shfl_xor(u, o);
                if (lane == 0) a.y[(size_t) pair * a.ys + r] = a.f32out ? (s / (1.0f + expf(-s))) * u : bfr(silu_bf(bfr(s)) * bfr(u));
            } else if (lane == 0) {
                if (MODE == MULTI) store_y(a.yj[job] + (size_t) t * a.ysj[job] + r, s, a.addj[job], a.f32out);
                else store_y(a.y + (size_t) (MODE == DENSE ? tg0 + t : pair) * a.ys + r, s, a.add, a.f32out);
            }
        }
    }
}

// ---- host side ----------------------------------------------------------------------------------------------------------
bool aligned16(const void* p) { return ((uintptr_t) p & 15u) == 0; }

// Fast-path geometry from K alone (and the entry point), so every token count takes the same arithmetic.
bool fast_shape(int fmt, int K, int mode, int* L, int* rpi, bool* shfl) {
    if (fmt != MF_SEED4P4 && fmt != MF_SEED4) return false;
    if (K % 64 || K / 64 > 128) return false;
    const int l = K / 64;
    int r = 256 / l;
    if (mode == GATEUP) r &= ~1;
    if (r < 1) return false;
    const bool pow2 = (l & (l - 1)) == 0;
    *L = l;
    *rpi = r;
    *shfl = pow2 && l <= (mode == GATEUP ? 32 : 64);
    return true;
}

// staged floats per 64-weight chunk; cols: the launch's P = 4 blocks go in the column form
int xpad_of(int fmt, bool cols = true) { return fmt == MF_SEED4P4 ? (cols ? xpad<4, true>() : xpad<4, false>()) : xpad<3>(); }
// launches of up to MV_MAXT tokens give every token the bits of a one-token call (the column form); longer ones trade that for
// the weights' form, which reads a third less LDS a token
bool cols_for(int T) { return T <= MV_MAXT; }

int cu_count() {
    static int n = 0;
    if (!n) {
        int dev = 0;
        hipDeviceProp_t pr;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&pr, dev) == hipSuccess) n = pr.multiProcessorCount;
        if (n <= 0) n = 256;
    }
    return n;
}

// virtual rows per workgroup: a multiple of rpi, sized so the grid has about 3 workgroups of 256 threads per CU (2 of 512, 1 of
// 1024) when the work allows
int pick_rows_per_wg(int V, int rpi, int ny, int nthr = 256) {
    const int iters = (V + rpi - 1) / rpi;
    const int want = (nthr >= 1024 ? 1 : nthr >= 512 ? 2 : 3) * cu_count();
    int per = (iters * ny + want - 1) / want;
    if (per < 1) per = 1;
    if (per > 64) per = 64;
    while (per > 1 && per * rpi > MV_YBUF) --per;   // a workgroup's results wait in LDS until its last iteration
    return per * rpi;
}
// Threads a workgroup for a one-token dense pass over V rows of L chunks: every workgroup fetches the activation row (K floats)
// and the decode tables, and at the start of a launch those fills compete with the first records for the same path into the
// CUs (C0: 512 workgroups of 256 threads brought in 8 MB of row copies beside 9.4 MB of records).  So a CU's share of the rows
// goes to ONE workgroup when it is more than four waves' worth: 512 or 1024 threads.
int pick_threads(int V, int L, bool shfl) {
    if (!shfl || L > 64) return 256;
    const long waves = ((long) V * L + 63) / 64, per_cu = (waves + cu_count() - 1) / cu_count();
    return per_cu > 8 ? 1024 : per_cu > 4 ? 512 : 256;
}

// kernels that stage activations may need more dynamic LDS than the default limit: raise it once per kernel, to what the
// CU's 160 KB leave beside the kernels' static arrays (under 32 KB each)
#define MV_LDS_MAX (128 * 1024)
// (the kernel is a template argument so that every kernel has its own "once": kernels of one signature share a pointer type)
template <auto K>
void allow_big_lds() {
    static const hipError_t once = hipFuncSetAttribute((const void*) K, hipFuncAttributeMaxDynamicSharedMemorySize, MV_LDS_MAX);
    (void) once;
}
template <int P, int MODE, int NT, bool COLS>
void launch_seed256(hipStream_t st, const MvArgs& a, bool shfl, dim3 grid, size_t lds) {
    if (shfl) {
        if (lds > 48 * 1024) allow_big_lds<k_mv_seed<P, MODE, NT, true, 256, COLS>>();
        hipLaunchKernelGGL((k_mv_seed<P, MODE, NT, true, 256, COLS>), grid, dim3(256), lds, st, a);
    } else {
        if (lds > 48 * 1024) allow_big_lds<k_mv_seed<P, MODE, NT, false, 256, COLS>>();
        hipLaunchKernelGGL((k_mv_seed<P, MODE, NT, false, 256, COLS>), grid, dim3(256), lds, st, a);
    }
}
template <int P, int MODE, int NT>
void launch_seed(hipStream_t st, const MvArgs& a, bool shfl, dim3 grid, size_t lds, int nthr = 256, bool cols = true) {
    if constexpr (NT == 1 && (MODE == DENSE || MODE == MULTI)) {
        if (shfl && nthr == 1024) { hipLaunchKernelGGL((k_mv_seed<P, MODE, NT, true, 1024>), grid, dim3(1024), lds, st, a); return; }
        if (shfl && nthr == 512) { hipLaunchKernelGGL((k_mv_seed<P, MODE, NT, true, 512>), grid, dim3(512), lds, st, a); return; }
    }
    if constexpr (P == 4 && NT > 2) {
        if (!cols) { launch_seed256<P, MODE, NT, false>(st, a, shfl, grid, lds); return; }
    }
    launch_seed256<P, MODE, NT, P == 4>(st, a, shfl, grid, lds);
}
template <int MODE, int NT>
void launch_seed_fmt(hipStream_t st, int fmt, const MvArgs& a, bool shfl, dim3 grid, size_t lds, int nthr = 256, bool cols = true) {
    if (fmt == MF_SEED4P4) launch_seed<4, MODE, NT>(st, a, shfl, grid, lds, nthr, cols);
    else launch_seed<3, MODE, NT>(st, a, shfl, grid, lds, nthr, cols);
}

// the wide path: BF16 / Q8 / Q4, whole blocks, 16-byte aligned activations and weights, staged activations within LDS
bool wide_ok(int fmt, int K, const void* x, int xs, int nt) {
    return (fmt == MF_BF16 || fmt == MF_Q8 || fmt == MF_Q4) && K % 8 == 0 && ((uintptr_t) x & 15u) == 0 && xs % 4 == 0 &&
           (size_t) nt * K * sizeof(float) <= MV_LDS_MAX;
}
template <int MODE>
void launch_wide(hipStream_t st, int fmt, const MvArgs& a, int ny) {
    const size_t lds = (size_t) (MODE == DENSE || MODE == MULTI ? a.nt : 1) * a.K * sizeof(float);
    // about 8 small workgroups a CU when the rows allow it; a wave then walks its rows with a grid stride
    int rows = a.R;
    if (MODE == MULTI) {
        rows = 0;
        for (int j = 0; j < a.nj; ++j) rows += a.Rj[j];
    }
    const int per_wg = MODE == DENSE && a.nt > 1 ? 4 * WIDE_RB : 4;   // (several tokens: a wave takes WIDE_RB rows at a time)
    int gx = (rows + per_wg - 1) / per_wg;
    const int cap = (8 * cu_count() + ny - 1) / ny;
    if (gx > cap) gx = cap < 1 ? 1 : cap;
    const dim3 grid((unsigned) gx, (unsigned) ny);
    // (one staged row of one matrix: the pipelined variant.  2880 x 2880 in Q4, one token: 5.9 -> 5.0 us; the multi-matrix launch of
    // three such took 11.1 instead of 9.6 us with it and the gate + up launch the same 7.3, so those keep the plain loop)
    const bool one = MODE == GATHER || (MODE == DENSE && (a.ttot > 0 ? a.ttot : a.nt) == 1 && !a.px);
#define NSLM_WIDE(F)                                                                         \
    do {                                                                                     \
        if (one) {                                                                           \
            if constexpr (MODE == DENSE || MODE == GATHER) {                                 \
                if (lds > 48 * 1024) allow_big_lds<k_mv_wide<F, MODE, true>>();                \
                hipLaunchKernelGGL((k_mv_wide<F, MODE, true>), grid, dim3(256), lds, st, a); \
            }                                                                                \
        } else if constexpr (MODE != GATHER) {                                               \
            if (lds > 48 * 1024) allow_big_lds<k_mv_wide<F, MODE, false>>();                   \
            hipLaunchKernelGGL((k_mv_wide<F, MODE, false>), grid, dim3(256), lds, st, a);    \
        }                                                                                    \
    } while (0)
    if (fmt == MF_BF16) NSLM_WIDE(MF_BF16);
    else if (fmt == MF_Q8) NSLM_WIDE(MF_Q8);
    else NSLM_WIDE(MF_Q4);
#undef NSLM_WIDE
}

void note_launch() { nslm::host_note_launch(); }

// Tokens a workgroup row of a wave-a-row dense launch takes (a token's result does not depend on its run): MV_MAXT at most; fewer
// while the rows alone do not fill the chip twice (a router's 128 rows at 32 tokens: 128 workgroups that each stage 64 KB of
// activations took 9.3 us); and, for a matrix small enough to be re-read from the caches by every run, few enough that several
// workgroups share a CU's LDS (eight rows of 2880 are 92 KB: one workgroup a CU).
int wide_run(int fmt, int K, int R, int T) {
    int run = T < MV_MAXT ? T : MV_MAXT;
    // (workgroups of a launch: four waves of WIDE_RB rows each, of one row where the run is a single token)
    auto wgs = [&](int run_) { const int per = run_ > 1 ? 4 * WIDE_RB : 4; return (long) ((R + per - 1) / per) * ((T + run_ - 1) / run_); };
    while (run > 1 && wgs(run) < 2L * cu_count()) run /= 2;
    const double bytes = (double) R * K * (fmt == MF_BF16 ? 2.0 : fmt == MF_Q8 ? 1.0625 : 0.5625);
    if (bytes <= 16e6)
        while (run > 1 && (size_t) run * K * sizeof(float) > 48 * 1024) run = (run + 1) / 2;
    return run;
}

#define MV_TG 4   // tokens a workgroup of the multi-token fast path stages in LDS
#define MV_MULTI_MAXT 64

}   // namespace

namespace nslm {
int host_store_f32() { return g_store_f32; }
void host_note_unsupported() { g_last_error = (int) hipErrorInvalidValue; }
void host_note_launch() {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) g_last_error = (int) e;
}
}   // namespace nslm

extern "C" {

void kc_store_f32(int on) { g_store_f32 = on; }
int kc_last_error(void) {
    const int e = g_last_error;
    g_last_error = 0;
    return e;
}

void kc_mv(kc_stream_t s, int fmt, WSlice w, int K, int R, const float* x, int xs, float* y, int ys, int T, int add,
           const uint32_t* G) {
    (void) G;
    if (T < 1 || R < 1) return;
    hipStream_t st = (hipStream_t) s;
    MvArgs a = {};
    a.wd = w; a.x = x; a.y = y; a.K = K; a.R = R; a.xdiv = 1; a.xs = xs; a.ys = ys; a.add = add; a.f32out = g_store_f32;
    int L, rpi;
    bool shfl;
    if (fast_shape(fmt, K, DENSE, &L, &rpi, &shfl) && aligned16(x) && xs % 4 == 0) {
        a.L = L; a.rpi = rpi;
        a.rows_per_wg = pick_rows_per_wg(R, rpi, 1);
        const dim3 grid((unsigned) ((R + a.rows_per_wg - 1) / a.rows_per_wg), 1);
        const int nthr = pick_threads(R, L, shfl);   // the one-token launches below
        MvArgs a1 = a;
        a1.rpi = nthr / L;
        a1.rows_per_wg = pick_rows_per_wg(R, a1.rpi, 1, nthr);
        const dim3 grid1((unsigned) ((R + a1.rows_per_wg - 1) / a1.rows_per_wg), 1);
        // Several tokens: their activations staged in LDS, MV_TG tokens a workgroup, the runs of MV_TG tokens dealt to grid.y
        // (a token's arithmetic does not depend on the run it is in).  One workgroup for all of 16 tokens needed 139 KB of
        // LDS, i.e. one workgroup a CU: 2048 x 2048 at 16 tokens 21.5 us, in runs of four 14.1 us (8 tokens: 12.6 -> 9.9).
        // Rows too long for the staging take one launch per token with the activations in registers.
        const bool cols = cols_for(T);
        if (T > 1 && (size_t) MV_TG * L * xpad_of(fmt, cols) * sizeof(float) <= MV_LDS_MAX) {
            a.ttot = T;
            launch_seed_fmt<DENSE, MV_TG>(st, fmt, a, shfl, dim3(grid.x, (unsigned) (T + MV_TG - 1) / MV_TG),
                                          (size_t) MV_TG * L * xpad_of(fmt, cols) * sizeof(float), 256, cols);
        } else {
            for (int t0 = 0; t0 < T; ++t0) {
                MvArgs b = a1;
                b.x = x + (size_t) t0 * xs;
                b.y = y + (size_t) t0 * ys;
                b.nt = 1;
                launch_seed_fmt<DENSE, 1>(st, fmt, b, shfl, grid1, (size_t) L * xpad_of(fmt) * sizeof(float), nthr);
            }
        }
        note_launch();
        return;
    }
    // Every other shape: the kernels' token loops hold MV_MAXT tokens, so more rows go in runs (a token's result does not depend on
    // the run it is in): for the wave-a-row kernel the runs of one launch, dealt to grid.y.
    if (T > 1 && wide_ok(fmt, K, x, xs, T < MV_MAXT ? T : MV_MAXT)) {
        MvArgs b = a;
        b.trun = wide_run(fmt, K, R, T);
        b.nt = b.trun;   // (sizes the staging)
        b.ttot = T;
        launch_wide<DENSE>(st, fmt, b, (T + b.trun - 1) / b.trun);
        note_launch();
        return;
    }
    for (int t0 = 0; t0 < T; t0 += MV_MAXT) {
        MvArgs b = a;
        b.x = x + (size_t) t0 * xs;
        b.y = y + (size_t) t0 * ys;
        b.nt = T - t0 < MV_MAXT ? T - t0 : MV_MAXT;
        if (wide_ok(fmt, K, b.x, xs, b.nt)) launch_wide<DENSE>(st, fmt, b, 1);
        else hipLaunchKernelGGL(k_mv_any<DENSE>, dim3((unsigned) (R + 3) / 4, 1), dim3(256), 0, st, fmt, b);
    }
    note_launch();
}

int kc_mv_pack(kc_stream_t s, int fmt, WSlice w, int K, int R, const float* x, int xs, float* y, int ys, int T, uint16_t* px) {
    if (T < 1 || T > MV_MULTI_MAXT || R < 1 || !wide_ok(fmt, K, x, xs, T < MV_MAXT ? T : MV_MAXT) || !aligned16(px)) return -1;
    MvArgs a = {};
    a.wd = w; a.x = x; a.y = y; a.K = K; a.R = R; a.xdiv = 1; a.xs = xs; a.ys = ys; a.f32out = g_store_f32;
    a.trun = wide_run(fmt, K, R, T);
    a.nt = T < a.trun ? T : a.trun;
    a.ttot = T;
    a.px = px;
    launch_wide<DENSE>((hipStream_t) s, fmt, a, (T + a.trun - 1) / a.trun);
    note_launch();
    return 0;
}

int kc_mv_multi(kc_stream_t s, int fmt, int n, const WSlice* w, const int* R, float* const* y, const int* ys, const int* add, int K,
                const float* x, int xs, int T, const float* norm_w, float norm_eps) {
    if (n >= 1 && n <= MV_MAXJ && T >= 1 && T <= MV_MAXT && !norm_w && wide_ok(fmt, K, x, xs, T)) {
        // BF16 / Q8 / Q4: a wave a row, the rows of the n matrices one after the other (the same row sums as kc_mv's)
        if (T > 1 && (size_t) T * K * sizeof(float) > 48 * 1024) {
            // several tokens of long rows: one dense launch a matrix, whose token runs keep several workgroups on a CU (eight tokens
            // of 2880 are 92 KB of staged activations - one workgroup a CU, and 91 us for three 2880 x 2880 matrices in Q4
            // against 11 us a dense launch)
            for (int j = 0; j < n; ++j) {
                if (R[j] < 1) return -1;
                kc_mv(s, fmt, w[j], K, R[j], x, xs, y[j], ys[j], T, add[j], nullptr);
            }
            return 0;
        }
        MvArgs a = {};
        a.x = x; a.K = K; a.xdiv = 1; a.xs = xs; a.f32out = g_store_f32; a.nj = n; a.nt = T;
        for (int j = 0; j < n; ++j) {
            if (R[j] < 1) return -1;
            a.wj[j] = w[j]; a.Rj[j] = R[j]; a.ysj[j] = ys[j]; a.addj[j] = add[j]; a.yj[j] = y[j];
        }
        launch_wide<MULTI>((hipStream_t) s, fmt, a, 1);
        note_launch();
        return 0;
    }
    int L, rpi;
    bool shfl;
    if (n < 1 || n > MV_MAXJ || T < 1 || T > MV_MULTI_MAXT || !fast_shape(fmt, K, DENSE, &L, &rpi, &shfl) || !aligned16(x) || xs % 4 ||
        (size_t) MV_TG * L * xpad_of(fmt, cols_for(T)) * sizeof(float) > MV_LDS_MAX)
        return -1;
    if (norm_w && (K > 256 * 16 || !aligned16(norm_w))) return -1;
    MvArgs a = {};
    a.x = x; a.K = K; a.xdiv = 1; a.xs = xs; a.f32out = g_store_f32; a.L = L; a.rpi = rpi; a.nj = n; a.nw = norm_w; a.neps = norm_eps;
    int total = 0;
    for (int j = 0; j < n; ++j) total += R[j];
    // (one token: the workgroup size kc_mv's one-token launches take for as many rows)
    const int nthr = T == 1 ? pick_threads(total, L, shfl) : 256;
    if (T == 1) a.rpi = nthr / L;
    a.rows_per_wg = pick_rows_per_wg(total, a.rpi, 1, nthr);
    for (int j = 0; j < n; ++j) {
        if (R[j] < 1) return -1;
        a.wj[j] = w[j]; a.Rj[j] = R[j]; a.ysj[j] = ys[j]; a.addj[j] = add[j];
        a.wg0[j + 1] = a.wg0[j] + (R[j] + a.rows_per_wg - 1) / a.rows_per_wg;
    }
    const dim3 grid((unsigned) a.wg0[n], 1);
    hipStream_t st = (hipStream_t) s;
    if (T == 1) {
        a.nt = 1;
        for (int j = 0; j < n; ++j) a.yj[j] = y[j];
        launch_seed_fmt<MULTI, 1>(st, fmt, a, shfl, grid, (size_t) L * xpad_of(fmt) * sizeof(float), nthr);
    } else {   // runs of MV_TG tokens over grid.y, as kc_mv's
        a.ttot = T;
        for (int j = 0; j < n; ++j) a.yj[j] = y[j];
        launch_seed_fmt<MULTI, MV_TG>(st, fmt, a, shfl, dim3(grid.x, (unsigned) (T + MV_TG - 1) / MV_TG),
                                      (size_t) MV_TG * L * xpad_of(fmt, cols_for(T)) * sizeof(float), 256, cols_for(T));
    }
    note_launch();
    return 0;
}

void kc_mv_sel(kc_stream_t s, int fmt, const WSlice* ws, int K, int R, const float* x, int xs, float* y, int ys,
               const int32_t* sel, int P, int xdiv, const uint32_t* G) {
    (void) G;
    if (P < 1 || R < 1) return;
    hipStream_t st = (hipStream_t) s;
    MvArgs a = {};
    a.ws = ws; a.x = x; a.y = y; a.sel = sel; a.K = K; a.R = R; a.xdiv = xdiv; a.xs = xs; a.ys = ys; a.nt = 1;
    a.f32out = g_store_f32;
    int L, rpi;
    bool shfl;
    if (fast_shape(fmt, K, GATHER, &L, &rpi, &shfl) && aligned16(x) && xs % 4 == 0) {
        a.L = L; a.rpi = rpi;
        a.rows_per_wg = pick_rows_per_wg(R, rpi, P);
        const dim3 grid((unsigned) ((R + a.rows_per_wg - 1) / a.rows_per_wg), (unsigned) P);
        launch_seed_fmt<GATHER, 1>(st, fmt, a, shfl, grid, (size_t) L * xpad_of(fmt) * sizeof(float));
        note_launch();
        return;
    }
    if (wide_ok(fmt, K, x, xs, 1)) launch_wide<GATHER>(st, fmt, a, P);
    else hipLaunchKernelGGL(k_mv_any<GATHER>, dim3((unsigned) (R + 3) / 4, (unsigned) P), dim3(256), 0, st, fmt, a);
    note_launch();
}

void kc_mv_gu(kc_stream_t s, int fmt, const WSlice* wg, const WSlice* wu, int K, int R, const float* x, int xs, float* a_,
              int ys, const int32_t* sel, int P, int xdiv, const uint32_t* G) {
    (void) G;
    if (P < 1 || R < 1) return;
    hipStream_t st = (hipStream_t) s;
    MvArgs a = {};
    a.ws = wg; a.wu = wu; a.x = x; a.y = a_; a.sel = sel; a.K = K; a.R = R; a.xdiv = xdiv; a.xs = xs; a.ys = ys; a.nt = 1;
    a.f32out = g_store_f32;
    int L, rpi;
    bool shfl;
    if (fast_shape(fmt, K, GATEUP, &L, &rpi, &shfl) && aligned16(x) && xs % 4 == 0) {
        a.L = L; a.rpi = rpi;
        a.rows_per_wg = pick_rows_per_wg(2 * R, rpi, P);
        const dim3 grid((unsigned) ((2 * R + a.rows_per_wg - 1) / a.rows_per_wg), (unsigned) P);
        launch_seed_fmt<GATEUP, 1>(st, fmt, a, shfl, grid, (size_t) L * xpad_of(fmt) * sizeof(float));
        note_launch();
        return;
    }
    if (wide_ok(fmt, K, x, xs, 1)) launch_wide<GATEUP>(st, fmt, a, P);
    else hipLaunchKernelGGL(k_mv_any<GATEUP>, dim3((unsigned) (R + 3) / 4, (unsigned) P), dim3(256), 0, st, fmt, a);
    note_launch();
}

}   // extern "C"
