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
};

enum { DENSE = 0, GATHER = 1, GATEUP = 2 };

// SHFL: L is a power of two <= 64 (<= 32 for GATEUP): row sums by wave shuffles, no barrier.  Otherwise through LDS.
template <int P, int MODE, int NT, bool SHFL>
__global__ void __launch_bounds__(256) k_mv_seed(MvArgs a) {
    extern __shared__ float xl[];                  // NT > 1: activations [token][chunk][XPAD]
    __shared__ uint32_t tab[NSLM_TAB_WORDS];
    __shared__ float part[SHFL ? 1 : 2][SHFL ? 1 : NT][SHFL ? 1 : 256];
    const int tid = threadIdx.x, L = a.L, rpi = a.rpi;
    const int lr = tid / L, ch = tid - lr * L;
    const bool active = lr < rpi;
    const int pair = MODE == DENSE ? 0 : (int) blockIdx.y;
    const int V = MODE == GATEUP ? 2 * a.R : a.R;   // virtual rows: gate row r = 2r, up row r = 2r + 1
    const int v0 = (int) blockIdx.x * a.rows_per_wg, v1 = min(v0 + a.rows_per_wg, V);
    WSlice wA = a.wd, wB = a.wd;
    if (MODE != DENSE) {
        const int sl = a.sel[pair];
        wA = a.ws[sl];
        if (MODE == GATEUP) wB = a.wu[sl];
    }
    const float* xrow = a.x + (size_t) (MODE == DENSE ? 0 : pair / a.xdiv) * a.xs;

    const bool al = streams_aligned(P, wA) && (MODE != GATEUP || streams_aligned(P, wB));

    // first records in flight before anything else
    int v = v0 + lr;
    auto fetch = [&](int vv) {
        const bool ok = active && vv < v1;
        const int r = MODE == GATEUP ? vv >> 1 : vv;
        const WSlice& w = (MODE == GATEUP && (vv & 1)) ? wB : wA;
        return load_chunk<P>(w, (uint32_t) r * (uint32_t) L + (uint32_t) ch, ok, al);
    };
    Chunk cur = fetch(v);

    load_tables(tab);
    float xreg[NT == 1 ? 64 : 1];
    if (NT == 1) {
        if (active) {
            const float4* xp = (const float4*) (xrow + (size_t) ch * 64);
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float4 q = xp[i];
                xreg[4 * i] = q.x; xreg[4 * i + 1] = q.y; xreg[4 * i + 2] = q.z; xreg[4 * i + 3] = q.w;
            }
        }
    } else {
        for (int t = 0; t < a.nt; ++t)
            for (int i = tid; i < a.K / 4; i += 256) {
                const float4 q = ((const float4*) (a.x + (size_t) t * a.xs))[i];
                *(float4*) &xl[(t * L + (i >> 4)) * XPAD + (i & 15) * 4] = q;
            }
    }
    __syncthreads();

    const int eA = wA.eb, eB = wB.eb;
    int par = 0;
    for (int vb = v0; vb < v1; vb += rpi, par ^= 1) {
        v = vb + lr;
        const Chunk nxt = fetch(v + rpi);
        float acc[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t] = 0.0f;
        const int eb = (MODE == GATEUP && (v & 1)) ? eB : eA;
        if (active && v < v1) {
            if (NT == 1) chunk_dot<P, NT>(cur, eb, tab, xreg, 0, 1, acc);
            else chunk_dot<P, NT>(cur, eb, tab, xl + ch * XPAD, L * XPAD, a.nt, acc);
        }
        if (SHFL) {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                if (NT > 1 && t >= a.nt) break;
                float s = acc[t];
                for (int o = L >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o);
                if (MODE == GATEUP) {
                    const float other = __shfl_xor(s, L);   // rows 2r and 2r+1 sit side by side in the wave
                    if (active && ch == 0 && !(v & 1) && v < v1) {
                        const float gs = s * NSLM_R32, us = other * NSLM_R32;
                        float* yo = a.y + (size_t) pair * a.ys + (v >> 1);
                        *yo = a.f32out ? (gs / (1.0f + expf(-gs))) * us : bfr(silu_bf(bfr(gs)) * bfr(us));
                    }
                } else if (active && ch == 0 && v < v1) {
                    store_y(a.y + (size_t) (MODE == DENSE ? t : pair) * a.ys + v, s * NSLM_R32, a.add, a.f32out);
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
                    float* yo = a.y + (size_t) pair * a.ys + ((vb >> 1) + tid);
                    *yo = a.f32out ? (gs / (1.0f + expf(-gs))) * us : bfr(silu_bf(bfr(gs)) * bfr(us));
                }
            } else if (tid < nrow * (NT > 1 ? a.nt : 1)) {
                const int t = tid / nrow, r = tid - t * nrow;
                float s = 0.0f;
                for (int j = 0; j < L; ++j) s += part[par][t][r * L + j];
                store_y(a.y + (size_t) (MODE == DENSE ? t : pair) * a.ys + (vb + r), s * NSLM_R32, a.add, a.f32out);
            }
        }
        cur = nxt;
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

// virtual rows per workgroup: a multiple of rpi, sized so the grid has about 3 workgroups per CU when the work allows
int pick_rows_per_wg(int V, int rpi, int ny) {
    const int iters = (V + rpi - 1) / rpi;
    const int want = 3 * cu_count();
    int per = (iters * ny + want - 1) / want;
    static const char* env = getenv("NSLM_MV_ITERS");   // tuning override: iterations per workgroup
    if (env && atoi(env) > 0) per = atoi(env);
    if (per < 1) per = 1;
    if (per > 64) per = 64;
    return per * rpi;
}

// kernels that stage activations may need more dynamic LDS than the default limit: raise it once per kernel
template <typename Kern>
void allow_big_lds(Kern k) {
    static const hipError_t once = hipFuncSetAttribute((const void*) k, hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024);
    (void) once;
}
template <int P, int MODE, int NT>
void launch_seed(hipStream_t st, const MvArgs& a, bool shfl, dim3 grid, size_t lds) {
    if (shfl) {
        if (lds > 48 * 1024) allow_big_lds(k_mv_seed<P, MODE, NT, true>);
        hipLaunchKernelGGL((k_mv_seed<P, MODE, NT, true>), grid, dim3(256), lds, st, a);
    } else {
        if (lds > 48 * 1024) allow_big_lds(k_mv_seed<P, MODE, NT, false>);
        hipLaunchKernelGGL((k_mv_seed<P, MODE, NT, false>), grid, dim3(256), lds, st, a);
    }
}
template <int MODE, int NT>
void launch_seed_fmt(hipStream_t st, int fmt, const MvArgs& a, bool shfl, dim3 grid, size_t lds) {
    static const char* pad = getenv("NSLM_MV_LDS");   // experiment: request this much LDS to cap workgroups per CU
    if (pad && (size_t) atoi(pad) > lds) lds = (size_t) atoi(pad);
    if (fmt == MF_SEED4P4) launch_seed<4, MODE, NT>(st, a, shfl, grid, lds);
    else launch_seed<3, MODE, NT>(st, a, shfl, grid, lds);
}

void note_launch() { nslm::host_note_launch(); }

#define MV_TG 4   // tokens per pass of the multi-token fast path (activations staged in LDS)

}   // namespace

namespace nslm {
int host_store_f32() { return g_store_f32; }
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
        // Tokens go in passes of at most MV_TG; a token's arithmetic is the same in every pass size.  Rows too long for
        // the LDS staging take one pass per token with the activations in registers.
        const bool stage = T > 1 && L <= 96;
        for (int t0 = 0; t0 < T; t0 += stage ? MV_TG : 1) {
            MvArgs b = a;
            b.x = x + (size_t) t0 * xs;
            b.y = y + (size_t) t0 * ys;
            b.nt = stage ? (T - t0 < MV_TG ? T - t0 : MV_TG) : 1;
            if (stage) launch_seed_fmt<DENSE, MV_TG>(st, fmt, b, shfl, grid, (size_t) MV_TG * L * XPAD * sizeof(float));
            else launch_seed_fmt<DENSE, 1>(st, fmt, b, shfl, grid, 0);
        }
        note_launch();
        return;
    }
    a.nt = T;
    hipLaunchKernelGGL(k_mv_any<DENSE>, dim3((unsigned) (R + 3) / 4, 1), dim3(256), 0, st, fmt, a);
    note_launch();
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
        launch_seed_fmt<GATHER, 1>(st, fmt, a, shfl, grid, 0);
        note_launch();
        return;
    }
    hipLaunchKernelGGL(k_mv_any<GATHER>, dim3((unsigned) (R + 3) / 4, (unsigned) P), dim3(256), 0, st, fmt, a);
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
        launch_seed_fmt<GATEUP, 1>(st, fmt, a, shfl, grid, 0);
        note_launch();
        return;
    }
    hipLaunchKernelGGL(k_mv_any<GATEUP>, dim3((unsigned) (R + 3) / 4, (unsigned) P), dim3(256), 0, st, fmt, a);
    note_launch();
}

}   // extern "C"
