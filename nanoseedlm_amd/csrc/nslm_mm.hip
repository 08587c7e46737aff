// nslm_mm.hip - the prefill GEMM on MFMA: Y[n][r] = sum_k W[r][k] X[n][k], dense (T tokens) or grouped (a tile table
// over pairs grouped by expert).  Replaces the reference's mm_body and its launchers (engine/kernels_moe.cu:405-525,
// 2354-2395).
//
// A workgroup of 4 waves owns 64 weight rows and up to 128 * MT tokens (MT = 4: 512 tokens, so a dense 512-token
// prefill decodes every weight tile exactly once).  Per K step of 32: each of the 256 threads decodes one 8-weight
// block (64 rows x 4 blocks) into LDS as BF16 - exact integer sums, one multiply by fl(R32 2^e), one rounding - and
// the activations of the step are staged as BF16; then wave w multiplies its 32 * MT tokens against all 64 rows with
// v_mfma_f32_32x32x16_bf16 (tokens on M, weight rows on N, so a lane's B fragment is one decoded block and the
// accumulator columns are consecutive output addresses).  f32 accumulation.  In exact mode (kc_seed_gemm_f32) a seed
// weight is carried as three BF16 terms hi + mid + lo whose sum is the f32 value, three MFMAs per step, as the reference.
// Other formats (BF16, Q8, Q4) dequantize to BF16 values exactly and take the same path.
#include "nslm_dev.h"

using namespace nslm;

namespace {

int g_seed_exact = 0;   // kc_seed_gemm_f32

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

struct MmArgs {
    int K, R, T, xs, ys, xdiv, add, f32out;
};

#define BM 64           // weight rows per workgroup
#define BK 32           // K per step
#define LDW 40          // LDS row stride in BF16 elements (80 bytes: 16-byte fragment reads are conflict-free)

// the 8 weights of block j of row r as f32 (seeds exact and unrounded; BF16 / Q8 / Q4 as their BF16 values)
__device__ __forceinline__ void tile_block(int fmt, const WSlice& w, const uint32_t* tab, int r, int K, int j, float (&o)[8]) {
    const int nbk = K / 8;
    if (fmt == MF_SEED4P4 || fmt == MF_SEED4) {
        const size_t g = (size_t) r * nbk + j;
        const uint32_t seed = ((const uint16_t*) w.p[0])[g], word = ((const uint16_t*) w.p[1])[g];
        int is[8], code;
        if (fmt == MF_SEED4P4) {
            block_isum<4>(tab, seed, word, is);
            code = (((const uint8_t*) w.p[3])[g >> 1] >> ((g & 1) * 4)) & 15;
        } else {
            block_isum<3>(tab, seed, word, is);
            code = (int) (word & 15u);
        }
        const float sc = pow2f(w.eb + code) * NSLM_R32;
#pragma unroll
        for (int c = 0; c < 8; ++c) o[c] = (float) is[c] * sc;
    } else if (fmt == MF_BF16) {
        const uint4 v = *(const uint4*) ((const uint16_t*) w.p[0] + (size_t) r * K + (size_t) j * 8);
        const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) { o[2 * i] = __uint_as_float(u[i] << 16); o[2 * i + 1] = __uint_as_float(u[i] & 0xFFFF0000u); }
    } else {
        const size_t e0 = (size_t) r * K + (size_t) j * 8, gi = e0 >> group_shift(w);
        const float s = bf(((const uint16_t*) w.p[1])[gi]), b = bf(((const uint16_t*) w.p[2])[gi]);
        if (fmt == MF_Q8) {
            const uint2 q = *(const uint2*) ((const uint32_t*) w.p[0] + e0 / 4);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                o[i] = bfr(s * (float) ((q.x >> (8 * i)) & 255u) + b);
                o[4 + i] = bfr(s * (float) ((q.y >> (8 * i)) & 255u) + b);
            }
        } else {
            const uint32_t q = ((const uint32_t*) w.p[0])[e0 / 8];
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] = bfr(s * (float) ((q >> (4 * i)) & 15u) + b);
        }
    }
}

// MT: 32-token tiles per wave (the workgroup covers 128 * MT tokens or pairs).  NTERM: BF16 terms per weight.
template <int MT, int NTERM, bool PACKED>
__global__ void __launch_bounds__(256) k_mm(int fmt, MmArgs a, WSlice wd, const WSlice* ws, const void* Xv, float* Y,
                                            const int32_t* perm, const MmTile* tiles, const int32_t* ntiles) {
    constexpr int BN = 128 * MT;
    __shared__ __attribute__((aligned(16))) uint16_t Wsm[NTERM][BM][LDW];
    __shared__ __attribute__((aligned(16))) uint16_t Xsm[BN][LDW];
    __shared__ int srow[BN], drow[BN];
    __shared__ uint32_t tab[NSLM_TAB_WORDS];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const bool grouped = tiles != nullptr;
    if (grouped && ntiles && (int) blockIdx.y >= *ntiles) return;
    const int r0 = (int) blockIdx.x * BM;
    int start, count;
    WSlice wt;
    if (grouped) {
        const MmTile tl = tiles[blockIdx.y];
        wt = ws[tl.slice];
        start = tl.start;
        count = tl.count;
    } else {
        wt = wd;
        start = (int) blockIdx.y * BN;
        count = min(BN, a.T - start);
    }
    load_tables(tab);
    for (int i = tid; i < BN; i += 256) {
        const bool ok = i < count;
        srow[i] = !ok ? -1 : grouped ? perm[start + i] / a.xdiv : start + i;
        drow[i] = !ok ? -1 : grouped ? perm[start + i] : start + i;
    }
    __syncthreads();

    f32x16 acc[MT][2];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < 2; ++n)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[m][n][i] = 0.0f;
    const int wtok = wv * 32 * MT;          // this wave's first token of the tile
    const bool wave_live = wtok < count;    // a wave whose tokens are all padding only helps to decode
    const int frow = lane & 31, fk = (lane >> 5) * 8;

    for (int k0 = 0; k0 < a.K; k0 += BK) {
        {   // weights: 64 rows x 4 blocks, one block per thread
            const int rr = tid >> 2, jb = tid & 3, row = r0 + rr;
            float f[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            if (row < a.R) tile_block(fmt, wt, tab, row, a.K, k0 / 8 + jb, f);
#pragma unroll
            for (int q = 0; q < NTERM; ++q) {   // f = hi + mid + lo: each term the BF16 value of what remains (exact)
                uint32_t h[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) { h[i] = tobf(f[i]); f[i] -= bf(h[i]); }
                *(uint4*) &Wsm[q][rr][jb * 8] = make_uint4(h[0] | h[1] << 16, h[2] | h[3] << 16, h[4] | h[5] << 16, h[6] | h[7] << 16);
            }
        }
        // activations: BN tokens x 32 k, 16 per thread per pass
        for (int i = tid; i < BN * 2; i += 256) {
            const int n = i >> 1, h = (i & 1) * 16, src = srow[n];
            uint4 v0 = make_uint4(0, 0, 0, 0), v1 = v0;
            if (src >= 0) {
                if (PACKED) {
                    const uint4* xr = (const uint4*) ((const uint16_t*) Xv + (size_t) src * a.xs + k0 + h);
                    v0 = xr[0];
                    v1 = xr[1];
                } else {
                    const float4* xr = (const float4*) ((const float*) Xv + (size_t) src * a.xs + k0 + h);
                    const float4 x0 = xr[0], x1 = xr[1], x2 = xr[2], x3 = xr[3];
                    v0 = make_uint4(pack_bf2(x0.x, x0.y), pack_bf2(x0.z, x0.w), pack_bf2(x1.x, x1.y), pack_bf2(x1.z, x1.w));
                    v1 = make_uint4(pack_bf2(x2.x, x2.y), pack_bf2(x2.z, x2.w), pack_bf2(x3.x, x3.y), pack_bf2(x3.z, x3.w));
                }
            }
            *(uint4*) &Xsm[n][h] = v0;
            *(uint4*) &Xsm[n][h + 8] = v1;
        }
        __syncthreads();
        if (wave_live) {
#pragma unroll
            for (int kk = 0; kk < BK; kk += 16) {
                bf16x8 af[MT];
#pragma unroll
                for (int m = 0; m < MT; ++m) af[m] = *(const bf16x8*) &Xsm[wtok + 32 * m + frow][kk + fk];
#pragma unroll
                for (int q = 0; q < NTERM; ++q)   // the largest term first
#pragma unroll
                    for (int n = 0; n < 2; ++n) {
                        const bf16x8 bfrag = *(const bf16x8*) &Wsm[q][32 * n + frow][kk + fk];
#pragma unroll
                        for (int m = 0; m < MT; ++m) acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[m], bfrag, acc[m][n], 0, 0, 0);
                    }
            }
        }
        __syncthreads();
    }
    if (!wave_live) return;
    // accumulator element v of lane l: token row 8 * (v / 4) + 4 * (l / 32) + v % 4, weight column l % 32
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < 2; ++n)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int tok = wtok + 32 * m + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3), row = r0 + 32 * n + (lane & 31);
                const int dst = drow[tok];
                if (dst < 0 || row >= a.R) continue;
                store_y(Y + (size_t) dst * a.ys + row, acc[m][n][v], a.add, a.f32out);
            }
}

template <int MT, bool PACKED>
void launch_mm(hipStream_t st, int fmt, const MmArgs& a, WSlice wd, const WSlice* ws, const void* X, float* Y, const int32_t* perm,
               const MmTile* tiles, const int32_t* ntiles, dim3 grid) {
    const bool exact = g_seed_exact && (fmt == MF_SEED4 || fmt == MF_SEED4P4);
    if (exact) hipLaunchKernelGGL((k_mm<MT, 3, PACKED>), grid, dim3(256), 0, st, fmt, a, wd, ws, X, Y, perm, tiles, ntiles);
    else hipLaunchKernelGGL((k_mm<MT, 1, PACKED>), grid, dim3(256), 0, st, fmt, a, wd, ws, X, Y, perm, tiles, ntiles);
}

template <bool PACKED>
void mm_dense(hipStream_t st, int fmt, WSlice w, int K, int R, const void* x, int xs, float* y, int ys, int T, int add) {
    if (T < 1 || R < 1) return;
    MmArgs a = {K, R, T, xs, ys, 1, add, host_store_f32()};
    const unsigned gx = (unsigned) (R + BM - 1) / BM;
    if (T > 256) launch_mm<4, PACKED>(st, fmt, a, w, nullptr, x, y, nullptr, nullptr, nullptr, dim3(gx, (unsigned) (T + 511) / 512));
    else if (T > 128) launch_mm<2, PACKED>(st, fmt, a, w, nullptr, x, y, nullptr, nullptr, nullptr, dim3(gx, 1));
    else launch_mm<1, PACKED>(st, fmt, a, w, nullptr, x, y, nullptr, nullptr, nullptr, dim3(gx, 1));
}
template <bool PACKED>
void mm_grouped(hipStream_t st, int fmt, const WSlice* ws, int K, int R, const void* x, int xs, float* y, int ys, int xdiv,
                const int32_t* perm, const MmTile* tiles, const int32_t* ntiles, int grid_tiles) {
    if (grid_tiles < 1 || R < 1) return;
    MmArgs a = {K, R, 0, xs, ys, xdiv, 0, host_store_f32()};
    WSlice none = {};
    launch_mm<1, PACKED>(st, fmt, a, none, ws, x, y, perm, tiles, ntiles, dim3((unsigned) (R + BM - 1) / BM, (unsigned) grid_tiles));
}

}   // namespace

extern "C" {

void kc_seed_gemm_f32(int on) { g_seed_exact = on; }

void kc_mm(kc_stream_t s, int fmt, WSlice w, int K, int R, const float* x, int xs, float* y, int ys, int T, int add,
           const uint32_t* G) {
    (void) G;
    mm_dense<false>((hipStream_t) s, fmt, w, K, R, x, xs, y, ys, T, add);
}
void kc_mm_packed(kc_stream_t s, int fmt, WSlice w, int K, int R, const uint16_t* x, int xs, float* y, int ys, int T,
                  int add, const uint32_t* G) {
    (void) G;
    mm_dense<true>((hipStream_t) s, fmt, w, K, R, x, xs, y, ys, T, add);
}
void kc_mm_grouped(kc_stream_t s, int fmt, const WSlice* ws, int K, int R, const float* x, int xs, float* y, int ys,
                   int xdiv, const int32_t* perm, const MmTile* tiles, int ntiles, const uint32_t* G) {
    (void) G;
    mm_grouped<false>((hipStream_t) s, fmt, ws, K, R, x, xs, y, ys, xdiv, perm, tiles, nullptr, ntiles);
}
void kc_mm_grouped_dev(kc_stream_t s, int fmt, const WSlice* ws, int K, int R, const float* x, int xs, float* y, int ys,
                       int xdiv, const int32_t* perm, const MmTile* tiles, const int32_t* ntiles, int max_tiles,
                       const uint32_t* G) {
    (void) G;
    mm_grouped<false>((hipStream_t) s, fmt, ws, K, R, x, xs, y, ys, xdiv, perm, tiles, ntiles, max_tiles);
}
void kc_mm_grouped_packed(kc_stream_t s, int fmt, const WSlice* ws, int K, int R, const uint16_t* x, int xs, float* y,
                          int ys, int xdiv, const int32_t* perm, const MmTile* tiles, const int32_t* nt, int max_tiles,
                          const uint32_t* G) {
    (void) G;
    mm_grouped<true>((hipStream_t) s, fmt, ws, K, R, x, xs, y, ys, xdiv, perm, tiles, nt, max_tiles);
}

}   // extern "C"
