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
#include <stdlib.h>

#include <type_traits>

#include "nslm_mv_dev.h"

using namespace nslm;

namespace {

int g_seed_exact = 0;   // kc_seed_gemm_f32

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

struct MmArgs {
    int K, R, T, xs, ys, xdiv, add, f32out;
    const WSlice* ws2;   // grouped launches of two matrices over the same tiles (grid.z = 2): the second slice table ..
    float* y2;           // .. and its output
    uint16_t* a16;       // non-null: a workgroup's 64 weight rows are 32 gate rows (ws) and the same 32 up rows (ws2), and what it
                         // stores is their SwiGLU as BF16 bits [pair][ys] (the two GEMMs and the SwiGLU + pack pass in one launch)
};

// A workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding global load of the
// wave, which would serialise the producers' prefetches (issued steps ahead on purpose) with each step.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

#define BM 64           // weight rows per workgroup
#define BK 32           // K per step
#define LDW 40          // LDS row stride in BF16 elements (80 bytes: 16-byte fragment reads are conflict-free)

// MT: 32-token tiles per consumer wave (the workgroup covers 128 * MT tokens or pairs).  NTERM: BF16 terms per weight.
//
// 512 threads: waves 0-3 are consumers (MFMA only: wave w owns tokens [32 MT w, 32 MT (w+1)) x all 64 rows), waves 4-7
// are producers (each thread decodes one 8-weight block per K step and stages its share of the step's activations).
// The two LDS buffers alternate per step with one workgroup barrier between steps; producers hold the global loads of
// the two following steps in registers, so a step's records and activations are requested three steps before the MFMAs
// read them and the matrix cores never wait on HBM or L2 latency.
struct MmRec {
    uint32_t seed, word, code;   // seeds: the block's raw fields
    uint4 raw[2];                // other formats: the block's packed words, scale and bias
};
template <int MT, bool PACKED>
struct MmX {
    uint4 v[PACKED ? 2 * MT : 4 * MT];   // this thread's share of a step: MT x 16 activations (BF16, or f32 before rounding)
};

template <int MT, int NTERM, bool PACKED>
__global__ void __launch_bounds__(512) k_mm(int fmt, MmArgs a, WSlice wd, const WSlice* ws, const void* Xv, float* Y,
                                            const int32_t* perm, const MmTile* tiles, const int32_t* ntiles) {
    constexpr int BN = 128 * MT;
    extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
    typedef uint16_t WTile[NTERM][BM][LDW];
    typedef uint16_t XTile[BN][LDW];
    WTile* Wsm = (WTile*) smem;                               // [2]
    XTile* Xsm = (XTile*) (smem + 2 * NTERM * BM * LDW);      // [2]
    __shared__ int srow[BN], drow[BN];
    __shared__ uint32_t tab[NSLM_TAB_WORDS];
    __shared__ __attribute__((aligned(16))) uint16_t rec_seed[2][BM][32], rec_word[2][BM][32];   // two super-steps of records
    __shared__ uint32_t rec_code[2][BM][4];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const bool producer = wv >= 4;
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
    for (int i = tid; i < BN; i += 512) {
        const bool ok = i < count;
        srow[i] = !ok ? -1 : grouped ? perm[start + i] / a.xdiv : start + i;
        drow[i] = !ok ? -1 : grouped ? perm[start + i] : start + i;
    }
    __syncthreads();
    const int nsteps = a.K / BK;

    // ---- producer side ---------------------------------------------------------------------------------------------------
    const int ptid = tid - 256, rr = ptid >> 2, jb = ptid & 3, row = r0 + rr, nbk = a.K / 8;
    const bool seedf = fmt == MF_SEED4P4 || fmt == MF_SEED4;
    // Seed records reach the decoder through LDS, one "super-step" of 8 K steps (32 blocks a row) at a time: thread
    // (rr, jb) fetches blocks [8 jb, 8 jb + 8) of the super-step with one 16-byte load of seeds, one of coefficient words
    // and a dword of codes, a whole super-step (microseconds) before they are decoded - the records stream from HBM
    // exactly once and nothing downstream may wait on that latency.
    const bool rec_fast = seedf && nbk % 8 == 0 && streams_aligned(fmt == MF_SEED4P4 ? 4 : 3, wt);
    auto load_super = [&](int S) {
        Chunk c;
        c.sd = c.cw = make_uint4(0, 0, 0, 0);
        c.codes = 0;
        const int b0 = 32 * S + 8 * jb;   // first block of this thread's share
        if (!seedf || row >= a.R || b0 >= nbk) return c;
        const size_t g = (size_t) row * nbk + b0;
        if (rec_fast) {
            c.sd = ldg16(gp<uint16_t>(wt.p[0]) + g);
            c.cw = ldg16(gp<uint16_t>(wt.p[1]) + g);
            if (fmt == MF_SEED4P4) c.codes = *(const NSLM_GLOBAL uint32_t*) (gp<uint8_t>(wt.p[3]) + (g >> 1));
        } else {
            uint32_t sd[8], cw[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const bool ok = b0 + i < nbk;
                sd[i] = ok ? gp<uint16_t>(wt.p[0])[g + i] : 0u;
                cw[i] = ok ? gp<uint16_t>(wt.p[1])[g + i] : 0u;
                if (ok && fmt == MF_SEED4P4) c.codes |= ((uint32_t) (gp<uint8_t>(wt.p[3])[(g + i) >> 1] >> (((g + i) & 1) * 4)) & 15u) << (4 * i);
            }
            c.sd = make_uint4(sd[0] | sd[1] << 16, sd[2] | sd[3] << 16, sd[4] | sd[5] << 16, sd[6] | sd[7] << 16);
            c.cw = make_uint4(cw[0] | cw[1] << 16, cw[2] | cw[3] << 16, cw[4] | cw[5] << 16, cw[6] | cw[7] << 16);
        }
        return c;
    };
    auto store_super = [&](int buf, const Chunk& c) {
        if (!seedf) return;
        *(uint4*) &rec_seed[buf][rr][8 * jb] = c.sd;
        *(uint4*) &rec_word[buf][rr][8 * jb] = c.cw;
        rec_code[buf][rr][jb] = c.codes;
    };
    // other formats: this thread's block of step s straight into registers
    auto load_rec = [&](int s, MmRec& r) {
        if (seedf || s >= nsteps || row >= a.R) return;
        const size_t g = (size_t) row * nbk + s * (BK / 8) + jb;
        if (fmt == MF_BF16) {
            r.raw[0] = ldg16(gp<uint16_t>(wt.p[0]) + g * 8);
        } else {
            const size_t gi = (g * 8) >> group_shift(wt);
            r.seed = gp<uint16_t>(wt.p[1])[gi];
            r.word = gp<uint16_t>(wt.p[2])[gi];
            if (fmt == MF_Q8) r.raw[0] = make_uint4(gp<uint32_t>(wt.p[0])[g * 2], gp<uint32_t>(wt.p[0])[g * 2 + 1], 0, 0);
            else r.raw[0] = make_uint4(gp<uint32_t>(wt.p[0])[g], 0, 0, 0);
        }
    };
    auto load_x = [&](int s, MmX<MT, PACKED>& x) {
        if (s >= nsteps) return;
        const int k0 = s * BK;
#pragma unroll
        for (int u = 0; u < MT; ++u) {
            const int i = ptid + 256 * u, n = i >> 1, h = (i & 1) * 16, src = srow[n];
            if (PACKED) {
                x.v[2 * u] = x.v[2 * u + 1] = make_uint4(0, 0, 0, 0);
                if (src >= 0) {
                    const uint4* xr = (const uint4*) ((const uint16_t*) Xv + (size_t) src * a.xs + k0 + h);
                    x.v[2 * u] = xr[0];
                    x.v[2 * u + 1] = xr[1];
                }
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q) x.v[4 * u + q] = make_uint4(0, 0, 0, 0);
                if (src >= 0) {
                    const uint4* xr = (const uint4*) ((const float*) Xv + (size_t) src * a.xs + k0 + h);
#pragma unroll
                    for (int q = 0; q < 4; ++q) x.v[4 * u + q] = xr[q];
                }
            }
        }
    };
    auto store_step = [&](int buf, int s, const MmRec& r, const MmX<MT, PACKED>& x) {
        float f[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        if (row < a.R) {
            if (seedf) {
                const int sb = (s >> 3) & 1, b = 4 * (s & 7) + jb;   // block b of the staged super-step
                const uint32_t seed = rec_seed[sb][rr][b], word = rec_word[sb][rr][b];
                int is[8], code;
                if (fmt == MF_SEED4P4) {
                    block_isum<4>(tab, seed, word, is);
                    code = (int) ((rec_code[sb][rr][b >> 3] >> (4 * (b & 7))) & 15u);
                } else {
                    block_isum<3>(tab, seed, word, is);
                    code = (int) (word & 15u);
                }
                const float sc = pow2f(wt.eb + code) * NSLM_R32;
#pragma unroll
                for (int c = 0; c < 8; ++c) f[c] = (float) is[c] * sc;
            } else if (fmt == MF_BF16) {
                const uint32_t u[4] = {r.raw[0].x, r.raw[0].y, r.raw[0].z, r.raw[0].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) { f[2 * i] = __uint_as_float(u[i] << 16); f[2 * i + 1] = __uint_as_float(u[i] & 0xFFFF0000u); }
            } else {
                const float sc = bf(r.seed), b = bf(r.word);
                if (fmt == MF_Q8) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        f[i] = bfr(sc * (float) ((r.raw[0].x >> (8 * i)) & 255u) + b);
                        f[4 + i] = bfr(sc * (float) ((r.raw[0].y >> (8 * i)) & 255u) + b);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) f[i] = bfr(sc * (float) ((r.raw[0].x >> (4 * i)) & 15u) + b);
                }
            }
        }
#pragma unroll
        for (int q = 0; q < NTERM; ++q) {   // f = hi + mid + lo: each term the BF16 value of what remains (exact)
            uint32_t h[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) { h[i] = tobf(f[i]); f[i] -= bf(h[i]); }
            *(uint4*) &Wsm[buf][q][rr][jb * 8] = make_uint4(h[0] | h[1] << 16, h[2] | h[3] << 16, h[4] | h[5] << 16, h[6] | h[7] << 16);
        }
#pragma unroll
        for (int u = 0; u < MT; ++u) {
            const int i = ptid + 256 * u, n = i >> 1, h = (i & 1) * 16;
            if (PACKED) {
                *(uint4*) &Xsm[buf][n][h] = x.v[2 * u];
                *(uint4*) &Xsm[buf][n][h + 8] = x.v[2 * u + 1];
            } else {
                const uint4 p0 = x.v[4 * u], p1 = x.v[4 * u + 1], p2 = x.v[4 * u + 2], p3 = x.v[4 * u + 3];
#define F(w) __uint_as_float(w)
                *(uint4*) &Xsm[buf][n][h] = make_uint4(pack_bf2(F(p0.x), F(p0.y)), pack_bf2(F(p0.z), F(p0.w)), pack_bf2(F(p1.x), F(p1.y)), pack_bf2(F(p1.z), F(p1.w)));
                *(uint4*) &Xsm[buf][n][h + 8] = make_uint4(pack_bf2(F(p2.x), F(p2.y)), pack_bf2(F(p2.z), F(p2.w)), pack_bf2(F(p3.x), F(p3.y)), pack_bf2(F(p3.z), F(p3.w)));
#undef F
            }
        }
    };

    // ---- the pipeline: each role runs its own loop (same barrier count) so neither carries the other's registers -----------
    // Step ps is produced into buffer ps & 1 while the consumers multiply step ps - 1 out of the other buffer.
    if (producer) {
        MmRec ra = {}, rb = {};
        MmX<MT, PACKED> xa, xb;
        load_x(0, xa);
        load_x(1, xb);
        load_rec(0, ra);
        load_rec(1, rb);
        Chunk rec = load_super(0);
        store_super(0, rec);
        rec = load_super(1);
        lds_barrier();   // super-step 0's records are in LDS
        for (int ps = 0; ps < nsteps; ps += 2) {
            if ((ps & 7) == 0) {   // the next super-step's records (fetched 8 steps ago) go to LDS, the one after is requested
                store_super(((ps >> 3) + 1) & 1, rec);
                rec = load_super((ps >> 3) + 2);
            }
            store_step(0, ps, ra, xa);
            load_x(ps + 2, xa);
            load_rec(ps + 2, ra);
            lds_barrier();
            if (ps + 1 >= nsteps) break;
            store_step(1, ps + 1, rb, xb);
            load_x(ps + 3, xb);
            load_rec(ps + 3, rb);
            lds_barrier();
        }
        return;
    }

    // ---- consumer side ---------------------------------------------------------------------------------------------------
    f32x16 acc[MT][2];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < 2; ++n)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[m][n][i] = 0.0f;
    const int wtok = wv * 32 * MT;          // this consumer wave's first token of the tile
    const bool wave_live = wtok < count;    // a consumer whose tokens are all padding has nothing to multiply
    const int frow = lane & 31, fk = (lane >> 5) * 8;
    auto consume = [&](int buf) {
        if (!wave_live) return;
#pragma unroll
        for (int kk = 0; kk < BK; kk += 16) {
            bf16x8 af[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) af[m] = *(const bf16x8*) &Xsm[buf][wtok + 32 * m + frow][kk + fk];
#pragma unroll
            for (int q = 0; q < NTERM; ++q)   // the largest term first
#pragma unroll
                for (int n = 0; n < 2; ++n) {
                    const bf16x8 bfrag = *(const bf16x8*) &Wsm[buf][q][32 * n + frow][kk + fk];
#pragma unroll
                    for (int m = 0; m < MT; ++m) acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[m], bfrag, acc[m][n], 0, 0, 0);
                }
        }
    };
    lds_barrier();   // pairs with the producers' barrier after the first records
    for (int s = 0; s < nsteps; ++s) {
        lds_barrier();   // step s is in buffer s & 1
        consume(s & 1);
    }
    if (!wave_live) return;
    // accumulator element v of lane l: token row 8 * (v / 4) + 4 * (l / 32) + v % 4, weight column l % 32
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int n = 0; n < 2; ++n)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int tok = wtok + 32 * m + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3), orow = r0 + 32 * n + (lane & 31);
                const int dst = drow[tok];
                if (dst < 0 || orow >= a.R) continue;
                store_y(Y + (size_t) dst * a.ys + orow, acc[m][n][v], a.add, a.f32out);
            }
}

// a kernel that asks for more dynamic LDS than the default limit has the limit raised to what it needs, once (the kernel is a
// template argument so that every kernel has its own "once": kernels of one signature share a pointer type)
template <auto K>
void allow_big_lds(size_t bytes) {
    static const hipError_t once = bytes > 48 * 1024 ? hipFuncSetAttribute((const void*) K, hipFuncAttributeMaxDynamicSharedMemorySize, (int) bytes)
                                                     : hipSuccess;
    (void) once;
}
template <int MT, int NTERM>
constexpr size_t mm_lds() { return (size_t) (2 * NTERM * BM * LDW + 2 * 128 * MT * LDW) * sizeof(uint16_t); }

template <int MT, bool PACKED>
void launch_mm(hipStream_t st, int fmt, const MmArgs& a, WSlice wd, const WSlice* ws, const void* X, float* Y, const int32_t* perm,
               const MmTile* tiles, const int32_t* ntiles, dim3 grid) {
    const bool exact = g_seed_exact && (fmt == MF_SEED4 || fmt == MF_SEED4P4);
    if (exact) {
        const size_t lds = mm_lds<MT, 3>();
        allow_big_lds<k_mm<MT, 3, PACKED>>(lds);
        hipLaunchKernelGGL((k_mm<MT, 3, PACKED>), grid, dim3(512), lds, st, fmt, a, wd, ws, X, Y, perm, tiles, ntiles);
    } else {
        const size_t lds = mm_lds<MT, 1>();
        allow_big_lds<k_mm<MT, 1, PACKED>>(lds);
        hipLaunchKernelGGL((k_mm<MT, 1, PACKED>), grid, dim3(512), lds, st, fmt, a, wd, ws, X, Y, perm, tiles, ntiles);
    }
    host_note_launch();
}

// ---- the streamed kernel: BF16 activations go from global memory straight into LDS -----------------------------------------
//
// For packed (BF16) activations and one BF16 term per weight.  512 threads: waves 0-3 are consumers, waves 4-7 producers.
//   * Weights move in steps of 64 K: producer thread (rr, jb) decodes blocks 2 jb and 2 jb + 1 of row rr (two independent
//     chains in one instruction stream) into one of two LDS tiles; one workgroup barrier per step hands the tile over.
//     The thread's records (a dword of seeds, a dword of coefficient words, a byte of codes) are requested four steps
//     before they are decoded and wait in registers; the four threads of a row read 16 consecutive bytes of each stream,
//     so every line comes from HBM once.
//   * Activations never touch a register on their way in: consumer wave w owns tokens [32 MT w, 32 MT (w + 1)) and fetches
//     its own rows with global_load_lds_dwordx4 (each lane lands 16 bytes at consecutive LDS addresses) into a ring of
//     four 32-K stages, three stages ahead of the MFMAs.  Only the owning wave reads those rows back, so the ring needs
//     no barrier - the wave waits on its own vector-memory counter.
//   * The 16-byte slots of a row (4 per 64-byte row) are stored XOR-swizzled by the row number so that the fragment reads
//     (32 rows x one slot per half wave) spread over all banks although the rows are unpadded; the swizzle is applied on
//     the global side, where every lane is free to pick the address it loads.
#define WK 64            // K per weight step
#define LDW2 72          // weight tile row stride in BF16 elements (144 bytes)
#define XCHUNK 2048      // BF16 elements of an activation chunk: 32 tokens x 64 K
#define RECD 4           // weight steps between a record's request and its decode

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t cvt_pk_bf16(float lo, float hi) {   // v_cvt_pk_bf16_f32: both round to nearest even
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ int x_swizzle(int row) { return ((row >> 1) & 7) ^ ((row & 1) << 2); }
template <int N>
__device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

struct MmRec2 {
    uint4 raw[2];      // BF16: the two blocks; Q8: raw[0]; Q4: raw[0].xy
    uint32_t u, v, c;  // seeds: two seeds, two coefficient words, the codes byte; Q8 / Q4: the group's scale and bias bits
};

template <int CT, int NCW, int XCH, int FMT>
__global__ void __launch_bounds__(64 * (NCW + 4)) k_mm_stream(MmArgs a, WSlice wd, const WSlice* ws, const uint16_t* X, float* Y,
                                                   const int32_t* perm, const MmTile* tiles, const int32_t* ntiles) {
    constexpr int BN = 32 * CT * NCW, NTHR = 64 * (NCW + 4);   // XCH: chunks in a consumer wave's ring
    constexpr bool seedf = FMT == MF_SEED4P4 || FMT == MF_SEED4;
    extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
    uint16_t* Xs = smem;                                   // [NCW waves][XCH chunks][32 rows][64 K], slots swizzled
    typedef uint16_t WTile[BM][LDW2];
    WTile* Wsm = (WTile*) (smem + NCW * XCH * XCHUNK);          // [2]
    __shared__ int srow[BN], drow[BN];
    __shared__ uint32_t tab[NSLM_TAB_WORDS];
    // FSYNC (one consumer wave: the grouped launches of a batched step, whose time is the decoders'): the weight tiles change hands
    // by counters in LDS instead of a workgroup barrier a step.  A decoder waits only for the consumer to have read the tile it
    // is about to overwrite (two steps back - it has, when the decode is what takes the time), never for the other decoders: with
    // the barrier every step cost each decoder wave the wait for the slowest of the four (C2 at 32 rows: 271.2 -> 263.5 us, C3 at 16:
    // 627 -> 609; with no hand-over at all and garbage computed: 247 and 540).  The dense 512-token GEMM with its eight consumer
    // waves is indifferent to the barrier and keeps it.
    constexpr bool FSYNC = NCW == 1;
    constexpr int NWT = FSYNC && XCH == 2 ? 3 : 2;   // weight tiles in LDS: a third one where the activation ring leaves room for it
    __shared__ __attribute__((aligned(16))) uint32_t flg[8];
    const int tid = threadIdx.x, lane = tid & 63, wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool producer = wv >= NCW;
    const bool grouped = tiles != nullptr;
    if (grouped && ntiles && (int) blockIdx.y >= *ntiles) return;
    const bool gu = a.a16 != nullptr;   // (grouped launches only)
    const int r0 = (int) blockIdx.x * (gu ? BM / 2 : BM);
    int start, count;
    WSlice wt;
    if (grouped) {
        const MmTile tl = tiles[blockIdx.y];
        if (blockIdx.z) {   // the launch's second matrix: same tiles and activations, its own slices and output
            ws = a.ws2;
            Y = a.y2;
        }
        // (gate / up tiles: the decoder waves of the tile's upper 32 rows read the up slice)
        wt = gu && tid >= 64 * NCW + 128 ? a.ws2[tl.slice] : ws[tl.slice];
        start = tl.start;
        count = min(tl.count, BN);   // (a tile never holds more than the launch was told: see mm_grouped)
        if (BN < MMT_BN && tl.count > BN) {
            // a broken promise is made visible: the pairs this launch cannot reach are stored as NaN, not left stale
            const int rows = gu ? BM / 2 : BM;
            for (int i = BN * rows + tid; i < tl.count * rows; i += NTHR) {
                const int orow = r0 + i % rows;
                const size_t at = (size_t) perm[tl.start + i / rows] * a.ys + orow;
                if (orow < a.R) {
                    if (gu) a.a16[at] = 0x7FC0u;
                    else Y[at] = __uint_as_float(0x7FC00000u);
                }
            }
        }
    } else {
        wt = wd;
        start = (int) blockIdx.y * BN;
        count = min(BN, a.T - start);
    }
    if (count < 1) return;
    if (seedf) load_tables(tab);
    if (FSYNC && tid < 8) flg[tid] = 0u;
    // flg[w], w < 4: weight steps decoder wave w has written; flg[4]: steps the consumer has read.  (One word a decoder, not a sum:
    // with two tiles a decoder may be a step ahead of another, and three waves a step ahead would make up for one a step behind.)
    // The polls and the posts are a few instructions of inline code with registers of their own: written in the language (volatile
    // reads in a loop, s_setprio builtins around it) they cost 20 registers and with them the fifth wave a SIMD, i.e. a resident
    // workgroup - a quarter more time instead of less.  A poll is bounded; a waiting wave drops to priority 0, so its polls take
    // only the issue slots nobody else wants.
    auto wait_written = [&](uint32_t need) {   // all four decoders have written `need` steps; back at priority 3
        uint32_t g0, g1, g2, g3, spins = 1u << 24;
        asm volatile("s_setprio 0\n\t"
                     "1:\n\t"
                     "ds_read_b32 %0, %5\n\t"
                     "ds_read_b32 %1, %5 offset:4\n\t"
                     "ds_read_b32 %2, %5 offset:8\n\t"
                     "ds_read_b32 %3, %5 offset:12\n\t"
                     "s_waitcnt lgkmcnt(0)\n\t"
                     "v_min3_u32 %0, %0, %1, %2\n\t"
                     "v_min_u32 %0, %0, %3\n\t"
                     "v_cmp_ge_u32 vcc, %0, %6\n\t"
                     "s_cbranch_vccnz 2f\n\t"
                     "s_sub_u32 %4, %4, 1\n\t"
                     "s_cmp_lg_u32 %4, 0\n\t"
                     "s_cbranch_scc1 1b\n\t"
                     "2:\n\t"
                     "s_setprio 3"
                     : "=&v"(g0), "=&v"(g1), "=&v"(g2), "=&v"(g3), "+s"(spins)
                     : "v"((uint32_t) (uintptr_t) &flg[0]), "v"(need)
                     : "vcc", "scc", "memory");
    };
    auto wait_read = [&](uint32_t need) {   // the consumer has read `need` steps; back at priority 2
        uint32_t got, spins = 1u << 24;
        asm volatile("s_setprio 0\n\t"
                     "1:\n\t"
                     "ds_read_b32 %0, %2\n\t"
                     "s_waitcnt lgkmcnt(0)\n\t"
                     "v_cmp_ge_u32 vcc, %0, %3\n\t"
                     "s_cbranch_vccnz 2f\n\t"
                     "s_sub_u32 %1, %1, 1\n\t"
                     "s_cmp_lg_u32 %1, 0\n\t"
                     "s_cbranch_scc1 1b\n\t"
                     "2:\n\t"
                     "s_setprio 2"
                     : "=&v"(got), "+s"(spins)
                     : "v"((uint32_t) (uintptr_t) &flg[4]), "v"(need)
                     : "vcc", "scc", "memory");
    };
    // (every lane stores the same word; the wave's LDS accesses before it are complete)
    auto post = [&](int which, uint32_t v) {
        asm volatile("s_waitcnt lgkmcnt(0)\n\tds_write_b32 %0, %1" ::"v"((uint32_t) (uintptr_t) &flg[which]), "v"(v) : "memory");
    };
    for (int i = tid; i < BN; i += NTHR) {
        const bool ok = i < count;
        const int j = start + (ok ? i : 0);   // padding rows load the tile's first row; their results are never stored
        srow[i] = grouped ? perm[j] / a.xdiv : j;
        drow[i] = !ok ? -1 : grouped ? perm[j] : j;
    }
    __syncthreads();
    const int nsteps = a.K / WK;

    if (producer) {
        if (FSYNC) __builtin_amdgcn_s_setprio(2);
        // rows past R decode row R - 1 again (never stored)
        const int ptid = tid - 64 * NCW, rr = ptid >> 2, jb = ptid & 3, row = min(r0 + (gu ? rr & 31 : rr), a.R - 1), nbk = a.K / 8;
        // This thread's two blocks of step s.  Always the same loads - steps past the end request the last step again, and a
        // stream at any 2-byte boundary is read by the same instruction (the load is typed with that alignment) - so that the
        // compiler knows how many loads are in flight at every use: with the loads inside conditions it had waited, after
        // every third and fourth step, for the records it had requested a moment before.
        typedef uint32_t u32_a2 __attribute__((aligned(2)));
        auto load_rec = [&](int s_, MmRec2& r) {
            const int s = min(s_, nsteps - 1);
            if (seedf) {
                const size_t g = (size_t) row * nbk + (size_t) s * (WK / 8) + 2 * jb;   // even: the pair shares a dword and a codes byte
                r.u = *(const NSLM_GLOBAL u32_a2*) (gp<uint16_t>(wt.p[0]) + g);
                r.v = *(const NSLM_GLOBAL u32_a2*) (gp<uint16_t>(wt.p[1]) + g);
                if (FMT == MF_SEED4P4) r.c = gp<uint8_t>(wt.p[3])[g >> 1];
                return;
            }
            const size_t e0 = (size_t) row * a.K + (size_t) s * WK + 16 * jb;   // first of 16 elements
            if (FMT == MF_BF16) {
                r.raw[0] = ldg16(gp<uint16_t>(wt.p[0]) + e0);
                r.raw[1] = ldg16(gp<uint16_t>(wt.p[0]) + e0 + 8);
            } else {
                const size_t gi = e0 >> group_shift(wt);
                r.u = gp<uint16_t>(wt.p[1])[gi];
                r.v = gp<uint16_t>(wt.p[2])[gi];
                if (FMT == MF_Q8) r.raw[0] = ldg16(gp<uint8_t>(wt.p[0]) + e0);
                else r.raw[0] = make_uint4(gp<uint32_t>(wt.p[0])[e0 / 8], gp<uint32_t>(wt.p[0])[e0 / 8 + 1], 0, 0);
            }
        };
        // seeds: the table reads of a step's two blocks are issued one step early (its records are in registers by then)
        struct Look { uint32_t g[2], qa[2], qb[2]; };
        auto lookup = [&](const MmRec2& r, Look& k) {
            if (!seedf) return;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t seed = h ? r.u >> 16 : r.u & 0xFFFFu, word = h ? r.v >> 16 : r.v & 0xFFFFu;
                k.g[h] = stream_of(tab, seed);
                k.qa[h] = FMT == MF_SEED4P4 ? tab[512 + (word & 0xFFu)] : tab[512 + ((word >> 4) & 0xFFu)];
                k.qb[h] = FMT == MF_SEED4P4 ? tab[512 + (word >> 8)] : tab[512 + (word >> 12)];
            }
        };
        auto produce = [&](int s, const MmRec2& r, const Look& k) {
            float f[2][8];
            {
                if (seedf) {
                    const uint32_t up[2] = {r.u << 16, r.u}, word[2] = {r.v & 0xFFFFu, r.v >> 16};
                    int is[2][8];
                    if (FMT == MF_SEED4P4) isum2_p4(up, k.g, k.qa, k.qb, is);
                    else isum2_p3(up, k.g, k.qa, k.qb, is);
                    float sc[2];
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int code = FMT == MF_SEED4P4 ? (int) ((r.c >> (4 * h)) & 15u) : (int) (word[h] & 15u);
                        sc[h] = pow2f(wt.eb + code) * NSLM_R32;
                    }
#pragma unroll
                    for (int c = 0; c < 8; ++c)
#pragma unroll
                        for (int h = 0; h < 2; ++h) f[h][c] = (float) is[h][c];
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int c = 0; c < 8; ++c)
#pragma unroll
                        for (int h = 0; h < 2; ++h) f[h][c] *= sc[h];
                    __builtin_amdgcn_sched_barrier(0);
                } else if (FMT == MF_BF16) {
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const uint32_t u[4] = {r.raw[h].x, r.raw[h].y, r.raw[h].z, r.raw[h].w};
#pragma unroll
                        for (int i = 0; i < 4; ++i) { f[h][2 * i] = __uint_as_float(u[i] << 16); f[h][2 * i + 1] = __uint_as_float(u[i] & 0xFFFF0000u); }
                    }
                } else {
                    const float sc = bf(r.u), b = bf(r.v);
                    const uint32_t u[4] = {r.raw[0].x, r.raw[0].y, r.raw[0].z, r.raw[0].w};
                    if (FMT == MF_Q8) {
#pragma unroll
                        for (int i = 0; i < 16; ++i) f[i >> 3][i & 7] = bfr(sc * (float) ((u[i >> 2] >> (8 * (i & 3))) & 255u) + b);
                    } else {
#pragma unroll
                        for (int i = 0; i < 16; ++i) f[i >> 3][i & 7] = bfr(sc * (float) ((u[i >> 3] >> (4 * (i & 7))) & 15u) + b);
                    }
                }
            }
            if (FSYNC && s >= NWT) wait_read((uint32_t) (s - NWT + 1));
#pragma unroll
            for (int h = 0; h < 2; ++h)
                *(uint4*) &Wsm[NWT == 2 ? s & 1 : s % NWT][rr][16 * jb + 8 * h] = make_uint4(cvt_pk_bf16(f[h][0], f[h][1]), cvt_pk_bf16(f[h][2], f[h][3]),
                                                                       cvt_pk_bf16(f[h][4], f[h][5]), cvt_pk_bf16(f[h][6], f[h][7]));
        };
        MmRec2 rec[RECD] = {};
        Look look[2] = {};
#pragma unroll
        for (int u = 0; u < RECD; ++u) load_rec(u, rec[u]);
        lookup(rec[0], look[0]);
        auto one = [&](int s, auto uc) {
            constexpr int u = decltype(uc)::value;
            lookup(rec[(u + 1) % RECD], look[(u + 1) & 1]);   // the next step's table reads travel under this step's decode
            produce(s, rec[u], look[u & 1]);
            load_rec(s + RECD, rec[u]);
            if (FSYNC) post(wv - NCW, (uint32_t) s + 1u);
            else lds_barrier();
        };
        // whole rounds of the record ring in a loop with one way out (a conditional exit per step costs the loop a
        // register move per record word and step), the steps left over after it
        int s0 = 0;
        for (; s0 + RECD <= nsteps; s0 += RECD) {
            one(s0, std::integral_constant<int, 0>{});
            one(s0 + 1, std::integral_constant<int, 1>{});
            one(s0 + 2, std::integral_constant<int, 2>{});
            one(s0 + 3, std::integral_constant<int, 3>{});
        }
        static_assert(RECD == 4, "the unrolling above");
        if (s0 < nsteps) one(s0, std::integral_constant<int, 0>{});
        if (s0 + 1 < nsteps) one(s0 + 1, std::integral_constant<int, 1>{});
        if (s0 + 2 < nsteps) one(s0 + 2, std::integral_constant<int, 2>{});
        return;
    }

    // ---- consumer side ---------------------------------------------------------------------------------------------------
    const int wtok = wv * 32 * CT;          // this wave's first token of the tile
    if (wtok >= count) {                    // a wave whose tokens are all padding has nothing to multiply
        if (FSYNC) post(4, 0x7FFFFFFFu);
        else for (int s = 0; s < nsteps; ++s) lds_barrier();
        return;
    }
    __builtin_amdgcn_s_setprio(FSYNC ? 3 : 2);   // the matrix pipeline's instruction stream goes first when both roles are ready
    f32x16 acc[CT][2];
#pragma unroll
    for (int m = 0; m < CT; ++m)
#pragma unroll
        for (int n = 0; n < 2; ++n)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[m][n][i] = 0.0f;
    // Chunk c = s MT + m is the 32 tokens of m-tile m x the 64 K of weight step s: 4 KB, four instructions, instruction i
    // landing rows 8 i + lane / 8, slot lane % 8 (whole 128-byte lines per row).  The wave's ring holds XCH chunks.
    // Offsets from X are 32-bit where the host has checked that they fit (MT > 1), so the loads take the scalar base +
    // vector offset form and cost no address arithmetic.
    typedef typename std::conditional<CT == 1, size_t, uint32_t>::type xoff_t;
    xoff_t xoff[4 * CT];
#pragma unroll
    for (int i = 0; i < 4 * CT; ++i) {
        const int row = 8 * (i & 3) + (lane >> 3), n = wtok + 32 * (i >> 2) + row, piece = (lane & 7) ^ x_swizzle(row);
        xoff[i] = (xoff_t) (((size_t) srow[n] * (size_t) a.xs + 8u * (size_t) piece) * 2u);
    }
    uint16_t* ring = Xs + wv * (XCH * XCHUNK);
    auto fetch = [&](int sf, int mf, int slot) {   // chunk (sf, mf) -> ring slot (past the end: a harmless reload of the last step)
        const char* src = (const char*) X + (size_t) min(sf, nsteps - 1) * WK * 2;
        uint16_t* dst = ring + slot * XCHUNK;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*) (src + xoff[4 * mf + i]),
                                             (__attribute__((address_space(3))) void*) (dst + i * 512), 16, 0, 0);
    };
    const int frow = lane & 31, fhi = lane >> 5, fsw = x_swizzle(frow);
    auto load_a = [&](int slot, bf16x8 (&af)[4]) {
        const uint16_t* ch = ring + slot * XCHUNK + frow * 64;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) af[kk] = *(const bf16x8*) (ch + ((2 * kk + fhi) ^ fsw) * 8);
    };
    // One weight step: chunk m multiplies out of fragment set (m even ? fa : fb) while the next chunk's fragments travel
    // into the other set; with MT odd the sets have swapped roles when the step ends.
    auto step = [&](int s, bf16x8 (&fa)[4], bf16x8 (&fb)[4]) {
        if (FSYNC) wait_written((uint32_t) s + 1u);
        else lds_barrier();   // weight step s is in tile s & 1
        bf16x8 bq[4][2];
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
#pragma unroll
            for (int n = 0; n < 2; ++n) bq[kk][n] = *(const bf16x8*) &Wsm[NWT == 2 ? s & 1 : s % NWT][32 * n + frow][16 * kk + 8 * fhi];
        if (FSYNC) post(4, (uint32_t) s + 1u);
#pragma unroll
        for (int m = 0; m < CT; ++m) {
            const int c = s * CT + m;
            fetch(s + (m + XCH - 1) / CT, (m + XCH - 1) % CT, (c + XCH - 1) % XCH);   // into the slot chunk c - 1 just left
            wait_vm<4 * (XCH - 2)>();   // chunks up to c + 1 have landed
            load_a((c + 1) % XCH, (m & 1) ? fa : fb);
#pragma unroll
            for (int kk = 0; kk < 4; ++kk)
#pragma unroll
                for (int n = 0; n < 2; ++n)
                    acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(((m & 1) ? fb : fa)[kk], bq[kk][n], acc[m][n], 0, 0, 0);
        }
    };
    if (nsteps > 0) {
#pragma unroll
        for (int c = 0; c < XCH - 1; ++c) fetch(c / CT, c % CT, c);
    }
    bf16x8 f0[4], f1[4];
    wait_vm<4 * (XCH - 2)>();   // chunk 0 has landed
    load_a(0, f0);
    for (int s = 0; s < nsteps; s += 2) {
        step(s, f0, f1);
        if (s + 1 >= nsteps) break;
        if (CT & 1) step(s + 1, f1, f0);
        else step(s + 1, f0, f1);
    }
    wait_vm<0>();
    // accumulator element v of lane l: token row 8 * (v / 4) + 4 * (l / 32) + v % 4, weight column l % 32
    const bool plain = !a.add && !a.f32out;
    if (gu) {   // n = 0: the gate rows, n = 1: the same rows of up, in the same lane: the values the two GEMMs would have stored
                // (rounded to BF16), then SwiGLU and its rounding, stored as BF16 bits
#pragma unroll
        for (int m = 0; m < CT; ++m)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int tok = wtok + 32 * m + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                const int dst = drow[tok], orow = r0 + (lane & 31);
                if (dst < 0 || orow >= a.R) continue;
                const float av = bfr(silu_bf(bfr(acc[m][0][v])) * bfr(acc[m][1][v]));
                a.a16[(size_t) dst * a.ys + orow] = (uint16_t) (__float_as_uint(av) >> 16);
            }
        return;
    }
#pragma unroll
    for (int m = 0; m < CT; ++m)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int tok = wtok + 32 * m + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
            const int dst = drow[tok];
            if (dst < 0) continue;
#pragma unroll
            for (int n = 0; n < 2; ++n) {
                const int orow = r0 + 32 * n + (lane & 31);
                if (orow >= a.R) continue;
                float* yo = Y + (size_t) dst * a.ys + orow;
                if (plain) __builtin_nontemporal_store(bfr(acc[m][n][v]), yo);
                else store_y(yo, acc[m][n][v], a.add, a.f32out);
            }
        }
}
template <int NCW, int XCH>
constexpr size_t mm_stream_lds() { return (size_t) (NCW * XCH * XCHUNK + (NCW == 1 && XCH == 2 ? 3 : 2) * BM * LDW2) * sizeof(uint16_t); }
// the streamed kernel takes BF16 activations in 16-byte aligned rows, one BF16 term per weight, K in whole weight steps
// (xrows > 0: the row count, for the variants that address rows by 32-bit byte offsets)
bool stream_ok(int fmt, int K, int xs, const void* x, long long xrows) {
    const bool exact = g_seed_exact && (fmt == MF_SEED4 || fmt == MF_SEED4P4);
    return !exact && K % WK == 0 && xs % 8 == 0 && ((uintptr_t) x & 15u) == 0 && (xrows * xs + K) * 2 < (1ll << 32);
}
template <int CT, int NCW, int XCH, int FMT>
void launch_mm_stream_f(hipStream_t st, const MmArgs& a, WSlice wd, const WSlice* ws, const void* X, float* Y, const int32_t* perm,
                        const MmTile* tiles, const int32_t* ntiles, dim3 grid) {
    const size_t lds = mm_stream_lds<NCW, XCH>();
    allow_big_lds<k_mm_stream<CT, NCW, XCH, FMT>>(lds);
    hipLaunchKernelGGL((k_mm_stream<CT, NCW, XCH, FMT>), grid, dim3(64 * (NCW + 4)), lds, st, a, wd, ws, (const uint16_t*) X, Y, perm, tiles, ntiles);
    host_note_launch();
}
template <int CT, int NCW, int XCH>
void launch_mm_stream(hipStream_t st, int fmt, const MmArgs& a, WSlice wd, const WSlice* ws, const void* X, float* Y, const int32_t* perm,
                      const MmTile* tiles, const int32_t* ntiles, dim3 grid) {
    switch (fmt) {
        case MF_SEED4P4: launch_mm_stream_f<CT, NCW, XCH, MF_SEED4P4>(st, a, wd, ws, X, Y, perm, tiles, ntiles, grid); break;
        case MF_SEED4: launch_mm_stream_f<CT, NCW, XCH, MF_SEED4>(st, a, wd, ws, X, Y, perm, tiles, ntiles, grid); break;
        case MF_BF16: launch_mm_stream_f<CT, NCW, XCH, MF_BF16>(st, a, wd, ws, X, Y, perm, tiles, ntiles, grid); break;
        case MF_Q8: launch_mm_stream_f<CT, NCW, XCH, MF_Q8>(st, a, wd, ws, X, Y, perm, tiles, ntiles, grid); break;
        default: launch_mm_stream_f<CT, NCW, XCH, MF_Q4>(st, a, wd, ws, X, Y, perm, tiles, ntiles, grid); break;
    }
}

template <bool PACKED>
void mm_dense(hipStream_t st, int fmt, WSlice w, int K, int R, const void* x, int xs, float* y, int ys, int T, int add) {
    if (T < 1 || R < 1) return;
    MmArgs a = {K, R, T, xs, ys, 1, add, host_store_f32(), nullptr, nullptr, nullptr};
    const unsigned gx = (unsigned) (R + BM - 1) / BM;
    if (PACKED && stream_ok(fmt, K, xs, x, T)) {
        if (T > 256) launch_mm_stream<2, 8, 4>(st, fmt, a, w, nullptr, x, y, nullptr, nullptr, nullptr, dim3(gx, (unsigned) (T + 511) / 512));
        else if (T > 128) launch_mm_stream<2, 4, 8>(st, fmt, a, w, nullptr, x, y, nullptr, nullptr, nullptr, dim3(gx, 1));
        else launch_mm_stream<1, 4, 8>(st, fmt, a, w, nullptr, x, y, nullptr, nullptr, nullptr, dim3(gx, 1));
        return;
    }
    if (T > 256) launch_mm<4, PACKED>(st, fmt, a, w, nullptr, x, y, nullptr, nullptr, nullptr, dim3(gx, (unsigned) (T + 511) / 512));
    else if (T > 128) launch_mm<2, PACKED>(st, fmt, a, w, nullptr, x, y, nullptr, nullptr, nullptr, dim3(gx, 1));
    else launch_mm<1, PACKED>(st, fmt, a, w, nullptr, x, y, nullptr, nullptr, nullptr, dim3(gx, 1));
}
template <bool PACKED>
void mm_grouped(hipStream_t st, int fmt, const WSlice* ws, int K, int R, const void* x, int xs, float* y, int ys, int xdiv,
                const int32_t* perm, const MmTile* tiles, const int32_t* ntiles, int grid_tiles, int tile_rows,
                const WSlice* ws2 = nullptr, float* y2 = nullptr) {
    if (grid_tiles < 1 || R < 1) return;
    MmArgs a = {K, R, 0, xs, ys, xdiv, 0, host_store_f32(), ws2, y2, nullptr};
    WSlice none = {};
    if (PACKED && stream_ok(fmt, K, xs, x, 0)) {
        // grouped tiles are mostly a few pairs of one expert: decode-bound, so a short ring buys two workgroups a CU - and
        // where the caller knows that no tile holds more than 32 pairs, one multiplying wave instead of four buys four
        const dim3 grid((unsigned) (R + BM - 1) / BM, (unsigned) grid_tiles, ws2 ? 2u : 1u);
        // (one multiplying wave: four workgroups a CU fit either three weight tiles and a ring of two activation chunks or two and
        // three.  C2 at 32 rows, P = 4: 260.3 against 263.5 us; C3 at 16 rows, P = 3, whose steps are shorter than an activation
        // chunk's way from memory: 620 against 609; three and three, three workgroups a CU: 265.2 and 615.6)
        if (tile_rows <= 32 && fmt == MF_SEED4P4) launch_mm_stream<1, 1, 2>(st, fmt, a, none, ws, x, y, perm, tiles, ntiles, grid);
        else if (tile_rows <= 32) launch_mm_stream<1, 1, 3>(st, fmt, a, none, ws, x, y, perm, tiles, ntiles, grid);
        else launch_mm_stream<1, 4, 3>(st, fmt, a, none, ws, x, y, perm, tiles, ntiles, grid);
        return;
    }
    launch_mm<1, PACKED>(st, fmt, a, none, ws, x, y, perm, tiles, ntiles, dim3((unsigned) (R + BM - 1) / BM, (unsigned) grid_tiles));
    if (ws2) {   // (the first-generation kernel takes one matrix a launch)
        a.ws2 = nullptr;
        a.y2 = nullptr;
        launch_mm<1, PACKED>(st, fmt, a, none, ws2, x, y2, perm, tiles, ntiles, dim3((unsigned) (R + BM - 1) / BM, (unsigned) grid_tiles));
    }
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
    mm_grouped<false>((hipStream_t) s, fmt, ws, K, R, x, xs, y, ys, xdiv, perm, tiles, nullptr, ntiles, MMT_BN);
}
void kc_mm_grouped_dev(kc_stream_t s, int fmt, const WSlice* ws, int K, int R, const float* x, int xs, float* y, int ys,
                       int xdiv, const int32_t* perm, const MmTile* tiles, const int32_t* ntiles, int max_tiles,
                       const uint32_t* G) {
    (void) G;
    mm_grouped<false>((hipStream_t) s, fmt, ws, K, R, x, xs, y, ys, xdiv, perm, tiles, ntiles, max_tiles, MMT_BN);
}
void kc_mm_grouped_packed(kc_stream_t s, int fmt, const WSlice* ws, int K, int R, const uint16_t* x, int xs, float* y,
                          int ys, int xdiv, const int32_t* perm, const MmTile* tiles, const int32_t* nt, int max_tiles,
                          const uint32_t* G) {
    (void) G;
    mm_grouped<true>((hipStream_t) s, fmt, ws, K, R, x, xs, y, ys, xdiv, perm, tiles, nt, max_tiles, MMT_BN);
}
void kc_mm_grouped_packed_rows(kc_stream_t s, int fmt, const WSlice* ws, int K, int R, const uint16_t* x, int xs, float* y,
                               int ys, int xdiv, const int32_t* perm, const MmTile* tiles, const int32_t* nt, int max_tiles,
                               int tile_rows) {
    mm_grouped<true>((hipStream_t) s, fmt, ws, K, R, x, xs, y, ys, xdiv, perm, tiles, nt, max_tiles, tile_rows < 1 ? MMT_BN : tile_rows);
}
int kc_mm_grouped_swiglu(kc_stream_t s, int fmt, const WSlice* gate, const WSlice* up, int K, int R, const uint16_t* x, int xs, uint16_t* a16,
                         int ys, int xdiv, const int32_t* perm, const MmTile* tiles, const int32_t* nt, int max_tiles, int tile_rows) {
    if (max_tiles < 1 || R < 1) return 0;
    if (!stream_ok(fmt, K, xs, x, 0) || host_store_f32()) return -1;
    MmArgs a = {K, R, 0, xs, ys, xdiv, 0, 0, up, nullptr, a16};
    WSlice none = {};
    const dim3 grid((unsigned) (R + BM / 2 - 1) / (BM / 2), (unsigned) max_tiles);
    if (tile_rows >= 1 && tile_rows <= 32 && fmt == MF_SEED4P4) launch_mm_stream<1, 1, 2>((hipStream_t) s, fmt, a, none, gate, x, nullptr, perm, tiles, nt, grid);   // (as in mm_grouped)
    else if (tile_rows >= 1 && tile_rows <= 32) launch_mm_stream<1, 1, 3>((hipStream_t) s, fmt, a, none, gate, x, nullptr, perm, tiles, nt, grid);
    else launch_mm_stream<1, 4, 3>((hipStream_t) s, fmt, a, none, gate, x, nullptr, perm, tiles, nt, grid);
    return 0;
}
void kc_mm_grouped_packed_pair(kc_stream_t s, int fmt, const WSlice* ws_a, const WSlice* ws_b, int K, int R, const uint16_t* x, int xs,
                               float* ya, float* yb, int ys, int xdiv, const int32_t* perm, const MmTile* tiles, const int32_t* nt,
                               int max_tiles, int tile_rows) {
    mm_grouped<true>((hipStream_t) s, fmt, ws_a, K, R, x, xs, ya, ys, xdiv, perm, tiles, nt, max_tiles, tile_rows < 1 ? MMT_BN : tile_rows,
                     ws_b, yb);
}

}   // extern "C"
