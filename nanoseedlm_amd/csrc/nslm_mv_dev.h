// nslm_mv_dev.h - device pieces of the seed matvec shared by the stand-alone kernels (nslm_mv.hip) and the fused MoE
// decode kernel (nslm_fused.hip): a chunk's records, the chunk x activations product, the generic block decoder.
#pragma once
#include "nslm_dev.h"

namespace nslm {

struct Chunk {
    uint4 sd, cw;
    uint32_t codes;
};

// A chunk's records: 16 bytes of seeds, 16 of coefficient (nibble) words, 4 of exponent codes.  The streams of a slice may start
// at any 2-byte (codes: 1-byte) boundary - the loads are typed with that alignment, and the target reads a misaligned
// unit in one instruction all the same - so there is one code path and no branch on the alignment.  The loads are
// unconditional (callers clamp `unit` to a chunk that exists): after a load under a condition the compiler no longer knows how
// many loads are in flight and waits for all of them before the next use of any loaded value - the activations' staging then
// waited for the records.
typedef uint32_t u32x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
typedef uint32_t u32_a1 __attribute__((aligned(1)));
template <int P>
__device__ __forceinline__ Chunk load_chunk(const WSlice& w, uint32_t unit) {
    Chunk c;
    c.codes = 0;
    // In pieces, in the order the blocks are decoded - the codes, then seeds and coefficient words of blocks 0..3, then of blocks
    // 4..7: a wave's loads return in the order they went out, and so do the whole launch's requests to the memory, so when every
    // wave asks for its records at once the first pieces of all of them arrive before any last piece does.  A thread starts
    // on its first blocks when 20 of its 36 bytes are there.
    typedef uint32_t u32x2_a2 __attribute__((ext_vector_type(2), aligned(2)));
    const NSLM_GLOBAL uint8_t* ps = gp<uint8_t>(w.p[0]) + (size_t) unit * 16;
    const NSLM_GLOBAL uint8_t* pc = gp<uint8_t>(w.p[1]) + (size_t) unit * 16;
    if (P == 4) c.codes = *(const NSLM_GLOBAL u32_a1*) (gp<uint8_t>(w.p[3]) + (size_t) unit * 4);
    const u32x2_a2 s0 = *(const NSLM_GLOBAL u32x2_a2*) ps, c0 = *(const NSLM_GLOBAL u32x2_a2*) pc;
    asm volatile("" ::: "memory");   // (keeps the halves apart: left alone, the compiler joins them into 16-byte loads again)
    const u32x2_a2 s1 = *(const NSLM_GLOBAL u32x2_a2*) (ps + 8), c1 = *(const NSLM_GLOBAL u32x2_a2*) (pc + 8);
    c.sd = make_uint4(s0.x, s0.y, s1.x, s1.y);
    c.cw = make_uint4(c0.x, c0.y, c1.x, c1.y);
    return c;
}
__device__ __forceinline__ bool streams_aligned(int P, const WSlice& w) {
    return (((uintptr_t) w.p[0] | (uintptr_t) w.p[1]) & 15u) == 0 && (P != 4 || ((uintptr_t) w.p[3] & 3u) == 0);
}

__device__ __forceinline__ uint32_t word_of(const uint4& v, int i) { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }

// ---- activations as the matvec reads them ----------------------------------------------------------------------------------
// P = 3: a block's 8 activations as they are.  P = 4: the 12 values of the nibble-column form (cols_p4 in nslm_dev.h):
// X(0..10), X(m) = x_m + 16 x_(m-1) + 256 x_(m-2) + 4096 x_(m-3) (terms outside 0..7 dropped), and CX = 2184 sum x.  One fixed
// order of operations, so every kernel that stages a row forms the same bits.
// COLS: the column form (P = 4 only; passes of more than two tokens read too much LDS with it - 48 bytes a token and block where
// the weights' form reads 32 - and are given COLS = false: the block's activations as they are, like P = 3).
template <int P, bool COLS = (P == 4)>
constexpr int xw() { return COLS ? 12 : 8; }          // floats a block
// LDS floats per 64-weight chunk (8 blocks + 4): 16-byte reads of 8 consecutive lanes land on 32 distinct banks (68 and 100 are 4 mod 32)
template <int P, bool COLS = (P == 4)>
constexpr int xpad() { return 8 * xw<P, COLS>() + 4; }
template <int P, bool COLS = (P == 4)>
__device__ __forceinline__ void xform_block(const float (&x)[8], float (&X)[xw<P, COLS>()]) {
    static_assert(!COLS || P == 4, "the column form is the P = 4 block's");
    if constexpr (COLS) {
#pragma unroll
        for (int m = 0; m < 11; ++m) {
            float v = m < 8 ? x[m] : 0.0f;
            if (m >= 1 && m <= 8) v = fmaf(16.0f, x[m - 1], v);
            if (m >= 2 && m <= 9) v = fmaf(256.0f, x[m - 2], v);
            if (m >= 3) v = fmaf(4096.0f, x[m - 3], v);
            X[m] = v;
        }
        X[11] = 2184.0f * (((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7])));
    } else {
#pragma unroll
        for (int c = 0; c < 8; ++c) X[c] = x[c];
    }
}
// block `blk` of a row into its place of a chunk-padded LDS row
template <int P, bool COLS = (P == 4)>
__device__ __forceinline__ void store_block(float* row, int blk, const float (&x)[8]) {
    float X[xw<P, COLS>()];
    xform_block<P, COLS>(x, X);
    float* dst = row + (blk >> 3) * xpad<P, COLS>() + (blk & 7) * xw<P, COLS>();
#pragma unroll
    for (int i = 0; i < xw<P, COLS>(); i += 4) *(float4*) (dst + i) = make_float4(X[i], X[i + 1], X[i + 2], X[i + 3]);
}

// One chunk (8 blocks) against NT tokens.  xr: this chunk's staged activations, token t at xr + t * xstride (registers when
// NT == 1 and the caller copied them, LDS otherwise).  acc[t] accumulates 2^e * (block . x) per block (R32 is applied to the row sum).
template <int P, int NT>
__device__ __forceinline__ void block_dot(const int (&is)[8], float e2, int b, const float* xr, int xstride, float (&acc)[NT]) {
    float w[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) w[c] = (float) is[c];
    if constexpr (NT == 1) {   // one token: its activations are in registers (or one LDS row)
        const float* xb = xr + 8 * b;
        float d = w[0] * xb[0];
#pragma unroll
        for (int c = 1; c < 8; ++c) d = fmaf(w[c], xb[c], d);
        acc[0] = fmaf(d, e2, acc[0]);
    } else {
        // Every token of the pass is computed (rows past nt hold whatever the LDS holds; their sums are never stored):
        // an early exit on the run-time count would make each token's LDS reads wait for the one before.
        float4 xa[NT][2];
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const float* xb = xr + t * xstride + 8 * b;
            xa[t][0] = *(const float4*) xb;
            xa[t][1] = *(const float4*) (xb + 4);
        }
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            float d = w[0] * xa[t][0].x;
            d = fmaf(w[1], xa[t][0].y, d);
            d = fmaf(w[2], xa[t][0].z, d);
            d = fmaf(w[3], xa[t][0].w, d);
            d = fmaf(w[4], xa[t][1].x, d);
            d = fmaf(w[5], xa[t][1].y, d);
            d = fmaf(w[6], xa[t][1].z, d);
            d = fmaf(w[7], xa[t][1].w, d);
            acc[t] = fmaf(d, e2, acc[t]);
        }
    }
}
// The column form of a P = 4 block against NT tokens' 12 staged values: every column's sum is converted and used as soon as it
// is formed (eleven sums and their float images held at once cost the persistent kernels their five waves a SIMD).
template <int NT>
__device__ __forceinline__ void cols_dot(uint32_t up, uint32_t g, uint32_t be, float e2, int b, const float* xr, int xstride, float (&acc)[NT]) {
    float4 xa[NT][3];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const float* xb = xr + t * xstride + 12 * b;
        xa[t][0] = *(const float4*) xb;
        xa[t][1] = *(const float4*) (xb + 4);
        xa[t][2] = *(const float4*) (xb + 8);
    }
    uint32_t G[6];
    col_bytes_p4(up, g, G);
    const uint32_t bo = be << 4;
    float d[NT];
    auto xv = [&](int t, int m) { const float4& q = xa[t][m >> 2]; return (m & 3) == 0 ? q.x : (m & 3) == 1 ? q.y : (m & 3) == 2 ? q.z : q.w; };
#pragma unroll
    for (int m = 0; m < 12; ++m) {
        const float z = (float) (m == 11 ? dot8ones(be) : dot8z(G[m >> 1], (m & 1) ? bo : be));
#pragma unroll
        for (int t = 0; t < NT; ++t) d[t] = m == 0 ? z * xv(t, 0) : fmaf(z, xv(t, m), d[t]);
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = fmaf(d[t], e2, acc[t]);
}
// The column form in two halves, for a caller that has a chunk's records before it has the activations: cols_pre forms the
// twelve exact column sums Z'(0..10), Q of every block (|Z'| <= 256: two to a register as int16), cols_post multiplies them with the
// staged values - the same converts, the same FMA chain in the same order as cols_dot, so the same bits.
__device__ __forceinline__ void cols_pre(const Chunk& ck, const uint32_t* tab, uint32_t (&zp)[8][6]) {
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const uint32_t ss = word_of(ck.sd, b >> 1), cc = word_of(ck.cw, b >> 1);
        const uint32_t g = stream_of(tab, (b & 1) ? ss >> 16 : ss & 0xFFFFu);
        const uint32_t up = (b & 1) ? ss : ss << 16;
        const uint32_t be = coef_bytes(cc, b & 1), bo = be << 4;
        uint32_t G[6];
        col_bytes_p4(up, g, G);
#pragma unroll
        for (int i = 0; i < 6; ++i) {
            const int z0 = dot8z(G[i], be), z1 = i == 5 ? dot8ones(be) : dot8z(G[i], bo);
            zp[b][i] = __builtin_amdgcn_perm((uint32_t) z1, (uint32_t) z0, 0x05040100u);   // { z0 as int16, z1 as int16 }
        }
        __builtin_amdgcn_sched_barrier(0);   // (a block at a time: 48 registers of results leave little room for eight blocks' temporaries)
    }
}
__device__ __forceinline__ void cols_post(const uint32_t (&zp)[8][6], uint32_t codes, int eb, const float* xr, float& acc) {
    const uint32_t ebase = (uint32_t) (eb + 127) << 23;
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const float* xb = xr + 12 * b;
        const float4 x0 = *(const float4*) xb, x1 = *(const float4*) (xb + 4), x2 = *(const float4*) (xb + 8);
        const float xs[12] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w, x2.x, x2.y, x2.z, x2.w};
        const float e2 = __uint_as_float((((codes >> (4 * b)) & 15u) << 23) + ebase);
        float d = 0.0f;
#pragma unroll
        for (int m = 0; m < 12; ++m) {
            const uint32_t p = zp[b][m >> 1];
            const float z = (m & 1) ? (float) ((int32_t) p >> 16) : (float) (int32_t) (int16_t) (p & 0xFFFFu);
            d = m == 0 ? z * xs[0] : fmaf(z, xs[m], d);
        }
        acc = fmaf(d, e2, acc);
    }
}
// PAIRED (P = 3 only): two blocks at a time in phase order (isum2_p3), as the GEMM's decoder waves decode: measured 1 % faster
// in the persistent MoE kernel (three waves a SIMD), 6 % slower in the stand-alone matvec, which keeps the compiler's own order.
template <int P, int NT, bool PAIRED = false, bool COLS = (P == 4)>
__device__ __forceinline__ void chunk_dot(const Chunk& ck, int eb, const uint32_t* tab, const float* xr, int xstride, int nt,
                                          float (&acc)[NT]) {
    (void) nt;
    static_assert(!PAIRED || P == 3 || COLS, "blocks in pairs: P = 3 only (the column form has one order)");
    if constexpr (COLS) {
        const uint32_t ebase = (uint32_t) (eb + 127) << 23;   // 2^eb as f32 bits: a block's scale is this plus its code in the exponent field
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const uint32_t ss = word_of(ck.sd, b >> 1), cc = word_of(ck.cw, b >> 1);
            const uint32_t g = stream_of(tab, (b & 1) ? ss >> 16 : ss & 0xFFFFu);
            const uint32_t up = (b & 1) ? ss : ss << 16;   // only the upper 16 bits are read
            const float e2 = __uint_as_float((((ck.codes >> (4 * b)) & 15u) << 23) + ebase);
            cols_dot<NT>(up, g, coef_bytes(cc, b & 1), e2, b, xr, xstride, acc);
        }
    } else if constexpr (PAIRED) {
#pragma unroll
        for (int b = 0; b < 8; b += 2) {   // blocks b and b + 1 share a word of seeds and a word of nibble words
            const uint32_t ss = word_of(ck.sd, b >> 1), cc = word_of(ck.cw, b >> 1);
            const uint32_t seed[2] = {ss & 0xFFFFu, ss >> 16}, word[2] = {cc & 0xFFFFu, cc >> 16};
            const uint32_t g[2] = {stream_of(tab, seed[0]), stream_of(tab, seed[1])}, up[2] = {ss << 16, ss};
            int is[2][8];
            const uint32_t q01[2] = {tab[512 + ((word[0] >> 4) & 0xFFu)], tab[512 + ((word[1] >> 4) & 0xFFu)]};
            const uint32_t q2[2] = {tab[512 + (word[0] >> 12)], tab[512 + (word[1] >> 12)]};
            isum2_p3(up, g, q01, q2, is);
            block_dot<P, NT>(is[0], pow2f(eb + (int) (word[0] & 15u)), b, xr, xstride, acc);
            block_dot<P, NT>(is[1], pow2f(eb + (int) (word[1] & 15u)), b + 1, xr, xstride, acc);
        }
    } else {
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const uint32_t ss = word_of(ck.sd, b >> 1), cc = word_of(ck.cw, b >> 1);
            const uint32_t seed16 = (b & 1) ? ss >> 16 : ss & 0xFFFFu, word16 = (b & 1) ? cc >> 16 : cc & 0xFFFFu;
            const uint32_t g = stream_of(tab, seed16);
            const uint32_t up = (b & 1) ? ss : ss << 16;   // only the upper 16 bits are read
            int is[8];
            if constexpr (P == 4) {   // the weights' form of a P = 4 block
                isum_p4(up, g, tab[512 + (word16 & 0xFFu)], tab[512 + (word16 >> 8)], is);
                block_dot<P, NT>(is, pow2f(eb + (int) ((ck.codes >> (4 * b)) & 15u)), b, xr, xstride, acc);
            } else {
                isum_p3(up, g, tab[512 + ((word16 >> 4) & 0xFFu)], tab[512 + (word16 >> 12)], is);
                block_dot<P, NT>(is, pow2f(eb + (int) (word16 & 15u)), b, xr, xstride, acc);
            }
        }
    }
}

// A P = 3 chunk's sum by 2^ls adjacent lanes (ls = 1 .. 3), lane s of the group taking blocks [s nb, (s + 1) nb), nb = 8 >> ls: each
// block's product with the activations as block_dot forms it, then block_dot's chain of multiply-adds over the blocks in block
// order, handed from lane to lane (lane s holds its final value after step s).  The group's last lane returns chunk_dot's bits.
__device__ __forceinline__ float chunk_dot_split(const Chunk& ck, int eb, const uint32_t* tab, const float* xr, int s, int ls) {
    const int nb = 8 >> ls, b0 = s * nb;
    float d[4] = {0.0f, 0.0f, 0.0f, 0.0f}, e2[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (i < nb) {
            const int b = b0 + i;
            const uint32_t ss = word_of(ck.sd, b >> 1), cc = word_of(ck.cw, b >> 1);
            const uint32_t seed16 = (b & 1) ? ss >> 16 : ss & 0xFFFFu, word16 = (b & 1) ? cc >> 16 : cc & 0xFFFFu;
            int is[8];
            isum_p3((b & 1) ? ss : ss << 16, stream_of(tab, seed16), tab[512 + ((word16 >> 4) & 0xFFu)], tab[512 + (word16 >> 12)], is);
            const float* xb = xr + 8 * b;
            float w[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) w[c] = (float) is[c];
            float dd = w[0] * xb[0];
#pragma unroll
            for (int c = 1; c < 8; ++c) dd = fmaf(w[c], xb[c], dd);
            d[i] = dd;
            e2[i] = pow2f(eb + (int) (word16 & 15u));
        }
    }
    float acc = 0.0f;
    for (int step = 0; step < (1 << ls); ++step) {
        // (the lane below, by a row shift of the wave's data path: the groups lie inside rows of 16 lanes)
        const float in = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, acc), 0x111, 0xF, 0xF, false));
        float v = s == 0 ? 0.0f : in;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (i < nb) v = fmaf(d[i], e2[i], v);
        acc = v;
    }
    return acc;
}

// The 8 weights of block j of row r as f32: seeds unscaled integers with *sc = 2^e R32; BF16 / Q8 as BF16 values; Q4 in
// MLX's matvec form s * q + b unrounded (reference engine/kernels_moe.cu:91-107, 171-189).
__device__ __forceinline__ void block_weights(int fmt, const WSlice& w, const uint32_t* tab, int r, int K, int j, float (&o)[8],
                                              float* sc) {
    const int nbk = K / 8;
    *sc = 1.0f;
    if (fmt == MF_SEED4P4 || fmt == MF_SEED4) {
        const size_t g = (size_t) r * nbk + j;
        const uint32_t seed = gp<uint16_t>(w.p[0])[g], word = gp<uint16_t>(w.p[1])[g];
        int is[8], code;
        if (fmt == MF_SEED4P4) {
            block_isum<4>(tab, seed, word, is);
            code = (gp<uint8_t>(w.p[3])[g >> 1] >> ((g & 1) * 4)) & 15;
        } else {
            block_isum<3>(tab, seed, word, is);
            code = (int) (word & 15u);
        }
#pragma unroll
        for (int c = 0; c < 8; ++c) o[c] = (float) is[c];
        *sc = pow2f(w.eb + code) * NSLM_R32;
    } else if (fmt == MF_BF16) {
        const NSLM_GLOBAL uint16_t* v = gp<uint16_t>(w.p[0]) + (size_t) r * K + (size_t) j * 8;
#pragma unroll
        for (int c = 0; c < 8; ++c) o[c] = bf(v[c]);
    } else {
        const size_t e0 = (size_t) r * K + (size_t) j * 8, gi = e0 >> group_shift(w);
        const float s = bf(gp<uint16_t>(w.p[1])[gi]), b = bf(gp<uint16_t>(w.p[2])[gi]);
        if (fmt == MF_Q8) {
            const NSLM_GLOBAL uint32_t* q = gp<uint32_t>(w.p[0]) + e0 / 4;
#pragma unroll
            for (int c = 0; c < 8; ++c) o[c] = bfr(s * (float) ((q[c >> 2] >> (8 * (c & 3))) & 255u) + b);
        } else {
            const uint32_t q = gp<uint32_t>(w.p[0])[e0 / 8];
#pragma unroll
            for (int c = 0; c < 8; ++c) o[c] = s * (float) ((q >> (4 * c)) & 15u) + b;
        }
    }
}


}   // namespace nslm
