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
// 16-byte unit in one instruction all the same - so there is one code path, no branch on the alignment and no join for the
// compiler to put a wait at.  `al` is kept in the signature for the callers and not used.
typedef uint32_t u32x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
typedef uint32_t u32_a1 __attribute__((aligned(1)));
template <int P>
__device__ __forceinline__ Chunk load_chunk(const WSlice& w, uint32_t unit, bool ok, bool al) {
    (void) al;
    Chunk c;
    c.sd = make_uint4(0, 0, 0, 0);
    c.cw = c.sd;
    c.codes = 0;
    if (!ok) return c;
    const u32x4_a2 s4 = *(const NSLM_GLOBAL u32x4_a2*) (gp<uint8_t>(w.p[0]) + (size_t) unit * 16);
    const u32x4_a2 c4 = *(const NSLM_GLOBAL u32x4_a2*) (gp<uint8_t>(w.p[1]) + (size_t) unit * 16);
    c.sd = make_uint4(s4.x, s4.y, s4.z, s4.w);
    c.cw = make_uint4(c4.x, c4.y, c4.z, c4.w);
    if (P == 4) c.codes = *(const NSLM_GLOBAL u32_a1*) (gp<uint8_t>(w.p[3]) + (size_t) unit * 4);
    return c;
}
__device__ __forceinline__ bool streams_aligned(int P, const WSlice& w) {
    return (((uintptr_t) w.p[0] | (uintptr_t) w.p[1]) & 15u) == 0 && (P != 4 || ((uintptr_t) w.p[3] & 3u) == 0);
}

__device__ __forceinline__ uint32_t word_of(const uint4& v, int i) { return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w; }

// One chunk (8 blocks) against NT tokens.  xr: this chunk's activations, token t at xr + t * xstride (registers when
// NT == 1, LDS otherwise).  acc[t] accumulates 2^(e+0) * sum_c isum_c x_c per block (R32 is applied to the row sum).
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
// PAIRED: two blocks at a time in phase order (isum2_*), as the GEMM's decoder waves decode: measured 1 % faster in the
// persistent MoE kernel (three waves a SIMD), 6 % slower in the stand-alone matvec, which keeps the compiler's own order.
template <int P, int NT, bool PAIRED = false>
__device__ __forceinline__ void chunk_dot(const Chunk& ck, int eb, const uint32_t* tab, const float* xr, int xstride, int nt,
                                          float (&acc)[NT]) {
    (void) nt;
    if constexpr (PAIRED) {
#pragma unroll
    for (int b = 0; b < 8; b += 2) {   // blocks b and b + 1 share a word of seeds and a word of coefficients
        const uint32_t ss = word_of(ck.sd, b >> 1), cc = word_of(ck.cw, b >> 1);
        const uint32_t seed[2] = {ss & 0xFFFFu, ss >> 16}, word[2] = {cc & 0xFFFFu, cc >> 16};
        const uint32_t g[2] = {stream_of(tab, seed[0]), stream_of(tab, seed[1])}, up[2] = {ss << 16, ss};
        int is[2][8], code[2];
        if (P == 4) {
            const uint32_t q01[2] = {tab[512 + (word[0] & 0xFFu)], tab[512 + (word[1] & 0xFFu)]};
            const uint32_t q23[2] = {tab[512 + (word[0] >> 8)], tab[512 + (word[1] >> 8)]};
            isum2_p4(up, g, q01, q23, is);
            code[0] = (int) ((ck.codes >> (4 * b)) & 15u);
            code[1] = (int) ((ck.codes >> (4 * b + 4)) & 15u);
        } else {
            const uint32_t q01[2] = {tab[512 + ((word[0] >> 4) & 0xFFu)], tab[512 + ((word[1] >> 4) & 0xFFu)]};
            const uint32_t q2[2] = {tab[512 + (word[0] >> 12)], tab[512 + (word[1] >> 12)]};
            isum2_p3(up, g, q01, q2, is);
            code[0] = (int) (word[0] & 15u);
            code[1] = (int) (word[1] & 15u);
        }
        block_dot<P, NT>(is[0], pow2f(eb + code[0]), b, xr, xstride, acc);
        block_dot<P, NT>(is[1], pow2f(eb + code[1]), b + 1, xr, xstride, acc);
    }
    } else {
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const uint32_t ss = word_of(ck.sd, b >> 1), cc = word_of(ck.cw, b >> 1);
        const uint32_t seed16 = (b & 1) ? ss >> 16 : ss & 0xFFFFu, word16 = (b & 1) ? cc >> 16 : cc & 0xFFFFu;
        const uint32_t g = stream_of(tab, seed16);
        const uint32_t up = (b & 1) ? ss : ss << 16;   // only the upper 16 bits are read
        int is[8];
        int code;
        if (P == 4) {
            isum_p4(up, g, tab[512 + (word16 & 0xFFu)], tab[512 + (word16 >> 8)], is);
            code = (int) ((ck.codes >> (4 * b)) & 15u);
        } else {
            isum_p3(up, g, tab[512 + ((word16 >> 4) & 0xFFu)], tab[512 + (word16 >> 12)], is);
            code = (int) (word16 & 15u);
        }
        block_dot<P, NT>(is, pow2f(eb + code), b, xr, xstride, acc);
    }
    }
}

#define XPAD 68   // LDS floats per 64-float chunk: 16-byte reads of 8 consecutive lanes land on 32 distinct banks

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
