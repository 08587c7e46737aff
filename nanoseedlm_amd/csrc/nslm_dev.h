// nslm_dev.h - device-side building blocks shared by the gfx950 kernels: BF16 rounding, the LFSR stream basis, and the
// exact integer decode of one 8-weight SeedLM block on 16-bit integer dot products.
//
// Arithmetic contract (reference: nslm/lfsr.h:4-10, nslm/search4.h:4-6): state_k of seed s is bits k..k+15 of the bit
// stream s | g(s) << 16, where g(s) is GF(2)-linear in s; weight c of a block is
//   isum_c = sum_p (state_(P*c+p+1) - 32768) * q_p   (exact, |isum| < 2^20),   w_c = (float) isum_c * fl(R32 * 2^e).
// Everything up to isum_c is done in integers here, so regenerated weights are bit-exact by construction.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels_hip.h"

namespace nslm {

// ---- global-memory pointers ---------------------------------------------------------------------------------------------
// Stream pointers arrive inside structs (WSlice), where the compiler cannot tell that they address global memory and would
// emit flat loads.  A flat load also counts against the LDS counter, so every LDS wait - and every barrier built on one -
// would wait for the HBM latency of loads issued steps ahead on purpose.  gp<T>(p) states the address space.
#define NSLM_GLOBAL __attribute__((address_space(1)))
template <typename T>
__device__ __forceinline__ const NSLM_GLOBAL T* gp(const void* p) { return (const NSLM_GLOBAL T*) p; }
// 16- and 8-byte global loads (uint4 / uint2 are class types and cannot be read through a qualified pointer directly)
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
template <typename P>
__device__ __forceinline__ uint4 ldg16(P p) {
    const u32x4 v = *(const NSLM_GLOBAL u32x4*) p;
    return make_uint4(v.x, v.y, v.z, v.w);
}
template <typename P>
__device__ __forceinline__ uint2 ldg8(P p) {
    const u32x2 v = *(const NSLM_GLOBAL u32x2*) p;
    return make_uint2(v.x, v.y);
}

// ---- BF16 (round to nearest even; reference engine/kernels_moe.cu:17-31) ---------------------------------------------
__device__ __forceinline__ float bfr(float x) {
    uint32_t u = __float_as_uint(x);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return __uint_as_float(u & 0xFFFF0000u);
}
__device__ __forceinline__ uint32_t tobf(float x) {
    uint32_t u = __float_as_uint(x);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return u >> 16;
}
__device__ __forceinline__ float bf(uint32_t h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ uint32_t pack_bf2(float a, float b) { return tobf(a) | (tobf(b) << 16); }
// nn.silu on a BF16 tensor: the sigmoid and the product are each rounded to BF16
__device__ __forceinline__ float silu_bf(float g) {
    const float s = bfr(1.0f / (1.0f + expf(-g)));
    return bfr(g * s);
}
// y = bf16(acc), or the residual form bf16(y + bf16(acc)); f32out keeps the unrounded sum (a switch of this backend)
__device__ __forceinline__ void store_y(float* yo, float s, int add, int f32out) {
    if (f32out) *yo = add ? *yo + s : s;
    else *yo = add ? bfr(*yo + bfr(s)) : bfr(s);
}

// ---- the stream basis -------------------------------------------------------------------------------------------------
// g(s) = the 32 stream bits that follow seed s: bit k = top bit of state k+1.  g is linear over GF(2), so
// g(s) = lo[s & 0xFF] ^ hi[s >> 8] with two 256-entry tables, built here at compile time from the LFSR definition
// (taps 0, 1, 3, 12; shift right; feedback into bit 15).  The P = 3 format reads the low 24 bits of the same table.
struct StreamBasis {
    uint32_t v[512];
};
constexpr uint32_t stream32_of(uint32_t s) {
    uint32_t g = 0;
    for (int k = 0; k < 32; ++k) {
        const uint32_t fb = (s ^ (s >> 1) ^ (s >> 3) ^ (s >> 12)) & 1u;
        s = (s >> 1) | (fb << 15);
        g |= (s >> 15) << k;
    }
    return g;
}
constexpr StreamBasis make_basis() {
    StreamBasis b{};
    for (uint32_t i = 0; i < 256; ++i) {
        b.v[i] = stream32_of(i);
        b.v[256 + i] = stream32_of(i << 8);
    }
    return b;
}
// Pairs of sign-extended int4 coefficients as packed int16: entry b = { sext4(b & 15), sext4(b >> 4) }.
struct CoefPairs {
    uint32_t v[256];
};
constexpr CoefPairs make_pairs() {
    CoefPairs t{};
    for (uint32_t b = 0; b < 256; ++b) {
        const int lo = (int) (b & 15u) - (int) ((b & 8u) << 1), hi = (int) (b >> 4) - (int) (((b >> 4) & 8u) << 1);
        t.v[b] = ((uint32_t) lo & 0xFFFFu) | ((uint32_t) hi << 16);
    }
    return t;
}
__device__ const StreamBasis kBasis = make_basis();
__device__ const CoefPairs kPairs = make_pairs();

// LDS copy of both tables: [0,512) stream basis, [512,768) coefficient pairs
#define NSLM_TAB_WORDS 768
__device__ __forceinline__ void load_tables(uint32_t* tab) {
    for (int i = threadIdx.x; i < 512; i += blockDim.x) tab[i] = kBasis.v[i];
    for (int i = threadIdx.x; i < 256; i += blockDim.x) tab[512 + i] = kPairs.v[i];
}
// The same for a workgroup of exactly NTHR threads (256, 512 or 1024), in two halves: a thread's loads are requested in
// tables_fetch() (put it beside the kernel's other first loads), and tables_store() writes them to LDS once they are needed -
// the loop above waits for every load in turn, one memory round trip each.
template <int NTHR>
struct TableWords {
    uint32_t w[(NSLM_TAB_WORDS + NTHR - 1) / NTHR];
};
template <int NTHR>
__device__ __forceinline__ TableWords<NTHR> tables_fetch() {
    TableWords<NTHR> t;
#pragma unroll
    for (int j = 0; j < (NSLM_TAB_WORDS + NTHR - 1) / NTHR; ++j) {
        const int i = min((int) threadIdx.x + NTHR * j, NSLM_TAB_WORDS - 1);   // clamped: the loads stay unconditional
        t.w[j] = i < 512 ? kBasis.v[i] : kPairs.v[i - 512];
    }
    return t;
}
template <int NTHR>
__device__ __forceinline__ void tables_store(uint32_t* tab, const TableWords<NTHR>& t) {
#pragma unroll
    for (int j = 0; j < (NSLM_TAB_WORDS + NTHR - 1) / NTHR; ++j) {
        const int i = (int) threadIdx.x + NTHR * j;
        if (i < NSLM_TAB_WORDS) tab[i] = t.w[j];
    }
}
// keeps the loads written above this line above it: left alone, the compiler moves a load down to its first use, and a load
// whose use sits in a conditional block becomes a load, a wait and a branch - one round trip per load instead of one for all
__device__ __forceinline__ void loads_issued() { asm volatile("" ::: "memory"); }
__device__ __forceinline__ uint32_t stream_of(const uint32_t* tab, uint32_t seed16) {
    return tab[seed16 & 0xFFu] ^ tab[256 + (seed16 >> 8)];
}

// ---- exact block decode -----------------------------------------------------------------------------------------------
// Written as the three-source encoding: left to itself the compiler prefers the accumulating two-source form, whose
// destination is tied to the addend, and pays a register move whenever the addend has another use or a different home.
__device__ __forceinline__ int dot2(uint32_t a, uint32_t b, int c) {
    int d;
    asm("v_dot2_i32_i16 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}
// the same with a zero addend: the three-source encoding takes the constant inline, where the accumulating two-source
// form the compiler picks for dot2(a, b, 0) would first spend a move on zeroing its destination
__device__ __forceinline__ int dot2z(uint32_t a, uint32_t b) {
    int d;
    asm("v_dot2_i32_i16 %0, %1, %2, 0" : "=v"(d) : "v"(a), "v"(b));
    return d;
}
// { word X's half hx, word Y's half hy } as one packed pair
__device__ __forceinline__ uint32_t halves(uint32_t X, int hx, uint32_t Y, int hy) {
    const uint32_t sel = (uint32_t) (2 * hx) | ((uint32_t) (2 * hx + 1) << 8) | ((uint32_t) (4 + 2 * hy) << 16) |
                         ((uint32_t) (5 + 2 * hy) << 24);
    return __builtin_amdgcn_perm(Y, X, sel);
}

// The 16 windows of a block's stream.  `up` is any word whose upper 16 bits are the seed, g the 32 bits that follow.
// A[k], k = 1..16: low half = state_k - 32768, high half = state_(k+16) - 32768 as int16 (state ^ 0x8000).
__device__ __forceinline__ void windows(uint32_t up, uint32_t g, uint32_t (&A)[17]) {
#pragma unroll
    for (int k = 1; k <= 15; ++k) A[k] = __builtin_amdgcn_alignbit(g, up, 16 + k) ^ 0x80008000u;
    A[16] = g ^ 0x80008000u;
}

// P = 4: weight c reads states 4c+1..4c+4; q01 = {q0,q1}, q23 = {q2,q3} as packed int16 (reference nslm/lib_search4.c:22-31)
__device__ __forceinline__ void isum_p4(uint32_t up, uint32_t g, uint32_t q01, uint32_t q23, int (&is)[8]) {
    uint32_t A[17];
    windows(up, g, A);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int k = 4 * c + 1;
        is[c] = dot2(halves(A[k], 0, A[k + 1], 0), q01, dot2z(halves(A[k + 2], 0, A[k + 3], 0), q23));
        is[c + 4] = dot2(halves(A[k], 1, A[k + 1], 1), q01, dot2z(halves(A[k + 2], 1, A[k + 3], 1), q23));
    }
}
// P = 3: weight c reads states 3c+1..3c+3; q01 = {q0,q1}, q2 = {q2,0} (reference nslm/lfsr.h:116-128)
__device__ __forceinline__ void isum_p3(uint32_t up, uint32_t g, uint32_t q01, uint32_t q2, int (&is)[8]) {
    uint32_t A[17];
    windows(up, g, A);
    const uint32_t q2hi = q2 << 16;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int k0 = 3 * c + 1, k1 = k0 + 1, k2 = k0 + 2;   // state k lives in A[k] low (k <= 16) or A[k-16] high
        const uint32_t pr = halves(A[k0 <= 16 ? k0 : k0 - 16], k0 > 16, A[k1 <= 16 ? k1 : k1 - 16], k1 > 16);
        const int third = k2 <= 16 ? dot2z(A[k2], q2) : dot2z(A[k2 - 16], q2hi);
        is[c] = dot2(pr, q01, third);
    }
}

// ---- P = 4 by nibble columns (the matvec's form) -----------------------------------------------------------------------------
// What a VALU instruction costs on this target was measured (issue slots of a SIMD with two or more waves resident): and / or /
// xor / shift right / add / mov / f32 mul, fma / int -> f32 convert ~2.5 cycles; everything with three sources or sub-word
// operands - v_alignbit, v_perm, v_bfe, shift left, the v_dot*, v_mad_* - ~4.3.  The exact decode above spends 47 of the
// expensive ones a block (15 windows, 16 pairings, 16 dot2).  A matvec does not need the eight sums themselves, only
// sum_c x_c isum_c, and that can be regrouped so that eleven v_dot8_i32_i4 do the 32 multiply-adds:
//   state_(4c+1+p) = sum_n 16^n N_p(c + n),  N_p(m) = the nibble at bits [4m+1+p, 4m+5+p) of the 48-bit stream S (m = 0..10);
//   sum_c x_c isum_c = sum_m Z(m) X(m) - 32768 Q SX,   Z(m) = sum_p q_p N_p(m),  X(m) = sum_n 16^n x_(m-n),  Q = sum_p q_p,  SX = sum_c x_c;
//   with signed nibbles N' = N - 8 (one xor):  = sum_m Z'(m) X(m) + Q CX,  Z'(m) = sum_p q_p N'_p(m),  CX = (8 * 4369 - 32768) SX = 2184 SX.
// N_p(m) is nibble m of V_p = S >> (1 + p), so byte j of V_0..V_3, gathered into one register (a 4 x 6 byte transpose: 12 v_perm),
// holds the columns m = 2j and 2j + 1, and v_dot8_i32_i4 against the coefficient nibbles spread to the even (odd) nibble
// positions gives Z'(2j) (Z'(2j + 1)).  Z' and Q are exact small integers; X and CX depend on the activations only and are
// formed once per activation row (xform_block in nslm_mv_dev.h).  The weights are never materialised: kernels that need
// them (the GEMM's decoder, kc_slice_deq) keep the exact sums above.
__device__ __forceinline__ int dot8z(uint32_t a, uint32_t b) {
    int d;
    asm("v_dot8_i32_i4 %0, %1, %2, 0" : "=v"(d) : "v"(a), "v"(b));
    return d;
}
// the coefficient nibbles q0..q3 of block `odd` (0 / 1) of a packed pair of coefficient words, one to a byte: the even-column operand
__device__ __forceinline__ uint32_t coef_bytes(uint32_t cc, int odd) {
    const uint32_t t = cc & 0x0F0F0F0Fu, u = (cc >> 4) & 0x0F0F0F0Fu;   // (q0, q2 | q0', q2'), (q1, q3 | q1', q3')
    return __builtin_amdgcn_perm(u, t, odd ? 0x07030602u : 0x05010400u);
}
// the sum of the four coefficients of a coefficient operand (even-column form): a dot product with ones, the constant from a scalar register
__device__ __forceinline__ int dot8ones(uint32_t a) {
    int d;
    asm("v_dot8_i32_i4 %0, %1, %2, 0" : "=v"(d) : "v"(a), "s"(0x01010101u));
    return d;
}
// up: any word whose upper 16 bits are the seed, g: stream bits 16..47.  G[j] = byte j of V_0..V_3 with the nibbles made signed:
// columns 2j (low nibbles) and 2j + 1 (high nibbles).  V_p's bytes 0..3 are one funnel shift of (g : up) by 17 + p, its bytes
// 4 and 5 one shift of g - no word of the stream's low 32 bits is formed first.
__device__ __forceinline__ void col_bytes_p4(uint32_t up, uint32_t g, uint32_t (&G)[6]) {
    uint32_t vl[4], vh[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        vl[p] = __builtin_amdgcn_alignbit(g, up, 17 + p);
        vh[p] = g >> (17 + p);
    }
    const uint32_t a01 = __builtin_amdgcn_perm(vl[1], vl[0], 0x05010400u), b01 = __builtin_amdgcn_perm(vl[1], vl[0], 0x07030602u);
    const uint32_t a23 = __builtin_amdgcn_perm(vl[3], vl[2], 0x05010400u), b23 = __builtin_amdgcn_perm(vl[3], vl[2], 0x07030602u);
    const uint32_t h01 = __builtin_amdgcn_perm(vh[1], vh[0], 0x05010400u), h23 = __builtin_amdgcn_perm(vh[3], vh[2], 0x05010400u);
    G[0] = __builtin_amdgcn_perm(a23, a01, 0x05040100u) ^ 0x88888888u;
    G[1] = __builtin_amdgcn_perm(a23, a01, 0x07060302u) ^ 0x88888888u;
    G[2] = __builtin_amdgcn_perm(b23, b01, 0x05040100u) ^ 0x88888888u;
    G[3] = __builtin_amdgcn_perm(b23, b01, 0x07060302u) ^ 0x88888888u;
    G[4] = __builtin_amdgcn_perm(h23, h01, 0x05040100u) ^ 0x88888888u;
    G[5] = __builtin_amdgcn_perm(h23, h01, 0x07060302u) ^ 0x88888888u;
}

// Two blocks at once, written in phases (all windows, then all sign flips, all pairings, all products) with the
// scheduler held to that order: a VALU result is not available to the next instruction slots, and a wave that has a SIMD's
// vector issue to itself (the GEMM's decoder waves) loses those slots unless dependent instructions sit far apart.  In
// phase order every operand is at least a dozen instructions old.
__device__ __forceinline__ void isum2_p4(const uint32_t (&up)[2], const uint32_t (&g)[2], const uint32_t (&q01)[2],
                                         const uint32_t (&q23)[2], int (&is)[2][8]) {
    uint32_t A[2][17], lo[2][8], hi[2][8];
#pragma unroll
    for (int k = 1; k <= 15; ++k)
#pragma unroll
        for (int h = 0; h < 2; ++h) A[h][k] = __builtin_amdgcn_alignbit(g[h], up[h], 16 + k);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int k = 1; k <= 16; ++k)
#pragma unroll
        for (int h = 0; h < 2; ++h) A[h][k] = (k < 16 ? A[h][k] : g[h]) ^ 0x80008000u;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 8; ++j)   // pair j = states 2j+1, 2j+2 (low halves) and 2j+17, 2j+18 (high halves)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            lo[h][j] = halves(A[h][2 * j + 1], 0, A[h][2 * j + 2], 0);
            hi[h][j] = halves(A[h][2 * j + 1], 1, A[h][2 * j + 2], 1);
        }
    __builtin_amdgcn_sched_barrier(0);
    int t[2][8];
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            t[h][c] = dot2z(lo[h][2 * c + 1], q23[h]);
            t[h][c + 4] = dot2z(hi[h][2 * c + 1], q23[h]);
        }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            is[h][c] = dot2(lo[h][2 * c], q01[h], t[h][c]);
            is[h][c + 4] = dot2(hi[h][2 * c], q01[h], t[h][c + 4]);
        }
    __builtin_amdgcn_sched_barrier(0);
}
__device__ __forceinline__ void isum2_p3(const uint32_t (&up)[2], const uint32_t (&g)[2], const uint32_t (&q01)[2],
                                         const uint32_t (&q2)[2], int (&is)[2][8]) {
    uint32_t A[2][17], pr[2][8];
#pragma unroll
    for (int k = 1; k <= 15; ++k)
#pragma unroll
        for (int h = 0; h < 2; ++h) A[h][k] = __builtin_amdgcn_alignbit(g[h], up[h], 16 + k);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int k = 1; k <= 16; ++k)
#pragma unroll
        for (int h = 0; h < 2; ++h) A[h][k] = (k < 16 ? A[h][k] : g[h]) ^ 0x80008000u;
    __builtin_amdgcn_sched_barrier(0);
    int t[2][8];
#pragma unroll
    for (int c = 0; c < 8; ++c)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k0 = 3 * c + 1, k1 = k0 + 1, k2 = k0 + 2;   // state k lives in A[k] low (k <= 16) or A[k-16] high
            pr[h][c] = halves(A[h][k0 <= 16 ? k0 : k0 - 16], k0 > 16, A[h][k1 <= 16 ? k1 : k1 - 16], k1 > 16);
            t[h][c] = k2 <= 16 ? dot2z(A[h][k2], q2[h]) : dot2z(A[h][k2 - 16], q2[h] << 16);
        }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int c = 0; c < 8; ++c)
#pragma unroll
        for (int h = 0; h < 2; ++h) is[h][c] = dot2(pr[h][c], q01[h], t[h][c]);
    __builtin_amdgcn_sched_barrier(0);
}

// One block of either seed format from its raw fields.  seed16 / word16: the 16-bit seed and coefficient (P = 4) or
// nibble (P = 3) word, zero-extended.  Returns the integer sums and the block's exponent e = eb + code.
template <int P>
__device__ __forceinline__ void block_isum(const uint32_t* tab, uint32_t seed16, uint32_t word16, int (&is)[8]) {
    const uint32_t g = stream_of(tab, seed16), up = seed16 << 16;
    if (P == 4) isum_p4(up, g, tab[512 + (word16 & 0xFFu)], tab[512 + (word16 >> 8)], is);
    else isum_p3(up, g, tab[512 + ((word16 >> 4) & 0xFFu)], tab[512 + (word16 >> 12)], is);
}
// 2^e as f32 bits; e in the normal range
__device__ __forceinline__ float pow2f(int e) { return __uint_as_float((uint32_t) (e + 127) << 23); }
#define NSLM_R32 (1.0f / 32767.0f)

__device__ __forceinline__ int group_shift(const WSlice& w) { return w.gs ? w.gs : 6; }

// process-wide switches and launch-error bookkeeping (defined in nslm_mv.hip)
int host_store_f32();
void host_note_launch();
void host_note_unsupported();   // a launcher refused its arguments: kc_last_error() reports an invalid value

// the sum of v over the workgroup's 256 threads, the same value in every thread (every thread must call)
__device__ __forceinline__ float wg_sum(float v, float* red) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    __syncthreads();   // red may still be read from a previous call
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}
// rsqrt(mean(x^2) + eps) of a row of g <= 256 NSLM_NORM_NR values, bit for bit as the RMSNorm kernel forms it (thread tid
// sums k = tid, tid + 256, .. in order, then the workgroup tree), so a consumer that normalises its own input,
// xn_k = x_k * r * (1 + w_k), computes what the separate kernel would have stored.  256 threads, every thread calls.
#define NSLM_NORM_NR 16
__device__ __forceinline__ float row_rnorm(const float* xi, int g, float eps, float* red) {
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < NSLM_NORM_NR; ++j) {
        const int k = (int) threadIdx.x + j * 256;
        const float xv = xi[min(k, g - 1)];   // unconditional (a conditional load waits for the loads before it)
        const float v = k < g ? xv : 0.0f;
        ss = fmaf(v, v, ss);
    }
    return rsqrtf(wg_sum(ss, red) / (float) g + eps);
}

}   // namespace nslm
