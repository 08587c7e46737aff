// nslm_mla.hip - decode attention over a latent KV cache (absorbed MLA) and what feeds it: per-head maps, RoPE with the
// cache write, the FP8 (E4M3 codes, one E8M0 scale per 32 values) cache codec, split-key latent attention and its reduce.
// Replaces the reference's k_heads_mv, k_mla_rope, k_mla_attn / k_mla_reduce, k_kv_f32 and the FP8 half of kvq_put /
// kvq_get8 (engine/kernels_moe.cu:955-1118,1147-1176,1177-1208,1217-1323; the codec's definition is nslm/kvq.h:19-80)
// behind the same launchers.  BF16 and FP8 caches; the FP4 cache format is not built.
//
// Per cached position the kernel reads r + rope values once for ALL heads of a workgroup (multi-query over the shared
// latent): 660 bytes at r = 512, rope 128, FP8 - so the attention of a 4096-token context moves 2.7 MB per row, and what
// it costs is the 2 x (r + rope) multiply-adds per (key, head).  Latent 512 + RoPE 64 runs them on the matrix cores
// (k_mla_attn_mfma: exact BF16 products, f32 sums, P as BF16 hi + lo, which holds the reference tests' bound of one BF16
// ulp + 2e-6 of a double-precision softmax); other shapes stay in f32 on the vector ALUs (k_mla_attn_any).
#include "nslm_mv_dev.h"

using namespace nslm;

namespace {

// ---- the FP8 codec (nslm/kvq.h) ----------------------------------------------------------------------------------------
__device__ __forceinline__ float e4m3_dec(uint32_t c) {
    const int e = (int) ((c >> 3) & 15u), m = (int) (c & 7u);
    const float v = e ? ldexpf(1.0f + (float) m / 8.0f, e - 7) : ldexpf((float) m, -9);
    return (c & 0x80u) ? -v : v;
}
// a >= 0: the E4M3 code of a, rounded to nearest even, saturated at 448
__device__ __forceinline__ uint32_t e4m3_enc_abs(float a) {
    if (!(a < 448.0f)) return 0x7Eu;
    if (a < 0.015625f) return (uint32_t) rintf(a * 512.0f);   // subnormals (8: the smallest normal)
    int e;
    const float f = frexpf(a, &e);   // a = 2f 2^(e - 1), 2f in [1, 2)
    int E = e - 1, m = (int) rintf((2.0f * f - 1.0f) * 8.0f);
    if (m == 8) { ++E; m = 0; }
    const int c = ((E + 7) << 3) | m;
    return (uint32_t) (c > 0x7E ? 0x7E : c);
}
// the E8M0 scale byte of a block with max |x| = amax
__device__ __forceinline__ uint32_t fp8_scale(float amax) {
    if (!(amax > 0.0f)) return 127u;
    int k;
    (void) frexpf(amax, &k);   // amax in [2^(k-1), 2^k); 448 2^(k-9) = 0.875 2^k
    int e = amax <= ldexpf(448.0f, k - 9) ? k - 9 : k - 8;
    e = e < -126 ? -126 : e > 127 ? 127 : e;
    return (uint32_t) (e + 127);
}
// one cached value as the f32 of its BF16 bits (a code times its scale is exact; truncation as the reference packs it)
__device__ __forceinline__ float fp8_value(uint32_t code, uint32_t sc) {
    return __uint_as_float(__float_as_uint(e4m3_dec(code) * ldexpf(1.0f, (int) sc - 127)) & 0xFFFF0000u);
}
// Store value v at dim d of FP8 row `row` (n values) when `store`: the 32 dims of a block are 32 consecutive lanes, which
// share the block's max |v|.  Every lane of the wave calls it.
__device__ __forceinline__ void fp8_put(bool store, float v, uint8_t* C, uint8_t* S, size_t row, int n, int d) {
    float a = fabsf(v);
    for (int o = 1; o < 32; o <<= 1) a = fmaxf(a, __shfl_xor(a, o));
    const uint32_t sc = fp8_scale(a);
    const uint32_t c = e4m3_enc_abs(ldexpf(fabsf(v), 127 - (int) sc));
    if (!store) return;
    C[row * (size_t) n + d] = (uint8_t) (c && v < 0.0f ? c | 0x80u : c);
    if (d % 32 == 0) S[row * (size_t) (n / 32) + d / 32] = (uint8_t) sc;
}

__device__ __forceinline__ KvSeg kv_seg(const KvView& kv, int pos, int* row) {
    if (pos < kv.nv) { *row = pos; return kv.a; }
    *row = pos - kv.nv;
    return kv.b;
}
// dims d .. d + 7 of a cache row (the RoPE key or the latent, n values a row) as f32
__device__ __forceinline__ void cache_get8(int fmt, const void* codes, const void* scales, size_t row, int n, int d, float (&o)[8]) {
    if (fmt == KV_BF16) {
        const uint4 q = ldg16(gp<uint16_t>(codes) + row * (size_t) n + d);
        const uint32_t u[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) { o[2 * i] = __uint_as_float(u[i] << 16); o[2 * i + 1] = __uint_as_float(u[i] & 0xFFFF0000u); }
    } else {
        const uint2 q = ldg8(gp<uint8_t>(codes) + row * (size_t) n + d);
        const uint32_t sc = gp<uint8_t>(scales)[row * (size_t) (n / 32) + d / 32];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[i] = fp8_value((q.x >> (8 * i)) & 255u, sc);
            o[4 + i] = fp8_value((q.y >> (8 * i)) & 255u, sc);
        }
    }
}

// softplus(x, beta = ln 2) in f32, then BF16 (engine/kernels_moe.cu:215-218)
__device__ __forceinline__ float softplus_gate(float g) {
    const float gx = g * 0.69314718055994531f;
    return bfr((fmaxf(gx, 0.0f) + logf(1.0f + expf(-fabsf(gx)))) / 0.69314718055994531f);
}

// ---- per-head maps: y[t][h][o] = bf16(W_h[o] . x[t * xs + h * hs ..]), optionally times bf16(softplus_ln2(g)) ----------
// LPR lanes per output row (a power of two, the row's blocks rounded up), 64 / LPR rows a wave; the lane's blocks and the
// FMA chain per block are k_mv_any's.  Seed maps take head h's exponent bias from W.p[2][h].
__global__ void __launch_bounds__(256) k_heads_mv(HmvArgs a, int fmt, WSlice W, const float* x, const float* g, float* y, int lpr) {
    __shared__ uint32_t tab[NSLM_TAB_WORDS];
    if (fmt == MF_SEED4P4 || fmt == MF_SEED4) {
        load_tables(tab);
        __syncthreads();
    }
    const int tid = threadIdx.x, rpw = 64 / lpr, sub = (tid & 63) / lpr, ln = tid & (lpr - 1);
    const int o = ((int) blockIdx.x * 4 + (tid >> 6)) * rpw + sub, h = (int) blockIdx.y, t = (int) blockIdx.z;
    const bool live = o < a.O;
    const float* xv = x + (size_t) t * a.xs + (size_t) h * a.hs;
    WSlice ws = W;
    if (fmt == MF_SEED4P4) ws.eb = gp<int32_t>(W.p[2])[h];
    float acc = 0.0f;
    if (live)
        for (int j = ln; j < a.I / 8; j += lpr) {
            float w[8], sc;
            block_weights(fmt, ws, tab, h * a.O + o, a.I, j, w, &sc);
            const float* xb = xv + (size_t) j * 8;
            float d = w[0] * xb[0];
#pragma unroll
            for (int c = 1; c < 8; ++c) d = fmaf(w[c], xb[c], d);
            acc = fmaf(d, sc, acc);
        }
    for (int s = lpr >> 1; s > 0; s >>= 1) acc += __shfl_xor(acc, s);
    if (live && ln == 0) {
        const size_t yi = ((size_t) t * a.H + h) * a.O + o;
        float v = bfr(acc);
        if (a.gate) v = bfr(v * softplus_gate(g[yi]));
        y[yi] = v;
    }
}

// ---- RoPE of the query RoPE parts (in place) and of the RoPE key into the cache; the latent into the cache -------------
// The work of a row is cut into jobs of one wave each: job 0 rotates the RoPE key and writes it, job 1 + j writes latent
// dims [64 j, 64 j + 64).  An FP8 block is 32 consecutive values, so it always sits in 32 consecutive lanes of one job and
// its maximum is five shuffles.  (The reference gives thread i latent dim i and, at once, rotation pair i % half of head
// i / half, engine/kernels_moe.cu:1177-1208; here the query heads are a loop of their own over a table of the row's
// sines and cosines, computed once instead of once per head.)
__device__ __forceinline__ void rotate(float x0, float x1, float cs, float sn, float* y0, float* y1) {
    *y0 = __fsub_rn(__fmul_rn(x0, cs), __fmul_rn(x1, sn));   // spelled out: the same bits wherever it is inlined
    *y1 = __fadd_rn(__fmul_rn(x1, cs), __fmul_rn(x0, sn));
}
__device__ __forceinline__ void cache_job(int job, const MlaArgs& a, int rope, const float* kr, const float* c, const KvView& kv, const RowInfo* ri,
                                          const float* inv, int t) {
    const int lane = threadIdx.x & 63, pos = ri[t].pos, half = rope / 2;
    int row;
    const KvSeg sg = kv_seg(kv, ri[t].kv0 + pos, &row);
    if (job == 0) {   // the key: lane p < half holds the pair (p, p + half)
        const bool on = lane < half;
        float y0 = 0.0f, y1 = 0.0f;
        if (on) {
            float sn, cs;
            sincosf((float) pos * inv[lane], &sn, &cs);
            rotate(kr[(size_t) t * rope + lane], kr[(size_t) t * rope + lane + half], cs, sn, &y0, &y1);
        }
        if (kv.fmt == KV_BF16) {
            if (on) {
                uint16_t* kc = (uint16_t*) sg.k + (size_t) row * rope;
                kc[lane] = (uint16_t) tobf(y0);
                kc[lane + half] = (uint16_t) tobf(y1);
            }
        } else {   // every lane runs the shuffles
            fp8_put(on, bfr(y0), (uint8_t*) sg.k, (uint8_t*) sg.ks, (size_t) row, rope, on ? lane : 0);
            fp8_put(on, bfr(y1), (uint8_t*) sg.k, (uint8_t*) sg.ks, (size_t) row, rope, on ? lane + half : 0);
        }
        return;
    }
    const int i = (job - 1) * 64 + lane;
    const bool on = i < a.r;
    const float v = on ? c[(size_t) t * a.r + i] : 0.0f;
    if (kv.fmt == KV_BF16) {
        if (on) ((uint16_t*) sg.v)[(size_t) row * a.r + i] = (uint16_t) tobf(v);
    } else {
        fp8_put(on, bfr(v), (uint8_t*) sg.v, (uint8_t*) sg.vs, (size_t) row, a.r, on ? i : 0);
    }
}
// one workgroup a row: the cache jobs dealt to the four waves, then every query head's pairs
__global__ void __launch_bounds__(256) k_mla_rope(MlaArgs a, int rope, float* qr, const float* kr, const float* c, KvView kv,
                                                  const RowInfo* ri, const float* inv) {
    __shared__ float cs_s[ATT_HD / 2], sn_s[ATT_HD / 2];
    const int t = (int) blockIdx.x, tid = threadIdx.x, half = rope / 2;
    if (tid < half) sincosf((float) ri[t].pos * inv[tid], &sn_s[tid], &cs_s[tid]);
    for (int job = tid >> 6; job < 1 + (a.r + 63) / 64; job += 4) cache_job(job, a, rope, kr, c, kv, ri, inv, t);
    __syncthreads();
    for (int i = tid; i < a.n_head * half; i += 256) {
        const int h = i / half, p = i - h * half;
        float* qh = qr + ((size_t) t * a.n_head + h) * rope;
        float y0, y1;
        rotate(qh[p], qh[p + half], cs_s[p], sn_s[p], &y0, &y1);
        qh[p] = bfr(y0);
        qh[p + half] = bfr(y1);
    }
}

// ---- the two maps of the query, its RoPE, and the cache write as ONE launch -----------------------------------------------
// Grid (1 + r / 64, n_head + 1, rows).  Head h < n_head: block 0 computes the `rope` rows of the RoPE mix
// (k_heads_mv's arithmetic), rotates them (k_mla_rope's) and stores them; block b > 0 computes latent-query rows
// [64 (b - 1), 64 b).  "Head" n_head: the blocks' waves take the cache jobs (the rotated key, the latent).
// The same bits as kc_heads_mv x 2 + kc_mla_rope.
__global__ void __launch_bounds__(256) k_qmaps_rope(MlaArgs a, int rope, HmvArgs hq, HmvArgs hl, int fmt, WSlice Wq, WSlice Wl, const float* q,
                                                   float* qr, float* ql, const float* kr, const float* c, KvView kv, const RowInfo* ri,
                                                   const float* inv, int lpr) {
    __shared__ uint32_t tab[NSLM_TAB_WORDS];
    __shared__ float qs[ATT_HD];
    const int tid = threadIdx.x, h = (int) blockIdx.y, t = (int) blockIdx.z, b = (int) blockIdx.x;
    if (h == a.n_head) {   // uniform over the block: cache jobs 4 b .. 4 b + 3
        const int job = b * 4 + (tid >> 6);
        if (job < 1 + (a.r + 63) / 64) cache_job(job, a, rope, kr, c, kv, ri, inv, t);
        return;
    }
    if (fmt == MF_SEED4P4 || fmt == MF_SEED4) {
        load_tables(tab);
        __syncthreads();
    }
    const bool mix = b == 0;
    const HmvArgs& hm = mix ? hq : hl;
    const int O = hm.O, o0 = mix ? 0 : 64 * (b - 1), o1 = mix ? O : min(o0 + 64, O);
    const int rpw = 64 / lpr, sub = (tid & 63) / lpr, ln = tid & (lpr - 1);
    const float* xv = q + (size_t) t * hm.xs + (size_t) h * hm.hs;
    WSlice ws = mix ? Wq : Wl;
    if (fmt == MF_SEED4P4) ws.eb = gp<int32_t>(ws.p[2])[h];
    for (int ob = o0; ob < o1; ob += 4 * rpw) {
        const int o = ob + (tid >> 6) * rpw + sub;
        const bool live = o < o1;
        float acc = 0.0f;
        if (live)
            for (int j = ln; j < hm.I / 8; j += lpr) {
                float w[8], sc;
                block_weights(fmt, ws, tab, h * O + o, hm.I, j, w, &sc);
                const float* xb = xv + (size_t) j * 8;
                float d = w[0] * xb[0];
#pragma unroll
                for (int cc = 1; cc < 8; ++cc) d = fmaf(w[cc], xb[cc], d);
                acc = fmaf(d, sc, acc);
            }
        for (int sft = lpr >> 1; sft > 0; sft >>= 1) acc += __shfl_xor(acc, sft);
        if (live && ln == 0) {
            if (mix) qs[o] = bfr(acc);
            else ql[((size_t) t * hl.H + h) * O + o] = bfr(acc);
        }
    }
    if (!mix) return;
    __syncthreads();
    const int half = rope / 2;
    if (tid < half) {
        float sn, cs;
        sincosf((float) ri[t].pos * inv[tid], &sn, &cs);
        float y0, y1;
        rotate(qs[tid], qs[tid + half], cs, sn, &y0, &y1);
        float* qh = qr + ((size_t) t * a.n_head + h) * rope;
        qh[tid] = bfr(y0);
        qh[tid + half] = bfr(y1);
    }
}

// ---- latent attention, any shape (f32 on the vector ALUs) ---------------------------------------------------------------------
// Workgroup (split, group of GA_HW heads, row), one query head a wave.  A tile of GA_KT keys (latent, then RoPE key) is decoded
// to f32 in LDS once for the workgroup's heads.
//   scores   lane (key u = lane / 4, quarter q = lane % 4) forms the part of s_u = q . k_u that falls into its quarter of the
//            r + rope dims - sequential reads of the key's LDS row and of the wave's staged query - and two quad shuffles add
//            the quarters: GA_KT scores a wave are ready at once (no wave-wide reduction per key);
//   softmax  the tile's maximum and its sum of exp over the 16 quads: four shuffles each, once a tile;
//   P c      lane l owns latent dims l, l + 64, ...; exp(s_u - m) reaches it as the broadcast of lane 4 u.
// n_splits > 1: partials [row][head][split] = (m, l, acc[r]) for the reduce; n_splits == 1: olat[row][head] = bf16(acc / l).
#define GA_KT 16
#define GA_HW 4
#define MLA_MAXL 16    // latent dims a lane (r <= 1024)
#define MLA_SPLITS_SHORT 32
__device__ __forceinline__ int mla_row_splits(const MlaArgs& a, int pos) {
    (void) pos;
    return a.pad[2] > 0 && a.n_splits > MLA_SPLITS_SHORT ? MLA_SPLITS_SHORT : a.n_splits;
}
// the keys [p0, p1) of split `split` of a row at position pos: the row's own 0..pos in equal runs, as few as `chunk` keys a run allow
__device__ __forceinline__ void split_range(const MlaArgs& a, int pos, int split, int* p0, int* p1) {
    const int ns = mla_row_splits(a, pos), want = (pos + a.chunk) / a.chunk, used = ns < want ? ns : want, run = (pos + used) / used;
    *p0 = split * run;
    *p1 = split < used ? min(pos + 1, *p0 + run) : *p0;
}
__global__ void __launch_bounds__(64 * GA_HW) k_mla_attn_any(MlaArgs a, int rope, const float* ql, const float* qr, KvView kv, const RowInfo* ri,
                                                            float* out) {
    extern __shared__ __attribute__((aligned(16))) float sm[];   // [GA_KT keys][ld] then [GA_HW queries][ld]
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, u = lane >> 2, qt = lane & 3;
    const int split = (int) blockIdx.x, t = (int) blockIdx.z, r = a.r, kw = r + rope, ld = kw + 4, nl = (r + 63) / 64;
    const int h = (int) blockIdx.y * GA_HW + wv;
    const bool live = h < a.n_head;
    float* keys = sm;
    float* qs = sm + GA_KT * ld + wv * ld;
    for (int i = lane; i < kw; i += 64) {   // the wave's query, scaled (its own rows of LDS: no barrier needed before the wave reads them)
        const int hh = live ? h : 0;
        qs[i] = a.scale * (i < r ? ql[((size_t) t * a.n_head + hh) * r + i] : qr[((size_t) t * a.n_head + hh) * rope + (i - r)]);
    }
    int p0, p1;
    split_range(a, ri[t].pos, split, &p0, &p1);
    const int q0 = qt * (kw / 4), q1 = q0 + kw / 4;   // kw % 8 == 0: whole pairs
    float acc[MLA_MAXL];
#pragma unroll
    for (int j = 0; j < MLA_MAXL; ++j) acc[j] = 0.0f;
    float m = -INFINITY, l = 0.0f;
    for (int p = p0; p < p1; p += GA_KT) {
        const int nk = min(GA_KT, p1 - p);
        __syncthreads();
        for (int e = tid; e < nk * (kw / 8); e += 64 * GA_HW) {   // 8 dims a thread (r and rope are multiples of 8)
            const int ku = e / (kw / 8), d = (e - ku * (kw / 8)) * 8;
            int row;
            const KvSeg sg = kv_seg(kv, ri[t].kv0 + p + ku, &row);
            float v[8];
            if (d < r) cache_get8(kv.fmt, sg.v, sg.vs, (size_t) row, r, d, v);
            else cache_get8(kv.fmt, sg.k, sg.ks, (size_t) row, rope, d - r, v);
            float* dst = keys + ku * ld + d;
            *(float4*) dst = make_float4(v[0], v[1], v[2], v[3]);
            *(float4*) (dst + 4) = make_float4(v[4], v[5], v[6], v[7]);
        }
        __syncthreads();
        float sc = 0.0f;
        if (u < nk) {
            const float* kr_ = keys + u * ld;
            for (int i = q0; i < q1; i += 2) {
                const float2 kk = *(const float2*) (kr_ + i), qq = *(const float2*) (qs + i);
                sc = fmaf(qq.x, kk.x, sc);
                sc = fmaf(qq.y, kk.y, sc);
            }
        }
        sc += __shfl_xor(sc, 1);
        sc += __shfl_xor(sc, 2);
        if (u >= nk) sc = -INFINITY;
        float mx = sc;
        for (int o = 4; o < 64; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
        mx = fmaxf(mx, m);
        const float cor = expf(m - mx), e = expf(sc - mx);   // exp(-inf) = 0: keys past the run, and the first tile's m
        float es = e;
        for (int o = 4; o < 64; o <<= 1) es += __shfl_xor(es, o);
        l = fmaf(l, cor, es);
        m = mx;
#pragma unroll
        for (int j = 0; j < MLA_MAXL; ++j) acc[j] *= cor;
#pragma unroll
        for (int ku = 0; ku < GA_KT; ++ku) {
            const float ek = __shfl(e, 4 * ku);
            if (ku >= nk) break;   // uniform
            const float* kr_ = keys + ku * ld;
#pragma unroll
            for (int j = 0; j < MLA_MAXL; ++j)
                if (j < nl && lane + 64 * j < r) acc[j] = fmaf(ek, kr_[lane + 64 * j], acc[j]);
        }
    }
    if (!live) return;
    if (a.n_splits == 1) {
        float* o = out + ((size_t) t * a.n_head + h) * r;
#pragma unroll
        for (int j = 0; j < MLA_MAXL; ++j)
            if (j < nl && lane + 64 * j < r) o[lane + 64 * j] = bfr(acc[j] / l);
    } else {
        float* pp = out + (((size_t) t * a.n_head + h) * a.n_splits + split) * (r + 2);
        if (lane == 0) { pp[0] = m; pp[1] = l; }
#pragma unroll
        for (int j = 0; j < MLA_MAXL; ++j)
            if (j < nl && lane + 64 * j < r) pp[2 + lane + 64 * j] = acc[j];
    }
}

// ---- latent attention on the matrix cores ---------------------------------------------------------------------------------
// Absorbed MLA is multi-query attention over the latent: the 16 heads of a group read the same keys, so a tile of keys is
// one MFMA operand for all of them (the reference's default path does the same on its tensor cores,
// engine/kernels_moe.cu:1388-1397, with the same rounding points: queries are BF16 values, products exact, f32 sums,
// f32 online softmax, P entering the second product as two BF16 terms hi + lo).
// Workgroup (split, group of 16 heads, row) of 4 waves; tile = 32 keys.  Per tile:
//   decode  the tile's cache rows -> BF16 in LDS twice: Ks[key][r + rope] (rows padded by 8) for the scores and
//           Vt[latent dim][key] for P c (MFMA contracts over the index that is contiguous in a lane's fragment).  A thread
//           owns 8 latent dims x 8 keys, so the transposition is 32 v_perm in registers.  FP8 -> BF16 is
//           v_cvt_scalef32_pk_bf16_fp8 (E4M3 code x E8M0 scale, exact); the codes 0x7F / 0xFF (never written by the
//           encoder; the reference's decoder reads them as +-480, the instruction as NaN) and scales outside 2^+-95
//           take the arithmetic decoder, so every byte decodes as in nslm/kvq.h.
//   scores  S^T[key][head] = Ks Q^T by v_mfma_f32_16x16x32_bf16, 18 k-slices x 2 key tiles; Q fragments stay in registers.
//           Wave w sums half of the k-slices of key tile w & 1; the four partial tiles meet in LDS (a third barrier, but a
//           quarter of the LDS reads of every wave computing all of S^T, which is what bounded the tile).
//   softmax lane (head l % 16, keys {4g .. 4g + 3, 16 + 4g .. 16 + 4g + 3}, g = l / 16): two shuffles for the tile's max.
//   P c     O^T[dim][head] += Vt P^T, wave w owns latent dims 128 w .. 128 w + 127 (8 accumulator tiles); the lane's P
//           values are already the B fragment when Vt holds key (16 u + 4 g + i) at column 8 g + 4 u + i.
// The next tile's cache bytes are loaded into registers before the current tile's MFMAs.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
#define MA_KB 32
template <int R, int ROPE>
constexpr int mla_mfma_lds() { return (MA_KB * (R + ROPE + 8) + R * MA_KB) * 2 + 4 * 64 * 16; }   // Vt (R x 32) also stages the 16 query rows

typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t bf2(float lo, float hi) {   // v_cvt_pk_bf16_f32: both round to nearest even
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

// NG = 2 (launches that leave most of the chip idle: a workgroup a CU or fewer): two groups of four waves, each with tiles of its
// own in LDS, take the split's key tiles alternately - the chain of tiles a workgroup walks is half as long - and group 1's running
// maximum, sum and accumulators are merged into group 0's through LDS before the split's partial result leaves, as two splits'
// would be by the reduce.  The groups meet at the same workgroup barriers (a group without a tile in an iteration only waits).
template <int R, int ROPE, int FMT, int NG>
__global__ void __launch_bounds__(256 * NG) k_mla_attn_mfma(MlaArgs a, const float* ql, const float* qr, KvView kv, const RowInfo* ri, float* out) {
    static_assert(R == 512 && ROPE == 64, "the thread mapping of the decode covers 64 latent dim groups and 8 RoPE dim groups");
    static_assert(NG == 1 || NG == 2, "one group of four waves, or two");
    constexpr int KW = R + ROPE, KLD = KW + 8, NKS = KW / 32, MT = R / 64, NW = FMT == KV_FP8 ? 2 : 4;
    extern __shared__ __attribute__((aligned(16))) uint8_t mla_lds[];
    const int grp = NG > 1 ? (int) threadIdx.x >> 8 : 0;
    uint16_t* Ks = (uint16_t*) (mla_lds + grp * mla_mfma_lds<R, ROPE>());
    uint16_t* Vt = Ks + MA_KB * KLD;
    f32x4* Sx = (f32x4*) (Vt + R * MA_KB);   // [wave][lane]: the waves' partial score tiles
    const int tid = (int) threadIdx.x & 255, w = tid >> 6, lane = tid & 63, c = lane & 15, g = lane >> 4;   // (tid, w: within the group)
    const int split = (int) blockIdx.x, t = (int) blockIdx.z, h = (int) blockIdx.y * 16 + c;
    const int pos = ri[t].pos, kv0 = ri[t].kv0;
    int p0, p1;
    split_range(a, pos, split, &p0, &p1);
    const bool live = h < a.n_head;

    // The group's queries, staged once for the four waves: thread e loads 4 consecutive values of head e / 128 (latent) or
    // e / 16 (RoPE part); heads past n_head read head 0 and are zeroed.  The loads are issued here and converted after the
    // first tile's loads are in flight.
    constexpr int QV = 16 * KW / 4 / 256;   // float4 a thread
    u32x4 qv[QV];
#pragma unroll
    for (int i = 0; i < QV; ++i) {
        const int e = tid + 256 * i, hh = e < 16 * R / 4 ? e / (R / 4) : (e - 16 * R / 4) / (ROPE / 4);
        const int hq = (int) blockIdx.y * 16 + hh;
        const size_t th = (size_t) t * a.n_head + (hq < a.n_head ? hq : 0);
        const NSLM_GLOBAL uint32_t* src = e < 16 * R / 4 ? gp<uint32_t>(ql) + th * R + 4 * (e % (R / 4)) : gp<uint32_t>(qr) + th * ROPE + 4 * ((e - 16 * R / 4) % (ROPE / 4));
        qv[i] = *(const NSLM_GLOBAL u32x4*) src;
    }
    // decode roles: latent dims 8 dg .. + 7 of keys {4 kap + j, 16 + 4 kap + j}; RoPE dims rd .. + 7 of key rkey
    constexpr int ES = FMT == KV_FP8 ? 1 : 2;   // bytes a cached value
    const int dgl = lane & 15, kap = lane >> 4, dg = 16 * w + dgl, par = dgl & 1, rkey = tid >> 3, rd = 8 * (tid & 7);
    const uint32_t selA = par ? 0x07060302u : 0x05040100u, selB = par ? 0x05040100u : 0x07060302u;
    uint32_t raw[8][NW] = {}, rraw[NW] = {}, rsc[8] = {127u, 127u, 127u, 127u, 127u, 127u, 127u, 127u}, rrsc = 127u;
    auto fetch = [&](const void* codes, const void* scales, int row, int n, int d, uint32_t (&x)[NW], uint32_t& sc) {
        if (FMT == KV_FP8) {
            const uint2 q = ldg8(gp<uint8_t>(codes) + (size_t) row * n + d);
            x[0] = q.x; x[1] = q.y;
            sc = gp<uint8_t>(scales)[(size_t) row * (n / 32) + d / 32];
        } else {
            const uint4 q = ldg16(gp<uint16_t>(codes) + (size_t) row * n + d);
            x[0] = q.x; x[1] = q.y; x[NW - 2] = q.z; x[NW - 1] = q.w;
        }
    };
    // Keys past the split's end read its last key (finite values; their scores are masked), so no load is conditional.
    auto load_tile = [&](int p) {
        const int rb = kv0 + p, last = p1 - 1 - p;
        if (rb + MA_KB <= kv.nv || rb >= kv.nv) {   // the tile lies in one segment of the view (uniform): 32-bit offsets from its first row
            const bool first = rb < kv.nv;
            const KvSeg sg = first ? kv.a : kv.b;
            const size_t r0 = (size_t) (first ? rb : rb - kv.nv);
            const NSLM_GLOBAL uint8_t* vb = gp<uint8_t>(sg.v) + r0 * (R * ES);
            const NSLM_GLOBAL uint8_t* kb = gp<uint8_t>(sg.k) + r0 * (ROPE * ES);
            const NSLM_GLOBAL uint8_t* vsb = gp<uint8_t>(sg.vs) + r0 * (R / 32);
            const NSLM_GLOBAL uint8_t* ksb = gp<uint8_t>(sg.ks) + r0 * (ROPE / 32);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t kj = (uint32_t) min(j < 4 ? 4 * kap + j : 12 + 4 * kap + j, last);
                if (FMT == KV_FP8) {
                    const uint2 q = ldg8(vb + (kj * (uint32_t) R + 8u * (uint32_t) dg));
                    raw[j][0] = q.x; raw[j][1] = q.y;
                    rsc[j] = vsb[kj * (uint32_t) (R / 32) + (uint32_t) (dg >> 2)];
                } else {
                    const uint4 q = ldg16(vb + (kj * (uint32_t) (2 * R) + 16u * (uint32_t) dg));
                    raw[j][0] = q.x; raw[j][1] = q.y; raw[j][NW - 2] = q.z; raw[j][NW - 1] = q.w;
                }
            }
            const uint32_t kr = (uint32_t) min(rkey, last);
            if (FMT == KV_FP8) {
                const uint2 q = ldg8(kb + (kr * (uint32_t) ROPE + (uint32_t) rd));
                rraw[0] = q.x; rraw[1] = q.y;
                rrsc = ksb[kr * (uint32_t) (ROPE / 32) + (uint32_t) (rd >> 5)];
            } else {
                const uint4 q = ldg16(kb + (kr * (uint32_t) (2 * ROPE) + 2u * (uint32_t) rd));
                rraw[0] = q.x; rraw[1] = q.y; rraw[NW - 2] = q.z; rraw[NW - 1] = q.w;
            }
        } else {   // the tile straddles the view's two segments: each key finds its own
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                int row;
                const KvSeg sg = kv_seg(kv, rb + min(j < 4 ? 4 * kap + j : 12 + 4 * kap + j, last), &row);
                fetch(sg.v, sg.vs, row, R, 8 * dg, raw[j], rsc[j]);
            }
            int row;
            const KvSeg sg = kv_seg(kv, rb + min(rkey, last), &row);
            fetch(sg.k, sg.ks, row, ROPE, rd, rraw, rrsc);
        }
    };
    // FP8 words that v_cvt_scalef32_pk_bf16_fp8 reads as the codec does: no all-ones magnitude (bit 7 of a byte of the
    // result set otherwise); a scale byte in [32, 222] keeps code x scale a normal BF16 value
    auto odd_codes = [](uint32_t x0, uint32_t x1) { return ((x0 & 0x7F7F7F7Fu) + 0x01010101u) | ((x1 & 0x7F7F7F7Fu) + 0x01010101u); };
    auto decode8 = [&](const uint32_t (&x)[NW], uint32_t sc, bool exact, uint32_t (&d)[4]) {
        if (FMT != KV_FP8) {
#pragma unroll
            for (int i = 0; i < 4; ++i) d[i] = x[i * NW / 4];
        } else if (!exact) {
            const float f = __uint_as_float(sc << 23);
            d[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(x[0], f, false));
            d[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(x[0], f, true));
            d[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(x[1], f, false));
            d[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(x[1], f, true));
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t wd = x[i >> 1] >> (16 * (i & 1));
                d[i] = (__float_as_uint(fp8_value(wd & 255u, sc)) >> 16) | (__float_as_uint(fp8_value((wd >> 8) & 255u, sc)) & 0xFFFF0000u);
            }
        }
    };
    auto store_tile = [&]() {
        uint32_t D[8][4], dr[4];
        bool exact = false;
        if (FMT == KV_FP8) {
            uint32_t odd = odd_codes(rraw[0], rraw[1]), far = rrsc - 32u;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                odd |= odd_codes(raw[j][0], raw[j][1]);
                far = max(far, rsc[j] - 32u);
            }
            exact = (odd & 0x80808080u) != 0u || far > 190u;
        }
        if (!exact) {
#pragma unroll
            for (int j = 0; j < 8; ++j) decode8(raw[j], rsc[j], false, D[j]);
            decode8(rraw, rrsc, false, dr);
        } else {   // the arithmetic decoder for this lane's whole share
#pragma unroll 1
            for (int rep = 0; rep < 1; ++rep) {
#pragma unroll
                for (int j = 0; j < 8; ++j) decode8(raw[j], rsc[j], true, D[j]);
                decode8(rraw, rrsc, true, dr);
            }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int key = j < 4 ? 4 * kap + j : 12 + 4 * kap + j;
            *(u32x4*) &Ks[key * KLD + 8 * dg] = u32x4{D[j][0], D[j][1], D[j][2], D[j][3]};
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {   // latent dims 8 dg + 2 q (+ 1): 8 keys each = one 16-byte block of a Vt row
            u32x4 oa, ob;
#pragma unroll
            for (int jp = 0; jp < 4; ++jp) {
                oa[jp] = __builtin_amdgcn_perm(D[2 * jp + 1][q], D[2 * jp][q], selA);
                ob[jp] = __builtin_amdgcn_perm(D[2 * jp + 1][q], D[2 * jp][q], selB);
            }
            const int blk = kap ^ (q & 3) ^ ((dg >> 1) & 3), row = 8 * dg + 2 * q;
            *(u32x4*) &Vt[(row + par) * MA_KB + 8 * blk] = oa;
            *(u32x4*) &Vt[(row + 1 - par) * MA_KB + 8 * blk] = ob;
        }
        *(u32x4*) &Ks[rkey * KLD + R + rd] = u32x4{dr[0], dr[1], dr[2], dr[3]};
    };

    // Online softmax against a reference score m per head that is raised only when a tile's maximum exceeds it by more than
    // MLA_LAZY (so P <= e^MLA_LAZY and the accumulators are rescaled on few tiles); l and acc are in the scale e^-m.
    constexpr float MLA_LAZY = 8.0f;
    f32x4 acc[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    float m = -INFINITY, l = 0.0f;
    if (p0 + grp * MA_KB < p1) load_tile(p0 + grp * MA_KB);
    // scores: wave w sums k-slices [9 (w >> 1), + 9) of key tile w & 1
    constexpr int KH = NKS / 2;
    const int su = w & 1, sk = (w >> 1) * KH;
    bf16x8 qf[KH];
    {   // queries -> BF16 rows in LDS (over Vt, which the first tile fills after the barrier below) -> the wave's B fragments
        uint16_t* Qs = Vt;
#pragma unroll
        for (int i = 0; i < QV; ++i) {
            const int e = tid + 256 * i, hh = e < 16 * R / 4 ? e / (R / 4) : (e - 16 * R / 4) / (ROPE / 4);
            const int d = e < 16 * R / 4 ? 4 * (e % (R / 4)) : R + 4 * ((e - 16 * R / 4) % (ROPE / 4));
            const uint32_t keep = (int) blockIdx.y * 16 + hh < a.n_head ? 0xFFFFFFFFu : 0u;
            *(u32x2*) &Qs[hh * KLD + d] = u32x2{bf2(__uint_as_float(qv[i][0]), __uint_as_float(qv[i][1])) & keep,
                                                bf2(__uint_as_float(qv[i][2]), __uint_as_float(qv[i][3])) & keep};
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < KH; ++ks) qf[ks] = *(const bf16x8*) &Qs[c * KLD + 32 * (sk + ks) + 8 * g];
        __syncthreads();
    }
    for (int pb = p0; pb < p1; pb += MA_KB * NG) {
        const int p = pb + grp * MA_KB;
        const bool mine = NG == 1 || p < p1;   // (uniform over the group)
        if (mine) store_tile();
        __syncthreads();
        if (p + MA_KB * NG < p1) load_tile(p + MA_KB * NG);
        f32x4 s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = s0;   // two chains over the wave's 9 k-slices
        if (mine) {
#pragma unroll
            for (int ks = 0; ks < KH; ++ks) {
                const bf16x8 a0 = *(const bf16x8*) &Ks[(16 * su + c) * KLD + 32 * (sk + ks) + 8 * g];
                if (ks & 1) s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, qf[ks], s1, 0, 0, 0);
                else s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, qf[ks], s0, 0, 0, 0);
            }
            Sx[tid] = s0 + s1;
        }
        __syncthreads();
        if (!mine) {   // no tile of this group's in the split's last iteration: the third barrier, nothing else
            __syncthreads();
            continue;
        }
        s0 = Sx[lane] + Sx[128 + lane];        // key tile 0: waves 0 and 2
        s1 = Sx[64 + lane] + Sx[192 + lane];   // key tile 1: waves 1 and 3
        float sv[8], mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int key = j < 4 ? 4 * g + j : 12 + 4 * g + j;
            sv[j] = p + key < p1 ? (j < 4 ? s0[j] : s1[j - 4]) * a.scale : -INFINITY;
            mx = fmaxf(mx, sv[j]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const bool up = mx > m + MLA_LAZY;   // true on the first tile (m = -inf; every tile has a key, so mx is finite)
        if (__any(up)) {
            const float cor = up ? __expf(m - mx) : 1.0f;
            m = up ? mx : m;
            l *= cor;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) acc[mt] *= cor;
        }
        u32x4 bh, bl;
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
            const float e0 = __expf(sv[j] - m), e1 = __expf(sv[j + 1] - m);   // masked keys: exp(-inf) = 0
            l += e0 + e1;
            bh[j >> 1] = bf2(e0, e1);
            bl[j >> 1] = bf2(e0 - __uint_as_float(bh[j >> 1] << 16), e1 - __uint_as_float(bh[j >> 1] & 0xFFFF0000u));
        }
        const bf16x8 ph = __builtin_bit_cast(bf16x8, bh), pl = __builtin_bit_cast(bf16x8, bl);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int tile = w * MT + mt;
            const bf16x8 vt = *(const bf16x8*) &Vt[(16 * tile + c) * MA_KB + 8 * (g ^ ((c >> 1) & 3) ^ (tile & 3))];
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt, ph, acc[mt], 0, 0, 0);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt, pl, acc[mt], 0, 0, 0);
        }
        __syncthreads();
    }
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    if (NG > 1) {   // group 1's state into group 0's, thread by thread (the same head, the same latent dims), as two splits merge
        float* mg = (float*) (mla_lds + mla_mfma_lds<R, ROPE>()) + tid * (4 * MT + 2);   // (group 1's tiles: read for the last time before the loop's last barrier)
        if (grp == 1) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int i = 0; i < 4; ++i) mg[4 * mt + i] = acc[mt][i];
            mg[4 * MT] = m;
            mg[4 * MT + 1] = l;
        }
        __syncthreads();
        if (grp == 1) return;
        const float m1 = mg[4 * MT], l1 = mg[4 * MT + 1], mn = fmaxf(m, m1);
        const float f0 = m == mn ? 1.0f : __expf(m - mn), f1 = m1 == mn ? 1.0f : __expf(m1 - mn);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[mt][i] = acc[mt][i] * f0 + mg[4 * mt + i] * f1;
        l = l * f0 + l1 * f1;
        m = mn;
    }
    if (!live) return;
    if (a.n_splits == 1) {
        float* o = out + ((size_t) t * a.n_head + h) * R;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i) o[16 * (w * MT + mt) + 4 * g + i] = bfr(acc[mt][i] / l);
    } else {
        float* pp = out + (((size_t) t * a.n_head + h) * a.n_splits + split) * (R + 2);
        if (w == 0 && g == 0) { pp[0] = m; pp[1] = l; }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i) pp[2 + 16 * (w * MT + mt) + 4 * g + i] = acc[mt][i];
    }
}

// Reduce the splits: olat[t][h][d] = bf16(acc / l).  Workgroup (head, row, 128 latent dims): the splits' maxima and
// weights exp(m_s - m) once per workgroup (threads stride the splits, so their loads are in flight together), then each
// thread sums its dim over the splits.
#define MLA_RED_MAXS 256
__global__ void __launch_bounds__(128) k_mla_reduce(MlaArgs a, const RowInfo* ri, const float* part, float* olat) {
    __shared__ float wts[MLA_RED_MAXS], red[4];
    const int h = (int) blockIdx.x, t = (int) blockIdx.y, r = a.r, w = r + 2, ns = mla_row_splits(a, ri[t].pos), tid = threadIdx.x;
    const NSLM_GLOBAL float* pp = gp<float>(part) + ((size_t) t * a.n_head + h) * a.n_splits * w;
    float ms[MLA_RED_MAXS / 128], m = -INFINITY;
#pragma unroll
    for (int i = 0; i < MLA_RED_MAXS / 128; ++i) {
        const int s = tid + 128 * i;
        ms[i] = s < ns ? pp[(size_t) s * w] : -INFINITY;
        m = fmaxf(m, ms[i]);
    }
    for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
    if ((tid & 63) == 0) red[tid >> 6] = m;
    __syncthreads();
    m = fmaxf(red[0], red[1]);
    float l = 0.0f;
#pragma unroll
    for (int i = 0; i < MLA_RED_MAXS / 128; ++i) {
        const int s = tid + 128 * i;
        if (s < ns) {
            const float c = ms[i] == -INFINITY ? 0.0f : expf(ms[i] - m);
            wts[s] = c;
            l = fmaf(pp[(size_t) s * w + 1], c, l);
        }
    }
    for (int o = 32; o > 0; o >>= 1) l += __shfl_xor(l, o);
    if ((tid & 63) == 0) red[2 + (tid >> 6)] = l;
    __syncthreads();
    l = red[2] + red[3];
    const int d = (int) blockIdx.z * 128 + tid;
    if (d >= r) return;
    float acc = 0.0f;
#pragma unroll 8
    for (int s = 0; s < ns; ++s) acc = fmaf(pp[(size_t) s * w + 2 + d], wts[s], acc);
    olat[((size_t) t * a.n_head + h) * r + d] = bfr(acc / l);
}

// The splits' reduce and the value-up map of a head in ONE launch: workgroup (row group, head, row) reduces the head's
// latent output into LDS (k_mla_reduce's arithmetic, all r dims: the map needs them all) and computes rows
// [RG g, RG (g + 1)) of y[t][h] = bf16(W_h . olat[t][h]) (k_heads_mv's arithmetic).  The same bits as the two kernels.
#define MLA_RV_GROUPS 16   // row groups a head at most: fewer when there are many (row, head) pairs, each group re-reads the partials
__global__ void __launch_bounds__(256) k_mla_reduce_vup(MlaArgs a, const RowInfo* ri, const float* part, HmvArgs hv, int fmt, WSlice W, float* y,
                                                       int lpr) {
    __shared__ uint32_t tab[NSLM_TAB_WORDS];
    __shared__ float wts[MLA_RED_MAXS], red[4];
    __shared__ __attribute__((aligned(16))) float ol[64 * MLA_MAXL];
    constexpr int PF = 32, NP = 2;   // splits / map passes whose loads are issued before anything waits
    const int g = (int) blockIdx.x, h = (int) blockIdx.y, t = (int) blockIdx.z, r = a.r, w = r + 2, ns = mla_row_splits(a, ri[t].pos), tid = threadIdx.x;
    const NSLM_GLOBAL float* pp = gp<float>(part) + ((size_t) t * a.n_head + h) * a.n_splits * w;
    const int rg = (hv.O + (int) gridDim.x - 1) / (int) gridDim.x, o0 = g * rg, o1 = min(o0 + rg, hv.O);
    const int rpw = 64 / lpr, sub = (tid & 63) / lpr, ln = tid & (lpr - 1);
    // Every load whose address is known now is in flight before the first wait: the splits' (m, l), this thread's two
    // output dims of the first PF splits, and (BF16 maps, one block a lane) the map rows of the first NP passes.
    // (loads are unconditional on clamped indices: a conditional load waits for the ones before it)
    float msv[MLA_RED_MAXS / 128], lsv[MLA_RED_MAXS / 128], pv[2][PF];
#pragma unroll
    for (int i = 0; i < MLA_RED_MAXS / 128; ++i) {
        const int s = tid + 128 * i, sc = min(s, ns - 1);
        const bool ok = tid < 128 && s < ns;
        const float mv = pp[(size_t) sc * w], lv = pp[(size_t) sc * w + 1];
        msv[i] = ok ? mv : -INFINITY;
        lsv[i] = ok ? lv : 0.0f;
    }
#pragma unroll
    for (int k = 0; k < 2; ++k)
#pragma unroll
        for (int s = 0; s < PF; ++s) pv[k][s] = pp[(size_t) min(s, ns - 1) * w + 2 + min(tid + 256 * k, r - 1)];
    const bool pre = fmt == MF_BF16 && hv.I / 8 == lpr && (((uintptr_t) W.p[0] | (uintptr_t) (2 * hv.I)) & 15u) == 0;
    uint4 wq[NP];
    if (pre) {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int o = min(o0 + i * 4 * rpw + (tid >> 6) * rpw + sub, hv.O - 1);
            wq[i] = ldg16(gp<uint16_t>(W.p[0]) + ((size_t) h * hv.O + o) * hv.I + (size_t) ln * 8);
        }
    }
    if (fmt == MF_SEED4P4 || fmt == MF_SEED4) load_tables(tab);
    // the splits' maximum and the sum of l exactly as k_mla_reduce forms them: its two waves, splits tid and tid + 128
    float m = -INFINITY, l = 0.0f;
    if (tid < 128) {
#pragma unroll
        for (int i = 0; i < MLA_RED_MAXS / 128; ++i) m = fmaxf(m, msv[i]);
        for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
        if ((tid & 63) == 0) red[tid >> 6] = m;
    }
    __syncthreads();
    m = fmaxf(red[0], red[1]);
    if (tid < 128) {
#pragma unroll
        for (int i = 0; i < MLA_RED_MAXS / 128; ++i) {
            const int s = tid + 128 * i;
            if (s < ns) {
                const float c = msv[i] == -INFINITY ? 0.0f : expf(msv[i] - m);
                wts[s] = c;
                l = fmaf(lsv[i], c, l);
            } else if (s < PF) wts[s] = 0.0f;   // the prefetched terms past the last split add x * 0
        }
        for (int o = 32; o > 0; o >>= 1) l += __shfl_xor(l, o);
        if ((tid & 63) == 0) red[2 + (tid >> 6)] = l;
    }
    __syncthreads();
    l = red[2] + red[3];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const int d = tid + 256 * k;
        if (d >= r) break;
        float acc = 0.0f;
#pragma unroll
        for (int s = 0; s < PF; ++s) acc = fmaf(pv[k][s], wts[s], acc);
        for (int s = PF; s < ns; ++s) acc = fmaf(pp[(size_t) s * w + 2 + d], wts[s], acc);
        ol[d] = bfr(acc / l);
    }
    for (int d = tid + 512; d < r; d += 256) {   // latent widths above 512
        float acc = 0.0f;
        for (int s = 0; s < ns; ++s) acc = fmaf(pp[(size_t) s * w + 2 + d], wts[s], acc);
        ol[d] = bfr(acc / l);
    }
    __syncthreads();
    WSlice ws = W;
    if (fmt == MF_SEED4P4) ws.eb = gp<int32_t>(W.p[2])[h];
    auto finish = [&](int o, bool live, float acc) {
        for (int sft = lpr >> 1; sft > 0; sft >>= 1) acc += __shfl_xor(acc, sft);
        if (live && ln == 0) y[((size_t) t * hv.H + h) * hv.O + o] = bfr(acc);
    };
    int ob = o0;
    if (pre) {   // one block a lane from the prefetched rows: the same products and sums as the loop below
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            if (ob >= o1) break;
            const int o = ob + (tid >> 6) * rpw + sub;
            const uint4 q = wq[i];
            const float* xb = ol + (size_t) ln * 8;
            float d = bf(q.x & 0xFFFFu) * xb[0];
            d = fmaf(bf(q.x >> 16), xb[1], d);
            d = fmaf(bf(q.y & 0xFFFFu), xb[2], d);
            d = fmaf(bf(q.y >> 16), xb[3], d);
            d = fmaf(bf(q.z & 0xFFFFu), xb[4], d);
            d = fmaf(bf(q.z >> 16), xb[5], d);
            d = fmaf(bf(q.w & 0xFFFFu), xb[6], d);
            d = fmaf(bf(q.w >> 16), xb[7], d);
            finish(o, o < o1, fmaf(d, 1.0f, 0.0f));
            ob += 4 * rpw;
        }
    }
    for (; ob < o1; ob += 4 * rpw) {
        const int o = ob + (tid >> 6) * rpw + sub;
        const bool live = o < o1;
        float acc = 0.0f;
        if (live)
            for (int j = ln; j < hv.I / 8; j += lpr) {
                float wv[8], sc;
                block_weights(fmt, ws, tab, h * hv.O + o, hv.I, j, wv, &sc);
                const float* xb = ol + (size_t) j * 8;
                float d = wv[0] * xb[0];
#pragma unroll
                for (int cc = 1; cc < 8; ++cc) d = fmaf(wv[cc], xb[cc], d);
                acc = fmaf(d, sc, acc);
            }
        finish(o, live, acc);
    }
}

// y = `rows` FP8 cache rows of n values, decoded (8 values a thread; for tests)
__global__ void k_kv_f32(int fmt, const uint8_t* C, const uint8_t* S, int n, int rows, float* y) {
    const int i = ((int) blockIdx.x * (int) blockDim.x + threadIdx.x) * 8;
    if (i >= n * rows) return;
    float v[8];
    cache_get8(fmt, C, S, (size_t) (i / n), n, i % n, v);
#pragma unroll
    for (int j = 0; j < 8; ++j) y[i + j] = v[j];
}

int rope_of(const MlaArgs& a) { return a.pad[0] > 0 ? a.pad[0] : ATT_HD; }

}   // namespace

extern "C" {

void kc_heads_mv(kc_stream_t s, HmvArgs a, int fmt, WSlice W, const uint32_t* G, const float* x, const float* g, float* y, int T) {
    (void) G;
    if (T < 1 || a.H < 1 || a.O < 1 || a.I < 8) return;
    int lpr = 1;
    while (lpr < 64 && lpr < a.I / 8) lpr <<= 1;
    const int rows_wg = 4 * (64 / lpr);
    hipLaunchKernelGGL(k_heads_mv, dim3((unsigned) (a.O + rows_wg - 1) / rows_wg, (unsigned) a.H, (unsigned) T), dim3(256), 0, (hipStream_t) s,
                       a, fmt, W, x, g ? g : x, y, lpr);
    host_note_launch();
}
void kc_mla_rope(kc_stream_t s, MlaArgs a, float* qr, const float* kr, const float* c, KvView kv, const RowInfo* ri, const float* inv,
                 int T) {
    const int rope = rope_of(a);
    if (T < 1 || (kv.fmt != KV_BF16 && kv.fmt != KV_FP8) || (rope != 64 && rope != 128) || a.r % 32) { host_note_unsupported(); return; }
    hipLaunchKernelGGL(k_mla_rope, dim3((unsigned) T), dim3(256), 0, (hipStream_t) s, a, rope, qr, kr, c, kv, ri, inv);
    host_note_launch();
}
int kc_mla_qmaps_rope(kc_stream_t s, MlaArgs a, HmvArgs hq, HmvArgs hl, int fmt, WSlice Wq, WSlice Wl, const float* q, float* qr, float* ql,
                      const float* kr, const float* c, KvView kv, const RowInfo* ri, const float* inv, int T) {
    const int rope = rope_of(a);
    int lpr = 1;
    while (lpr < 64 && lpr < hq.I / 8) lpr <<= 1;
    if (T < 1 || (kv.fmt != KV_BF16 && kv.fmt != KV_FP8) || (rope != 64 && rope != 128) || a.r % 64 || hq.O != rope || hl.O != a.r || hq.I != hl.I ||
        hq.I % 8 || hq.I / 8 > 64 || lpr != hq.I / 8 || hq.H != a.n_head || hl.H != a.n_head || hq.gate || hl.gate || hq.xs != hl.xs || hq.hs != hl.hs)
        return -1;
    const int bx = 1 + a.r / 64;   // >= the cache jobs' blocks: (1 + r / 64 + 3) / 4
    hipLaunchKernelGGL(k_qmaps_rope, dim3((unsigned) bx, (unsigned) a.n_head + 1, (unsigned) T), dim3(256), 0, (hipStream_t) s, a, rope, hq, hl, fmt,
                       Wq, Wl, q, qr, ql, kr, c, kv, ri, inv, lpr);
    host_note_launch();
    return 0;
}
// attention into the partials (n_splits > 1) or olat; the reduce when `reduce`.  false: unsupported, nothing launched
static bool mla_attn_launch(kc_stream_t s, MlaArgs a, const float* ql, const float* qr, KvView kv, const RowInfo* ri, float* part, float* olat,
                            int T, bool reduce) {
    const int rope = rope_of(a);
    if (T < 1 || (kv.fmt != KV_BF16 && kv.fmt != KV_FP8) || (rope != 64 && rope != 128) || a.r % 8 || a.r > 64 * MLA_MAXL || a.n_splits < 1) {
        host_note_unsupported();
        return false;
    }
    float* o = a.n_splits > 1 ? part : olat;
    if (a.n_splits > MLA_RED_MAXS) { host_note_unsupported(); return false; }
    if (a.r == 512 && rope == 64 && (((uintptr_t) ql | (uintptr_t) qr) & 15u) == 0) {   // the matrix-core kernel: 16 heads a workgroup
        constexpr int lds = mla_mfma_lds<512, 64>();
        static const hipError_t once[4] = {
            hipFuncSetAttribute((const void*) k_mla_attn_mfma<512, 64, KV_BF16, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, lds),
            hipFuncSetAttribute((const void*) k_mla_attn_mfma<512, 64, KV_FP8, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, lds),
            hipFuncSetAttribute((const void*) k_mla_attn_mfma<512, 64, KV_BF16, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * lds),
            hipFuncSetAttribute((const void*) k_mla_attn_mfma<512, 64, KV_FP8, 2>, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * lds)};
        (void) once;
        const dim3 grid((unsigned) a.n_splits, (unsigned) (a.n_head + 15) / 16, (unsigned) T);
        // a workgroup a CU or fewer: two groups of waves a workgroup walk a split's tiles (a step of a few rows is a chain of tiles)
        const bool two = (long) grid.x * grid.y * grid.z <= 256;
        if (two && kv.fmt == KV_FP8) hipLaunchKernelGGL((k_mla_attn_mfma<512, 64, KV_FP8, 2>), grid, dim3(512), 2 * lds, (hipStream_t) s, a, ql, qr, kv, ri, o);
        else if (two) hipLaunchKernelGGL((k_mla_attn_mfma<512, 64, KV_BF16, 2>), grid, dim3(512), 2 * lds, (hipStream_t) s, a, ql, qr, kv, ri, o);
        else if (kv.fmt == KV_FP8) hipLaunchKernelGGL((k_mla_attn_mfma<512, 64, KV_FP8, 1>), grid, dim3(256), lds, (hipStream_t) s, a, ql, qr, kv, ri, o);
        else hipLaunchKernelGGL((k_mla_attn_mfma<512, 64, KV_BF16, 1>), grid, dim3(256), lds, (hipStream_t) s, a, ql, qr, kv, ri, o);
    } else {
        const size_t lds = sizeof(float) * (size_t) (GA_KT + GA_HW) * (size_t) (a.r + rope + 4);
        static const hipError_t once = hipFuncSetAttribute((const void*) k_mla_attn_any, hipFuncAttributeMaxDynamicSharedMemorySize,
                                                           (int) (sizeof(float) * (GA_KT + GA_HW) * (64 * MLA_MAXL + ATT_HD + 4)));
        (void) once;
        hipLaunchKernelGGL(k_mla_attn_any, dim3((unsigned) a.n_splits, (unsigned) (a.n_head + GA_HW - 1) / GA_HW, (unsigned) T), dim3(64 * GA_HW), lds,
                           (hipStream_t) s, a, rope, ql, qr, kv, ri, o);
    }
    if (a.n_splits > 1 && reduce)
        hipLaunchKernelGGL(k_mla_reduce, dim3((unsigned) a.n_head, (unsigned) T, (unsigned) (a.r + 127) / 128), dim3(128), 0, (hipStream_t) s, a, ri,
                           part, olat);
    host_note_launch();
    return true;
}
void kc_mla_attn(kc_stream_t s, MlaArgs a, const float* ql, const float* qr, KvView kv, const RowInfo* ri, float* part, float* olat,
                 int T) {
    (void) mla_attn_launch(s, a, ql, qr, kv, ri, part, olat, T, true);
}
int kc_mla_attn_vup(kc_stream_t s, MlaArgs a, const float* ql, const float* qr, KvView kv, const RowInfo* ri, float* part, HmvArgs hv, int fmt,
                    WSlice W, float* y, int T) {
    int lpr = 1;
    while (lpr < 64 && lpr < hv.I / 8) lpr <<= 1;
    if (a.n_splits < 2 || a.n_splits > MLA_RED_MAXS || hv.I != a.r || a.r % 8 || a.r > 64 * MLA_MAXL || hv.H != a.n_head || hv.gate ||
        (lpr != hv.I / 8 && hv.I / 8 <= 64) || hv.O < 1)
        return -1;
    if (!mla_attn_launch(s, a, ql, qr, kv, ri, part, NULL, T, false)) return -1;
    int groups = 1024 / (a.n_head * T);   // about a thousand workgroups
    groups = groups < 1 ? 1 : groups > MLA_RV_GROUPS ? MLA_RV_GROUPS : groups;
    hipLaunchKernelGGL(k_mla_reduce_vup, dim3((unsigned) groups, (unsigned) a.n_head, (unsigned) T), dim3(256), 0, (hipStream_t) s, a, ri, part, hv, fmt,
                       W, y, lpr);
    host_note_launch();
    return 0;
}
void kc_kv_f32(kc_stream_t s, int fmt, const uint8_t* codes, const uint8_t* scales, int n, int rows, float* y) {
    if (rows < 1 || n < 8 || (fmt != KV_BF16 && fmt != KV_FP8)) { host_note_unsupported(); return; }
    hipLaunchKernelGGL(k_kv_f32, dim3((unsigned) ((n * rows / 8 + 127) / 128)), dim3(128), 0, (hipStream_t) s, fmt, codes, scales, n, rows, y);
    host_note_launch();
}

}   // extern "C"
