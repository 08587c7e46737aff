// nslm_mla.hip - decode attention over a latent KV cache (absorbed MLA) and what feeds it: per-head maps, RoPE with the
// cache write, the FP8 (E4M3 codes, one E8M0 scale per 32 values) cache codec, split-key latent attention and its reduce.
// Replaces the reference's k_heads_mv, k_mla_rope, k_mla_attn / k_mla_reduce, k_kv_f32 and the FP8 half of kvq_put /
// kvq_get8 (engine/kernels_moe.cu:955-1118,1147-1176,1177-1208,1217-1323; the codec's definition is nslm/kvq.h:19-80)
// behind the same launchers.  BF16 and FP8 caches; the FP4 cache format is not built.
//
// Per cached position the kernel reads r + rope values once for ALL heads of a workgroup (multi-query over the shared
// latent): 660 bytes at r = 512, rope 128, FP8 - so the attention of a 4096-token context moves 2.7 MB per row, and what
// it costs is the 2 x (r + rope) multiply-adds per (key, head).  Those stay in f32 on the vector ALUs: the reference's
// tests hold the output to one BF16 ulp + 2e-6 of a double-precision softmax, which BF16 matrix products of the scores
// would not meet.
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
// Thread i: latent dim i (i < r) and the pair (i % half, + half) of head i / half (head n_head: the key), half = rope / 2.
__global__ void __launch_bounds__(64) k_mla_rope(MlaArgs a, int rope, float* qr, const float* kr, const float* c, KvView kv,
                                                 const RowInfo* ri, const float* inv) {
    const int i = (int) blockIdx.x * 64 + threadIdx.x, t = (int) blockIdx.y, pos = ri[t].pos, half = rope / 2;
    int row;
    const KvSeg sg = kv_seg(kv, ri[t].kv0 + pos, &row);
    const int head = i / half, p = i % half;
    const bool lat = i < a.r, key = head == a.n_head;
    float y0 = 0.0f, y1 = 0.0f;
    if (head <= a.n_head) {
        float sn, cs;
        sincosf((float) pos * inv[p], &sn, &cs);
        float* qh = qr + ((size_t) t * a.n_head + (key ? 0 : head)) * rope;
        const float* xh = key ? kr + (size_t) t * rope : qh;
        const float x0 = xh[p], x1 = xh[p + half];
        y0 = x0 * cs - x1 * sn;
        y1 = x1 * cs + x0 * sn;
        if (!key) { qh[p] = bfr(y0); qh[p + half] = bfr(y1); }
    }
    if (kv.fmt == KV_BF16) {
        if (lat) ((uint16_t*) sg.v)[(size_t) row * a.r + i] = (uint16_t) tobf(c[(size_t) t * a.r + i]);
        if (key) {
            uint16_t* kc = (uint16_t*) sg.k + (size_t) row * rope;
            kc[p] = (uint16_t) tobf(y0);
            kc[p + half] = (uint16_t) tobf(y1);
        }
        return;
    }
    // FP8 (uniform over the grid): every lane runs the shuffles; 32 consecutive lanes are one block
    fp8_put(lat, lat ? bfr(c[(size_t) t * a.r + i]) : 0.0f, (uint8_t*) sg.v, (uint8_t*) sg.vs, (size_t) row, a.r, lat ? i : 0);
    fp8_put(key, bfr(y0), (uint8_t*) sg.k, (uint8_t*) sg.ks, (size_t) row, rope, p);
    fp8_put(key, bfr(y1), (uint8_t*) sg.k, (uint8_t*) sg.ks, (size_t) row, rope, p + half);
}

// ---- latent attention -----------------------------------------------------------------------------------------------------
// Workgroup (split, head group, row) of HG waves, one query head a wave; lane l holds latent dims l, l + 64, .. (up to
// MAXL) and RoPE dims l (, l + 64).  Each step stages KU keys (latent, then RoPE key) decoded to f32 in LDS once for the
// workgroup's heads.  Score = scale (ql . c + qr . k), online softmax, f32 sums.  n_splits > 1: partials
// [row][head][split] = (m, l, acc[r]) for k_mla_reduce; n_splits == 1: olat[row][head] = bf16(acc / l).
#define MLA_KU 8
#define MLA_MAXL 16    // latent dims a lane (r <= 1024)
#define MLA_SPLITS_SHORT 32
__device__ __forceinline__ int mla_row_splits(const MlaArgs& a, int pos) {
    (void) pos;
    return a.pad[2] > 0 && a.n_splits > MLA_SPLITS_SHORT ? MLA_SPLITS_SHORT : a.n_splits;
}
template <int HG>
__global__ void __launch_bounds__(64 * HG) k_mla_attn(MlaArgs a, int rope, const float* ql, const float* qr, KvView kv, const RowInfo* ri,
                                                     float* out) {
    __shared__ __attribute__((aligned(16))) float sh[MLA_KU * (64 * MLA_MAXL + ATT_HD)];
    const int lane = threadIdx.x & 63, tid = threadIdx.x, ntg = 64 * HG;
    const int split = (int) blockIdx.x, t = (int) blockIdx.z, r = a.r, nl = (r + 63) / 64, kw = r + rope;
    const int h = (int) blockIdx.y * HG + (tid >> 6);
    const int pos = ri[t].pos, ns = mla_row_splits(a, pos);
    const int nsr = min(ns, (pos + a.chunk) / a.chunk);
    const int chunk = (pos + nsr) / nsr;
    const int p0 = split * chunk, p1 = split < nsr ? min(pos + 1, p0 + chunk) : p0;
    const bool live = h < a.n_head;
    float q[MLA_MAXL], acc[MLA_MAXL], qp[2];
    const float* qlh = ql + ((size_t) t * a.n_head + (live ? h : 0)) * r;
    const float* qrh = qr + ((size_t) t * a.n_head + (live ? h : 0)) * rope;
#pragma unroll
    for (int j = 0; j < MLA_MAXL; ++j) {
        q[j] = j < nl && lane + 64 * j < r ? qlh[lane + 64 * j] * a.scale : 0.0f;
        acc[j] = 0.0f;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) qp[j] = lane + 64 * j < rope ? qrh[lane + 64 * j] * a.scale : 0.0f;
    float m = -INFINITY, l = 0.0f;
    for (int p = p0; p < p1; p += MLA_KU) {
        const int nk = min(MLA_KU, p1 - p);
        __syncthreads();
        for (int e = tid; e < nk * (kw / 8); e += ntg) {   // 8 dims at a time (r and rope: multiples of 8)
            const int u = e / (kw / 8), d = (e - u * (kw / 8)) * 8;
            int row;
            const KvSeg sg = kv_seg(kv, ri[t].kv0 + p + u, &row);
            float v[8];
            if (d < r) cache_get8(kv.fmt, sg.v, sg.vs, (size_t) row, r, d, v);
            else cache_get8(kv.fmt, sg.k, sg.ks, (size_t) row, rope, d - r, v);
            float* dst = sh + u * kw + d;
            *(float4*) dst = make_float4(v[0], v[1], v[2], v[3]);
            *(float4*) (dst + 4) = make_float4(v[4], v[5], v[6], v[7]);
        }
        __syncthreads();
        float s[MLA_KU];
        float mx = m;
#pragma unroll
        for (int u = 0; u < MLA_KU; ++u) {
            float d = 0.0f;
            if (u < nk) {
                const float* kk = sh + u * kw;
#pragma unroll
                for (int j = 0; j < MLA_MAXL; ++j)
                    if (j < nl && lane + 64 * j < r) d = fmaf(q[j], kk[lane + 64 * j], d);
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    if (lane + 64 * j < rope) d = fmaf(qp[j], kk[r + lane + 64 * j], d);
            }
            for (int o = 32; o > 0; o >>= 1) d += __shfl_xor(d, o);
            s[u] = u < nk ? d : -INFINITY;
            mx = fmaxf(mx, s[u]);
        }
        const float cor = expf(m - mx);
        l *= cor;
#pragma unroll
        for (int j = 0; j < MLA_MAXL; ++j) acc[j] *= cor;
#pragma unroll
        for (int u = 0; u < MLA_KU; ++u) {
            if (u >= nk) break;
            const float e = expf(s[u] - mx);
            l += e;
            const float* kk = sh + u * kw;
#pragma unroll
            for (int j = 0; j < MLA_MAXL; ++j)
                if (j < nl && lane + 64 * j < r) acc[j] = fmaf(e, kk[lane + 64 * j], acc[j]);
        }
        m = mx;
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
// Reduce the splits: olat[t][h][d] = bf16(acc / l).  Workgroup (head, row); threads stride d.
__global__ void __launch_bounds__(128) k_mla_reduce(MlaArgs a, const RowInfo* ri, const float* part, float* olat) {
    const int h = (int) blockIdx.x, t = (int) blockIdx.y, r = a.r, w = r + 2, ns = mla_row_splits(a, ri[t].pos);
    const float* pp = part + ((size_t) t * a.n_head + h) * a.n_splits * w;
    float m = -INFINITY;
    for (int s = 0; s < ns; ++s) m = fmaxf(m, pp[s * w]);
    for (int d = (int) (blockIdx.z * blockDim.x + threadIdx.x); d < r; d += (int) (gridDim.z * blockDim.x)) {
        float l = 0.0f, acc = 0.0f;
        for (int s = 0; s < ns; ++s) {
            const float ms = pp[s * w];
            if (ms == -INFINITY) continue;
            const float c = expf(ms - m);
            l = fmaf(pp[s * w + 1], c, l);
            acc = fmaf(pp[s * w + 2 + d], c, acc);
        }
        olat[((size_t) t * a.n_head + h) * r + d] = bfr(acc / l);
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
    const int nx = (a.n_head + 1) * (rope / 2) > a.r ? (a.n_head + 1) * (rope / 2) : a.r;
    hipLaunchKernelGGL(k_mla_rope, dim3((unsigned) (nx + 63) / 64, (unsigned) T), dim3(64), 0, (hipStream_t) s, a, rope, qr, kr, c, kv, ri, inv);
    host_note_launch();
}
void kc_mla_attn(kc_stream_t s, MlaArgs a, const float* ql, const float* qr, KvView kv, const RowInfo* ri, float* part, float* olat,
                 int T) {
    const int rope = rope_of(a);
    if (T < 1 || (kv.fmt != KV_BF16 && kv.fmt != KV_FP8) || (rope != 64 && rope != 128) || a.r % 8 || a.r > 64 * MLA_MAXL || a.n_splits < 1) {
        host_note_unsupported();
        return;
    }
    float* o = a.n_splits > 1 ? part : olat;
    if (a.n_head > 8)
        hipLaunchKernelGGL(k_mla_attn<16>, dim3((unsigned) a.n_splits, (unsigned) (a.n_head + 15) / 16, (unsigned) T), dim3(1024), 0, (hipStream_t) s,
                           a, rope, ql, qr, kv, ri, o);
    else
        hipLaunchKernelGGL(k_mla_attn<8>, dim3((unsigned) a.n_splits, 1, (unsigned) T), dim3(512), 0, (hipStream_t) s, a, rope, ql, qr, kv, ri, o);
    if (a.n_splits > 1)
        hipLaunchKernelGGL(k_mla_reduce, dim3((unsigned) a.n_head, (unsigned) T, (unsigned) (a.r + 127) / 128), dim3(128), 0, (hipStream_t) s, a, ri,
                           part, olat);
    host_note_launch();
}
void kc_kv_f32(kc_stream_t s, int fmt, const uint8_t* codes, const uint8_t* scales, int n, int rows, float* y) {
    if (rows < 1 || n < 8 || (fmt != KV_BF16 && fmt != KV_FP8)) { host_note_unsupported(); return; }
    hipLaunchKernelGGL(k_kv_f32, dim3((unsigned) ((n * rows / 8 + 127) / 128)), dim3(128), 0, (hipStream_t) s, fmt, codes, scales, n, rows, y);
    host_note_launch();
}

}   // extern "C"
