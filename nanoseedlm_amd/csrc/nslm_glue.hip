// nslm_glue.hip - the small kernels that sit either side of the seed matmuls in a full decode step: embedding rows,
// the two RMSNorm forms, greedy arg-max over the vocabulary.  They replace the reference's k_embed, k_gnorm
// (engine/kernels_moe.cu:676-713), k_argmax (:2115-2151) and k_q4_norm1p (engine/kernels_qwen4.cu:205-236) behind the same
// launchers.  All of them move a few hundred KB at most per token: what matters is one pass over the data with wide
// loads, 64-lane reductions and no second kernel.
#include "nslm_mv_dev.h"

using namespace nslm;

namespace {

// x[t][c] = the BF16 value of weight (ids[t], c): BF16 rows as stored, Q8 / Q4 as bf16(s q + b), seed rows as the
// BF16-rounded exact weight.  One thread per 8-weight block.
__global__ void __launch_bounds__(256) k_embed(int fmt, WSlice w, int d, const int32_t* ids, float* x) {
    __shared__ uint32_t tab[NSLM_TAB_WORDS];
    const bool seedf = fmt == MF_SEED4P4 || fmt == MF_SEED4;
    if (seedf) {
        load_tables(tab);
        __syncthreads();
    }
    const int j = (int) (blockIdx.x * 256 + threadIdx.x), t = (int) blockIdx.y;
    if (j >= d / 8) return;
    const int row = ids[t];
    float o[8], sc;
    if (fmt == MF_Q4) {   // block_weights gives Q4 in the unrounded matvec form; the embedding is the dequantized value
        const size_t e0 = (size_t) row * d + (size_t) j * 8, gi = e0 >> group_shift(w);
        const float s = bf(gp<uint16_t>(w.p[1])[gi]), b = bf(gp<uint16_t>(w.p[2])[gi]);
        const uint32_t q = gp<uint32_t>(w.p[0])[e0 / 8];
#pragma unroll
        for (int c = 0; c < 8; ++c) o[c] = bfr(s * (float) ((q >> (4 * c)) & 15u) + b);
        sc = 1.0f;
    } else {
        block_weights(fmt, w, tab, row, d, j, o, &sc);
    }
    float* xo = x + (size_t) t * d + (size_t) j * 8;
#pragma unroll
    for (int c = 0; c < 8; ++c) xo[c] = seedf ? bfr(o[c] * sc) : o[c];
}


// One workgroup per (token, group): y = f(x * rsqrt(mean_group(x^2) + eps), w).  The group's values stay in registers
// between the sum and the scaling when the group is at most 256 * NR long; longer groups read x twice.
// MODE 0: the MoVA grouped norm, BF16 weights, y = bf16(w * (x * r));  MODE 1: the Qwen form, f32 weights, y = x r (1 + w).
#define NR NSLM_NORM_NR
template <int MODE>
__global__ void __launch_bounds__(256) k_rmsnorm(const float* x, int len, int g, const void* wv, float eps, float* y) {
    __shared__ float red[4];
    const int groups = len / g, t = (int) blockIdx.x / groups, a = ((int) blockIdx.x % groups) * g, tid = threadIdx.x;
    const float* xi = x + (size_t) t * len + a;
    float* yi = y + (size_t) t * len + a;
    auto out = [&](int k, float v, float r) {
        if (MODE == 0) yi[k] = bfr(bf(((const uint16_t*) wv)[a + k]) * (v * r));
        else yi[k] = v * r * (1.0f + ((const float*) wv)[a + k]);
    };
    if (g <= 256 * NSLM_NORM_NR) {
        float v[NR], ss = 0.0f;
#pragma unroll
        for (int j = 0; j < NR; ++j) {
            const int k = tid + j * 256;
            v[j] = k < g ? xi[k] : 0.0f;
            ss = fmaf(v[j], v[j], ss);
        }
        const float r = rsqrtf(wg_sum(ss, red) / (float) g + eps);
#pragma unroll
        for (int j = 0; j < NR; ++j)
            if (tid + j * 256 < g) out(tid + j * 256, v[j], r);
    } else {
        float ss = 0.0f;
        for (int k = tid; k < g; k += 256) ss = fmaf(xi[k], xi[k], ss);
        const float r = rsqrtf(wg_sum(ss, red) / (float) g + eps);
        for (int k = tid; k < g; k += 256) out(k, xi[k], r);
    }
}

// Greedy arg-max of row t (ties: the lowest index; NaNs never win), optionally with its softmax probability
// 1 / sum exp(l - max).  One workgroup of 1024 per row, 16-byte loads where the row allows them.
__device__ __forceinline__ void take(float v, int i, float& best, int& idx) {
    if (v > best || (v == best && i < idx)) { best = v; idx = i; }
}
__global__ void __launch_bounds__(1024) k_argmax(const float* logits, int32_t* out, float* prob, int V) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    const int t = (int) blockIdx.x, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const float* l = logits + (size_t) t * V;
    const bool vec = (((uintptr_t) l) & 15u) == 0;
    const int V4 = vec ? V / 4 : 0;
    float best = -INFINITY;
    int idx = V;   // "nothing yet": any real index is lower
    // eight loads a thread are requested before the first is compared (clamped indices, so they are unconditional): one
    // workgroup reads the whole row, and a load a round trip was 25 us for 152 k logits
    for (int i0 = tid; i0 < V4; i0 += 8 * 1024) {
        float4 q[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) q[u] = ((const float4*) l)[min(i0 + u * 1024, V4 - 1)];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = i0 + u * 1024;
            if (i < V4) {
                take(q[u].x, 4 * i, best, idx);
                take(q[u].y, 4 * i + 1, best, idx);
                take(q[u].z, 4 * i + 2, best, idx);
                take(q[u].w, 4 * i + 3, best, idx);
            }
        }
    }
    for (int i = 4 * V4 + tid; i < V; i += 1024) take(l[i], i, best, idx);
    for (int o = 32; o > 0; o >>= 1) take(__shfl_xor(best, o), __shfl_xor(idx, o), best, idx);
    if (lane == 0) { bv[wv] = best; bi[wv] = idx; }
    __syncthreads();
    best = bv[0];
    idx = bi[0];
#pragma unroll
    for (int s = 1; s < 16; ++s) take(bv[s], bi[s], best, idx);
    if (idx >= V) idx = 0;   // a row of NaNs or -inf: the reference answers 0
    if (tid == 0) out[t] = idx;
    if (!prob) return;
    float s = 0.0f;
    for (int i = tid; i < V4; i += 1024) {
        const float4 q = ((const float4*) l)[i];
        s += __expf(q.x - best) + __expf(q.y - best) + __expf(q.z - best) + __expf(q.w - best);
    }
    for (int i = 4 * V4 + tid; i < V; i += 1024) s += __expf(l[i] - best);
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
    __syncthreads();   // every thread has read bv
    if (lane == 0) bv[wv] = s;
    __syncthreads();
    if (tid == 0) {
        float tot = 0.0f;
        for (int w = 0; w < 16; ++w) tot += bv[w];
        prob[t] = 1.0f / tot;
    }
}

// ---- what a host that runs a whole synthetic model needs beside the reference's kernels ---------------------------------
// x = bf16(x + bf16(a + b)): the residual stream takes a block's two branch outputs, BF16 at the tensor boundary as the
// MoVA engine keeps it (engine/kernels_moe.cu:780-788 does the same for its expert sum + shared expert)
__global__ void __launch_bounds__(256) k_residual_add(float* x, const float* a, const float* b, size_t n) {
    const size_t i = (size_t) blockIdx.x * 256 + threadIdx.x;
    if (i < n) x[i] = bfr(x[i] + bfr(a[i] + (b ? b[i] : 0.0f)));
}
__global__ void k_rows_advance(RowInfo* ri, int T) {
    const int t = (int) (blockIdx.x * blockDim.x + threadIdx.x);
    if (t < T) {   // pad[0] > 0: the sequence slot's length; a row on its last position stays there (the cache write stays inside the slot)
        const int lim = ri[t].pad[0], nxt = ri[t].pos + 1;
        ri[t].pos = lim > 0 && nxt >= lim ? lim - 1 : nxt;
    }
}
// splitmix64 of the word index: reproducible pseudo-random bytes for synthetic packs (any bytes are valid seed records)
__device__ __forceinline__ uint64_t mix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
__global__ void __launch_bounds__(256) k_fill_random(uint64_t* p, size_t nwords, uint64_t seed) {
    for (size_t i = (size_t) blockIdx.x * 256 + threadIdx.x; i < nwords; i += (size_t) gridDim.x * 256) p[i] = mix64(seed ^ (i * 0xD1342543DE82EF95ull));
}
// Random E4M3 codes as the cache's encoder can write them: it saturates at 0x7E, so the all-ones magnitude never occurs
__global__ void __launch_bounds__(256) k_fill_fp8_codes(uint64_t* p, size_t nwords, uint64_t seed) {
    for (size_t i = (size_t) blockIdx.x * 256 + threadIdx.x; i < nwords; i += (size_t) gridDim.x * 256) {
        const uint64_t x = mix64(seed ^ (i * 0xD1342543DE82EF95ull));
        const uint64_t ones = ((x & 0x7F7F7F7F7F7F7F7Full) + 0x0101010101010101ull) & 0x8080808080808080ull;
        p[i] = x & ~(ones >> 7);
    }
}
// BF16 values uniform in [-scale, scale]
__global__ void __launch_bounds__(256) k_fill_bf16(uint16_t* p, size_t n, uint64_t seed, float scale) {
    for (size_t i = (size_t) blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t) gridDim.x * 256) {
        const uint32_t u = (uint32_t) (mix64(seed ^ (i * 0xD1342543DE82EF95ull)) >> 40);   // 24 bits
        p[i] = (uint16_t) tobf(((float) u * (1.0f / 8388608.0f) - 1.0f) * scale);
    }
}

}   // namespace

extern "C" {

void kc_residual_add(kc_stream_t s, float* x, const float* a, const float* b, size_t n) {
    if (!n) return;
    hipLaunchKernelGGL(k_residual_add, dim3((unsigned) ((n + 255) / 256)), dim3(256), 0, (hipStream_t) s, x, a, b, n);
    host_note_launch();
}
void kc_rows_advance(kc_stream_t s, RowInfo* ri, int T) {
    if (T < 1) return;
    hipLaunchKernelGGL(k_rows_advance, dim3((unsigned) (T + 63) / 64), dim3(64), 0, (hipStream_t) s, ri, T);
    host_note_launch();
}
void kc_fill_random(kc_stream_t s, void* p, size_t nbytes, uint64_t seed) {
    if (nbytes < 8) return;
    hipLaunchKernelGGL(k_fill_random, dim3(2048), dim3(256), 0, (hipStream_t) s, (uint64_t*) p, nbytes / 8, seed);
    host_note_launch();
}
void kc_fill_fp8_codes(kc_stream_t s, void* p, size_t nbytes, uint64_t seed) {
    if (nbytes < 8) return;
    hipLaunchKernelGGL(k_fill_fp8_codes, dim3(2048), dim3(256), 0, (hipStream_t) s, (uint64_t*) p, nbytes / 8, seed);
    host_note_launch();
}
void kc_fill_bf16(kc_stream_t s, uint16_t* p, size_t n, uint64_t seed, float scale) {
    if (!n) return;
    hipLaunchKernelGGL(k_fill_bf16, dim3(2048), dim3(256), 0, (hipStream_t) s, p, n, seed, scale);
    host_note_launch();
}

void kc_embed(kc_stream_t s, int fmt, WSlice w, int d, const int32_t* ids, float* x, int T) {
    if (T < 1 || d < 8) return;
    hipLaunchKernelGGL(k_embed, dim3((unsigned) (d / 8 + 255) / 256, (unsigned) T), dim3(256), 0, (hipStream_t) s, fmt, w, d, ids, x);
    host_note_launch();
}
void kc_gnorm(kc_stream_t s, int d, float eps, const float* x, const uint16_t* w, float* y, int T) {
    if (T < 1 || d < 2) return;
    hipLaunchKernelGGL(k_rmsnorm<0>, dim3((unsigned) (2 * T)), dim3(256), 0, (hipStream_t) s, x, d, d / 2, (const void*) w, eps, y);
    host_note_launch();
}
void kq4_norm1p(kc_stream_t s, const float* x, int len, int g, const float* w, float eps, float* y, int T) {
    if (T < 1 || g < 1 || len < g) return;
    hipLaunchKernelGGL(k_rmsnorm<1>, dim3((unsigned) (T * (len / g))), dim3(256), 0, (hipStream_t) s, x, len, g, (const void*) w, eps, y);
    host_note_launch();
}
void kc_argmax(kc_stream_t s, const float* logits, int32_t* out, int V, int n) {
    if (n < 1 || V < 1) return;
    hipLaunchKernelGGL(k_argmax, dim3((unsigned) n), dim3(1024), 0, (hipStream_t) s, logits, out, (float*) nullptr, V);
    host_note_launch();
}
void kc_argmax_p(kc_stream_t s, const float* logits, int32_t* out, float* prob, int V, int n) {
    if (n < 1 || V < 1) return;
    hipLaunchKernelGGL(k_argmax, dim3((unsigned) n), dim3(1024), 0, (hipStream_t) s, logits, out, prob, V);
    host_note_launch();
}

}   // extern "C"
