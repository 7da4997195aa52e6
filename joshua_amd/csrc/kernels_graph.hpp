// The non-matmul pieces of the dense Qwen3 decoder layer, in f32 as the
// reference runs them: RMSNorm, per-head Q/K RMSNorm + half-split RoPE, KV-cache
// append, grouped-query attention over the cache, SwiGLU, residual add, argmax
// (reference: src/embedding.rs:297-396, src/quantized_qwen3_moe.rs:231-386,776-819).
#pragma once
#include "kernels_moe.hpp"

namespace jq {

__device__ __forceinline__ float block_sum(float v, float *red) {  // blockDim.x <= 1024
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float t = 0.0f;
    for (int i = 0; i < nw; i++) t += red[i];
    return t;
}

// out[r, :] = x[r, :] / sqrt(mean(x[r, :]^2) + eps) * w   (+ res[r, :] first when given:
// the sum is also written to res_out so the residual stream stays materialised)
__global__ __launch_bounds__(256) void rmsnorm_rows(const float *__restrict__ x, const float *__restrict__ w, float eps,
                                                     float *__restrict__ out, int h) {
    __shared__ float red[16];
    const float *xr = x + (size_t)blockIdx.x * h;
    float ss = 0.0f;
    for (int c = threadIdx.x; c < h; c += blockDim.x) ss = fmaf(xr[c], xr[c], ss);
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)h + eps);
    for (int c = threadIdx.x; c < h; c += blockDim.x) out[(size_t)blockIdx.x * h + c] = xr[c] * inv * w[c];
}

// Per-head RMSNorm over head_dim, then half-split rotary embedding at position
// pos0 + t; one wave per (token, head).  v: [T, n_heads*d] in place.
// inv_freq_i = theta^(-2i/d); pairs (i, i + d/2)
// (reference: src/quantized_qwen3_moe.rs:237-262,345-354; closed form in its test :867-895).
__global__ __launch_bounds__(64) void headnorm_rope(float *__restrict__ v, const float *__restrict__ w, float eps,
                                                     int n_heads, int d, int pos0, float theta) {
    const int t = blockIdx.x / n_heads, hd = blockIdx.x % n_heads, lane = threadIdx.x;
    float *p = v + ((size_t)t * n_heads + hd) * d;
    float ss = 0.0f;
    for (int c = lane; c < d; c += 64) ss = fmaf(p[c], p[c], ss);
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
    const int half = d / 2;
    const float pos = (float)(pos0 + t);
    for (int i = lane; i < half; i += 64) {
        const float a = p[i] * inv * w[i], b = p[i + half] * inv * w[i + half];
        const float freq = 1.0f / powf(theta, (float)(2 * i) / (float)d);
        const float ang = pos * freq, c = cosf(ang), s = sinf(ang);
        p[i] = a * c - b * s;
        p[i + half] = a * s + b * c;
    }
}

// cache[kvh, pos0 + t, :] = src[t, kvh*d .. +d]
__global__ __launch_bounds__(256) void kv_append(const float *__restrict__ src, float *__restrict__ cache, int T,
                                                  int n_kv, int d, int pos0, int n_ctx) {
    const size_t total = (size_t)T * n_kv * d;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const int c = (int)(i % d), kvh = (int)((i / d) % n_kv), t = (int)(i / ((size_t)d * n_kv));
        cache[((size_t)kvh * n_ctx + pos0 + t) * d + c] = src[i];
    }
}

// One workgroup per (token, query head): softmax(q . K^T / sqrt(d)) . V over the
// keys 0 .. pos0 + t (causal), K/V of head hq / (n_head / n_kv)
// (reference: src/quantized_qwen3_moe.rs:366-379; mask :776-789).
__global__ __launch_bounds__(256) void attention_rows(const float *__restrict__ q, const float *__restrict__ kc,
                                                       const float *__restrict__ vc, float *__restrict__ out,
                                                       int n_head, int n_kv, int d, int pos0, int n_ctx, float sqrt_d) {
    extern __shared__ float sm[];  // q[d], scores[n_keys], red[16]
    const int t = blockIdx.x / n_head, hq = blockIdx.x % n_head;
    const int kvh = hq / (n_head / n_kv), n_keys = pos0 + t + 1;
    float *qs = sm, *sc = sm + d, *red = sm + d + n_keys;
    const float *qp = q + ((size_t)t * n_head + hq) * d;
    for (int c = threadIdx.x; c < d; c += blockDim.x) qs[c] = qp[c];
    __syncthreads();
    const float *kb = kc + (size_t)kvh * n_ctx * d;
    float mx = -INFINITY;
    for (int j = threadIdx.x; j < n_keys; j += blockDim.x) {
        const float *kr = kb + (size_t)j * d;
        float acc = 0.0f;
        for (int c = 0; c < d; c += 4) {
            const float4 kv = ld<float4>((const uint8_t *)(kr + c));
            acc = fmaf(qs[c], kv.x, acc);
            acc = fmaf(qs[c + 1], kv.y, acc);
            acc = fmaf(qs[c + 2], kv.z, acc);
            acc = fmaf(qs[c + 3], kv.w, acc);
        }
        acc = acc / sqrt_d;  // the reference divides by sqrt(head_dim) (src/embedding.rs:386)
        sc[j] = acc;
        mx = fmaxf(mx, acc);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
    __syncthreads();
    for (int i = 0; i < (int)(blockDim.x >> 6); i++) mx = fmaxf(mx, red[i]);
    float sum = 0.0f;
    for (int j = threadIdx.x; j < n_keys; j += blockDim.x) {
        const float e = expf(sc[j] - mx);
        sc[j] = e;
        sum += e;
    }
    sum = block_sum(sum, red);
    for (int j = threadIdx.x; j < n_keys; j += blockDim.x) sc[j] = sc[j] / sum;
    __syncthreads();
    const float *vb = vc + (size_t)kvh * n_ctx * d;
    for (int c = threadIdx.x; c < d; c += blockDim.x) {
        float acc = 0.0f;
        for (int j = 0; j < n_keys; j++) acc = fmaf(sc[j], vb[(size_t)j * d + c], acc);
        out[((size_t)t * n_head + hq) * d + c] = acc;
    }
}

__global__ __launch_bounds__(256) void add_rows(const float *__restrict__ a, const float *__restrict__ b,
                                                 float *__restrict__ out, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
        out[i] = a[i] + b[i];
}

// Index of the largest value; of equal values the LAST one, as the reference's
// greedy pick does (Iterator::max_by, src/engine.rs:2371-2378).  One workgroup.
__global__ __launch_bounds__(1024) void argmax_last(const float *__restrict__ v, int n, uint32_t *__restrict__ out) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    float best = -INFINITY;
    int idx = -1;
    for (int i = threadIdx.x; i < n; i += blockDim.x)
        if (v[i] >= best) {  // i increases within a thread: >= keeps the last
            best = v[i];
            idx = i;
        }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ob = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(idx, off, 64);
        if (ob > best || (ob == best && oi > idx)) {
            best = ob;
            idx = oi;
        }
    }
    if ((threadIdx.x & 63) == 0) {
        bv[threadIdx.x >> 6] = best;
        bi[threadIdx.x >> 6] = idx;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < (int)(blockDim.x >> 6); i++)
            if (bv[i] > best || (bv[i] == best && bi[i] > idx)) {
                best = bv[i];
                idx = bi[i];
            }
        out[0] = (uint32_t)(idx < 0 ? 0 : idx);
    }
}

}  // namespace jq
