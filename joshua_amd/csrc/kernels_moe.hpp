// Mixture-of-experts layer kernels: router, gating + top-k, grouping of the
// routed (token, slot) pairs by expert, expert matmuls over the groups, and the
// weighted combine.  Everything stays on the device: the reference's one host
// sync per layer (reading the k expert ids back,
// src/quantized_qwen3_moe.rs:511) has no counterpart here.
#pragma once
#include "kernels_valu.hpp"

namespace jq {

// logits[t, e] = x[t, :] . router[e, :]   (reference: src/quantized_qwen3_moe.rs:425,
// src/quantized_deepseek2.rs:528; an f32 matmul there too)
__global__ __launch_bounds__(256) void moe_router_logits(const float *__restrict__ Wr, const float *__restrict__ X,
                                                          float *__restrict__ logits, int T, int h, int E) {
    const int lane = threadIdx.x & 63;
    const int e = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (e >= E) return;
    const float *wr = Wr + (size_t)e * h;
    for (int t0 = 0; t0 < T; t0 += 4) {
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        for (int c = lane * 4; c < h; c += 256) {
            const float4 w = ld<float4>((const uint8_t *)(wr + c));
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if (t0 + i < T) {
                    const float4 x = ld<float4>((const uint8_t *)(X + (size_t)(t0 + i) * h + c));
                    acc[i] = fmaf(x.x, w.x, acc[i]);
                    acc[i] = fmaf(x.y, w.y, acc[i]);
                    acc[i] = fmaf(x.z, w.z, acc[i]);
                    acc[i] = fmaf(x.w, w.w, acc[i]);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float s = wave_sum(acc[i]);
            if (lane == 0 && t0 + i < T) logits[(size_t)(t0 + i) * E + e] = s;
        }
    }
}

struct MoeGateParams {
    int E, k_used;
    int sigmoid;      // 0: softmax over experts, 1: sigmoid per expert
    int norm_topk;    // divide the k weights by their sum (clamped below at 2^-14)
    float scale;      // multiply the weights (0 or 1: leave alone)
    int n_group, topk_group;
};

// One wave per token: probabilities, selection scores (bias, group limit),
// the k best experts in descending score order and their weights
// (reference: src/quantized_qwen3_moe.rs:424-436, src/quantized_deepseek2.rs:527-551,563-597).
// Equal scores are ordered by expert index (the reference's sort order on ties
// is that of a third-party argsort and is not pinned).
__global__ __launch_bounds__(64) void moe_gate_topk(const float *__restrict__ logits, const float *__restrict__ bias,
                                                     MoeGateParams p, uint32_t *__restrict__ ids,
                                                     float *__restrict__ wts) {
    extern __shared__ float sm[];  // probs[E], sel[E], gscore[n_group]
    float *probs = sm, *sel = sm + p.E, *gscore = sm + 2 * p.E;
    const int t = blockIdx.x, lane = threadIdx.x;
    const float *lg = logits + (size_t)t * p.E;
    if (p.sigmoid) {
        for (int e = lane; e < p.E; e += 64) probs[e] = 1.0f / (1.0f + expf(-lg[e]));
    } else {
        float mx = -INFINITY;
        for (int e = lane; e < p.E; e += 64) mx = fmaxf(mx, lg[e]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        float sum = 0.0f;
        for (int e = lane; e < p.E; e += 64) {
            const float v = expf(lg[e] - mx);
            probs[e] = v;
            sum += v;
        }
        sum = wave_sum(sum);
        for (int e = lane; e < p.E; e += 64) probs[e] = probs[e] / sum;
    }
    for (int e = lane; e < p.E; e += 64) sel[e] = probs[e] + (bias ? bias[e] : 0.0f);
    __syncthreads();
    if (p.n_group > 1) {
        const int per = p.E / p.n_group;
        for (int g = lane; g < p.n_group; g += 64) {
            float b1 = -INFINITY, b2 = -INFINITY;  // two best of the group
            for (int i = 0; i < per; i++) {
                const float v = sel[g * per + i];
                if (v > b1) {
                    b2 = b1;
                    b1 = v;
                } else if (v > b2) {
                    b2 = v;
                }
            }
            gscore[g] = p.sigmoid ? b1 + b2 : b1;
        }
        __syncthreads();
        for (int e = lane; e < p.E; e += 64) {
            const int g = e / per;
            int rank = 0;
            for (int o = 0; o < p.n_group; o++) rank += gscore[o] > gscore[g] || (gscore[o] == gscore[g] && o < g);
            // selection + (mask*1e30 - 1e30): unchanged inside the kept groups
            if (rank >= p.topk_group) sel[e] = sel[e] + (0.0f * 1e30f - 1e30f);
        }
        __syncthreads();
    }
    for (int e = lane; e < p.E; e += 64) {
        const float v = sel[e];
        int rank = 0;
        for (int o = 0; o < p.E; o++) rank += sel[o] > v || (sel[o] == v && o < e);
        if (rank < p.k_used) {
            ids[(size_t)t * p.k_used + rank] = (uint32_t)e;
            wts[(size_t)t * p.k_used + rank] = probs[e];
        }
    }
    __syncthreads();
    if (lane == 0) {
        float *w = wts + (size_t)t * p.k_used;
        if (p.norm_topk) {
            float s = 0.0f;
            for (int i = 0; i < p.k_used; i++) s += w[i];
            s = fmaxf(s, 6.103515625e-5f);
            for (int i = 0; i < p.k_used; i++) w[i] = w[i] / s;
        }
        if (p.scale != 0.0f && p.scale != 1.0f)
            for (int i = 0; i < p.k_used; i++) w[i] = w[i] * p.scale;
    }
}

// Groups the T*k routed (token, slot) pairs by expert, keeping pair order inside
// a group (the reference buckets the same way on the host,
// src/quantized_qwen3_moe.rs:459-480).  Group e is expert e:
//   offsets[e] .. offsets[e+1]  positions of the expert's pairs
//   xrow[pos]  activation row (token) of the pair,  yrow[pos]  the pair index
__global__ __launch_bounds__(256) void moe_group_pairs(const uint32_t *__restrict__ ids, int T, int k_used, int E,
                                                       int *__restrict__ gexp, int *__restrict__ offsets,
                                                       int *__restrict__ xrow, int *__restrict__ yrow) {
    extern __shared__ int cnt[];  // [E + 1]
    const int P = T * k_used;
    for (int e = threadIdx.x; e <= E; e += blockDim.x) cnt[e] = 0;
    __syncthreads();
    for (int pidx = threadIdx.x; pidx < P; pidx += blockDim.x) {
        const uint32_t e = ids[pidx];
        if (e < (uint32_t)E) atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int run = 0;
        for (int e = 0; e < E; e++) {
            const int c = cnt[e];
            cnt[e] = run;
            run += c;
        }
        cnt[E] = run;
    }
    __syncthreads();
    for (int e = threadIdx.x; e <= E; e += blockDim.x) offsets[e] = cnt[e];
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        gexp[e] = e;
        int pos = cnt[e];
        for (int pidx = 0; pidx < P; pidx++) {
            if (ids[pidx] == (uint32_t)e) {
                xrow[pos] = pidx / k_used;
                yrow[pos] = pidx;
                pos++;
            }
        }
    }
}

// Few pairs (decode): every pair is its own group, its expert read from ids.
__global__ __launch_bounds__(256) void moe_pairs_as_groups(const uint32_t *__restrict__ ids, int P, int k_used,
                                                           int *__restrict__ gexp, int *__restrict__ offsets,
                                                           int *__restrict__ xrow, int *__restrict__ yrow) {
    for (int pidx = threadIdx.x; pidx <= P; pidx += blockDim.x) {
        offsets[pidx] = pidx;
        if (pidx < P) {
            gexp[pidx] = (int)ids[pidx];
            xrow[pidx] = pidx / k_used;
            yrow[pidx] = pidx;
        }
    }
}

__device__ __forceinline__ float silu(float v) { return v / (1.0f + expf(-v)); }

// Expert matmuls over the grouped pairs: blockIdx.y = group (its expert is
// gexp[group]), rows of the expert's weight over blockIdx.x.  The activation row of the pair at sorted
// position pos is X[xsel[pos]]; with SWIGLU it is silu(X[...]) * X2[...]
// (reference: src/quantized_qwen3_moe.rs:397-401).  Results go to Y[yrow[pos]].
template <class Q, int MT, bool SWIGLU>
__global__ __launch_bounds__(64 * ROWS_PER_WG) void moe_rows_valu(const uint8_t *const *__restrict__ Wptr,
                                                                   size_t row_bytes, const float *__restrict__ X,
                                                                   const float *__restrict__ X2,
                                                                   const int *__restrict__ gexp,
                                                                   const int *__restrict__ offsets,
                                                                   const int *__restrict__ xsel,
                                                                   const int *__restrict__ yrow,
                                                                   float *__restrict__ Y, int k, int n) {
    const int grp = blockIdx.y;
    const int beg = offsets[grp], cnt = offsets[grp + 1] - beg;
    if (cnt == 0) return;
    const int e = gexp[grp];
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * ROWS_PER_WG + (threadIdx.x >> 6);
    if (row >= n) return;
    const uint8_t *rp = Wptr[e] + (size_t)row * row_bytes;
    const int units = (k / Q::BLOCK_ELEMS) * Q::UNITS;
    constexpr int UE = Q::SEGS * Q::SEGLEN;
    for (int m0 = 0; m0 < cnt; m0 += MT) {
        float acc[MT];
        int xr[MT];
#pragma unroll
        for (int i = 0; i < MT; i++) {
            acc[i] = 0.0f;
            xr[i] = xsel[beg + min(m0 + i, cnt - 1)];
        }
        for (int u = lane; u < units; u += 64) {
            const int b = u / Q::UNITS, ub = u % Q::UNITS;
            float w[UE];
            Q::decode(rp + (size_t)b * Q::BLOCK_BYTES, ub, w);
            const int xoff = b * Q::BLOCK_ELEMS + Q::elem_base(ub);
#pragma unroll
            for (int i = 0; i < MT; i++) {
                if (m0 + i < cnt) {
                    const float *xp = X + (size_t)xr[i] * k + xoff;
                    const float *xp2 = SWIGLU ? X2 + (size_t)xr[i] * k + xoff : nullptr;
#pragma unroll
                    for (int s = 0; s < Q::SEGS; s++) {
#pragma unroll
                        for (int el = 0; el < Q::SEGLEN; el += 4) {
                            float4 xv = ld<float4>((const uint8_t *)(xp + s * Q::SEG_STRIDE + el));
                            if (SWIGLU) {
                                const float4 uv = ld<float4>((const uint8_t *)(xp2 + s * Q::SEG_STRIDE + el));
                                xv = float4{silu(xv.x) * uv.x, silu(xv.y) * uv.y, silu(xv.z) * uv.z, silu(xv.w) * uv.w};
                            }
                            acc[i] = fmaf(xv.x, w[s * Q::SEGLEN + el + 0], acc[i]);
                            acc[i] = fmaf(xv.y, w[s * Q::SEGLEN + el + 1], acc[i]);
                            acc[i] = fmaf(xv.z, w[s * Q::SEGLEN + el + 2], acc[i]);
                            acc[i] = fmaf(xv.w, w[s * Q::SEGLEN + el + 3], acc[i]);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < MT; i++) {
            const float s = wave_sum(acc[i]);
            if (lane == 0 && m0 + i < cnt) Y[(size_t)yrow[beg + m0 + i] * n + row] = s;
        }
    }
}

// y[t, :] = sum_s w[t, s] * out[t*k + s, :]  (+ shared_out[t, :] of the shared expert),
// slots added in order s = 0..k-1 (reference: src/quantized_qwen3_moe.rs:516-518,
// src/quantized_deepseek2.rs:553-557).
__global__ __launch_bounds__(256) void moe_combine(const float *__restrict__ out, const float *__restrict__ wts, int T,
                                                    int k_used, int h, const float *__restrict__ shared_out,
                                                    float *__restrict__ y) {
    const size_t total = (size_t)T * h;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t t = i / h, c = i % h;
        float acc = 0.0f;
        for (int s = 0; s < k_used; s++) acc += out[(t * k_used + s) * h + c] * wts[t * k_used + s];
        if (shared_out) acc += shared_out[i];
        y[i] = acc;
    }
}

}  // namespace jq

namespace jq {

// h[i] = silu(g[i]) * u[i]  (the shared expert's activation)
__global__ __launch_bounds__(256) void swiglu_rows(const float *__restrict__ g, const float *__restrict__ u,
                                                    float *__restrict__ h, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
        h[i] = silu(g[i]) * u[i];
}

}  // namespace jq
