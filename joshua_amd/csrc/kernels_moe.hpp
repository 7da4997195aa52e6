// Mixture-of-experts layer kernels: router, gating + top-k, grouping of the
// routed (token, slot) pairs by expert, expert matmuls over the groups, and the
// weighted combine.  Everything stays on the device: the reference's one host
// sync per layer (reading the k expert ids back,
// src/quantized_qwen3_moe.rs:511) has no counterpart here.
#pragma once
#include "kernels_valu.hpp"

namespace jq {

// Activations as 15-bit fixed point per 32-element block, two int8 planes (X = 256 hi + lo) and the
// block's scale: what the formats with an integer dot product (Q::dot8) multiply against.
struct ActsI8 {
    uint32_t *xl, *xh;  // [rows][k / 4]: four elements a word
    float *sx, *sxs;    // [rows][k / 32]: the block's scale, and scale * sum of its fixed-point values
};

// Elements 4 i .. 4 i + 3 of X: eight consecutive lanes (i a multiple of 8 in the first) make one block of 32.
__device__ __forceinline__ void acts_i8_quantize(const float *__restrict__ X, size_t i, const ActsI8 &out) {
    const float4 v = *(const float4 *)(X + 4 * i);
    float amax = fmaxf(fmaxf(mag_or_inf(v.x), mag_or_inf(v.y)), fmaxf(mag_or_inf(v.z), mag_or_inf(v.w)));
    amax = max_row8(amax);
    const bool live = amax > 0.0f && amax < INFINITY;
    const float inv = live ? 32639.0f / amax : 0.0f;
    const int Xq[4] = {__float2int_rn(v.x * inv), __float2int_rn(v.y * inv), __float2int_rn(v.z * inv),
                       __float2int_rn(v.w * inv)};
    uint32_t wl = 0, wh = 0;
    int sum = 0;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int lo = ((Xq[e] + 128) & 255) - 128, hi = (Xq[e] - lo) >> 8;
        wl |= (uint32_t)(lo & 255) << (8 * e);
        wh |= (uint32_t)(hi & 255) << (8 * e);
        sum += Xq[e];
    }
    out.xl[i] = wl;
    out.xh[i] = wh;
    sum = isum_row8(sum);
    if ((i & 7) == 0) {
        const float s = fixed_scale(amax, 32639.0f);
        out.sx[i >> 3] = s;
        out.sxs[i >> 3] = s * (float)sum;
    }
}

// logits[t, e] = x[t, :] . router[e, :]   (reference: src/quantized_qwen3_moe.rs:425,
// src/quantized_deepseek2.rs:528; an f32 matmul there too)
constexpr int ROUTER_TOKENS_PER_WG = 8;

__device__ __forceinline__ void moe_router_logits_body(const float *__restrict__ Wr, const float *__restrict__ X,
                                                       float *__restrict__ logits, int T, int h, int E, ActsI8 planes) {
    // one workgroup per (expert row of the router, run of 8 tokens): every load of the row in
    // flight at once; a logit's arithmetic does not depend on how the tokens are split
    __shared__ float red[4][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, e = blockIdx.x;
    const float *wr = Wr + (size_t)e * h;
    const int t_begin = blockIdx.y * ROUTER_TOKENS_PER_WG, t_end = min(T, t_begin + ROUTER_TOKENS_PER_WG);
    // With `planes` (h a multiple of 32): the tokens' activations as fixed-point planes for the expert kernels
    // that follow, one launch less.  Workgroup e makes blocks e, e + E, .. of its tokens: eight lanes a block.
    if (planes.xl && (int)threadIdx.x < 8 * (t_end - t_begin)) {
        const size_t t = (size_t)t_begin + (threadIdx.x >> 3);
        for (int b = e; b < h / 32; b += E) acts_i8_quantize(X, t * (size_t)(h / 4) + 8 * b + (threadIdx.x & 7), planes);
    }
    for (int t0 = t_begin; t0 < t_end; t0 += 4) {
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        for (int c = threadIdx.x * 4; c < h; c += 1024) {
            const float4 w = ld<float4>((const uint8_t *)(wr + c));
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if (t0 + i < t_end) {
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
            if (lane == 0) red[wave][i] = s;
        }
        __syncthreads();
        if (threadIdx.x < 4 && t0 + threadIdx.x < t_end)
            logits[(size_t)(t0 + threadIdx.x) * E + e] =
                (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
        __syncthreads();
    }
}

__global__ __launch_bounds__(256) void moe_router_logits(const float *__restrict__ Wr, const float *__restrict__ X,
                                                          float *__restrict__ logits, int T, int h, int E, ActsI8 planes) {
    moe_router_logits_body(Wr, X, logits, T, h, E, planes);
}

// The router's logits of ONE token with the decoder layer's residual add and RMSNorm in front
// (reference: src/quantized_qwen3_moe.rs:806-812: x + moe(norm(x))), a launch less: every workgroup adds res to x and
// normalises the row for itself (h floats, read twice, the second time from cache), workgroup 0 stores x + res to
// x_out (a buffer other than x: the others are still reading x) and the normalised row to hn_out, where the expert
// kernels behind this launch read it.  Column c of the row goes to the thread that takes it in moe_router_logits, and
// the logit is accumulated and reduced in the same order, so given the same normalised row the two give the same bits.
struct MoePreNormArgs {
    const float *x, *res, *w;
    float eps;
    float *x_out, *hn_out;
};

__global__ __launch_bounds__(256) void moe_router_logits_norm(const float *__restrict__ Wr, MoePreNormArgs nm,
                                                               float *__restrict__ logits, int h, int E) {
    __shared__ float red[2][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, e = blockIdx.x;
    const float *wr = Wr + (size_t)e * h;
    float ss = 0.0f;
    for (int c = threadIdx.x * 4; c < h; c += 1024) {
        float4 v = ld<float4>((const uint8_t *)(nm.x + c));
        if (nm.res) {
            const float4 r = ld<float4>((const uint8_t *)(nm.res + c));
            v.x += r.x, v.y += r.y, v.z += r.z, v.w += r.w;
        }
        ss = fmaf(v.x, v.x, ss), ss = fmaf(v.y, v.y, ss), ss = fmaf(v.z, v.z, ss), ss = fmaf(v.w, v.w, ss);
    }
    ss = wave_sum(ss);
    if (lane == 0) red[0][wave] = ss;
    __syncthreads();
    const float inv = 1.0f / sqrtf(((red[0][0] + red[0][1]) + (red[0][2] + red[0][3])) / (float)h + nm.eps);
    float acc = 0.0f;
    for (int c = threadIdx.x * 4; c < h; c += 1024) {
        float4 v = ld<float4>((const uint8_t *)(nm.x + c));
        if (nm.res) {
            const float4 r = ld<float4>((const uint8_t *)(nm.res + c));
            v.x += r.x, v.y += r.y, v.z += r.z, v.w += r.w;
        }
        const float4 g = ld<float4>((const uint8_t *)(nm.w + c)), w = ld<float4>((const uint8_t *)(wr + c));
        const float4 hn = float4{v.x * inv * g.x, v.y * inv * g.y, v.z * inv * g.z, v.w * inv * g.w};
        if (e == 0) *(float4 *)(nm.x_out + c) = v, *(float4 *)(nm.hn_out + c) = hn;
        acc = fmaf(hn.x, w.x, acc);
        acc = fmaf(hn.y, w.y, acc);
        acc = fmaf(hn.z, w.z, acc);
        acc = fmaf(hn.w, w.w, acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) red[1][wave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) logits[e] = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
}

// The same logits for several tokens: one workgroup per (8 router rows, 8 tokens), so a token's activations are read
// once per eight experts instead of once per expert (512 tokens x 256 experts of 7168: 228 -> 60 us).  Every
// logit is accumulated by the same thread over the same columns in the same order as in moe_router_logits and
// reduced the same way, so the two kernels give the same bits.
// With `planes` (h a multiple of 32) the launch also leaves the tokens' activations as fixed-point planes for the expert
// kernels behind it: the workgroups of a token tile share its 8 h / 32 blocks, eight lanes a block.
__global__ __launch_bounds__(256) void moe_router_logits_tile(const float *__restrict__ Wr, const float *__restrict__ X,
                                                               float *__restrict__ logits, int T, int h, int E,
                                                               ActsI8 planes = ActsI8{nullptr, nullptr, nullptr, nullptr}) {
    __shared__ float red[4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int e0 = 8 * (int)blockIdx.x, t0 = 8 * (int)blockIdx.y;
    if (planes.xl) {
        const int bpt = h / 32, units = 8 * bpt;  // blocks a token, blocks of the tile
        for (int u = 32 * (int)blockIdx.x + ((int)threadIdx.x >> 3); u < units; u += 32 * (int)gridDim.x) {
            const int t = t0 + u / bpt, b = u % bpt;
            // (the eight lanes of a block stay together: u depends on threadIdx.x >> 3 only)
            if (t < T) acts_i8_quantize(X, (size_t)t * (size_t)(h / 4) + 8 * b + (threadIdx.x & 7), planes);
        }
    }
    float acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 8; j++) acc[i][j] = 0.0f;
    for (int c = threadIdx.x * 4; c < h; c += 1024) {
        float4 w[8], x[8];
#pragma unroll
        for (int i = 0; i < 8; i++) w[i] = ld<float4>((const uint8_t *)(Wr + (size_t)min(e0 + i, E - 1) * h + c));
#pragma unroll
        for (int j = 0; j < 8; j++) x[j] = ld<float4>((const uint8_t *)(X + (size_t)min(t0 + j, T - 1) * h + c));
#pragma unroll
        for (int i = 0; i < 8; i++)
#pragma unroll
            for (int j = 0; j < 8; j++) {
                acc[i][j] = fmaf(x[j].x, w[i].x, acc[i][j]);
                acc[i][j] = fmaf(x[j].y, w[i].y, acc[i][j]);
                acc[i][j] = fmaf(x[j].z, w[i].z, acc[i][j]);
                acc[i][j] = fmaf(x[j].w, w[i].w, acc[i][j]);
            }
    }
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float s = wave_sum(acc[i][j]);
            if (lane == 0) red[wave][8 * i + j] = s;
        }
    __syncthreads();
    if (threadIdx.x < 64) {
        const int i = threadIdx.x >> 3, j = threadIdx.x & 7;
        if (e0 + i < E && t0 + j < T)
            logits[(size_t)(t0 + j) * E + e0 + i] =
                (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
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
// Where moe_gate_topk writes the pair groups itself (null gexp: a separate grouping kernel runs).
// n_extra = 1 appends, per token, a pair for the shared expert (table index E, output row P + t).
struct MoePairGroups {
    int *gexp, *offsets, *xrow, *yrow;
    int n_extra;
};

__global__ __launch_bounds__(256) void moe_gate_topk(const float *__restrict__ logits, const float *__restrict__ bias,
                                                      MoeGateParams p, uint32_t *__restrict__ ids,
                                                      float *__restrict__ wts, MoePairGroups pg) {
    extern __shared__ __attribute__((aligned(16))) float sm[];  // probs[E], sel[E], gscore[n_group], selw[k_used], red[4]
    float *probs = sm, *sel = sm + p.E, *gscore = sm + 2 * p.E, *selw = gscore + (p.n_group > 1 ? p.n_group : 1);
    float *red = selw + p.k_used;
    const int t = blockIdx.x, lane = threadIdx.x, wv = threadIdx.x >> 6;  // `lane` strides the experts by 256
    constexpr int NT = 256;
    const float *lg = logits + (size_t)t * p.E;
    if (p.sigmoid) {
        for (int e = lane; e < p.E; e += NT) probs[e] = 1.0f / (1.0f + expf(-lg[e]));
    } else {
        float mx = -INFINITY;
        for (int e = lane; e < p.E; e += NT) mx = fmaxf(mx, lg[e]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        if ((lane & 63) == 0) red[wv] = mx;
        __syncthreads();
        mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        __syncthreads();
        float sum = 0.0f;
        for (int e = lane; e < p.E; e += NT) {
            const float v = expf(lg[e] - mx);
            probs[e] = v;
            sum += v;
        }
        sum = wave_sum(sum);
        if ((lane & 63) == 0) red[wv] = sum;
        __syncthreads();
        sum = (red[0] + red[1]) + (red[2] + red[3]);
        for (int e = lane; e < p.E; e += NT) probs[e] = probs[e] / sum;
    }
    for (int e = lane; e < p.E; e += NT) sel[e] = probs[e] + (bias ? bias[e] : 0.0f);
    __syncthreads();
    if (p.n_group > 1) {
        const int per = p.E / p.n_group;
        for (int g = lane; g < p.n_group; g += NT) {
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
        for (int e = lane; e < p.E; e += NT) {
            const int g = e / per;
            int rank = 0;
            for (int o = 0; o < p.n_group; o++) rank += gscore[o] > gscore[g] || (gscore[o] == gscore[g] && o < g);
            // selection + (mask*1e30 - 1e30): unchanged inside the kept groups
            if (rank >= p.topk_group) sel[e] = sel[e] + (0.0f * 1e30f - 1e30f);
        }
        __syncthreads();
    }
    for (int e = lane; e < p.E; e += NT) {
        const float v = sel[e];
        int rank = 0;
        // how many experts come before e: four scores a read, sixteen reads in flight (one score a read,
        // each waited for in turn, made this loop two thirds of the kernel's time)
        int o = 0;
        if ((p.E & 3) == 0) {
            const float4 *sel4 = (const float4 *)sel;  // sm is 16-byte aligned and E a multiple of 4
#pragma unroll 4
            for (; o < p.E; o += 4) {
                const float4 q = sel4[o >> 2];
                rank += (q.x > v || (q.x == v && o < e)) + (q.y > v || (q.y == v && o + 1 < e)) +
                        (q.z > v || (q.z == v && o + 2 < e)) + (q.w > v || (q.w == v && o + 3 < e));
            }
        }
        for (; o < p.E; o++) rank += sel[o] > v || (sel[o] == v && o < e);
        if (rank < p.k_used) {
            ids[(size_t)t * p.k_used + rank] = (uint32_t)e;
            selw[rank] = probs[e];
            if (pg.gexp) {  // decode-sized call: every (token, slot) pair is its own group
                const int pidx = t * p.k_used + rank;
                pg.gexp[pidx] = e, pg.offsets[pidx] = pidx, pg.xrow[pidx] = t, pg.yrow[pidx] = pidx;
            }
        }
    }
    __syncthreads();
    for (int i = lane; i < p.k_used; i += NT) {
        float w = selw[i];
        if (p.norm_topk) {
            float s = 0.0f;
            for (int j = 0; j < p.k_used; j++) s += selw[j];
            w = w / fmaxf(s, 6.103515625e-5f);
        }
        if (p.scale != 0.0f && p.scale != 1.0f) w = w * p.scale;
        wts[(size_t)t * p.k_used + i] = w;
    }
    if (pg.gexp && lane == 0) {
        const int P = (int)gridDim.x * p.k_used, total = P + pg.n_extra * (int)gridDim.x;
        if (t == 0) pg.offsets[total] = total;
        if (pg.n_extra) {  // the shared expert as one more pair of this token
            const int pidx = P + t;
            pg.gexp[pidx] = p.E, pg.offsets[pidx] = pidx, pg.xrow[pidx] = t, pg.yrow[pidx] = pidx;
        }
    }
}

// The same gating by ONE wave per token, for layers without expert groups and with at most 256 experts: lane l
// holds experts l, l + 64, ..., the softmax and each of the k_used arg-max rounds are register-to-register
// reductions (no LDS, no barrier), where moe_gate_topk's 256 threads meet at eight barriers and rank every
// expert against every other through LDS: 3 us a launch instead of 7.  Equal scores go to the lower expert
// index, as there.
// The gating of token t by one wave.  Lane r < k_used ends with slot r's expert in *slot_e; `write`: the slots go
// to ids / wts and the pair groups as well (a kernel that runs the gating in every workgroup writes them once).
template <int NE>
__device__ __forceinline__ void moe_gate_topk_wave_body(int t, int T, int lane, const float *__restrict__ logits,
                                                        const float *__restrict__ bias, const MoeGateParams &p,
                                                        uint32_t *__restrict__ ids, float *__restrict__ wts,
                                                        const MoePairGroups &pg, bool write, int *slot_e) {
    const float *lg = logits + (size_t)t * p.E;
    float prob[NE], sel[NE];
    {
        float v[NE];
#pragma unroll
        for (int i = 0; i < NE; i++) v[i] = lane + 64 * i < p.E ? lg[lane + 64 * i] : -INFINITY;
        if (p.sigmoid) {
#pragma unroll
            for (int i = 0; i < NE; i++) prob[i] = 1.0f / (1.0f + expf(-v[i]));
        } else {
            float mx = v[0];
#pragma unroll
            for (int i = 1; i < NE; i++) mx = fmaxf(mx, v[i]);
            mx = wave_max(mx);
            float sum = 0.0f;
#pragma unroll
            for (int i = 0; i < NE; i++) {
                prob[i] = lane + 64 * i < p.E ? expf(v[i] - mx) : 0.0f;
                sum += prob[i];
            }
            sum = wave_sum(sum);
#pragma unroll
            for (int i = 0; i < NE; i++) prob[i] = prob[i] / sum;
        }
#pragma unroll
        for (int i = 0; i < NE; i++)
            sel[i] = lane + 64 * i < p.E ? prob[i] + (bias ? bias[lane + 64 * i] : 0.0f) : -INFINITY;
    }
    int my_e = 0;
    float my_p = 0.0f;  // lane r keeps slot r
    for (int r = 0; r < p.k_used; r++) {
        float best = sel[0];
#pragma unroll
        for (int i = 1; i < NE; i++) best = fmaxf(best, sel[i]);
        const float top = wave_max(best);
        // the lowest expert index holding the maximum: the first slot any lane holds it in, and there the first
        // lane (scalar work on the lanes' votes; scores that compare with nothing, from activations that are not
        // numbers, leave slot r to expert r)
        int slot = 0, owner = r & 63;
#pragma unroll
        for (int i = NE - 1; i >= 0; i--) {
            const unsigned long long votes = __ballot(sel[i] == top);
            if (votes) slot = i, owner = __builtin_ctzll(votes);
        }
        const int e = min(owner + 64 * slot, p.E - 1);  // (in range whatever the scores were)
        float pw = 0.0f;
#pragma unroll
        for (int i = 0; i < NE; i++) {
            if (i == slot) {
                pw = prob[i];
                if (lane == owner) sel[i] = -INFINITY;
            }
        }
        pw = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, pw), owner));
        if (lane == r) my_e = e, my_p = pw;
    }
    float w = my_p;
    if (p.norm_topk) {
        float s = 0.0f;
        for (int j = 0; j < p.k_used; j++) s += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_p), j));
        w = w / fmaxf(s, 6.103515625e-5f);
    }
    if (p.scale != 0.0f && p.scale != 1.0f) w = w * p.scale;
    *slot_e = my_e;
    if (!write) return;
    if (lane < p.k_used) {
        const int pidx = t * p.k_used + lane;
        ids[pidx] = (uint32_t)my_e;
        wts[pidx] = w;
        if (pg.gexp) pg.gexp[pidx] = my_e, pg.offsets[pidx] = pidx, pg.xrow[pidx] = t, pg.yrow[pidx] = pidx;
    }
    if (pg.gexp && lane == 0) {
        const int P = T * p.k_used, total = P + pg.n_extra * T;
        if (t == 0) pg.offsets[total] = total;
        if (pg.n_extra) {  // the shared expert as one more pair of this token
            const int pidx = P + t;
            pg.gexp[pidx] = p.E, pg.offsets[pidx] = pidx, pg.xrow[pidx] = t, pg.yrow[pidx] = pidx;
        }
    }
}

template <int NE>
__global__ __launch_bounds__(64) void moe_gate_topk_wave(const float *__restrict__ logits, const float *__restrict__ bias,
                                                          MoeGateParams p, uint32_t *__restrict__ ids,
                                                          float *__restrict__ wts, MoePairGroups pg) {
    int slot_e;
    moe_gate_topk_wave_body<NE>((int)blockIdx.x, (int)gridDim.x, (int)threadIdx.x, logits, bias, p, ids, wts, pg, true, &slot_e);
}

// Groups the T*k routed (token, slot) pairs by expert, keeping pair order inside
// a group (the reference buckets the same way on the host,
// src/quantized_qwen3_moe.rs:459-480).  Group e is expert e:
//   offsets[e] .. offsets[e+1]  positions of the expert's pairs
//   xrow[pos]  activation row (token) of the pair,  yrow[pos]  the pair index
constexpr int GROUP_PAIRS_THREADS = 1024;

__global__ __launch_bounds__(GROUP_PAIRS_THREADS) void moe_group_pairs(const uint32_t *__restrict__ ids, int T,
                                                                       int k_used, int E, int *__restrict__ gexp,
                                                                       int *__restrict__ offsets,
                                                                       int *__restrict__ xrow, int *__restrict__ yrow,
                                                                       int shared_group, int ids_in_lds) {
    extern __shared__ int cnt[];  // [E + 1], then the pair list [P] when ids_in_lds
    const int P = T * k_used;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    uint32_t *ids_lds = (uint32_t *)(cnt + E + 1);
    for (int e = threadIdx.x; e <= E; e += blockDim.x) cnt[e] = 0;
    __syncthreads();
    for (int pidx = threadIdx.x; pidx < P; pidx += blockDim.x) {
        const uint32_t e = ids[pidx];
        if (ids_in_lds) ids_lds[pidx] = e;
        if (e < (uint32_t)E) atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    if (wave == 0) {  // counts -> start positions: each lane a run of experts, a wave scan between the runs
        const int per = (E + 63) / 64, b = lane * per;
        int local = 0;
        for (int i = 0; i < per; i++)
            if (b + i < E) local += cnt[b + i];
        int incl = local;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int v = __shfl_up(incl, off, 64);
            if (lane >= off) incl += v;
        }
        int run = incl - local;
        for (int i = 0; i < per; i++) {
            if (b + i < E) {
                const int c = cnt[b + i];
                cnt[b + i] = run;
                run += c;
            }
        }
        if (lane == 63) cnt[E] = incl;
    }
    __syncthreads();
    for (int e = threadIdx.x; e <= E; e += blockDim.x) offsets[e] = cnt[e];
    if (shared_group) {  // group E: the shared expert over every token, output rows P .. P + T - 1
        if (threadIdx.x == 0) gexp[E] = E, offsets[E + 1] = P + T;
        for (int t = threadIdx.x; t < T; t += blockDim.x) xrow[P + t] = t, yrow[P + t] = P + t;
    }
    // a wave per expert walks the pair list 64 pairs at a time, in order (from the LDS copy when
    // it fits): a pair's place is the expert's start + the matches before it
    const uint32_t *scan = ids_in_lds ? ids_lds : ids;
    for (int e = wave; e < E; e += waves) {
        if (lane == 0) gexp[e] = e;
        int pos = cnt[e];
        for (int base = 0; base < P; base += 64) {
            const int pidx = base + lane;
            const bool hit = pidx < P && scan[pidx] == (uint32_t)e;
            const unsigned long long mask = __ballot(hit);
            if (hit) {
                const int at = pos + __popcll(mask & ((1ull << lane) - 1ull));
                xrow[at] = pidx / k_used;
                yrow[at] = pidx;
            }
            pos += __popcll(mask);
        }
    }
}

// The same grouping for pair lists of up to GROUP_RANK_CHUNKS * 64 pairs, by ranks instead of one pass over
// the list per expert: a wave takes 64 consecutive pairs, every lane counts the lanes before it that name its
// expert (its rank within the chunk), the last lane of an expert in the chunk records the chunk's count of
// that expert in hist[chunk][expert]; prefix sums over the chunks and then over the experts turn the counts
// into start positions, and a pair's place is its expert's start + the earlier chunks' count + its rank.
// LDS: chunks * E + E + 1 ints.
constexpr int GROUP_RANK_CHUNKS = 64, GROUP_RANK_PER_WAVE = GROUP_RANK_CHUNKS * 64 / GROUP_PAIRS_THREADS;

__global__ __launch_bounds__(GROUP_PAIRS_THREADS) void moe_group_pairs_ranked(const uint32_t *__restrict__ ids, int T,
                                                                              int k_used, int E, int *__restrict__ gexp,
                                                                              int *__restrict__ offsets,
                                                                              int *__restrict__ xrow, int *__restrict__ yrow,
                                                                              int shared_group) {
    extern __shared__ int hist[];  // [chunks][E], then start[E + 1]
    const int P = T * k_used, chunks = (P + 63) / 64;
    int *start = hist + chunks * E;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    constexpr int WAVES = GROUP_PAIRS_THREADS / 64;
    for (int i = threadIdx.x; i < chunks * E; i += GROUP_PAIRS_THREADS) hist[i] = 0;
    __syncthreads();
    uint32_t mine[GROUP_RANK_PER_WAVE];
    int rank[GROUP_RANK_PER_WAVE];
#pragma unroll
    for (int c = 0; c < GROUP_RANK_PER_WAVE; c++) {
        const int chunk = wave + WAVES * c, pidx = 64 * chunk + lane;
        mine[c] = 0xFFFFFFFFu, rank[c] = 0;
        if (chunk >= chunks) continue;  // the same for the whole wave
        const uint32_t e = pidx < P ? ids[pidx] : 0xFFFFFFFFu;
        int before = 0, after = 0;
        for (int j = 0; j < 64; j++) {
            const bool same = (uint32_t)__shfl((int)e, j, 64) == e;
            before += same && j < lane;
            after += same && j > lane;
        }
        mine[c] = e, rank[c] = before;
        if (e < (uint32_t)E && after == 0) hist[chunk * E + (int)e] = before + 1;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += GROUP_PAIRS_THREADS) {  // counts -> counts in earlier chunks; the expert's total
        int run = 0;
        for (int ch = 0; ch < chunks; ch++) {
            const int c = hist[ch * E + e];
            hist[ch * E + e] = run;
            run += c;
        }
        start[e] = run;
    }
    __syncthreads();
    if (wave == 0) {  // totals -> start positions: each lane a run of experts, a wave scan between the runs
        const int per = (E + 63) / 64, b = lane * per;
        int local = 0;
        for (int i = 0; i < per; i++)
            if (b + i < E) local += start[b + i];
        int incl = local;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int v = __shfl_up(incl, off, 64);
            if (lane >= off) incl += v;
        }
        int run = incl - local;
        for (int i = 0; i < per; i++) {
            if (b + i < E) {
                const int c = start[b + i];
                start[b + i] = run;
                run += c;
            }
        }
        if (lane == 63) start[E] = incl;
    }
    __syncthreads();
    for (int e = threadIdx.x; e <= E; e += GROUP_PAIRS_THREADS) {
        offsets[e] = start[e];
        if (e < E) gexp[e] = e;
    }
    if (shared_group) {  // group E: the shared expert over every token, output rows P .. P + T - 1
        if (threadIdx.x == 0) gexp[E] = E, offsets[E + 1] = P + T;
        for (int t = threadIdx.x; t < T; t += GROUP_PAIRS_THREADS) xrow[P + t] = t, yrow[P + t] = P + t;
    }
#pragma unroll
    for (int c = 0; c < GROUP_RANK_PER_WAVE; c++) {
        const int chunk = wave + WAVES * c, pidx = 64 * chunk + lane;
        if (mine[c] < (uint32_t)E) {
            const int at = start[mine[c]] + hist[chunk * E + (int)mine[c]] + rank[c];
            xrow[at] = pidx / k_used;
            yrow[at] = pidx;
        }
    }
}


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
                                                                   float *__restrict__ Y, int k, int n, MoeClamp cl) {
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
                                xv = float4{swiglu(xv.x, uv.x, cl, e), swiglu(xv.y, uv.y, cl, e), swiglu(xv.z, uv.z, cl, e),
                                            swiglu(xv.w, uv.w, cl, e)};
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

// The grouped expert matmul with the weight rows staged through LDS (see matmul_rows_staged): a
// wave pulls the packed bytes of its 64 / L consecutive rows with coalesced asynchronous loads,
// then L lanes work on each row (L = 16, 32 or 64, so that short rows still fill the wave).
// DUAL: the same rows of two weight tables (gate and up) against one activation row, result
// silu(gate . x) * (up . x) (reference: src/quantized_qwen3_moe.rs:397-401) without a round trip
// of the two vectors through memory.
template <class Q, int MT, bool DUAL, int G>
__global__ __launch_bounds__(64 * ROWS_PER_WG) void moe_rows_staged(const uint8_t *const *__restrict__ Wa,
                                                                     const uint8_t *const *__restrict__ Wb,
                                                                     size_t row_bytes, const float *__restrict__ X,
                                                                     const int *__restrict__ gexp,
                                                                     const int *__restrict__ offsets,
                                                                     const int *__restrict__ xsel,
                                                                     const int *__restrict__ yrow,
                                                                     float *__restrict__ Y, int k, int n, int L,
                                                                     int wave_lds, MoeClamp cl) {
    extern __shared__ __attribute__((aligned(16))) uint8_t staged_moe[];
    const auto *table = stage_table<Q>(staged_moe);  // before any wave leaves: it holds a barrier
    const int grp = blockIdx.y;
    const int beg = offsets[grp], cnt = offsets[grp + 1] - beg;
    if (cnt == 0) return;
    const int e = gexp[grp];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int R = 64 / L;
    const int row0 = (blockIdx.x * ROWS_PER_WG + wave) * R;
    if (row0 >= n) return;  // wave-uniform; the kernel has no barrier
    const int nrows = min(R, n - row0);
    uint8_t *ra = staged_moe + table_bytes<Q>() + (size_t)wave * wave_lds, *rb = ra + (DUAL ? wave_lds / 2 : 0);
    {
        const int pieces = (int)((size_t)nrows * row_bytes / G);
        const uint8_t *sa = Wa[e] + (size_t)row0 * row_bytes;
        const uint8_t *sb = DUAL ? Wb[e] + (size_t)row0 * row_bytes : nullptr;
        for (int p0 = 0; p0 < pieces; p0 += 64) {
            if (p0 + lane < pieces) {
                if (G == 16) {
                    async_load16(sa + (size_t)(p0 + lane) * 16, lds_offset_of(ra + (size_t)p0 * 16));
                    if (DUAL) async_load16(sb + (size_t)(p0 + lane) * 16, lds_offset_of(rb + (size_t)p0 * 16));
                } else {
                    async_load4(sa + (size_t)(p0 + lane) * 4, lds_offset_of(ra + (size_t)p0 * 4));
                    if (DUAL) async_load4(sb + (size_t)(p0 + lane) * 4, lds_offset_of(rb + (size_t)p0 * 4));
                }
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    const int sub = lane % L, rl = lane / L, row = row0 + rl;
    const bool active = rl < nrows;
    const uint8_t *rpa = ra + (size_t)rl * row_bytes, *rpb = rb + (size_t)rl * row_bytes;
    const int units = (k / Q::BLOCK_ELEMS) * Q::UNITS;
    constexpr int UE = Q::SEGS * Q::SEGLEN;
    for (int m0 = 0; m0 < cnt; m0 += MT) {
        float acc[MT], acc2[MT];
        int xr[MT];
#pragma unroll
        for (int i = 0; i < MT; i++) {
            acc[i] = acc2[i] = 0.0f;
            xr[i] = xsel[beg + min(m0 + i, cnt - 1)];
        }
        if (active) {
            for (int u = sub; u < units; u += L) {
                const int b = u / Q::UNITS, ub = u % Q::UNITS;
                float w[UE], w2[DUAL ? UE : 1];
                decode_staged<Q>(table, rpa + (size_t)b * Q::BLOCK_BYTES, ub, w);
                if (DUAL) decode_staged<Q>(table, rpb + (size_t)b * Q::BLOCK_BYTES, ub, w2);
                const int xoff = b * Q::BLOCK_ELEMS + Q::elem_base(ub);
#pragma unroll
                for (int i = 0; i < MT; i++) {
                    if (m0 + i < cnt) {
                        const float *xp = X + (size_t)xr[i] * k + xoff;
#pragma unroll
                        for (int s = 0; s < Q::SEGS; s++) {
#pragma unroll
                            for (int el = 0; el < Q::SEGLEN; el += 4) {
                                const float4 xv = ld<float4>((const uint8_t *)(xp + s * Q::SEG_STRIDE + el));
                                acc[i] = fmaf(xv.x, w[s * Q::SEGLEN + el + 0], acc[i]);
                                acc[i] = fmaf(xv.y, w[s * Q::SEGLEN + el + 1], acc[i]);
                                acc[i] = fmaf(xv.z, w[s * Q::SEGLEN + el + 2], acc[i]);
                                acc[i] = fmaf(xv.w, w[s * Q::SEGLEN + el + 3], acc[i]);
                                if (DUAL) {
                                    acc2[i] = fmaf(xv.x, w2[s * Q::SEGLEN + el + 0], acc2[i]);
                                    acc2[i] = fmaf(xv.y, w2[s * Q::SEGLEN + el + 1], acc2[i]);
                                    acc2[i] = fmaf(xv.z, w2[s * Q::SEGLEN + el + 2], acc2[i]);
                                    acc2[i] = fmaf(xv.w, w2[s * Q::SEGLEN + el + 3], acc2[i]);
                                }
                            }
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < MT; i++) {
            float s = acc[i], s2 = acc2[i];
            for (int off = L >> 1; off > 0; off >>= 1) {
                s += __shfl_xor(s, off, 64);
                if (DUAL) s2 += __shfl_xor(s2, off, 64);
            }
            if (sub == 0 && active && m0 + i < cnt)
                Y[(size_t)yrow[beg + m0 + i] * n + row] = DUAL ? swiglu(s, s2, cl, e) : s;
        }
    }
}

__global__ __launch_bounds__(256) void acts_i8_prep(const float *__restrict__ X, size_t rows, int k, ActsI8 out) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;  // four elements a thread, eight threads a block
    if (i >= rows * (size_t)(k / 4)) return;  // whole groups of 8 lanes leave together (k % 32 == 0)
    acts_i8_quantize(X, i, out);
}

// The decode-shaped grouped expert matmul (one activation row a group) on integer dot products: rows
// staged through LDS as in moe_rows_staged, every unit of 32 or 64 elements multiplied by Q::dot8
// against the group's activation row as 15-bit fixed point per 32-element block (ActsI8).  OWN_PREP:
// the workgroup quantises the row itself into LDS while its rows are on their way (short rows: cheaper
// than one more launch); otherwise the planes come from acts_i8_prep (long rows: quantising 7168
// elements in each of thousands of workgroups costs more than it saves).
// Y[yrow[beg]] = W[e] x, or silu(Wa[e] x) * (Wb[e] x) with DUAL.
// Dynamic LDS: the format's table, ROWS_PER_WG * wave_lds of staged rows, with OWN_PREP 2.25 k more.
template <class Q, bool DUAL, int G, bool OWN_PREP>
__global__ __launch_bounds__(64 * ROWS_PER_WG) void moe_rows_dot8(const uint8_t *const *__restrict__ Wa,
                                                                   const uint8_t *const *__restrict__ Wb,
                                                                   size_t row_bytes, const float *__restrict__ X,
                                                                   ActsI8 xq, const int *__restrict__ gexp,
                                                                   const int *__restrict__ offsets,
                                                                   const int *__restrict__ xsel,
                                                                   const int *__restrict__ yrow,
                                                                   float *__restrict__ Y, int k, int n, int L,
                                                                   int wave_lds, MoeClamp cl) {
    static_assert(Q::SEGS == 1 && Q::SEGLEN % 32 == 0, "units of 32 or 64 consecutive elements");
    constexpr int XW = Q::SEGLEN / 4, NS = Q::SEGLEN / 32;  // activation words a plane, scales a unit
    extern __shared__ __attribute__((aligned(16))) uint8_t staged_moe[];
    const auto *table = stage_table<Q>(staged_moe);  // before any wave leaves: it holds a barrier
    const int grp = blockIdx.y;
    const int beg = offsets[grp], cnt = offsets[grp + 1] - beg;
    if (cnt == 0) return;  // the whole workgroup
    const int e = gexp[grp];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int R = 64 / L;
    const int row0 = (blockIdx.x * ROWS_PER_WG + wave) * R;
    const int nrows = min(R, n - row0);  // <= 0: this wave has no rows and only helps with the activations
    uint8_t *ra = staged_moe + table_bytes<Q>() + (size_t)wave * wave_lds, *rb = ra + (DUAL ? wave_lds / 2 : 0);
    if (nrows > 0) {
        const int pieces = (int)((size_t)nrows * row_bytes / G);
        const uint8_t *sa = Wa[e] + (size_t)row0 * row_bytes;
        const uint8_t *sb = DUAL ? Wb[e] + (size_t)row0 * row_bytes : nullptr;
        for (int p0 = 0; p0 < pieces; p0 += 64) {
            if (p0 + lane < pieces) {
                if (G == 16) {
                    async_load16(sa + (size_t)(p0 + lane) * 16, lds_offset_of(ra + (size_t)p0 * 16));
                    if (DUAL) async_load16(sb + (size_t)(p0 + lane) * 16, lds_offset_of(rb + (size_t)p0 * 16));
                } else {
                    async_load4(sa + (size_t)(p0 + lane) * 4, lds_offset_of(ra + (size_t)p0 * 4));
                    if (DUAL) async_load4(sb + (size_t)(p0 + lane) * 4, lds_offset_of(rb + (size_t)p0 * 4));
                }
            }
        }
    }
    const size_t xr = (size_t)xsel[beg];
    const uint32_t *xlp = xq.xl + xr * (size_t)(k / 4), *xhp = xq.xh + xr * (size_t)(k / 4);
    const float *sxp = xq.sx + xr * (size_t)(k / 32), *sxsp = xq.sxs + xr * (size_t)(k / 32);
    if (OWN_PREP) {  // four elements a thread, eight threads a 32-element block (k % 32 == 0)
        uint32_t *xl_lds = (uint32_t *)(staged_moe + table_bytes<Q>() + (size_t)ROWS_PER_WG * wave_lds), *xh_lds = xl_lds + k / 4;
        float *sx_lds = (float *)(xh_lds + k / 4), *sxs_lds = sx_lds + k / 32;
        const float *xrow = X + xr * k;
        for (int i = threadIdx.x; i < k / 4; i += 64 * ROWS_PER_WG) {
            const float4 v = *(const float4 *)(xrow + 4 * i);
            float amax = fmaxf(fmaxf(mag_or_inf(v.x), mag_or_inf(v.y)), fmaxf(mag_or_inf(v.z), mag_or_inf(v.w)));
            amax = max_row8(amax);
            const bool live = amax > 0.0f && amax < INFINITY;
            const float inv = live ? 32639.0f / amax : 0.0f;
            const int Xq[4] = {__float2int_rn(v.x * inv), __float2int_rn(v.y * inv), __float2int_rn(v.z * inv),
                               __float2int_rn(v.w * inv)};
            uint32_t wl = 0, wh = 0;
            int sum = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int lo = ((Xq[j] + 128) & 255) - 128, hi = (Xq[j] - lo) >> 8;
                wl |= (uint32_t)(lo & 255) << (8 * j);
                wh |= (uint32_t)(hi & 255) << (8 * j);
                sum += Xq[j];
            }
            xl_lds[i] = wl;
            xh_lds[i] = wh;
            sum = isum_row8(sum);
            if ((i & 7) == 0) {
                const float s = fixed_scale(amax, 32639.0f);
                sx_lds[i >> 3] = s;
                sxs_lds[i >> 3] = s * (float)sum;
            }
        }
        __syncthreads();
        xlp = xl_lds, xhp = xh_lds, sxp = sx_lds, sxsp = sxs_lds;
    }
    if (nrows <= 0) return;
    const int sub = lane % L, rl = lane / L, row = row0 + rl;
    const bool active = rl < nrows;
    const uint8_t *rpa = ra + (size_t)rl * row_bytes, *rpb = rb + (size_t)rl * row_bytes;
    const int units = (k / Q::BLOCK_ELEMS) * Q::UNITS;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the rows landed (this wave's own data)
    float acc = 0.0f, acc2 = 0.0f;
    if (active) {
        for (int u = sub; u < units; u += L) {
            const int b = u / Q::UNITS, ub = u % Q::UNITS;
            const int el = b * Q::BLOCK_ELEMS + Q::elem_base(ub);  // a multiple of 32
            uint32_t xl[XW], xh[XW];
            float sx[NS], sxs[NS];
#pragma unroll
            for (int i = 0; i < XW; i += 4) {
                const uint4 lw = *(const uint4 *)(xlp + el / 4 + i), hw = *(const uint4 *)(xhp + el / 4 + i);
                xl[i] = lw.x, xl[i + 1] = lw.y, xl[i + 2] = lw.z, xl[i + 3] = lw.w;
                xh[i] = hw.x, xh[i + 1] = hw.y, xh[i + 2] = hw.z, xh[i + 3] = hw.w;
            }
#pragma unroll
            for (int i = 0; i < NS; i++) sx[i] = sxp[el / 32 + i], sxs[i] = sxsp[el / 32 + i];
            acc += Q::dot8(table, rpa + (size_t)b * Q::BLOCK_BYTES, ub, xl, xh, sx, sxs);
            if (DUAL) acc2 += Q::dot8(table, rpb + (size_t)b * Q::BLOCK_BYTES, ub, xl, xh, sx, sxs);
        }
    }
    for (int off = L >> 1; off > 0; off >>= 1) {
        acc += __shfl_xor(acc, off, 64);
        if (DUAL) acc2 += __shfl_xor(acc2, off, 64);
    }
    if (sub == 0 && active) Y[(size_t)yrow[beg] * n + row] = DUAL ? swiglu(acc, acc2, cl, e) : acc;
}

// Groups of several pairs (bucketed by expert), formats with Q::decode_i8: the expert's rows are decoded ONCE, to
// signed int8 words held in registers (a lane keeps UL units of 32 elements of its row, or of gate's and up's row
// with DUAL; the rows come through LDS, 16 or 4 bytes a lane and load), and the group's pairs stream past them: a
// pair's activation planes (acts_i8_prep's, row xsel[pair]) are copied into LDS once for the workgroup's four
// waves, two pairs in flight, and every unit costs sixteen v_dot4 a matrix.  Per-pair kernels re-read a pair's
// planes in every wave (2.1 bytes an element and wave, from L2: at DeepSeek-V3's sizes that traffic, not the
// weights, bounds calls of 64 tokens and more) and decode the weights again for every pair.  The rows' staging
// area becomes the activation buffers once every wave has decoded.  Groups are taken from the last down: a
// folded shared expert, the one group with a pair per token, is the last group and starts first.  A pair's
// buffer holds, for units = k / 32: the first four words of every unit of the low plane, the last four, the
// same of the high plane, the units' scales and, for formats with an offset a sub-block (Q4_K), the units' scaled
// sums.
// Dynamic LDS: the format's table and its I8_EXTRA_ENTRIES words of 8 bytes, then
// max(4 * wave_lds, x_at + 2 * (68 or 72) * units) bytes.
constexpr int EXPERT_DOT8_WAVES = 4;
template <class Q, bool DUAL, int G, int UL>
__global__ __launch_bounds__(64 * EXPERT_DOT8_WAVES) void moe_expert_dot8(
    const uint8_t *const *__restrict__ Wa, const uint8_t *const *__restrict__ Wb, size_t row_bytes, ActsI8 xq,
    const int *__restrict__ gexp, const int *__restrict__ offsets, const int *__restrict__ xsel,
    const int *__restrict__ yrow, float *__restrict__ Y, int k, int n, int L, int wave_lds, int x_at, MoeClamp cl) {
    static_assert(Q::HAS_DECODE_I8 && Q::BLOCK_ELEMS == 32 * Q::I8_UNITS, "units of 32 consecutive elements");
    constexpr int XB = 68 + (Q::I8_HAS_MIN ? 4 : 0);  // bytes of a pair's buffer a unit
    extern __shared__ __attribute__((aligned(16))) uint8_t staged_moe[];
    const int grp = (int)gridDim.y - 1 - (int)blockIdx.y;
    const int beg = offsets[grp], cnt = offsets[grp + 1] - beg;
    if (cnt == 0) return;  // the whole workgroup
    const int e = gexp[grp];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int units = k / 32, x_lds = XB * units;
    const int chunks = 4 * units + (Q::I8_HAS_MIN ? 2 : 1) * (units / 4);  // 16-byte pieces of a pair's planes and scales
    uint8_t *base = staged_moe + table_bytes<Q>() + 8 * Q::I8_EXTRA_ENTRIES;
    auto copy = [&](int p, int buf) {
        const size_t xr = (size_t)xsel[beg + p];
        const uint8_t *xl = (const uint8_t *)(xq.xl + xr * (size_t)(k / 4)), *xh = (const uint8_t *)(xq.xh + xr * (size_t)(k / 4));
        const uint8_t *sx = (const uint8_t *)(xq.sx + xr * (size_t)(k / 32)), *sxs = (const uint8_t *)(xq.sxs + xr * (size_t)(k / 32));
        uint8_t *dst = base + x_at + (size_t)buf * x_lds;
        for (int c0 = 64 * wave; c0 < chunks; c0 += 64 * EXPERT_DOT8_WAVES) {
            const int c = c0 + lane;
            if (c < chunks) {
                const uint8_t *src;
                if (c < 4 * units) {
                    const int q = c / units, u = c - q * units;  // q: low plane first half, second half, high plane ...
                    src = ((q & 2) ? xh : xl) + 32 * u + 16 * (q & 1);
                } else if (!Q::I8_HAS_MIN || c < 4 * units + units / 4) {
                    src = sx + 16 * (c - 4 * units);
                } else {
                    src = sxs + 16 * (c - 4 * units - units / 4);
                }
                async_load16(src, lds_offset_of(dst + (size_t)c0 * 16));
            }
        }
    };
    const int R = 64 / L;
    const int row0 = (blockIdx.x * EXPERT_DOT8_WAVES + wave) * R;
    const int nrows = min(R, n - row0);  // <= 0: this wave has no rows; it still copies activations and meets the barriers
    uint8_t *ra = base + (size_t)wave * wave_lds, *rb = ra + (DUAL ? wave_lds / 2 : 0);
    if (nrows > 0) {
        const int pieces = (int)((size_t)nrows * row_bytes / G);
        const uint8_t *sa = Wa[e] + (size_t)row0 * row_bytes;
        const uint8_t *sb = DUAL ? Wb[e] + (size_t)row0 * row_bytes : nullptr;
        for (int p0 = 0; p0 < pieces; p0 += 64) {
            if (p0 + lane < pieces) {
                if (G == 16) {
                    async_load16(sa + (size_t)(p0 + lane) * 16, lds_offset_of(ra + (size_t)p0 * 16));
                    if (DUAL) async_load16(sb + (size_t)(p0 + lane) * 16, lds_offset_of(rb + (size_t)p0 * 16));
                } else {
                    async_load4(sa + (size_t)(p0 + lane) * 4, lds_offset_of(ra + (size_t)p0 * 4));
                    if (DUAL) async_load4(sb + (size_t)(p0 + lane) * 4, lds_offset_of(rb + (size_t)p0 * 4));
                }
            }
        }
    }
    if (x_at) copy(0, 0);  // the activations have room of their own: the first pair comes in beside the rows
    if ((int)threadIdx.x < Q::I8_EXTRA_ENTRIES)
        ((uint64_t *)(staged_moe + table_bytes<Q>()))[threadIdx.x] = Q::i8_extra_entry((int)threadIdx.x);
    const auto *table = stage_table<Q>(staged_moe);  // holds a barrier when the format has a table
    const int sub = lane % L, rl = lane / L, row = row0 + rl;
    const bool active = rl < nrows;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the rows landed (this wave's own data)
    int wa[UL][8], wb[DUAL ? UL : 1][8];
    float da[UL], db[DUAL ? UL : 1], oa[Q::I8_HAS_MIN ? UL : 1], ob[Q::I8_HAS_MIN && DUAL ? UL : 1];
#pragma unroll
    for (int j = 0; j < UL; j++) {
        const int u = sub + L * j;
        if (active && u < units) {
            const size_t at = (size_t)rl * row_bytes + (size_t)(u / Q::I8_UNITS) * Q::BLOCK_BYTES;
            float o, o2 = 0.0f;
            Q::decode_i8(table, ra + at, u % Q::I8_UNITS, wa[j], da[j], o);
            if (DUAL) Q::decode_i8(table, rb + at, u % Q::I8_UNITS, wb[j], db[j], o2);
            if (Q::I8_HAS_MIN) {
                oa[j] = o;
                if (DUAL) ob[j] = o2;
            }
        } else {
            if (Q::I8_HAS_MIN) {
                oa[j] = 0.0f;
                if (DUAL) ob[j] = 0.0f;
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
                wa[j][i] = 0;
                if (DUAL) wb[j][i] = 0;
            }
            da[j] = 0.0f;
            if (DUAL) db[j] = 0.0f;
        }
    }
    if (!x_at) {
        __syncthreads();  // every wave holds its weights: the rows' LDS now takes the activations
        copy(0, 0);
    }
    for (int p = 0; p < cnt; p++) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();  // pair p's planes are in; every wave is done with pair p - 1's buffer
        if (p + 1 < cnt) copy(p + 1, (p + 1) & 1);
        const uint8_t *xb = base + x_at + (size_t)(p & 1) * x_lds;
        float acc = 0.0f, acc2 = 0.0f;
        // a unit's activations: eight words of each plane and the scale.  The next unit's are asked for before
        // this unit's products; the fences keep the compiler from asking for every unit's at once (17 registers
        // a unit, which with the weights would not fit).
        struct UnitX {
            uint4 l0, l1, h0, h1;
            float sx, sxs;
        };
        auto unit_x = [&](int j) {
            const int u = min(sub + L * j, units - 1);  // past the row's end: zero weights against the last unit
            UnitX x;
            x.l0 = *(const uint4 *)(xb + 16 * u), x.l1 = *(const uint4 *)(xb + 16 * (units + u));
            x.h0 = *(const uint4 *)(xb + 16 * (2 * units + u)), x.h1 = *(const uint4 *)(xb + 16 * (3 * units + u));
            x.sx = *(const float *)(xb + 64 * units + 4 * u);
            x.sxs = Q::I8_HAS_MIN ? *(const float *)(xb + 68 * units + 4 * u) : 0.0f;
            return x;
        };
        UnitX cur = unit_x(0);
#pragma unroll
        for (int j = 0; j < UL; j++) {
            UnitX nxt = cur;
            if (j + 1 < UL) nxt = unit_x(j + 1);
            __builtin_amdgcn_sched_barrier(0);
            const int xl[8] = {(int)cur.l0.x, (int)cur.l0.y, (int)cur.l0.z, (int)cur.l0.w,
                               (int)cur.l1.x, (int)cur.l1.y, (int)cur.l1.z, (int)cur.l1.w};
            const int xh[8] = {(int)cur.h0.x, (int)cur.h0.y, (int)cur.h0.z, (int)cur.h0.w,
                               (int)cur.h1.x, (int)cur.h1.y, (int)cur.h1.z, (int)cur.h1.w};
            int pl = 0, ph = 0, pl2 = 0, ph2 = 0;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                pl = __builtin_amdgcn_sdot4(wa[j][i], xl[i], pl, false);
                ph = __builtin_amdgcn_sdot4(wa[j][i], xh[i], ph, false);
                if (DUAL) {
                    pl2 = __builtin_amdgcn_sdot4(wb[j][i], xl[i], pl2, false);
                    ph2 = __builtin_amdgcn_sdot4(wb[j][i], xh[i], ph2, false);
                }
            }
            acc = fmaf(cur.sx * da[j], (float)((ph << 8) + pl), acc);
            if (Q::I8_HAS_MIN) acc = fmaf(-oa[j], cur.sxs, acc);
            if (DUAL) {
                acc2 = fmaf(cur.sx * db[j], (float)((ph2 << 8) + pl2), acc2);
                if (Q::I8_HAS_MIN) acc2 = fmaf(-ob[j], cur.sxs, acc2);
                // both sums are due here: left alone, the second matrix's products of every unit are put after
                // the first's, with every unit's activations held until then
                asm volatile("" : "+v"(acc), "+v"(acc2));
            }
            __builtin_amdgcn_sched_barrier(0);
            cur = nxt;
        }
        if (L >= 64) acc = sum_xor32(acc);  // L is 16, 32 or 64: whole rows of 16 lanes
        if (L >= 32) acc = sum_xor16(acc);
        acc = sum_row16(acc);
        if (DUAL) {
            if (L >= 64) acc2 = sum_xor32(acc2);
            if (L >= 32) acc2 = sum_xor16(acc2);
            acc2 = sum_row16(acc2);
        }
        if (sub == 0 && active) Y[(size_t)yrow[beg + p] * n + row] = DUAL ? swiglu(acc, acc2, cl, e) : acc;
    }
}

// The decode-sized down projection with the weighted combine in the same kernel.  Workgroup (tile of
// output rows, token t) walks the token's pairs: its k_used routed experts in slot order (pair
// t * k_used + s, weight wts[pair]) and then, with n_extra, the shared expert (pair P + t, weight 1).  Pair p
// multiplies row p of X (the activations silu(gate) * up of that pair) by expert gexp[p]'s rows.  All
// pairs' rows of a wave are asked for at once (S times the bytes in flight of moe_rows_dot8, and a ninth
// of its workgroups at DeepSeek-V3's sizes), and
//   y[t, row] = sum_s w_s * (W[e_s] x_s)[row]  (+ the shared expert's)
// is formed in the order moe_combine adds in, without the trip of the per-pair results through memory
// or the launch of moe_combine.  The S activation rows are fixed-point planes: quantised into LDS by the
// workgroup itself with OWN_PREP, else read from acts_i8_prep's output (copying those into LDS as well
// leaves room for one workgroup a compute unit at DeepSeek-V3's sizes and measured a quarter slower).
// Dynamic LDS: the format's table, ROWS_PER_WG * S * slot_lds of staged rows, with OWN_PREP S * 2.25 k more.
template <class Q, int G, bool OWN_PREP>
__global__ __launch_bounds__(64 * ROWS_PER_WG) void moe_down_combine_dot8(const uint8_t *const *__restrict__ Wa,
                                                                           size_t row_bytes, const float *__restrict__ X,
                                                                           ActsI8 xq, const int *__restrict__ gexp,
                                                                           const float *__restrict__ wts,
                                                                           float *__restrict__ y, int k, int n, int L,
                                                                           int slot_lds, int k_used, int n_extra, int P) {
    static_assert(Q::SEGS == 1 && Q::SEGLEN % 32 == 0, "units of 32 or 64 consecutive elements");
    constexpr int XW = Q::SEGLEN / 4, NS = Q::SEGLEN / 32;
    extern __shared__ __attribute__((aligned(16))) uint8_t staged_moe[];
    const auto *table = stage_table<Q>(staged_moe);  // holds a barrier
    const int t = blockIdx.y, S = k_used + n_extra;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int R = 64 / L;
    const int row0 = (blockIdx.x * ROWS_PER_WG + wave) * R;
    const int nrows = min(R, n - row0);  // <= 0: this wave has no rows and only helps with the activations
    uint8_t *ra = staged_moe + table_bytes<Q>() + (size_t)wave * S * slot_lds;
    if (nrows > 0) {
        const int pieces = (int)((size_t)nrows * row_bytes / G);
        for (int sl = 0; sl < S; sl++) {
            const int pair = sl < k_used ? t * k_used + sl : P + t;
            const uint8_t *sa = Wa[gexp[pair]] + (size_t)row0 * row_bytes;
            uint8_t *dst = ra + (size_t)sl * slot_lds;
            for (int p0 = 0; p0 < pieces; p0 += 64) {
                if (p0 + lane < pieces) {
                    if (G == 16) async_load16(sa + (size_t)(p0 + lane) * 16, lds_offset_of(dst + (size_t)p0 * 16));
                    else async_load4(sa + (size_t)(p0 + lane) * 4, lds_offset_of(dst + (size_t)p0 * 4));
                }
            }
        }
    }
    const int kw = k / 4, kb = k / 32;
    uint32_t *xl_lds = (uint32_t *)(staged_moe + table_bytes<Q>() + (size_t)ROWS_PER_WG * S * slot_lds);
    uint32_t *xh_lds = xl_lds + (size_t)S * kw;
    float *sx_lds = (float *)(xh_lds + (size_t)S * kw), *sxs_lds = sx_lds + (size_t)S * kb;
    if (OWN_PREP) {  // four elements a thread, eight threads a 32-element block (k % 32 == 0)
        for (int i = threadIdx.x; i < S * kw; i += 64 * ROWS_PER_WG) {
            const int sl = i / kw, j = i - sl * kw;
            const int pair = sl < k_used ? t * k_used + sl : P + t;
            const float4 v = *(const float4 *)(X + (size_t)pair * k + 4 * j);
            float amax = fmaxf(fmaxf(mag_or_inf(v.x), mag_or_inf(v.y)), fmaxf(mag_or_inf(v.z), mag_or_inf(v.w)));
            amax = max_row8(amax);
            const bool live = amax > 0.0f && amax < INFINITY;
            const float inv = live ? 32639.0f / amax : 0.0f;
            const int Xq[4] = {__float2int_rn(v.x * inv), __float2int_rn(v.y * inv), __float2int_rn(v.z * inv),
                               __float2int_rn(v.w * inv)};
            uint32_t wl = 0, wh = 0;
            int sum = 0;
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const int lo = ((Xq[c] + 128) & 255) - 128, hi = (Xq[c] - lo) >> 8;
                wl |= (uint32_t)(lo & 255) << (8 * c);
                wh |= (uint32_t)(hi & 255) << (8 * c);
                sum += Xq[c];
            }
            xl_lds[i] = wl;
            xh_lds[i] = wh;
            sum = isum_row8(sum);
            if ((i & 7) == 0) {
                const float sc = fixed_scale(amax, 32639.0f);
                sx_lds[i >> 3] = sc;
                sxs_lds[i >> 3] = sc * (float)sum;
            }
        }
        __syncthreads();
    }
    if (nrows <= 0) return;
    const int sub = lane % L, rl = lane / L, row = row0 + rl;
    const bool active = rl < nrows;
    const int units = (k / Q::BLOCK_ELEMS) * Q::UNITS;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the rows landed (this wave's own data)
    float total = 0.0f;
    for (int sl = 0; sl < S; sl++) {
        const size_t pair = sl < k_used ? (size_t)t * k_used + sl : (size_t)P + t;
        const uint32_t *xlp = OWN_PREP ? xl_lds + (size_t)sl * kw : xq.xl + pair * kw;
        const uint32_t *xhp = OWN_PREP ? xh_lds + (size_t)sl * kw : xq.xh + pair * kw;
        const float *sxp = OWN_PREP ? sx_lds + (size_t)sl * kb : xq.sx + pair * kb;
        const float *sxsp = OWN_PREP ? sxs_lds + (size_t)sl * kb : xq.sxs + pair * kb;
        const uint8_t *rpa = ra + (size_t)sl * slot_lds + (size_t)rl * row_bytes;
        float acc = 0.0f;
        if (active) {
            for (int u = sub; u < units; u += L) {
                const int b = u / Q::UNITS, ub = u % Q::UNITS;
                const int el = b * Q::BLOCK_ELEMS + Q::elem_base(ub);  // a multiple of 32
                uint32_t xl[XW], xh[XW];
                float sx[NS], sxs[NS];
#pragma unroll
                for (int i = 0; i < XW; i += 4) {
                    const uint4 lw = *(const uint4 *)(xlp + el / 4 + i), hw = *(const uint4 *)(xhp + el / 4 + i);
                    xl[i] = lw.x, xl[i + 1] = lw.y, xl[i + 2] = lw.z, xl[i + 3] = lw.w;
                    xh[i] = hw.x, xh[i + 1] = hw.y, xh[i + 2] = hw.z, xh[i + 3] = hw.w;
                }
#pragma unroll
                for (int i = 0; i < NS; i++) sx[i] = sxp[el / 32 + i], sxs[i] = sxsp[el / 32 + i];
                acc += Q::dot8(table, rpa + (size_t)b * Q::BLOCK_BYTES, ub, xl, xh, sx, sxs);
            }
        }
        for (int off = L >> 1; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
        total = sl < k_used ? fmaf(acc, wts[t * k_used + sl], total) : total + acc;
    }
    if (sub == 0 && active) y[(size_t)t * n + row] = total;
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

// h[i] = silu(g[i]) * u[i], both clamped first when limit > 0  (the shared expert's activation; the decoder's)
__global__ __launch_bounds__(256) void swiglu_rows(const float *__restrict__ g, const float *__restrict__ u,
                                                    float *__restrict__ h, size_t total, float limit) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
        h[i] = swiglu(g[i], u[i], limit);
}

// g[i] = silu(g[i]) * u[i] in place (gate and up results of the grouped GEMM, in front of the down projection)
__global__ __launch_bounds__(256) void swiglu_in_place(float *__restrict__ g, const float *__restrict__ u, size_t total,
                                                        float limit) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
        g[i] = swiglu(g[i], u[i], limit);
}

}  // namespace jq
