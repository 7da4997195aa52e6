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

// x[r, :] += res[r, :] when res is given (the residual add of the layer before), then
// out[r, :] = x[r, :] / sqrt(mean(x[r, :]^2) + eps) * w.  One workgroup of 1024 per row,
// float4 per thread, the row kept in registers between the two passes (h <= 8192),
// so a 4096-wide row costs one memory round trip instead of sixteen.
__global__ __launch_bounds__(1024) void rmsnorm_rows(float *__restrict__ x, const float *__restrict__ res,
                                                      const float *__restrict__ w, float eps,
                                                      float *__restrict__ out, int h) {
    __shared__ float red[16];
    float *xr = x + (size_t)blockIdx.x * h;
    const float *rr = res ? res + (size_t)blockIdx.x * h : nullptr;
    const int nv = h >> 2;  // h % 4 == 0
    float4 keep[2];
    float ss = 0.0f;
    int slot = 0;
    for (int c = threadIdx.x; c < nv; c += 1024, slot++) {
        float4 v = ((const float4 *)xr)[c];
        if (rr) {
            const float4 r = ((const float4 *)rr)[c];
            v.x += r.x, v.y += r.y, v.z += r.z, v.w += r.w;
            ((float4 *)xr)[c] = v;
        }
        if (slot < 2) keep[slot] = v;
        ss = fmaf(v.x, v.x, ss), ss = fmaf(v.y, v.y, ss), ss = fmaf(v.z, v.z, ss), ss = fmaf(v.w, v.w, ss);
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)h + eps);
    slot = 0;
    for (int c = threadIdx.x; c < nv; c += 1024, slot++) {
        const float4 v = slot < 2 ? keep[slot] : ((const float4 *)xr)[c];
        const float4 g = ((const float4 *)w)[c];
        ((float4 *)(out + (size_t)blockIdx.x * h))[c] = float4{v.x * inv * g.x, v.y * inv * g.y, v.z * inv * g.z, v.w * inv * g.w};
    }
}

// Per-head RMSNorm over head_dim then half-split rotary embedding at position
// pos0 + t, one wave per (token, head) over the q heads, the k heads and the v heads of
// a token: q is rewritten in place, k goes normed and rotated straight into the K
// cache, v is copied into the V cache.  inv_freq_i = theta^(-2i/d); pairs (i, i + d/2)
// (reference: src/quantized_qwen3_moe.rs:237-262,345-364; closed form in its test :867-895).
// cache layout [kv_head, n_ctx, d]; *pos_ptr is the number of tokens already cached.  A token's q, k and v
// heads start qs, ks and vs floats after the previous token's (the three may be parts of one product's rows).
__global__ __launch_bounds__(64) void qkv_norm_rope_cache(float *__restrict__ q, const float *__restrict__ k,
                                                           const float *__restrict__ v, const float *__restrict__ wq,
                                                           const float *__restrict__ wk, float eps, int n_head, int n_kv,
                                                           int d, const int *__restrict__ pos_ptr, float theta,
                                                           float *__restrict__ kc, float *__restrict__ vc, int n_ctx,
                                                           int qs, int ks, int vs) {
    const int per = n_head + 2 * n_kv;
    const int t = blockIdx.x / per, j = blockIdx.x % per, lane = threadIdx.x;
    const int pos = *pos_ptr + t;
    if (j >= n_head + n_kv) {  // v head: plain copy
        const int hd = j - n_head - n_kv;
        const float *src = v + (size_t)t * vs + (size_t)hd * d;
        float *dst = vc + ((size_t)hd * n_ctx + pos) * d;
        for (int c = lane; c < d; c += 64) dst[c] = src[c];
        return;
    }
    const bool is_q = j < n_head;
    const int hd = is_q ? j : j - n_head;
    const float *src = is_q ? q + (size_t)t * qs + (size_t)hd * d : k + (size_t)t * ks + (size_t)hd * d;
    float *dst = is_q ? q + (size_t)t * qs + (size_t)hd * d : kc + ((size_t)hd * n_ctx + pos) * d;
    const float *w = is_q ? wq : wk;
    float ss = 0.0f;
    for (int c = lane; c < d; c += 64) ss = fmaf(src[c], src[c], ss);
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
    const int half = d / 2;
    for (int i = lane; i < half; i += 64) {
        const float a = src[i] * inv * w[i], b = src[i + half] * inv * w[i + half];
        const float freq = 1.0f / powf(theta, (float)(2 * i) / (float)d);
        const float ang = (float)pos * freq, c = cosf(ang), s = sinf(ang);
        dst[i] = a * c - b * s;
        dst[i + half] = a * s + b * c;
    }
}

// One workgroup per (token, query head): softmax(q . K^T / sqrt(d)) . V over the
// keys 0 .. pos0 + t (causal), K/V of head hq / (n_head / n_kv)
// (reference: src/quantized_qwen3_moe.rs:366-379; mask :776-789).  The keys go by in chunks of
// AR_CHUNK with a running maximum and sum (each chunk's scores wait in LDS, the value sums are rescaled
// when the maximum moves), so the LDS a launch needs does not grow with the context.  d <= 4 * 256.
constexpr int AR_CHUNK = 1024, AR_MAX_D = 1024;

__global__ __launch_bounds__(256) void attention_rows(const float *__restrict__ q, const float *__restrict__ kc,
                                                       const float *__restrict__ vc, float *__restrict__ out,
                                                       int n_head, int n_kv, int d, const int *__restrict__ pos_ptr,
                                                       int n_ctx, float sqrt_d, int q_stride) {
    extern __shared__ float sm[];  // q[d], scores[AR_CHUNK], red[16]
    const int t = blockIdx.x / n_head, hq = blockIdx.x % n_head;
    const int kvh = hq / (n_head / n_kv), n_keys = *pos_ptr + t + 1;
    float *qs = sm, *sc = sm + d, *red = sm + d + AR_CHUNK;
    const float *qp = q + (size_t)t * q_stride + (size_t)hq * d;  // a token's heads start q_stride floats apart
    for (int c = threadIdx.x; c < d; c += blockDim.x) qs[c] = qp[c];
    __syncthreads();
    const float *kb = kc + (size_t)kvh * n_ctx * d, *vb = vc + (size_t)kvh * n_ctx * d;
    float m_run = -INFINITY, l_run = 0.0f, acc[AR_MAX_D / 256] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int j0 = 0; j0 < n_keys; j0 += AR_CHUNK) {
        const int nj = min(AR_CHUNK, n_keys - j0);
        float mx = -INFINITY;
        for (int j = threadIdx.x; j < nj; j += blockDim.x) {
            const float *kr = kb + (size_t)(j0 + j) * d;
            float a = 0.0f;
            for (int c = 0; c < d; c += 4) {
                const float4 kv = ld<float4>((const uint8_t *)(kr + c));
                a = fmaf(qs[c], kv.x, a);
                a = fmaf(qs[c + 1], kv.y, a);
                a = fmaf(qs[c + 2], kv.z, a);
                a = fmaf(qs[c + 3], kv.w, a);
            }
            a = a / sqrt_d;  // the reference divides by sqrt(head_dim) (src/embedding.rs:386)
            sc[j] = a;
            mx = fmaxf(mx, a);
        }
        mx = wave_max(mx);
        __syncthreads();  // the previous chunk's readers of red are done
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = mx;
        __syncthreads();
        for (int i = 0; i < (int)(blockDim.x >> 6); i++) mx = fmaxf(mx, red[i]);
        const float m_new = fmaxf(m_run, mx), rescale = expf(m_run - m_new);  // exp(-inf) = 0 in front of the first chunk
        float sum = 0.0f;
        for (int j = threadIdx.x; j < nj; j += blockDim.x) {
            const float e = expf(sc[j] - m_new);
            sc[j] = e;
            sum += e;
        }
        sum = block_sum(sum, red);
        l_run = fmaf(l_run, rescale, sum);
        m_run = m_new;
        __syncthreads();
#pragma unroll
        for (int i = 0; i < AR_MAX_D / 256; i++) {
            const int c = threadIdx.x + 256 * i;
            if (c >= d) break;
            float a = acc[i] * rescale;
            for (int j = 0; j < nj; j++) a = fmaf(sc[j], vb[(size_t)(j0 + j) * d + c], a);
            acc[i] = a;
        }
        __syncthreads();  // sc is rewritten by the next chunk
    }
#pragma unroll
    for (int i = 0; i < AR_MAX_D / 256; i++) {
        const int c = threadIdx.x + 256 * i;
        if (c < d) out[((size_t)t * n_head + hq) * d + c] = acc[i] / l_run;
    }
}

// The same attention for a step of many tokens, on the f32 matrix cores.  One workgroup per (tile of 16
// tokens, KV head), one wave per query head of that KV head (G = n_head / n_kv waves), so the G heads
// share every K and V row the workgroup stages.  Keys go by in tiles of 16 through LDS (the next tile's
// rows travel into registers while the current one is multiplied); per tile and wave
//   S^T = K Q^T   (16 keys x 16 tokens; 32 v_mfma_f32_16x16x4_f32 over the D = 128 head dimensions),
//   running maximum and sum per token, p = exp(s - max)   (online softmax, keys after a token masked),
//   O += P V      (32 more, 8 tiles of 16 dimensions)
// Lane (n = lane % 16, g = lane / 16) holds S^T[key 4 g + j][token n], j < 4, which is the A operand of
// P V as it stands when the product's inner index g stands for key 4 g + j in step j on both sides; the
// outputs come out as O[token 4 g + j][dimension], so a token's rescaling factor is fetched from the lane
// that holds its statistics.  Scores are divided by sqrt(d) as the reference does (src/embedding.rs:386).
constexpr int AT_PAD = 4;  // floats a staged row is longer than D: 16 rows then fall into different banks

// KS = 2 splits a tile's keys between two sets of G waves (key tiles of even and odd number), each with a
// running maximum, sum and output of its own, merged through LDS at the end: the workgroups of the last
// tokens, which walk the most key tiles and set the time of a causal prefill, take half as many steps.
template <int D, int G, int KS>
__global__ __launch_bounds__(64 * G * KS) void attention_tiles(const float *__restrict__ q, const float *__restrict__ kc,
                                                               const float *__restrict__ vc, float *__restrict__ out,
                                                               int T, int n_head, const int *__restrict__ pos_ptr,
                                                               int n_ctx, float sqrt_d, int q_stride) {
    static_assert(KS == 1 || KS == 2, "one or two key splits");
    constexpr int NT = 64 * G, STRIDE = D + AT_PAD, PIECES = 16 * (D / 4), PER = (PIECES + NT - 1) / NT;
    constexpr int MERGE = KS == 2 ? G * 64 * (D / 4 + 2) : 0;  // floats: a split's outputs, maximum and sum per lane
    constexpr int STAGE = 2 * KS * 16 * STRIDE;                 // the key and value tile of each split
    // the merge reuses the tiles' memory: every wave has left the loop by then
    __shared__ __attribute__((aligned(16))) float lds[STAGE > MERGE ? STAGE : MERGE];
    static_assert(sizeof(float) * (STAGE > MERGE ? STAGE : MERGE) <= 65536, "static LDS");
    const int lane = threadIdx.x & 63, wave_all = threadIdx.x >> 6, wave = wave_all % G, sp = wave_all / G;
    const int tid = threadIdx.x - NT * sp;  // within the split's G waves, which stage the split's tiles
    const int n = lane & 15, g = lane >> 4;
    float *ks = lds + sp * 16 * STRIDE, *vs = lds + (KS + sp) * 16 * STRIDE, *merge = lds;
    const int t0 = 16 * (int)blockIdx.x, kvh = blockIdx.y, hq = kvh * G + wave, pos0 = *pos_ptr;
    const int last_key = pos0 + min(t0 + 15, T - 1);        // the last key any token of the tile may see
    const int n_tiles = last_key / 16 + 1, n_steps = (n_tiles + KS - 1) / KS;
    const float *kb = kc + (size_t)kvh * n_ctx * D, *vb = vc + (size_t)kvh * n_ctx * D;

    typedef float f4 __attribute__((ext_vector_type(4)));
    // this lane's share of Q^T as B operands: token n, dimensions 4 s + g
    float qr[D / 4];
    {
        const float *qp = q + (size_t)min(t0 + n, T - 1) * q_stride + (size_t)hq * D + g;  // tokens q_stride floats apart
#pragma unroll
        for (int s_ = 0; s_ < D / 4; s_++) qr[s_] = qp[4 * s_];
    }
    f4 o[D / 16];
#pragma unroll
    for (int dt = 0; dt < D / 16; dt++) o[dt] = f4{0.f, 0.f, 0.f, 0.f};
    float mx = -INFINITY, sum = 0.0f;                       // of token n (the same in the four lanes that hold it)

    float4 kpre[PER], vpre[PER];
    auto fetch = [&](int tile) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int piece = tid + NT * i, row = piece / (D / 4), c4 = piece % (D / 4), key = 16 * tile + row;
            kpre[i] = vpre[i] = float4{0.f, 0.f, 0.f, 0.f};  // rows after the last key: the cache holds nothing there
            if (piece < PIECES && key <= last_key) {
                kpre[i] = *(const float4 *)(kb + (size_t)key * D + 4 * c4);
                vpre[i] = *(const float4 *)(vb + (size_t)key * D + 4 * c4);
            }
        }
    };
    fetch(sp);
    for (int step = 0; step < n_steps; step++) {
        const int tile = KS * step + sp;  // past the last tile (the odd split, in the last step): all keys masked
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int piece = tid + NT * i, row = piece / (D / 4), c4 = piece % (D / 4);
            if (piece < PIECES) {
                *(float4 *)(ks + row * STRIDE + 4 * c4) = kpre[i];
                *(float4 *)(vs + row * STRIDE + 4 * c4) = vpre[i];
            }
        }
        __syncthreads();
        if (step + 1 < n_steps) fetch(tile + KS);
        if (tile < n_tiles) {
            // S^T: keys 16 tile + (4 g + j) x token n
            f4 st = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s_ = 0; s_ < D / 4; s_++)
                st = __builtin_amdgcn_mfma_f32_16x16x4f32(ks[n * STRIDE + 4 * s_ + g], qr[s_], st, 0, 0, 0);
            float p[4], tmax = -INFINITY;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int key = 16 * tile + 4 * g + j;
                p[j] = key <= pos0 + t0 + n ? st[j] / sqrt_d : -INFINITY;
                tmax = fmaxf(tmax, p[j]);
            }
            tmax = max_xor32(max_xor16(tmax));
            // a token that sees none of this tile's keys (the odd split's first tile may lie past a token's
            // last key) keeps its state: exp(-inf - -inf) would be NaN
            const float mnew = fmaxf(mx, tmax), rescale = mnew == -INFINITY ? 1.0f : expf(mx - mnew);
            float tsum = 0.0f;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                p[j] = mnew == -INFINITY ? 0.0f : expf(p[j] - mnew);
                tsum += p[j];
            }
            tsum = sum_xor32(sum_xor16(tsum));
            sum = fmaf(sum, rescale, tsum);
            mx = mnew;
            // O rows are tokens 4 g + j: their factors live in the lanes of those tokens
            float rs[4];
#pragma unroll
            for (int j = 0; j < 4; j++) rs[j] = __shfl(rescale, 4 * g + j, 64);
#pragma unroll
            for (int dt = 0; dt < D / 16; dt++) {
                f4 acc = f4{o[dt][0] * rs[0], o[dt][1] * rs[1], o[dt][2] * rs[2], o[dt][3] * rs[3]};
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc = __builtin_amdgcn_mfma_f32_16x16x4f32(p[j], vs[(4 * g + j) * STRIDE + 16 * dt + n], acc, 0, 0, 0);
                o[dt] = acc;
            }
        }
        __syncthreads();
    }
    if constexpr (KS == 2) {
        // the odd split hands its state over; the even split (which always holds key 0) rescales both to the
        // common maximum
        float *mine = merge + (size_t)(wave * 64 + lane) * (D / 4 + 2);
        if (sp == 1) {
#pragma unroll
            for (int dt = 0; dt < D / 16; dt++)
#pragma unroll
                for (int j = 0; j < 4; j++) mine[4 * dt + j] = o[dt][j];
            mine[D / 4] = mx, mine[D / 4 + 1] = sum;
        }
        __syncthreads();
        if (sp == 1) return;
        const float m1 = mine[D / 4], s1 = mine[D / 4 + 1];
        const float mnew = fmaxf(mx, m1), f0 = expf(mx - mnew), f1 = m1 == -INFINITY ? 0.0f : expf(m1 - mnew);
        sum = sum * f0 + s1 * f1;
        float F0[4], F1[4];
#pragma unroll
        for (int j = 0; j < 4; j++) F0[j] = __shfl(f0, 4 * g + j, 64), F1[j] = __shfl(f1, 4 * g + j, 64);
#pragma unroll
        for (int dt = 0; dt < D / 16; dt++)
#pragma unroll
            for (int j = 0; j < 4; j++) o[dt][j] = o[dt][j] * F0[j] + mine[4 * dt + j] * F1[j];
    }
    float inv[4];
#pragma unroll
    for (int j = 0; j < 4; j++) inv[j] = 1.0f / __shfl(sum, 4 * g + j, 64);
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int t = t0 + 4 * g + j;
        if (t >= T) continue;
        float *op = out + ((size_t)t * n_head + hq) * D + n;
#pragma unroll
        for (int dt = 0; dt < D / 16; dt++) op[16 * dt] = o[dt][j] * inv[j];
    }
}

// *pos = p, and the rotary angles of the T positions p .. p + T - 1 of a step: cs[t][i] = (cos, sin) of
// (p + t) * theta^(-2i/d), i < d/2 — the arithmetic of qkv_norm_rope_cache, done once a step for the
// attention kernel that applies head norm and rotation itself.
__global__ __launch_bounds__(256) void rope_table(int *pos, int p, int T, int d, float theta, float2 *__restrict__ cs) {
    if (threadIdx.x == 0) *pos = p;
    const int half = d / 2;
    for (int e = threadIdx.x; e < T * half; e += blockDim.x) {
        const int t = e / half, i = e % half;
        const float freq = 1.0f / powf(theta, (float)(2 * i) / (float)d);
        const float ang = (float)(p + t) * freq;
        cs[e] = float2{cosf(ang), sinf(ang)};
    }
}

// One head row held by 16 lanes (lane `sub` has elements 4 sub + 64 i + c, i < D / 64, c < 4):
// RMSNorm over the head with weight w, then the half-split rotation by the angles cs[0 .. D/2)
// (reference: src/quantized_qwen3_moe.rs:237-262,345-364).  Same arithmetic as qkv_norm_rope_cache.
template <int D>
__device__ __forceinline__ void head_norm_rope(float4 (&x)[D / 64], const float *__restrict__ w, float eps,
                                               const float2 *__restrict__ cs, int sub) {
    constexpr int QI = D / 64;
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < QI; i++)
        ss = fmaf(x[i].x, x[i].x, ss), ss = fmaf(x[i].y, x[i].y, ss), ss = fmaf(x[i].z, x[i].z, ss), ss = fmaf(x[i].w, x[i].w, ss);
    ss = sum_row16(ss);
    const float inv = 1.0f / sqrtf(ss / (float)D + eps);
    float v[QI][4];
#pragma unroll
    for (int i = 0; i < QI; i++) {
        const float4 g = *(const float4 *)(w + 4 * sub + 64 * i);
        v[i][0] = x[i].x * inv * g.x, v[i][1] = x[i].y * inv * g.y, v[i][2] = x[i].z * inv * g.z, v[i][3] = x[i].w * inv * g.w;
    }
    if constexpr (QI >= 2) {  // element e < D/2 and its partner e + D/2 sit in the same lane
#pragma unroll
        for (int i = 0; i < QI / 2; i++) {
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const float2 r = cs[4 * sub + 64 * i + c];
                const float a = v[i][c], b = v[i + QI / 2][c];
                v[i][c] = a * r.x - b * r.y;
                v[i + QI / 2][c] = a * r.y + b * r.x;
            }
        }
    } else {  // D = 64: the partner is 8 lanes away
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const float other = dpp_f<0x128>(v[0][c]);  // row_ror:8
            const bool low = sub < 8;
            const float2 r = cs[(4 * sub + c) & 31];
            const float a = low ? v[0][c] : other, b = low ? other : v[0][c];
            v[0][c] = low ? a * r.x - b * r.y : a * r.y + b * r.x;
        }
    }
#pragma unroll
    for (int i = 0; i < QI; i++) x[i] = float4{v[i][0], v[i][1], v[i][2], v[i][3]};
}

// Decode-shaped attention (few query tokens, long cache), split over the keys so the
// whole chip works on it: one workgroup per (token, query head, chunk of ATT_CHUNK keys)
// computes its chunk's scores, their maximum m, l = sum exp(s - m) and the unnormalised
// sum exp(s - m) v, and writes (m, l, acc[d]) to part[(t*n_head + hq)*n_chunks + chunk];
// attention_merge rescales the chunks to the common maximum and divides by the total.
// 16 lanes per key (4 keys per wave step), head_dim 64, 128 or 256.  Chunks past the causal
// limit write l = 0 and are skipped by the merge.
// q, k, v are the step's raw projections: the kernel applies the per-head RMSNorm and the rotation to
// its query row and to the keys of the step's own tokens (positions pos0 and up, not in the cache
// yet) itself, and the workgroups of a kv head's first query head store the new key and value rows
// into the cache for the steps to come.
constexpr int ATT_CHUNK = 64;

template <int D>  // head_dim: 64, 128 or 256
__global__ __launch_bounds__(256) void attention_split(int n_head, int n_kv, int n_chunks, int n_tri, int pos0, int n_ctx,
                                                        const float *__restrict__ q, const float *__restrict__ k,
                                                        const float *__restrict__ v, float *kc, float *vc,
                                                        const float *__restrict__ wq, const float *__restrict__ wk,
                                                        const float2 *__restrict__ cs, float *__restrict__ part,
                                                        float eps, float sqrt_d) {
    // (what the first loads need comes first in the argument list: the leading 16 words of arguments
    // arrive in scalar registers with the wave, the rest by a scalar load)
    constexpr int d = D, QI = D / 64;          // float4 of q (and of a key) per lane
    constexpr int NG = D / 4, KP = 256 / NG;   // column groups of four, key parts
    constexpr int VI = ATT_CHUNK / KP;         // keys per thread in the value sum
    __shared__ float sc[ATT_CHUNK];
    __shared__ float4 accs[256];               // [key part][column group]
    // Workgroup ids 8 apart run on the same XCD (ids go round the 8 XCDs in turn) and share its L2: the
    // query heads of one KV head and chunk read the same key and value rows, so they get ids 8 apart and
    // the rows come from HBM once.  id = x + 8 (g + group y): g the query head within its group, 8 y + x
    // the (token, KV head, chunk) triple; ids past the last triple have nothing to do.
    const int group = n_head / n_kv;
    const int tri = 8 * ((int)(blockIdx.x >> 3) / group) + (int)(blockIdx.x & 7);
    if (tri >= n_tri) return;
    const int chunk = tri % n_chunks, kvh = (tri / n_chunks) % n_kv, t = tri / (n_chunks * n_kv);
    const int hq = kvh * group + (int)(blockIdx.x >> 3) % group, n_keys = pos0 + t + 1;
    const int j0 = chunk * ATT_CHUNK, nj = min(ATT_CHUNK, n_keys - j0);
    float *po = part + ((size_t)(t * n_head + hq) * n_chunks + chunk) * (d + 2);
    if (nj <= 0) {
        if (threadIdx.x == 0) po[0] = -INFINITY, po[1] = 0.0f;
        return;
    }
    const bool keeper = hq % group == 0;  // stores this token's new key and value rows
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, sub = lane & 15, kq = lane >> 4;
    const float *qp = q + ((size_t)t * n_head + hq) * d;
    const int cg = threadIdx.x % NG, kp = threadIdx.x / NG;
    // every global read of this workgroup is issued here, before any of them is needed: the query slice,
    // this lane's slices of its four keys, this thread's VI value rows (rows past the chunk's end are
    // read from its last valid row and not used); rows of this step's tokens come from k and v
    float4 qv[QI], kv[4][QI], vv[VI];
#pragma unroll
    for (int i = 0; i < QI; i++) qv[i] = *(const float4 *)(qp + 4 * sub + 64 * i);
#pragma unroll
    for (int s = 0; s < 4; s++) {
        const int jg = j0 + min(wave * 4 + kq + 16 * s, nj - 1);
        const float *row = jg >= pos0 ? k + ((size_t)(jg - pos0) * n_kv + kvh) * d : kc + ((size_t)kvh * n_ctx + jg) * d;
#pragma unroll
        for (int i = 0; i < QI; i++) kv[s][i] = *(const float4 *)(row + 4 * sub + 64 * i);
    }
#pragma unroll
    for (int s = 0; s < VI; s++) {
        const int jg = j0 + min(kp + KP * s, nj - 1);
        const float *row = jg >= pos0 ? v + ((size_t)(jg - pos0) * n_kv + kvh) * d : vc + ((size_t)kvh * n_ctx + jg) * d;
        vv[s] = *(const float4 *)(row + 4 * cg);
    }
    head_norm_rope<D>(qv, wq, eps, cs + (size_t)t * (d / 2), sub);
#pragma unroll
    for (int s = 0; s < 4; s++) {
        const int jg = j0 + min(wave * 4 + kq + 16 * s, nj - 1);
        if (jg >= pos0) {  // a key of this step: the same for the 16 lanes that hold it
            head_norm_rope<D>(kv[s], wk, eps, cs + (size_t)(jg - pos0) * (d / 2), sub);
            if (keeper && jg == pos0 + t) {
                float *dst = kc + ((size_t)kvh * n_ctx + jg) * d;
#pragma unroll
                for (int i = 0; i < QI; i++) *(float4 *)(dst + 4 * sub + 64 * i) = kv[s][i];
            }
        }
    }

#pragma unroll
    for (int s = 0; s < 4; s++) {
        const int j = wave * 4 + kq + 16 * s;
        float acc = 0.0f;
#pragma unroll
        for (int i = 0; i < QI; i++) {
            acc = fmaf(qv[i].x, kv[s][i].x, acc), acc = fmaf(qv[i].y, kv[s][i].y, acc);
            acc = fmaf(qv[i].z, kv[s][i].z, acc), acc = fmaf(qv[i].w, kv[s][i].w, acc);
        }
        acc = sum_row16(acc);
        if (sub == 0) sc[j] = j < nj ? acc / sqrt_d : -INFINITY;
    }
    __syncthreads();
    float mx = sc[lane];  // ATT_CHUNK == 64: every wave holds the whole chunk
    mx = wave_max(mx);
    const float e = expf(sc[lane] - mx);  // exp(-inf) = 0 for the masked tail
    const float l = wave_sum(e);
    __syncthreads();
    if (wave == 0) sc[lane] = e;
    __syncthreads();
    // acc[c] = sum_j e_j v[j, c]: thread (column group, key part) over the keys kp, kp + KP, ...
    float4 acc = float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < VI; s++) {
        const int j = kp + KP * s;
        const float e_j = j < nj ? sc[j] : 0.0f;
        acc.x = fmaf(e_j, vv[s].x, acc.x), acc.y = fmaf(e_j, vv[s].y, acc.y);
        acc.z = fmaf(e_j, vv[s].z, acc.z), acc.w = fmaf(e_j, vv[s].w, acc.w);
    }
    accs[kp * NG + cg] = acc;
    __syncthreads();
    if (threadIdx.x < NG) {
        float4 a = accs[threadIdx.x];
        for (int pt = 1; pt < KP; pt++) {
            const float4 o = accs[pt * NG + threadIdx.x];
            a.x += o.x, a.y += o.y, a.z += o.z, a.w += o.w;
        }
        po[2 + 4 * threadIdx.x + 0] = a.x, po[2 + 4 * threadIdx.x + 1] = a.y;
        po[2 + 4 * threadIdx.x + 2] = a.z, po[2 + 4 * threadIdx.x + 3] = a.w;
    }
    if (threadIdx.x == 0) po[0] = mx, po[1] = l;
    if (keeper) {  // this token's value row into the cache (its key row went in above)
#pragma unroll
        for (int s = 0; s < VI; s++) {
            const int jg = j0 + min(kp + KP * s, nj - 1);
            if (jg == pos0 + t) *(float4 *)(vc + ((size_t)kvh * n_ctx + jg) * d + 4 * cg) = vv[s];
        }
    }
}

// out[(t, head), :] = sum_ch exp(m_ch - m) acc_ch / sum_ch exp(m_ch - m) l_ch over the chunks with keys.
// Every read of the partials is issued side by side (a thread per chunk for m and l, 16 chunks at a
// time for the sums): the kernel is a few round trips to memory long, whatever the chunk count.
__global__ __launch_bounds__(128) void attention_merge(const float *__restrict__ part, float *__restrict__ out, int d,
                                                        int n_chunks) {
    extern __shared__ float wch[];  // [n_chunks] maxima, then rescaling weights; [n_chunks] l
    float *lch = wch + n_chunks;
    const float *pp = part + (size_t)blockIdx.x * n_chunks * (d + 2);
    for (int ch = threadIdx.x; ch < n_chunks; ch += 128) {
        const float2 ml = *(const float2 *)(pp + (size_t)ch * (d + 2));
        wch[ch] = ml.x, lch[ch] = ml.y;
    }
    __syncthreads();
    float mx = -INFINITY;
    for (int ch = 0; ch < n_chunks; ch++) mx = fmaxf(mx, wch[ch]);
    __syncthreads();
    for (int ch = threadIdx.x; ch < n_chunks; ch += 128) wch[ch] = lch[ch] > 0.0f ? expf(wch[ch] - mx) : 0.0f;
    __syncthreads();
    float tot = 0.0f;
    for (int ch = 0; ch < n_chunks; ch++) tot = fmaf(lch[ch], wch[ch], tot);
    for (int c = threadIdx.x; c < d; c += 128) {
        float a = 0.0f;
        for (int ch0 = 0; ch0 < n_chunks; ch0 += 16) {
            float v[16];
#pragma unroll
            for (int j = 0; j < 16; j++) v[j] = pp[(size_t)min(ch0 + j, n_chunks - 1) * (d + 2) + 2 + c];
#pragma unroll
            for (int j = 0; j < 16; j++) {
                // a chunk past a token's last key holds no sums, only whatever the buffer held before: its
                // slots may be inf or NaN, and 0 * NaN is NaN, so such a chunk is left out, not weighted by 0
                const float wgt = ch0 + j < n_chunks ? wch[ch0 + j] : 0.0f;
                a = wgt > 0.0f ? fmaf(wgt, v[j], a) : a;
            }
        }
        out[(size_t)blockIdx.x * d + c] = a / tot;
    }
}

// out[i] = silu(gu[2i]) * gu[2i + 1]: the activation over a product with a row-paired gate|up matrix
__global__ __launch_bounds__(256) void swiglu_pairs(const float *__restrict__ gu, float *__restrict__ out, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const float2 v = ((const float2 *)gu)[i];
        out[i] = silu(v.x) * v.y;
    }
}

__global__ void set_int(int *p, int v) { *p = v; }

__global__ __launch_bounds__(256) void add_rows(const float *__restrict__ a, const float *__restrict__ b,
                                                 float *__restrict__ out, size_t total) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x)
        out[i] = a[i] + b[i];
}

// Index of the largest value; of equal values the LAST one, as the reference's
// greedy pick does (Iterator::max_by, src/engine.rs:2371-2378).  Two launches: ARGMAX_PARTS
// workgroups each find the pick of a contiguous slice, one workgroup picks among those.
constexpr int ARGMAX_PARTS = 256;

// (best, idx) over a workgroup; a later index wins among equal values.  Valid in thread 0.
__device__ __forceinline__ void argmax_last_block(float &best, int &idx, float *bv, int *bi) {
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
    }
}

__global__ __launch_bounds__(256) void argmax_last_parts(const float *__restrict__ v, int n, float *__restrict__ pv,
                                                         int *__restrict__ pi) {
    __shared__ float bv[4];
    __shared__ int bi[4];
    const int per = (n + (int)gridDim.x - 1) / (int)gridDim.x;
    const int lo = (int)blockIdx.x * per, hi = min(n, lo + per);
    float best = -INFINITY;
    int idx = -1;
    for (int i = lo + (int)threadIdx.x; i < hi; i += blockDim.x)
        if (v[i] >= best) {  // i increases within a thread: >= keeps the last
            best = v[i];
            idx = i;
        }
    argmax_last_block(best, idx, bv, bi);
    if (threadIdx.x == 0) pv[blockIdx.x] = best, pi[blockIdx.x] = idx;
}

__global__ __launch_bounds__(ARGMAX_PARTS) void argmax_last_merge(const float *__restrict__ pv, const int *__restrict__ pi,
                                                                  uint32_t *__restrict__ out) {
    __shared__ float bv[ARGMAX_PARTS / 64];
    __shared__ int bi[ARGMAX_PARTS / 64];
    float best = pv[threadIdx.x];
    int idx = pi[threadIdx.x];
    if (idx < 0) best = -INFINITY;  // an empty slice, or one of NaNs only
    argmax_last_block(best, idx, bv, bi);
    if (threadIdx.x == 0) out[0] = (uint32_t)(idx < 0 ? 0 : idx);
}

}  // namespace jq
