// Multi-head latent attention (DeepSeek-V2 / V3 / Kimi-K2) in its absorbed form, f32 throughout.
//
// The reference (src/quantized_deepseek2.rs:422-499) expands every new token's latent through the KV
// up-projection into per-head keys and values and caches those: n_head * (qk_nope + qk_rope +
// v_head_dim) floats a token (160 KB at V3 size), all of which a decode step reads back.  The same
// numbers come out of the latent itself: with W_k[h] (qk_nope x kv_lora_rank) and W_v[h] (v_head_dim x
// kv_lora_rank) the rows of the up-projection for head h,
//     q_nope[h] . (W_k[h] c_t)  =  (W_k[h]^T q_nope[h]) . c_t
//     sum_t p_t (W_v[h] c_t)    =  W_v[h] (sum_t p_t c_t)
// so the cache holds, per token, the normed latent c_t (kv_lora_rank) and the rotated shared key k_pe
// (qk_rope): 2.3 KB at V3 size, shared by all heads.  A step is
//   mla_rope_latent   rotate q_pe in place; norm the latent, rotate k_pe, append both to the cache
//   mla_absorb_q      q_abs[h] = W_k[h]^T q_nope[h]
//   mla_attention     scores over the cached latents, running softmax, o_lat[h] = sum p_t c_t, the
//                     context split over workgroups (partial maximum, sum and vector per split)
//   mla_merge         merge the splits into o_lat[h]
//   mla_vproj         ctx[h] = W_v[h] o_lat[h]
// around the quantized projections (q, kv_a, o), which run on the matmul kernels.
#pragma once
#include "kernels_graph.hpp"

namespace jq {

// grid (n_head + 1, S), one wave.  Workgroups x < n_head rotate the rope slice of q[s, x] in place
// (neighbouring pairs (2i, 2i+1), candle's rope_i; cs[p][i] = (cos, sin) of position p, pair i, already
// scaled by the YaRN mscale; reference :302-311).  Workgroup x == n_head norms the latent
// comp[s, 0:lkv] (RMSNorm, weight w) into lat[pos0 + s] and rotates comp[s, lkv:] into kpe[pos0 + s].
__device__ __forceinline__ void mla_rope_latent_wave(float *__restrict__ q, const float *__restrict__ comp,
                                                     const float *__restrict__ w, const float2 *__restrict__ cs,
                                                     float *__restrict__ lat, float *__restrict__ kpe, int n_head,
                                                     int nope, int rope, int lkv, int pos0, float eps, int bx, int s,
                                                     int lane) {
    const int half = rope >> 1;
    const float2 *c = cs + (size_t)(pos0 + s) * half;
    if (bx < n_head) {
        float *v = q + ((size_t)s * n_head + bx) * (nope + rope) + nope;
        for (int i = lane; i < half; i += 64) {
            const float a = v[2 * i], b = v[2 * i + 1];
            v[2 * i] = a * c[i].x - b * c[i].y;
            v[2 * i + 1] = a * c[i].y + b * c[i].x;
        }
        return;
    }
    const float *x = comp + (size_t)s * (lkv + rope);
    float ss = 0.0f;
    for (int i = lane; i < lkv; i += 64) ss = fmaf(x[i], x[i], ss);
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)lkv + eps);
    float *l = lat + (size_t)(pos0 + s) * lkv, *k = kpe + (size_t)(pos0 + s) * rope;
    for (int i = lane; i < lkv; i += 64) l[i] = x[i] * inv * w[i];
    for (int i = lane; i < half; i += 64) {
        const float a = x[lkv + 2 * i], b = x[lkv + 2 * i + 1];
        k[2 * i] = a * c[i].x - b * c[i].y;
        k[2 * i + 1] = a * c[i].y + b * c[i].x;
    }
}

__global__ __launch_bounds__(64) void mla_rope_latent(float *__restrict__ q, const float *__restrict__ comp,
                                                       const float *__restrict__ w, const float2 *__restrict__ cs,
                                                       float *__restrict__ lat, float *__restrict__ kpe, int n_head,
                                                       int nope, int rope, int lkv, int pos0, float eps) {
    mla_rope_latent_wave(q, comp, w, cs, lat, kpe, n_head, nope, rope, lkv, pos0, eps, (int)blockIdx.x, (int)blockIdx.y,
                         (int)threadIdx.x);
}

// q_abs[s, h, c] = sum_r q[s, h, r] * Wkv[h * (nope + vh) + r, c], r < nope.  grid (n_head, ceil(S / ST)),
// 512 threads: thread (row quarter, column group of CW) walks a quarter of the head's nope rows (the
// rows are read coalesced, once per ST tokens, whose query values wait in LDS); the four quarters sum
// through LDS.  CW = 4 (16-byte loads) needs lkv % 4 == 0 and lkv <= 512; CW = 1 any lkv <= 128.
constexpr int MLA_MAX_NOPE = 256, MLA_MAX_LKV = 512;
template <int ST, int CW>
__device__ __forceinline__ void mla_absorb_q_workgroup(const float *__restrict__ q, const float *__restrict__ Wkv,
                                                       float *__restrict__ qabs, int S, int n_head, int nope, int rope,
                                                       int vh, int lkv, int h, int s0) {
    __shared__ float qs[MLA_MAX_NOPE][ST];
    __shared__ float red[3][ST][128 * CW];
    const int qd = nope + rope;
    for (int e = threadIdx.x; e < nope * ST; e += 512) {
        const int r = e / ST, j = e % ST;
        qs[r][j] = s0 + j < S ? q[((size_t)(s0 + j) * n_head + h) * qd + r] : 0.0f;
    }
    __syncthreads();
    const float *W = Wkv + (size_t)h * (nope + vh) * lkv;
    const int part = threadIdx.x >> 7, c = (threadIdx.x & 127) * CW;
    const int r0 = part * ((nope + 3) >> 2), r1 = min(nope, r0 + ((nope + 3) >> 2));
    float acc[ST][CW];
#pragma unroll
    for (int j = 0; j < ST; j++)
#pragma unroll
        for (int i = 0; i < CW; i++) acc[j][i] = 0.0f;
    if (c < lkv) {
#pragma unroll 8
        for (int r = r0; r < r1; r++) {
            float wv[CW];
            if constexpr (CW == 4) {
                const float4 v = *(const float4 *)(W + (size_t)r * lkv + c);
                wv[0] = v.x, wv[1] = v.y, wv[2] = v.z, wv[3] = v.w;
            } else {
                wv[0] = W[(size_t)r * lkv + c];
            }
#pragma unroll
            for (int j = 0; j < ST; j++)
#pragma unroll
                for (int i = 0; i < CW; i++) acc[j][i] = fmaf(qs[r][j], wv[i], acc[j][i]);
        }
    }
    if (part > 0) {
#pragma unroll
        for (int j = 0; j < ST; j++)
#pragma unroll
            for (int i = 0; i < CW; i++) red[part - 1][j][c + i] = acc[j][i];
    }
    __syncthreads();
    if (part == 0 && c < lkv) {
#pragma unroll
        for (int j = 0; j < ST; j++)
#pragma unroll
            for (int i = 0; i < CW; i++) {
                const float v = acc[j][i] + red[0][j][c + i] + red[1][j][c + i] + red[2][j][c + i];
                if (s0 + j < S) qabs[((size_t)(s0 + j) * n_head + h) * lkv + c + i] = v;
            }
    }
}

template <int ST, int CW>
__global__ __launch_bounds__(512) void mla_absorb_q(const float *__restrict__ q, const float *__restrict__ Wkv,
                                                     float *__restrict__ qabs, int S, int n_head, int nope, int rope,
                                                     int vh, int lkv) {
    mla_absorb_q_workgroup<ST, CW>(q, Wkv, qabs, S, n_head, nope, rope, vh, lkv, (int)blockIdx.x, (int)blockIdx.y * ST);
}

// mla_rope_latent and mla_absorb_q of a single-token step as one launch: grid n_head + 1, 512 threads.  The
// first wave of workgroup x does what workgroup x of mla_rope_latent does (it touches the rope slice of
// q[x], the absorption reads the other slice); workgroup n_head has nothing else to do.
template <int CW>
__global__ __launch_bounds__(512) void mla_absorb_rope(float *__restrict__ q, const float *__restrict__ Wkv,
                                                        float *__restrict__ qabs, int n_head, int nope, int rope, int vh,
                                                        int lkv, const float *__restrict__ comp, const float *__restrict__ w,
                                                        const float2 *__restrict__ cs, float *__restrict__ lat,
                                                        float *__restrict__ kpe, int pos0, float eps) {
    if (threadIdx.x < 64)
        mla_rope_latent_wave(q, comp, w, cs, lat, kpe, n_head, nope, rope, lkv, pos0, eps, (int)blockIdx.x, 0, (int)threadIdx.x);
    if ((int)blockIdx.x == n_head) return;
    mla_absorb_q_workgroup<1, CW>(q, Wkv, qabs, 1, n_head, nope, rope, vh, lkv, (int)blockIdx.x, 0);
}

// Scores, running softmax and the weighted latent sum for G heads of one query token over one split of
// its context.  grid (n_head / G, n_split, S), four waves; wave w takes tokens t0 + w, t0 + w + 4, ... of
// the split: a lane holds LPL consecutive latent elements (and one rope element) of the token, loaded
// once for the G heads, and the same elements of every head's absorbed query; a score is the wave sum
// of the products.  The four waves' (maximum, sum, vector) merge through LDS into
// part[s, h, split] = {m, l, o[lkv]}, unnormalised.  lkv <= 64 LPL, rope <= 64.  Query token s sees
// cache tokens 0 .. pos0 + s (the causal mask of the reference, :875-889).
constexpr int MLA_SPLIT_MAX = 64;
template <int G, int LPL>
__global__ __launch_bounds__(256) void mla_attention(const float *__restrict__ qabs, const float *__restrict__ q,
                                                      const float *__restrict__ lat, const float *__restrict__ kpe,
                                                      float *__restrict__ part, int n_head, int nope, int rope, int lkv,
                                                      int pos0, int n_split, float scale) {
    __shared__ float wm[4][G], wl[4][G];
    __shared__ float wo[4][G][64 * LPL];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h0 = blockIdx.x * G, split = blockIdx.y, s = blockIdx.z;
    const int T = pos0 + s + 1, chunk = (T + n_split - 1) / n_split;
    const int t0 = split * chunk, t1 = min(T, t0 + chunk);
    const bool vec = lkv == 64 * LPL && LPL % 4 == 0;  // whole float4 loads
    const int e0 = lane * LPL;

    float qa[G][LPL], qp[G], m[G], l[G], o[G][LPL];
#pragma unroll
    for (int g = 0; g < G; g++) {
        const float *qv = qabs + ((size_t)s * n_head + h0 + g) * lkv;
#pragma unroll
        for (int i = 0; i < LPL; i++) qa[g][i] = e0 + i < lkv ? qv[e0 + i] : 0.0f, o[g][i] = 0.0f;
        qp[g] = lane < rope ? q[((size_t)s * n_head + h0 + g) * (nope + rope) + nope + lane] : 0.0f;
        m[g] = -INFINITY, l[g] = 0.0f;
    }
    for (int t = t0 + wave; t < t1; t += 4) {
        float c[LPL];
        const float *cv = lat + (size_t)t * lkv;
        bool loaded = false;
        if constexpr (LPL % 4 == 0) {
            if (vec) {
#pragma unroll
                for (int i = 0; i < LPL; i += 4) {
                    const float4 v = *(const float4 *)(cv + e0 + i);
                    c[i] = v.x, c[i + 1] = v.y, c[i + 2] = v.z, c[i + 3] = v.w;
                }
                loaded = true;
            }
        }
        if (!loaded) {
#pragma unroll
            for (int i = 0; i < LPL; i++) c[i] = e0 + i < lkv ? cv[e0 + i] : 0.0f;
        }
        const float kp = lane < rope ? kpe[(size_t)t * rope + lane] : 0.0f;
#pragma unroll
        for (int g = 0; g < G; g++) {
            float sc = qp[g] * kp;
#pragma unroll
            for (int i = 0; i < LPL; i++) sc = fmaf(qa[g][i], c[i], sc);
            sc = wave_sum(sc) * scale;
            const float mn = fmaxf(m[g], sc);
            const float a = __expf(m[g] - mn), p = __expf(sc - mn);  // the first token: a = exp(-inf) = 0
            l[g] = fmaf(l[g], a, p);
#pragma unroll
            for (int i = 0; i < LPL; i++) o[g][i] = fmaf(o[g][i], a, p * c[i]);
            m[g] = mn;
        }
    }
#pragma unroll
    for (int g = 0; g < G; g++) {
        if (lane == 0) wm[wave][g] = m[g], wl[wave][g] = l[g];
#pragma unroll
        for (int i = 0; i < LPL; i++) wo[wave][g][e0 + i] = o[g][i];
    }
    __syncthreads();
    for (int e = threadIdx.x; e < G * 64 * LPL; e += 256) {
        const int g = e / (64 * LPL), i = e % (64 * LPL);
        const float M = fmaxf(fmaxf(wm[0][g], wm[1][g]), fmaxf(wm[2][g], wm[3][g]));
        float ov = 0.0f, lv = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float f = wm[w][g] == -INFINITY ? 0.0f : __expf(wm[w][g] - M);  // a wave without tokens
            ov = fmaf(wo[w][g][i], f, ov);
            lv = fmaf(wl[w][g], f, lv);
        }
        float *p = part + (((size_t)s * n_head + h0 + g) * n_split + split) * (lkv + 2);
        if (i < lkv) p[2 + i] = ov;
        if (i == 0) p[0] = M, p[1] = lv;
    }
}

// The same scores and latent sums on the f32 matrix cores (v_mfma_f32_32x32x2_f32: exact f32 products,
// f32 sums), for the geometry every DeepSeek MLA model has: 512 latent + 64 rope elements, heads in
// groups of 32.  grid (n_head / 32, n_split, S), eight waves.  A tile is 32 heads x 32 tokens; the
// tokens' rows [latent | rope key] (576 floats) wait in LDS.
//   scores  = Q[32 x 576] . C^T[576 x 32]: wave w multiplies columns 72 w .. 72 w + 71 (36 steps of 2;
//             its slice of Q stays in 36 registers), the eight partial tiles sum through LDS;
//   softmax: 16 threads a head, two tokens each, running maximum and sum in registers;
//   o_lat  += P[32 x 32] . C[32 x 512]: wave w owns latent columns 64 w .. 64 w + 63 (two tiles of 32,
//             32 accumulator registers), 16 steps of 2 tokens.
// The next tile's rows are fetched into registers while a tile is worked on.  Output as mla_attention.
constexpr int MLA_M_LKV = 512, MLA_M_ROPE = 64, MLA_M_KT = MLA_M_LKV + MLA_M_ROPE, MLA_M_STRIDE = MLA_M_KT + 4;
typedef float mla_f16v __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(512) void mla_attention_mfma(const float *__restrict__ qabs, const float *__restrict__ q,
                                                           const float *__restrict__ lat, const float *__restrict__ kpe,
                                                           float *__restrict__ part, int n_head, int nope, int pos0,
                                                           int n_split, float scale) {
    __shared__ __attribute__((aligned(16))) float ct[32][MLA_M_STRIDE];
    __shared__ float sp[8][32][33];
    __shared__ float ps[32][33];
    __shared__ __attribute__((aligned(16))) float al[32];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 31, lk = lane >> 5;
    const int h0 = blockIdx.x * 32, split = blockIdx.y, s = blockIdx.z;
    const int T = pos0 + s + 1, chunk = (T + n_split - 1) / n_split;
    const int t0 = split * chunk, t1 = min(T, t0 + chunk);

    // 32 rows (tokens of a tile, or the heads' queries) x 144 pieces of 16 bytes (128 latent, 16 rope) = 9 a thread
    float4 pre[9];
    auto load_tile = [&](int tb) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 9; u++) {
            const int idx = tid + 512 * u, tok = idx / 144, f = idx % 144, t = tb + tok;
            if (t < t1) pre[u] = f < 128 ? *(const float4 *)(lat + (size_t)t * MLA_M_LKV + 4 * f)
                                         : *(const float4 *)(kpe + (size_t)t * MLA_M_ROPE + 4 * (f - 128));
            else pre[u] = float4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    };
    if (t0 < t1) load_tile(t0);
    // this wave's slice of the 32 heads' queries, element 72 wave + 2 ks + lk of head li, by way of LDS
    // (rows [absorbed query | rotated rope query] read whole, then picked apart)
    float qreg[36];
    {
#pragma unroll
        for (int u = 0; u < 9; u++) {
            const int idx = tid + 512 * u, i = idx / 144, f = idx % 144;
            const size_t row = (size_t)s * n_head + h0 + i;
            *(float4 *)&ct[i][4 * f] = f < 128 ? *(const float4 *)(qabs + row * MLA_M_LKV + 4 * f)
                                               : *(const float4 *)(q + row * (nope + MLA_M_ROPE) + nope + 4 * (f - 128));
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < 36; ks++) qreg[ks] = ct[li][72 * wave + 2 * ks + lk];
        __syncthreads();
    }
    mla_f16v o[2];
#pragma unroll
    for (int nt = 0; nt < 2; nt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[nt][r] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;  // of head tid / 16, the same in its 16 threads

    for (int tb = t0; tb < t1; tb += 32) {
        if (tb > t0) __syncthreads();  // every wave is done with the rows of the tile before
#pragma unroll
        for (int u = 0; u < 9; u++) {
            const int idx = tid + 512 * u, tok = idx / 144, f = idx % 144;
            *(float4 *)&ct[tok][4 * f] = pre[u];
        }
        __syncthreads();
        if (tb + 32 < t1) load_tile(tb + 32);

        mla_f16v sc;
#pragma unroll
        for (int r = 0; r < 16; r++) sc[r] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 36; ks++)
            sc = __builtin_amdgcn_mfma_f32_32x32x2f32(qreg[ks], ct[li][72 * wave + 2 * ks + lk], sc, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 16; r++) sp[wave][8 * (r >> 2) + 4 * lk + (r & 3)][li] = sc[r];  // row = head, column = token
        __syncthreads();
        {
            const int i = tid >> 4, j = 2 * (tid & 15);
            float s0 = 0.0f, s1 = 0.0f;
#pragma unroll
            for (int w = 0; w < 8; w++) s0 += sp[w][i][j], s1 += sp[w][i][j + 1];
            s0 = tb + j < t1 ? s0 * scale : -INFINITY;
            s1 = tb + j + 1 < t1 ? s1 * scale : -INFINITY;
            const float mn = fmaxf(m_run, max_row16(fmaxf(s0, s1)));  // finite: token tb is inside the split
            const float p0 = __expf(s0 - mn), p1 = __expf(s1 - mn), a = __expf(m_run - mn);
            l_run = fmaf(l_run, a, sum_row16(p0 + p1));
            m_run = mn;
            ps[i][j] = p0, ps[i][j + 1] = p1;
            if ((tid & 15) == 0) al[i] = a;
        }
        __syncthreads();
#pragma unroll
        for (int b = 0; b < 4; b++) {
            const float4 a = *(const float4 *)&al[8 * b + 4 * lk];
#pragma unroll
            for (int nt = 0; nt < 2; nt++) o[nt][4 * b] *= a.x, o[nt][4 * b + 1] *= a.y, o[nt][4 * b + 2] *= a.z, o[nt][4 * b + 3] *= a.w;
        }
#pragma unroll
        for (int kk = 0; kk < 16; kk++) {
            const float pa = ps[li][2 * kk + lk];
#pragma unroll
            for (int nt = 0; nt < 2; nt++)
                o[nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(pa, ct[2 * kk + lk][64 * wave + 32 * nt + li], o[nt], 0, 0, 0);
        }
    }
#pragma unroll
    for (int nt = 0; nt < 2; nt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int i = 8 * (r >> 2) + 4 * lk + (r & 3);
            part[(((size_t)s * n_head + h0 + i) * n_split + split) * (MLA_M_LKV + 2) + 2 + 64 * wave + 32 * nt + li] = o[nt][r];
        }
    if ((tid & 15) == 0) {
        float *p = part + (((size_t)s * n_head + h0 + (tid >> 4)) * n_split + split) * (MLA_M_LKV + 2);
        p[0] = m_run, p[1] = l_run;
    }
}

// grid (n_head, S, ceil(lkv / 128)), 128 threads, one latent column each: merges the splits of (s, h)
// into the normalised latent sum olat[s, h, :] = sum_i f_i o_i / sum_i f_i l_i, f_i = exp(m_i - max m).
__global__ __launch_bounds__(128) void mla_merge(const float *__restrict__ part, float *__restrict__ olat, int n_head,
                                                  int lkv, int n_split) {
    __shared__ float f[MLA_SPLIT_MAX];
    __shared__ float Linv;
    const int h = blockIdx.x, s = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float *p = part + ((size_t)s * n_head + h) * n_split * (lkv + 2);
    if (wave == 0) {  // n_split <= 64
        const float mi = lane < n_split ? p[(size_t)lane * (lkv + 2)] : -INFINITY;
        const float M = wave_max(mi);
        const float fi = mi == -INFINITY ? 0.0f : __expf(mi - M);  // an empty split
        const float L = wave_sum(lane < n_split ? p[(size_t)lane * (lkv + 2) + 1] * fi : 0.0f);
        f[lane] = fi;
        if (lane == 0) Linv = 1.0f / L;
    }
    __syncthreads();
    const int c = blockIdx.z * 128 + threadIdx.x;
    if (c >= lkv) return;
    float v = 0.0f;
#pragma unroll 8
    for (int i = 0; i < n_split; i++) v = fmaf(p[(size_t)i * (lkv + 2) + 2 + c], f[i], v);
    olat[((size_t)s * n_head + h) * lkv + c] = v * Linv;
}

// ctx[s, h * vh + j] = Wkv[h * (nope + vh) + nope + j, :] . olat[s, h, :].  grid (n_head, ceil(vh / 16),
// ceil(S / ST)), four waves: a wave takes four value rows, read coalesced (16-byte loads when VEC:
// lkv % 4 == 0) once for the ST tokens whose latent sums wait in LDS.
template <int ST, bool VEC>
__global__ __launch_bounds__(256) void mla_vproj(const float *__restrict__ olat, const float *__restrict__ Wkv,
                                                  float *__restrict__ ctx, int S, int n_head, int nope, int vh, int lkv) {
    __shared__ __attribute__((aligned(16))) float ol[ST][MLA_MAX_LKV];
    const int h = blockIdx.x, s0 = blockIdx.z * ST, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int e = threadIdx.x; e < ST * lkv; e += 256) {
        const int j = e / lkv, c = e % lkv;
        ol[j][c] = s0 + j < S ? olat[((size_t)(s0 + j) * n_head + h) * lkv + c] : 0.0f;
    }
    __syncthreads();
    const float *W = Wkv + ((size_t)h * (nope + vh) + nope) * lkv;
#pragma unroll
    for (int rr = 0; rr < 4; rr++) {
        const int j = blockIdx.y * 16 + wave * 4 + rr;
        if (j >= vh) break;  // the whole wave
        float acc[ST];
#pragma unroll
        for (int t = 0; t < ST; t++) acc[t] = 0.0f;
        if constexpr (VEC) {
            for (int c = 4 * lane; c < lkv; c += 256) {
                const float4 wv = *(const float4 *)(W + (size_t)j * lkv + c);
#pragma unroll
                for (int t = 0; t < ST; t++) {
                    const float4 o = *(const float4 *)&ol[t][c];
                    acc[t] = fmaf(wv.x, o.x, fmaf(wv.y, o.y, fmaf(wv.z, o.z, fmaf(wv.w, o.w, acc[t]))));
                }
            }
        } else {
            for (int c = lane; c < lkv; c += 64) {
                const float wv = W[(size_t)j * lkv + c];
#pragma unroll
                for (int t = 0; t < ST; t++) acc[t] = fmaf(wv, ol[t][c], acc[t]);
            }
        }
#pragma unroll
        for (int t = 0; t < ST; t++) {
            const float v = wave_sum(acc[t]);
            if (lane == 0 && s0 + t < S) ctx[((size_t)(s0 + t) * n_head + h) * vh + j] = v;
        }
    }
}

}  // namespace jq
