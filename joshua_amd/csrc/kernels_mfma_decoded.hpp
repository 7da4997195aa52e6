// Any block format times more than 16 activation rows on the matrix cores: the weights are decoded
// (the format's own decode, as in the f32 kernels) into LDS as two f16 planes per (row, 256-element
// chunk), w * 2048 / max|w| = hi + lo; the activations arrive from acts_f16_prep split the same way per
// (row, chunk); v_mfma_f32_16x16x32_f16 adds hi*hi + hi*lo + lo*hi into one f32 accumulator per chunk,
// which is scaled by the two maxima and added to the result.  Either operand is good to 22 bits, so the
// result differs from f32 arithmetic by accumulation order only (one f16 plane of weights fails the
// 1e-3 bound in the tails of a 4096 x 4096 product).  Scaling into +-2048 keeps the low planes above
// the f16 denormal range.
//
// Workgroup: 64 weight rows x 64 activation rows, 4 waves (16 weight rows each), chunks of 256
// elements: the raw block bytes of the chunk (4-byte loads from the word at or below each row's
// unaligned start) and the activation planes go to LDS, 256 threads decode one or two units each,
// then 8 k-steps x 4 column tiles x 2 planes of MFMA per wave.  The next chunk's global data travels into
// registers while the current chunk is decoded and multiplied; the stages themselves run one after the
// other (the kernel replaces f32 row kernels that run at 5 to 9 TFLOP/s).
#pragma once
#include "kernels_mfma_q4k_gemm.hpp"
#include "kernels_valu.hpp"

namespace jq {

constexpr int GD_NT = 64, GD_MT = 64, GD_KC = 256;
constexpr int GD_STRIDE = GD_KC + 8;  // halves a row in LDS: 528 bytes, so that 16 rows spread over the banks

// v = hi + lo in f16, hi the nearest f16 and lo the rest (exact when |v| <= 2048 and not tiny).  The low
// part is computed against the very bits that are stored as the high part (the empty asm keeps the
// compiler from rounding a second time with another instruction, which differs at ties).
__device__ __forceinline__ void split_f16x2(float v0, float v1, uint32_t &hi, uint32_t &lo) {
    hi = __builtin_bit_cast(uint32_t, qg_h2{(_Float16)v0, (_Float16)v1});
    asm volatile("" : "+v"(hi));
    const qg_h2 h = __builtin_bit_cast(qg_h2, hi);
    lo = __builtin_bit_cast(uint32_t, qg_h2{(_Float16)(v0 - (float)h.x), (_Float16)(v1 - (float)h.y)});
}

struct ActsF16 {
    _Float16 *hi, *lo;  // [m_pad][k], rows beyond m zero
    float *s;           // [m_pad][k / 256]
};

__global__ __launch_bounds__(256) void acts_f16_prep(const float *__restrict__ X, int m, int m_pad, int k, ActsF16 out) {
    const int unit = (int)((blockIdx.x * 256 + threadIdx.x) >> 6);  // one (row, 256-element chunk) a wave
    const int nc = k >> 8;
    if (unit >= m_pad * nc) return;
    const int row = unit / nc, c = unit % nc, lane = threadIdx.x & 63;
    float4 v = float4{0.f, 0.f, 0.f, 0.f};
    if (row < m) v = *(const float4 *)(X + (size_t)row * k + 256 * c + 4 * lane);
    float amax = fmaxf(fmaxf(mag_or_inf(v.x), mag_or_inf(v.y)), fmaxf(mag_or_inf(v.z), mag_or_inf(v.w)));
    amax = wave_max(amax);
    const bool live = amax > 0.0f && amax < INFINITY;
    const float inv = live ? 2048.0f / amax : 0.0f;
    const float x[4] = {v.x * inv, v.y * inv, v.z * inv, v.w * inv};
    uint32_t h01, l01, h23, l23;
    split_f16x2(x[0], x[1], h01, l01);
    split_f16x2(x[2], x[3], h23, l23);
    const size_t at = (size_t)row * k + 256 * c + 4 * lane;
    *(uint2 *)(out.hi + at) = uint2{h01, h23};
    *(uint2 *)(out.lo + at) = uint2{l01, l23};
    if (lane == 0) out.s[(size_t)row * nc + c] = fixed_scale(amax, 2048.0f);
}

template <class Q>
// Split over k: blockIdx.z takes the z-th of gridDim.z contiguous runs of chunks and stores its partial
// sums at Y + z * split_stride (splitk_sum adds them in order); one run and stride 0 give the result.
__global__ __launch_bounds__(256) void gemm_decoded_mfma(const uint8_t *__restrict__ W, size_t row_bytes, ActsF16 acts,
                                                         float *__restrict__ Y, int m, int k, int n, size_t split_stride) {
    constexpr int CB = Q::BLOCK_BYTES * (GD_KC / Q::BLOCK_ELEMS);  // bytes of a row's chunk
    constexpr int NDW = (CB + 3 + 3) / 4;                          // words that cover it from any byte offset
    constexpr int UE = Q::SEGS * Q::SEGLEN, UPR = GD_KC / UE;      // elements a unit, units a row chunk
    __shared__ __attribute__((aligned(16))) _Float16 a_lds[2][GD_NT][GD_STRIDE];
    __shared__ float sw_lds[GD_NT];
    __shared__ __attribute__((aligned(16))) _Float16 b_lds[2][GD_MT][GD_STRIDE];
    __shared__ __attribute__((aligned(16))) uint32_t raw[GD_NT][NDW];
    __shared__ float s_lds[GD_MT];
    __shared__ __attribute__((aligned(16))) uint8_t table_lds[table_bytes<Q>() > 0 ? table_bytes<Q>() : 16];
    const auto *table = stage_table<Q>(table_lds);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n0 = blockIdx.x * GD_NT, m0 = blockIdx.y * GD_MT;
    const int r16 = lane & 15, kg = lane >> 4;
    qg_f4 acc[4];
#pragma unroll
    for (int ct = 0; ct < 4; ct++) acc[ct] = qg_f4{0.f, 0.f, 0.f, 0.f};

    const int nc = k >> 8;
    // The next chunk's global data (raw block bytes, activation planes, activation scales) is asked for
    // into registers before the decode and MFMA stages of the current one and stored into LDS at the top
    // of the next iteration, so the trip to memory runs beside the arithmetic.
    constexpr int RAW_IT = (GD_NT * NDW + 255) / 256, B_IT = GD_MT * (GD_KC / 8) / 256;
    uint32_t raw_r[RAW_IT];
    qg_u4 bh_r[B_IT], bl_r[B_IT];
    float s_r = 0.0f;
    auto fetch = [&](int c) __attribute__((always_inline)) {
        // row r's words from the word at or below its first byte
#pragma unroll
        for (int it = 0; it < RAW_IT; it++) {
            const int idx = tid + 256 * it;
            const int r = idx / NDW, dw = idx % NDW;
            raw_r[it] = 0u;
            if (idx < GD_NT * NDW) {
                const uintptr_t src = (uintptr_t)(W + (size_t)min(n0 + r, n - 1) * row_bytes + (size_t)c * CB);
                const uint32_t *wp = (const uint32_t *)(src & ~(uintptr_t)3) + dw;
                // the last word may lie past the chunk: it is read only when it still holds bytes of it
                if ((uintptr_t)wp < src + CB) raw_r[it] = *wp;
            }
        }
        // the activation planes of the 64 rows m0 .. m0 + 63 (prepared, zero beyond m)
#pragma unroll
        for (int it = 0; it < B_IT; it++) {
            const int idx = tid + 256 * it;
            const int col = idx / (GD_KC / 8), part = idx % (GD_KC / 8);
            const size_t at = (size_t)(m0 + col) * k + (size_t)c * GD_KC + 8 * part;
            bh_r[it] = *(const qg_u4 *)(acts.hi + at);
            bl_r[it] = *(const qg_u4 *)(acts.lo + at);
        }
        if (tid < GD_MT) s_r = acts.s[(size_t)(m0 + tid) * nc + c];
    };
    const int c_begin = (int)((long)blockIdx.z * nc / gridDim.z), c_end = (int)((long)(blockIdx.z + 1) * nc / gridDim.z);
    Y += (size_t)blockIdx.z * split_stride;
    fetch(c_begin);
    for (int c = c_begin; c < c_end; c++) {
#pragma unroll
        for (int it = 0; it < RAW_IT; it++) {
            const int idx = tid + 256 * it;
            if (idx < GD_NT * NDW) raw[idx / NDW][idx % NDW] = raw_r[it];
        }
#pragma unroll
        for (int it = 0; it < B_IT; it++) {
            const int idx = tid + 256 * it;
            const int col = idx / (GD_KC / 8), part = idx % (GD_KC / 8);
            *(qg_u4 *)&b_lds[0][col][8 * part] = bh_r[it];
            *(qg_u4 *)&b_lds[1][col][8 * part] = bl_r[it];
        }
        if (tid < GD_MT) s_lds[tid] = s_r;
        __syncthreads();
        if (c + 1 < c_end) fetch(c + 1);
        // ---- decode: unit u of row r -> f16 in operand order ----
        for (int id = tid; id < GD_NT * UPR; id += 256) {
            const int r = id / UPR, u = id % UPR, b = u / Q::UNITS, ub = u % Q::UNITS;
            const uintptr_t src = (uintptr_t)(W + (size_t)min(n0 + r, n - 1) * row_bytes + (size_t)c * CB);
            const uint8_t *blk = (const uint8_t *)&raw[r][0] + (src & 3) + (size_t)b * Q::BLOCK_BYTES;
            float w[UE];
            decode_staged<Q>(table, blk, ub, w);
            // the row chunk's maximum: its UPR units sit in neighbouring lanes
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < UE; i++) amax = fmaxf(amax, mag_or_inf(w[i]));
            amax = fmaxf(amax, dpp_f<0xB1>(amax));
            amax = fmaxf(amax, dpp_f<0x4E>(amax));
            if (UPR == 8) amax = fmaxf(amax, dpp_f<0x141>(amax));
            const float inv = amax > 0.0f && amax < INFINITY ? 2048.0f / amax : 0.0f;
            if (u == 0) sw_lds[r] = fixed_scale(amax, 2048.0f);
            const int base = b * Q::BLOCK_ELEMS + Q::elem_base(ub);
#pragma unroll
            for (int s = 0; s < Q::SEGS; s++) {
#pragma unroll
                for (int e = 0; e < Q::SEGLEN; e += 2) {
                    uint32_t hi, lo;
                    split_f16x2(w[s * Q::SEGLEN + e] * inv, w[s * Q::SEGLEN + e + 1] * inv, hi, lo);
                    *(uint32_t *)&a_lds[0][r][base + s * Q::SEG_STRIDE + e] = hi;
                    *(uint32_t *)&a_lds[1][r][base + s * Q::SEG_STRIDE + e] = lo;
                }
            }
        }
        __syncthreads();
        // ---- 16 weight rows of this wave x 64 activation rows, both planes into one accumulator ----
        qg_f4 part[4];
#pragma unroll
        for (int ct = 0; ct < 4; ct++) part[ct] = qg_f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < GD_KC / 32; ks++) {
            const qg_h8 ah = *(const qg_h8 *)&a_lds[0][16 * wave + r16][32 * ks + 8 * kg];
            const qg_h8 al = *(const qg_h8 *)&a_lds[1][16 * wave + r16][32 * ks + 8 * kg];
#pragma unroll
            for (int ct = 0; ct < 4; ct++) {
                const qg_h8 bh = *(const qg_h8 *)&b_lds[0][16 * ct + r16][32 * ks + 8 * kg];
                const qg_h8 bl = *(const qg_h8 *)&b_lds[1][16 * ct + r16][32 * ks + 8 * kg];
                part[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, bh, part[ct], 0, 0, 0);
                part[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, bl, part[ct], 0, 0, 0);
                part[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(al, bh, part[ct], 0, 0, 0);
            }
        }
        float sw[4];
#pragma unroll
        for (int j = 0; j < 4; j++) sw[j] = sw_lds[16 * wave + 4 * kg + j];
#pragma unroll
        for (int ct = 0; ct < 4; ct++) {
            const float s = s_lds[16 * ct + r16];
#pragma unroll
            for (int j = 0; j < 4; j++) acc[ct][j] = fmaf(s * sw[j], part[ct][j], acc[ct][j]);
        }
        __syncthreads();
    }
    // results: weight row n0 + 16 wave + 4 kg + j, activation row m0 + 16 ct + r16
#pragma unroll
    for (int ct = 0; ct < 4; ct++) {
        const int mm = m0 + 16 * ct + r16;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int nn = n0 + 16 * wave + 4 * kg + j;
            if (mm < m && nn < n) Y[(size_t)mm * n + nn] = acc[ct][j];
        }
    }
}

}  // namespace jq
