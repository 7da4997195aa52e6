// Q4_K decode GEMV (m = 1..4) on the int8 matrix cores.
//
// Work split
//   workgroup = 4 waves = one tile of 16 weight rows over the whole k;
//   wave w takes the tile's super-blocks b = w, w+4, ...; lane (n = l%16,
//   g = l/16) loads, for row n, the 16-byte header and the 32 bytes of
//   chunk g of each of its super-blocks: two 128-bit loads of packed nibbles,
//   all issued before anything else happens.
//
// Arithmetic
//   The activations are turned once per workgroup into 23-bit fixed point per
//   group of 32 elements (one Q4_K sub-block): X = round(x * (2^22-1)/max|x|),
//   held as three signed byte planes D0,D1,D2 (the bytes of X + 2^22, the low
//   two re-centred by -128) with X = D2*65536 + D1*256 + D0 - 4161408.
//   Nibbles are exact small integers, so
//       sum_i q_i * X_i = 65536*S2 + 256*S1 + S0 - 4161408*Sq
//   with S_p = sum q*D_p and Sq = sum q, all exact int32 sums from
//   v_mfma_i32_16x16x64_i8.  Per sub-block the f32 result is
//       y += (d*sc) * s_x * (sum q*X) - (dmin*m) * sum_x
//   (d*sc and dmin*m rounded to f32 first, as in the reference,
//   src/kquant_dot.rs:439-441; sum_x is the f32 sum of the group's x).
//   The fixed-point error is at most 2^-23 of the group's largest |x| per
//   element, i.e. below f32 rounding of the products the reference adds up.
//
// MFMA operand layout (16x16x64: A row = l%16, k-slots 16*(l/16)..+15; B column
// = l%16, same k-slots; C rows 4*(l/16)..+3, column l%16)
//   B: lane (n, g) supplies the 16 low (or high) nibbles of 16 bytes of chunk g
//      of row n as int8: one AND (or shift+AND) per dword.
//   A: rows 4g..4g+3 are nonzero only in k-slot group g, where they hold planes
//      D0, D1, D2 of the matching 16 activations and a row of ones.  So one
//      MFMA gives, for all 16 rows and all four chunks at once, S0,S1,S2,Sq of
//      half a sub-block; two chained MFMAs finish the even sub-blocks
//      (low nibbles), two more the odd ones (high nibbles).  Lane (n, g) ends
//      up with the four sums of sub-blocks 2g and 2g+1 of row n: exactly the
//      ones whose scales sit in the header it loaded.
#pragma once
#include "blocks.hpp"

namespace jq {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int Q4K_MFMA_WAVES = 4;
constexpr int Q4K_LDS_DIGITS_PER_BLOCK = 768;  // [op 4][g 4][plane 3][16 B]
constexpr int Q4K_LDS_SCALES_PER_BLOCK = 64;   // [g 4]{s_even, s_odd, sum_even, sum_odd}
constexpr int Q4K_LDS_CONST = 640;             // span an inactive lane may read: 3*192 + 16, padded

__host__ __device__ constexpr size_t q4k_mfma_lds_bytes(int blocks_per_row, int mt) {
    return (size_t)mt * blocks_per_row * (Q4K_LDS_DIGITS_PER_BLOCK + Q4K_LDS_SCALES_PER_BLOCK) + 2 * Q4K_LDS_CONST +
           Q4K_MFMA_WAVES * 16 * 4 * sizeof(float);
}

// Quantizes activation rows [m0, m0+MT) into LDS (digits + group scale/sum).
template <int MT>
__device__ __forceinline__ void q4k_stage_activations(const float *__restrict__ X, int m0, int m, int k, int bpr,
                                                      uint8_t *digits, float *scales) {
    const int chunks = k / 16;
    for (int mi = 0; mi < MT; mi++) {
        const bool live = m0 + mi < m;
        const float *xr = X + (size_t)(live ? m0 + mi : m0) * k;
        uint8_t *dg = digits + (size_t)mi * bpr * Q4K_LDS_DIGITS_PER_BLOCK;
        float *sc = scales + (size_t)mi * bpr * (Q4K_LDS_SCALES_PER_BLOCK / 4);
        // Adjacent threads take adjacent 16-element chunks, so lanes (2j, 2j+1)
        // share one 32-element group.  chunks is a multiple of 16: a wave is
        // either fully inside the loop or fully out of it.
        for (int ch = threadIdx.x; ch < chunks; ch += blockDim.x) {
            float x[16];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float4 v = ld<float4>((const uint8_t *)(xr + 16 * ch + 4 * i));
                x[4 * i] = v.x; x[4 * i + 1] = v.y; x[4 * i + 2] = v.z; x[4 * i + 3] = v.w;
            }
            float amax = 0.0f, sum = 0.0f;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                amax = fmaxf(amax, fabsf(x[i]));
                sum += x[i];
            }
            amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
            sum += __shfl_xor(sum, 1, 64);
            const float inv = amax > 0.0f ? 4194303.0f / amax : 0.0f;
            const float s = amax / 4194303.0f;
            uint32_t u[16];
#pragma unroll
            for (int i = 0; i < 16; i++)  // low 23 bits = round(x*inv) + 2^22
                u[i] = __float_as_uint(fmaf(x[i], inv, 12582912.0f)) & 0x7FFFFFu;
            uint32_t p0[4], p1[4], p2[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t a = u[4 * i], b = u[4 * i + 1], c = u[4 * i + 2], d = u[4 * i + 3];
                // __builtin_amdgcn_perm(hi, lo, sel): byte j of the result is byte sel_j of {hi:lo} (lo = bytes 0..3)
                const uint32_t ab01 = __builtin_amdgcn_perm(b, a, 0x05010400u);  // a0 b0 a1 b1
                const uint32_t cd01 = __builtin_amdgcn_perm(d, c, 0x05010400u);
                const uint32_t ab2 = __builtin_amdgcn_perm(b, a, 0x06020602u);   // a2 b2 a2 b2
                const uint32_t cd2 = __builtin_amdgcn_perm(d, c, 0x06020602u);
                p0[i] = __builtin_amdgcn_perm(cd01, ab01, 0x05040100u) ^ 0x80808080u;  // a0 b0 c0 d0, minus 128
                p1[i] = __builtin_amdgcn_perm(cd01, ab01, 0x07060302u) ^ 0x80808080u;  // a1 b1 c1 d1, minus 128
                p2[i] = __builtin_amdgcn_perm(cd2, ab2, 0x05040100u);                  // a2 b2 c2 d2 (0..127 as is)
            }
            const int b = ch >> 4, e0 = (ch & 15) * 16;
            const int g = e0 >> 6, odd = (e0 >> 5) & 1, second = (e0 >> 4) & 1;
            uint8_t *dst = dg + b * Q4K_LDS_DIGITS_PER_BLOCK + (odd * 2 + second) * 192 + g * 48;
            *(uint4 *)(dst) = uint4{p0[0], p0[1], p0[2], p0[3]};
            *(uint4 *)(dst + 16) = uint4{p1[0], p1[1], p1[2], p1[3]};
            *(uint4 *)(dst + 32) = uint4{p2[0], p2[1], p2[2], p2[3]};
            if (!second) {
                float *sp = sc + b * 16 + g * 4 + odd;
                sp[0] = live ? s : 0.0f;
                sp[2] = live ? sum : 0.0f;
            }
        }
    }
}

template <int MT>
__global__ __launch_bounds__(64 * Q4K_MFMA_WAVES) void q4k_gemv_mfma(const uint8_t *__restrict__ W, size_t row_bytes,
                                                                      const float *__restrict__ X,
                                                                      float *__restrict__ Y, int m0, int m, int k,
                                                                      int n) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int bpr = k / 256;
    uint8_t *digits = lds;
    float *scales = (float *)(lds + (size_t)MT * bpr * Q4K_LDS_DIGITS_PER_BLOCK);
    uint8_t *zeros = (uint8_t *)(scales + (size_t)MT * bpr * (Q4K_LDS_SCALES_PER_BLOCK / 4));
    uint8_t *ones = zeros + Q4K_LDS_CONST;
    float *partial = (float *)(ones + Q4K_LDS_CONST);  // [wave][MT<=4][16]

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nl = lane & 15, g = lane >> 4;
    const int row0 = blockIdx.x * 16;
    const int row = min(row0 + nl, n - 1);  // tail tile: re-read the last row, discard later
    const uint8_t *rp = W + (size_t)row * row_bytes;

    // ---- issue the loads of this wave's first four super-blocks ----------------
    constexpr int NB = 4;
    uint4 hdr[NB], qa[NB], qb[NB];
#pragma unroll
    for (int j = 0; j < NB; j++) {
        const int b = min(wave + Q4K_MFMA_WAVES * j, bpr - 1);
        const uint8_t *bp = rp + (size_t)b * 144;
        hdr[j] = ld<uint4>(bp);
        qa[j] = ld<uint4>(bp + 16 + 32 * g);
        qb[j] = ld<uint4>(bp + 32 + 32 * g);
    }

    // ---- activations -> fixed-point digit planes in LDS ------------------------
    for (int i = threadIdx.x; i < Q4K_LDS_CONST / 4; i += blockDim.x) {
        ((uint32_t *)zeros)[i] = 0u;
        ((uint32_t *)ones)[i] = 0x01010101u;
    }
    q4k_stage_activations<MT>(X, m0, m, k, bpr, digits, scales);
    __syncthreads();

    // A-operand addressing: lane (row = l%16, k-group = l/16) is live when
    // row/4 == k-group; row%4 < 3 selects a digit plane, row%4 == 3 the ones.
    const int arow = lane & 15, agrp = lane >> 4, aslot = arow & 3;
    const bool a_live = (arow >> 2) == agrp;
    const bool a_digit = a_live && aslot < 3;
    const uint8_t *a_base = a_digit ? digits + agrp * 48 + aslot * 16 : (a_live ? ones : zeros);
    const int a_stride = a_digit ? Q4K_LDS_DIGITS_PER_BLOCK : 0;
    const int a_mstride = a_digit ? bpr * Q4K_LDS_DIGITS_PER_BLOCK : 0;

    float acc[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) acc[mi] = 0.0f;

    for (int j0 = 0; wave + Q4K_MFMA_WAVES * j0 < bpr; j0 += NB) {
        if (j0 > 0) {
#pragma unroll
            for (int j = 0; j < NB; j++) {
                const int b = min(wave + Q4K_MFMA_WAVES * (j0 + j), bpr - 1);
                const uint8_t *bp = rp + (size_t)b * 144;
                hdr[j] = ld<uint4>(bp);
                qa[j] = ld<uint4>(bp + 16 + 32 * g);
                qb[j] = ld<uint4>(bp + 32 + 32 * g);
            }
        }
#pragma unroll
        for (int j = 0; j < NB; j++) {
            const int b = wave + Q4K_MFMA_WAVES * (j0 + j);
            if (b >= bpr) break;  // wave-uniform
            // scale/min pairs 2g and 2g+1 of this lane's row (reference: src/kquant_dot.rs:108-118)
            const float d = f16_bits(hdr[j].x), dmin = f16_bits(hdr[j].x >> 16);
            const int sh = 16 * (g & 1);
            const uint32_t a16 = (hdr[j].y >> sh) & 0xFFFFu, b16 = (hdr[j].z >> sh) & 0xFFFFu,
                           e16 = (hdr[j].w >> sh) & 0xFFFFu;
            uint32_t sc2, mn2;  // two packed bytes each: pair 2g in byte 0, pair 2g+1 in byte 1
            if (g < 2) {
                sc2 = a16 & 0x3F3Fu;
                mn2 = b16 & 0x3F3Fu;
            } else {
                sc2 = (e16 & 0x0F0Fu) | ((a16 >> 2) & 0x3030u);
                mn2 = ((e16 >> 4) & 0x0F0Fu) | ((b16 >> 2) & 0x3030u);
            }
            const float d_e = d * (float)(sc2 & 0xFFu), d_o = d * (float)(sc2 >> 8);
            const float m_e = dmin * (float)(mn2 & 0xFFu), m_o = dmin * (float)(mn2 >> 8);

            const v4i bl_a = {(int)(qa[j].x & 0x0F0F0F0Fu), (int)(qa[j].y & 0x0F0F0F0Fu), (int)(qa[j].z & 0x0F0F0F0Fu),
                              (int)(qa[j].w & 0x0F0F0F0Fu)};
            const v4i bl_b = {(int)(qb[j].x & 0x0F0F0F0Fu), (int)(qb[j].y & 0x0F0F0F0Fu), (int)(qb[j].z & 0x0F0F0F0Fu),
                              (int)(qb[j].w & 0x0F0F0F0Fu)};
            const v4i bh_a = {(int)((qa[j].x >> 4) & 0x0F0F0F0Fu), (int)((qa[j].y >> 4) & 0x0F0F0F0Fu),
                              (int)((qa[j].z >> 4) & 0x0F0F0F0Fu), (int)((qa[j].w >> 4) & 0x0F0F0F0Fu)};
            const v4i bh_b = {(int)((qb[j].x >> 4) & 0x0F0F0F0Fu), (int)((qb[j].y >> 4) & 0x0F0F0F0Fu),
                              (int)((qb[j].z >> 4) & 0x0F0F0F0Fu), (int)((qb[j].w >> 4) & 0x0F0F0F0Fu)};
#pragma unroll
            for (int mi = 0; mi < MT; mi++) {
                const uint8_t *ap = a_base + b * a_stride + mi * a_mstride;
                const v4i a00 = *(const v4i *)(ap), a01 = *(const v4i *)(ap + 192);
                const v4i a10 = *(const v4i *)(ap + 384), a11 = *(const v4i *)(ap + 576);
                const float4 sx = *(const float4 *)(scales + ((size_t)mi * bpr + b) * 16 + g * 4);
                v4i ce = {0, 0, 0, 0}, co = {0, 0, 0, 0};
                ce = __builtin_amdgcn_mfma_i32_16x16x64_i8(a00, bl_a, ce, 0, 0, 0);
                co = __builtin_amdgcn_mfma_i32_16x16x64_i8(a10, bh_a, co, 0, 0, 0);
                ce = __builtin_amdgcn_mfma_i32_16x16x64_i8(a01, bl_b, ce, 0, 0, 0);
                co = __builtin_amdgcn_mfma_i32_16x16x64_i8(a11, bh_b, co, 0, 0, 0);
                // sum q*X = 65536*S2 + 256*S1 + S0 - 4161408*Sq.  |sum q*X| <= 32*15*(2^22-1) < 2^31,
                // so evaluating it in wrapping 32-bit arithmetic is exact.
                const float ve = (float)(int)(((uint32_t)ce[2] << 16) + ((uint32_t)ce[1] << 8) + (uint32_t)ce[0] -
                                              __umul24((uint32_t)ce[3], 4161408u));
                const float vo = (float)(int)(((uint32_t)co[2] << 16) + ((uint32_t)co[1] << 8) + (uint32_t)co[0] -
                                              __umul24((uint32_t)co[3], 4161408u));
                acc[mi] = fmaf(ve, d_e * sx.x, acc[mi]);
                acc[mi] = fmaf(-m_e, sx.z, acc[mi]);
                acc[mi] = fmaf(vo, d_o * sx.y, acc[mi]);
                acc[mi] = fmaf(-m_o, sx.w, acc[mi]);
            }
        }
    }

    // ---- sum the four chunk lanes of a row, then the four waves ----------------
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
        float v = acc[mi];
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        if (lane < 16) partial[(wave * MT + mi) * 16 + lane] = v;
    }
    __syncthreads();
    if (threadIdx.x < 16 * MT) {
        const int mi = threadIdx.x >> 4, r = threadIdx.x & 15;
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < Q4K_MFMA_WAVES; w++) v += partial[(w * MT + mi) * 16 + r];
        if (row0 + r < n && m0 + mi < m) Y[(size_t)(m0 + mi) * n + row0 + r] = v;
    }
}

}  // namespace jq
