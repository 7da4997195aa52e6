// Q4_K decode GEMV (m = 1..4 activation rows per launch) on the int8 matrix
// cores of gfx950.
//
// Work split
//   A "unit" is 16 weight rows x 4 consecutive super-blocks (576 contiguous
//   bytes per row).  One wave owns one unit; a workgroup holds all the units of
//   one or more 16-row tiles (up to 16 waves), so the activations are staged
//   once per workgroup and the per-tile sums never leave it.
//   A row's 576 bytes are 36 pieces of 16 bytes: piece 9b is the header of
//   super-block b (d, dmin, 12 scale bytes), pieces 9b+1..9b+8 its 128 bytes
//   of nibbles.  Lane (n = l%16, g = l/16) loads piece 4i+g of row n with its
//   i-th 128-bit load, i = 0..8: every load instruction covers 64 contiguous
//   bytes of each of 16 rows, and all nine are issued before anything else.
//
// Arithmetic
//   Activations are turned, once per workgroup, into 23-bit fixed point per
//   group of 16 elements: X = round(x * 4161407 / max|x|), held as three
//   signed byte planes with X = 65536*D2 + 256*D1 + D0 exactly.  (The planes
//   are the bytes of the f32 word x*inv + 12615808: its mantissa is
//   2^22 + X + 0x8080, so byte0-128, byte1-128 and byte2-64 are balanced
//   digits.)  Nibbles q are exact small integers, so for the 16 elements of a
//   piece
//       sum q*X = 65536*S2 + 256*S1 + S0,   S_p = sum q*D_p,
//   with every S_p an exact int32 sum out of v_mfma_i32_16x16x64_i8 and
//   |sum q*X| <= 16*15*4161407 < 2^31.  The f32 result adds, per piece,
//       (d*sc) * s_x * (sum q*X)  -  (dmin*m) * sum_x
//   with d*sc and dmin*m rounded to f32 first as the reference does
//   (src/kquant_dot.rs:439-441), s_x = max|x|/4161407 and sum_x the f32 sum of
//   the group's activations.  The fixed-point step is at most 2^-23 of the
//   group's largest |x| per element: below the f32 rounding of the products the
//   reference adds up.
//
// MFMA operand layout (16x16x64 i8: A row = l%16, k-slots 16*(l/16)..+15;
// B column = l%16, same k-slots; C rows 4*(l/16)..+3, column l%16)
//   B: lane (n, g) supplies the 16 low (or high) nibbles of its piece as int8:
//      one AND (or shift+AND) per dword.
//   A: rows 4g..4g+2 are nonzero only in k-slot group g, where they hold planes
//      D0, D1, D2 of the 16 activations that piece 4i+g multiplies (nothing for
//      a header piece).  One MFMA therefore yields S0,S1,S2 for 16 rows x 4
//      pieces at once, and lane (n, g) receives exactly the sums of its own
//      piece.
//   Headers reach the lanes that need them through LDS: the lane holding a
//   header decodes all eight (d*sc, dmin*m) pairs once and publishes them.
#pragma once
#include "blocks.hpp"

namespace jq {

typedef int v4i __attribute__((ext_vector_type(4)));

#ifndef Q4K_EARLY_MASK
#define Q4K_EARLY_MASK 0x1FF  // which of the nine weight loads go out before the activations are staged
#endif
constexpr int Q4K_UNIT_BLOCKS = 4;    // super-blocks per unit
constexpr int Q4K_MAX_WAVES = 16;     // waves per workgroup
constexpr int Q4K_PLANE_PAD = 64;     // bytes between digit planes beyond k
constexpr int Q4K_DEC_ROW = 80;       // bytes per (block,row) of decoded scale pairs (64 used)
constexpr int Q4K_DEC_WAVE = Q4K_UNIT_BLOCKS * 16 * Q4K_DEC_ROW;
constexpr int Q4K_ZERO_BYTES = 64;
constexpr float Q4K_ACT_RANGE = 4161407.0f;   // 2^22 - 1 - 0x8080
constexpr float Q4K_ACT_MAGIC = 12615808.0f;  // 1.5 * 2^23 + 0x8080

struct Q4kLds {
    int planes, scl, dec, zeros, partial, total;  // byte offsets
};

__host__ __device__ inline Q4kLds q4k_lds_layout(int k, int mt, int waves) {
    Q4kLds L;
    L.planes = 0;
    L.scl = L.planes + mt * 3 * (k + Q4K_PLANE_PAD);
    L.dec = L.scl + mt * (k / 256) * 128;
    L.zeros = L.dec + waves * Q4K_DEC_WAVE;
    L.partial = L.zeros + Q4K_ZERO_BYTES;
    L.total = L.partial + waves * mt * 16 * (int)sizeof(float);
    return L;
}

// For load i and lane group g: which piece of the unit the lane holds.
// Low 6 bits: 16*b + 4*c + h (block b, chunk c, half h: the piece's low nibbles
// are elements 256*b + 64*c + 16*h + [0,16), its high nibbles the same + 32);
// bit 7: the piece is a block header.
__host__ __device__ constexpr uint32_t q4k_piece_codes(int i) {
    uint32_t packed = 0;
    for (int g = 0; g < 4; g++) {
        const int p = 4 * i + g, b = p / 9, r = p % 9;
        const uint32_t code = r == 0 ? (0x80u | (uint32_t)(16 * b)) : (uint32_t)(16 * b + 4 * ((r - 1) >> 1) + ((r - 1) & 1));
        packed |= code << (8 * g);
    }
    return packed;
}

template <int MT>
__global__ __launch_bounds__(64 * Q4K_MAX_WAVES) void q4k_gemv_mfma(const uint8_t *__restrict__ W, size_t row_bytes,
                                                                     const float *__restrict__ X,
                                                                     float *__restrict__ Y, int m0, int m, int k, int n,
                                                                     int units_per_tile) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int nthreads = blockDim.x, nwaves = nthreads >> 6;
    const int bpr = k >> 8;
    const Q4kLds L = q4k_lds_layout(k, MT, nwaves);
    const int pstride = k + Q4K_PLANE_PAD;

    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nl = lane & 15, g = lane >> 4;
    const int tiles_per_wg = nwaves / units_per_tile;
    const int tile_in_wg = wave / units_per_tile, uq = wave - tile_in_wg * units_per_tile;
    const bool wave_live = tile_in_wg < tiles_per_wg;
    const int row0 = (blockIdx.x * tiles_per_wg + tile_in_wg) * 16;
    const int nbv = min(Q4K_UNIT_BLOCKS, bpr - Q4K_UNIT_BLOCKS * uq);  // valid blocks of this unit

    // ---- 1. activation loads first (VMEM returns in order), then the weights ----
    const int kq = k >> 2;  // float4s per activation row
    constexpr int XP = 2;  // float4s per thread and row fetched ahead of the weight loads
    float4 xpre[MT][XP];
#pragma unroll
    for (int mi = 0; mi < MT; mi++)
#pragma unroll
        for (int j = 0; j < XP; j++)
            xpre[mi][j] = ld<float4>((const uint8_t *)(X + (size_t)min(m0 + mi, m - 1) * k +
                                                       4 * min((int)threadIdx.x + j * nthreads, kq - 1)));

    // Weight loads selected by Q4K_EARLY_MASK are issued now, the others once the
    // activations are staged.  Measured on MI355X at 14336 x 4096: issuing all
    // nine at once is fastest, although the activation loads then wait in the
    // memory queues behind other waves' weight loads for several microseconds.
    uint4 t[9];
    const int wrow = min(max(row0, 0) + nl, n - 1);  // tail tile: re-read the last row, discard later
    const uint8_t *up = W + (size_t)wrow * row_bytes + (size_t)uq * (Q4K_UNIT_BLOCKS * 144) + 16 * g;
    const int valid_bytes = wave_live ? 144 * nbv : 0;
    auto load_piece = [&](int i) {
        const int off = 64 * i + 16 * g < valid_bytes ? 64 * i : -16 * g - (int)(uq * Q4K_UNIT_BLOCKS * 144);
        t[i] = ld<uint4>(up + off);  // out-of-unit pieces re-read the row's first 16 bytes
    };
#pragma unroll
    for (int i = 0; i < 9; i++)
        if ((Q4K_EARLY_MASK >> i) & 1) load_piece(i);
    __builtin_amdgcn_sched_barrier(0);

    // ---- 2. stage the activations: digit planes + (scale, sum) per 16 elements ----
    if (threadIdx.x < Q4K_ZERO_BYTES / 4) ((uint32_t *)(lds + L.zeros))[threadIdx.x] = 0u;
    auto stage = [&](int mi, int fi, float4 v) {
        const bool live = m0 + mi < m;
        float amax = fmaxf(fmaxf(mag_or_inf(v.x), mag_or_inf(v.y)), fmaxf(mag_or_inf(v.z), mag_or_inf(v.w)));
        float sum = (v.x + v.y) + (v.z + v.w);
        // lanes 4j..4j+3 hold 16 consecutive elements: one quantization group
        amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
        sum += __shfl_xor(sum, 1, 64);
        amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
        sum += __shfl_xor(sum, 2, 64);
        const float inv = amax > 0.0f ? Q4K_ACT_RANGE / amax : 0.0f;
        const uint32_t a = __float_as_uint(fmaf(v.x, inv, Q4K_ACT_MAGIC)), b = __float_as_uint(fmaf(v.y, inv, Q4K_ACT_MAGIC));
        const uint32_t c = __float_as_uint(fmaf(v.z, inv, Q4K_ACT_MAGIC)), d = __float_as_uint(fmaf(v.w, inv, Q4K_ACT_MAGIC));
        // __builtin_amdgcn_perm(hi, lo, sel): result byte j = byte sel_j of {hi:lo} (lo = bytes 0..3; sel 0x0c = 0)
        const uint32_t ab01 = __builtin_amdgcn_perm(b, a, 0x05010400u);  // a0 b0 a1 b1
        const uint32_t cd01 = __builtin_amdgcn_perm(d, c, 0x05010400u);
        const uint32_t ab2 = __builtin_amdgcn_perm(b, a, 0x0c0c0602u);   // a2 b2 0 0
        const uint32_t cd2 = __builtin_amdgcn_perm(d, c, 0x0c0c0602u);
        const uint32_t p0 = __builtin_amdgcn_perm(cd01, ab01, 0x05040100u) ^ 0x80808080u;               // byte0 - 128
        const uint32_t p1 = __builtin_amdgcn_perm(cd01, ab01, 0x07060302u) ^ 0x80808080u;               // byte1 - 128
        const uint32_t p2 = (__builtin_amdgcn_perm(cd2, ab2, 0x05040100u) + 0x40404040u) ^ 0x80808080u;  // byte2 - 64
        uint8_t *pl = lds + L.planes + mi * 3 * pstride + 4 * fi;
        *(uint32_t *)(pl) = p0;
        *(uint32_t *)(pl + pstride) = p1;
        *(uint32_t *)(pl + 2 * pstride) = p2;
        if ((lane & 3) == 0) {
            const int grp = fi >> 2;  // 16-element group within the row: 16*b + 4*c + 2*hi + h
            const int blk = grp >> 4, cc = (grp >> 2) & 3, hi = (grp >> 1) & 1, hh = grp & 1;
            float2 *sp = (float2 *)(lds + L.scl + ((mi * bpr + blk) * 8 + cc * 2 + hh) * 16 + hi * 8);
            *sp = float2{live ? amax / Q4K_ACT_RANGE : 0.0f, live ? sum : 0.0f};
        }
    };
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
#pragma unroll
        for (int j = 0; j < XP; j++)
            if ((int)threadIdx.x + j * nthreads < kq) stage(mi, (int)threadIdx.x + j * nthreads, xpre[mi][j]);
        // longer rows: these loads queue behind the weight loads already in flight
        for (int fi = (int)threadIdx.x + XP * nthreads; fi < kq; fi += nthreads)
            stage(mi, fi, ld<float4>((const uint8_t *)(X + (size_t)min(m0 + mi, m - 1) * k + 4 * fi)));
    }

    __syncthreads();
#pragma unroll
    for (int i = 0; i < 9; i++)
        if (!((Q4K_EARLY_MASK >> i) & 1)) load_piece(i);

    // ---- 3. the lane holding block g's header decodes its 8 scale pairs --------
    //      (reference: src/kquant_dot.rs:108-118; d*sc and dmin*m rounded to f32)
    uint8_t *dec = lds + L.dec + wave * Q4K_DEC_WAVE;
    {
        // piece 9g sits in load 2g.  The candidates go through an empty asm so the
        // compiler keeps this a register select instead of indexing t[] in memory
        // (the memory clobber keeps it, and the wait for the loads, below the barrier).
        asm volatile("" : "+v"(t[0].x), "+v"(t[0].y), "+v"(t[0].z), "+v"(t[0].w), "+v"(t[2].x), "+v"(t[2].y), "+v"(t[2].z), "+v"(t[2].w)::"memory");
        asm volatile("" : "+v"(t[4].x), "+v"(t[4].y), "+v"(t[4].z), "+v"(t[4].w), "+v"(t[6].x), "+v"(t[6].y), "+v"(t[6].z), "+v"(t[6].w)::"memory");
        uint4 h;
        h.x = g == 0 ? t[0].x : (g == 1 ? t[2].x : (g == 2 ? t[4].x : t[6].x));
        h.y = g == 0 ? t[0].y : (g == 1 ? t[2].y : (g == 2 ? t[4].y : t[6].y));
        h.z = g == 0 ? t[0].z : (g == 1 ? t[2].z : (g == 2 ? t[4].z : t[6].z));
        h.w = g == 0 ? t[0].w : (g == 1 ? t[2].w : (g == 2 ? t[4].w : t[6].w));
        const float dd = f16_bits(h.x), dmin = f16_bits(h.x >> 16);
        const uint32_t sc_a = h.y & 0x3F3F3F3Fu, mn_a = h.z & 0x3F3F3F3Fu;  // pairs 0..3
        const uint32_t sc_b = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);          // pairs 4..7
        const uint32_t mn_b = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
        float4 *dp = (float4 *)(dec + (g * 16 + nl) * Q4K_DEC_ROW);
        dp[0] = float4{dd * (float)(sc_a & 0xFFu), dmin * (float)(mn_a & 0xFFu), dd * (float)((sc_a >> 8) & 0xFFu),
                       dmin * (float)((mn_a >> 8) & 0xFFu)};
        dp[1] = float4{dd * (float)((sc_a >> 16) & 0xFFu), dmin * (float)((mn_a >> 16) & 0xFFu),
                       dd * (float)(sc_a >> 24), dmin * (float)(mn_a >> 24)};
        dp[2] = float4{dd * (float)(sc_b & 0xFFu), dmin * (float)(mn_b & 0xFFu), dd * (float)((sc_b >> 8) & 0xFFu),
                       dmin * (float)((mn_b >> 8) & 0xFFu)};
        dp[3] = float4{dd * (float)((sc_b >> 16) & 0xFFu), dmin * (float)((mn_b >> 16) & 0xFFu),
                       dd * (float)(sc_b >> 24), dmin * (float)(mn_b >> 24)};
    }

    // ---- 4. nine pieces per lane: MFMA sums, then scale and accumulate ----------
    // A-operand role of this lane: row l%16 of k-slot group g is live when
    // row/4 == g and row%4 < 3 (the digit plane).
    const int arow = lane & 15, aslot = arow & 3;
    const bool a_role = (arow >> 2) == g && aslot < 3;
    const int a_plane = L.planes + aslot * pstride + uq * (Q4K_UNIT_BLOCKS * 256);
    const int scl_unit = L.scl + (Q4K_UNIT_BLOCKS * uq) * 128;

    float acc[MT];
#pragma unroll
    for (int mi = 0; mi < MT; mi++) acc[mi] = 0.0f;

#pragma unroll
    for (int i = 0; i < 9; i++) {
        if (i % 3 == 0) __builtin_amdgcn_sched_barrier(0);  // schedule three pieces at a time
        const uint32_t code = (q4k_piece_codes(i) >> (8 * g)) & 0xFFu;
        const int blk = (code >> 4) & 3;
        const bool live = code < 0x80u && blk < nbv && wave_live;
        const int idx = live ? (int)code : 0;  // 16*b + 4*c + h
        const int a_off = a_role && live ? a_plane + 16 * idx : L.zeros;
        const int s_off = live ? scl_unit + ((idx >> 4) * 8 + ((idx >> 2) & 3) * 2 + (idx & 1)) * 16 : L.zeros;
        const float4 dq = *(const float4 *)(dec + (blk * 16 + nl) * Q4K_DEC_ROW + ((idx >> 2) & 3) * 16);

        const v4i b_lo = {(int)(t[i].x & 0x0F0F0F0Fu), (int)(t[i].y & 0x0F0F0F0Fu), (int)(t[i].z & 0x0F0F0F0Fu),
                          (int)(t[i].w & 0x0F0F0F0Fu)};
        const v4i b_hi = {(int)((t[i].x >> 4) & 0x0F0F0F0Fu), (int)((t[i].y >> 4) & 0x0F0F0F0Fu),
                          (int)((t[i].z >> 4) & 0x0F0F0F0Fu), (int)((t[i].w >> 4) & 0x0F0F0F0Fu)};
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            const int a_m = a_role && live ? mi * 3 * pstride : 0;
            const int s_m = live ? mi * bpr * 128 : 0;
            const v4i a_lo = *(const v4i *)(lds + a_off + a_m);
            const v4i a_hi = *(const v4i *)(lds + a_off + a_m + 32);
            const float4 sx = *(const float4 *)(lds + s_off + s_m);  // s_lo, sum_lo, s_hi, sum_hi
            v4i c_lo = {0, 0, 0, 0}, c_hi = {0, 0, 0, 0};
            c_lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_lo, b_lo, c_lo, 0, 0, 0);
            c_hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(a_hi, b_hi, c_hi, 0, 0, 0);
            const float v_lo = (float)(int)(((uint32_t)c_lo[2] << 16) + ((uint32_t)c_lo[1] << 8) + (uint32_t)c_lo[0]);
            const float v_hi = (float)(int)(((uint32_t)c_hi[2] << 16) + ((uint32_t)c_hi[1] << 8) + (uint32_t)c_hi[0]);
            acc[mi] = fmaf(v_lo, dq.x * sx.x, acc[mi]);
            acc[mi] = fmaf(-dq.y, sx.y, acc[mi]);
            acc[mi] = fmaf(v_hi, dq.z * sx.z, acc[mi]);
            acc[mi] = fmaf(-dq.w, sx.w, acc[mi]);
            // finish every third piece before more MFMA results pile up in registers
            if (i % 3 == 2) asm volatile("" : "+v"(acc[mi]));
        }
    }

    // ---- 5. sum a row's four lanes, then the tile's units in a fixed order -----
    float *partial = (float *)(lds + L.partial);
#pragma unroll
    for (int mi = 0; mi < MT; mi++) {
        float v = acc[mi];
        v = sum_xor16(v);
        v = sum_xor32(v);
        if (lane < 16) partial[(wave * MT + mi) * 16 + lane] = v;
    }
    __syncthreads();
    if (wave_live && uq == 0 && lane < 16) {
#pragma unroll
        for (int mi = 0; mi < MT; mi++) {
            float v = 0.0f;
            for (int u = 0; u < units_per_tile; u++) v += partial[((wave + u) * MT + mi) * 16 + lane];
            if (row0 + lane < n && m0 + mi < m) Y[(size_t)(m0 + mi) * n + row0 + lane] = v;
        }
    }
}

}  // namespace jq
