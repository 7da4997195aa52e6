// Q4_K, Q6_K, Q2_K and Q8_0 matmul for many activation rows on the int8 matrix cores.  The arithmetic is
// written out for Q4_K; Q6_K (w = d sc (q - 32), signed 8-bit sc, no min term) takes the same path with
// p = sc (q - 32), Q2_K with a one-byte p = sc q and sixteen sub-blocks in I2, Q8_0 with eight blocks put on
// a common scale (QiQ2K, QiQ8_0 below).
//
// Per 256-element super-block B of weight row n and activation row m (reference arithmetic
// w = d sc q - dmin m, src/kquant_dot.rs:440-465):
//
//   sum_k x_k w_k = s (d I1 - dmin I2),   I1 = sum_k (sc_j(k) q_k) X_k,   I2 = sum_j m_j XS_j
//
// with the activations in 16-bit fixed point per (row, super-block), X = round(x / s), s = amax_B |x| / 32639,
// and XS_j the sum of X over sub-block j.  Both factors of I1 are split into two signed bytes,
//
//   X = 256 Xh + Xl          p = sc q = 256 Ph + Pl   (p <= 945: Ph = (p + 128) >> 8 in 0..4, Pl in -128..127)
//   I1 = 65536 HH + 256 MID + LL,   HH = sum Xh Ph,  MID = sum Xh Pl + Xl Ph,  LL = sum Xl Pl
//
// so that the 6-bit sub-block scales are part of the integer operand and every super-block costs four
// v_mfma_i32_16x16x64_i8 per 64 k and 16 x 16 outputs, with int32 sums that are exact, and one conversion
// to f32 per super-block (seven vector instructions an output) instead of one per sub-block.  I2 is one
// v_mfma_f32_16x16x32_f16 per super-block over exact f16 integers (XS = 1024 a1 + a0 against m and 1024 m).
// A single scale per 256 activations leaves an error of at most 2^-16 of the super-block's largest
// magnitude per element: rows whose values span many orders of magnitude inside one super-block are
// resolved relative to the largest of them, like the reference's own 8-bit Q8_K activations
// (src/kquant_dot.rs:407-483) but with 256 times the resolution.
//
// Workgroup: NW waves, tile 32 NW activation rows x 16 NG weight rows; a wave owns 32 activation rows (two
// groups of 16) against all 16 NG weight rows.  Each thread takes the packed bytes of (weight row, 64-k
// chunk) units from global memory an iteration ahead, multiplies the nibbles by their scales (two elements an
// instruction), splits the products and stores them into LDS as MFMA B operands: two buffers, one barrier a
// super-block, an eighth of the work in every eighth of the iteration.  The activation operands come
// prepared in operand order (q4k_gemm_i8_prep) straight from global memory (L2) into registers, one chunk of
// one row group at a time, three quarters of a half iteration before the MFMAs want them.
//
// What bounds it (counters at 512 x 4096 x 14336): the matrix cores are busy 59 % of the cycles and the
// vector ALU most of the rest: on this part an MFMA and a vector instruction of the same SIMD hardly
// overlap (a loop of independent MFMAs slows by about 2.7 cycles for every vector instruction put between
// them, with two waves a SIMD), so the seven instructions an output and super-block of the conversion and the
// ~150 of the unpack add to the MFMA time instead of hiding under it.
#pragma once
#include "kernels_mfma_q4k_rows16.hpp"

namespace jq {

typedef _Float16 qi_h2 __attribute__((ext_vector_type(2)));
typedef _Float16 qi_h8 __attribute__((ext_vector_type(8)));

// Prepared activations, per (group of 16 activation rows, super-block): 4 chunks x 2 planes (Xh, Xl) x 64
// lanes x 16 bytes (lane (i = lane % 16, g = lane / 16): elements 64 c + 16 g .. + 15 of row i), then the I2
// operand (64 lanes x 8 halves: g = 0 holds a0 of the 8 sub-blocks, g = 1 a1, g = 2, 3 zero), then s of the
// 16 rows.
constexpr int QI_PLANES = 4 * 2 * 64 * 16, QI_MIN = QI_PLANES, QI_SCALE = QI_PLANES + 1024, QI_REC = QI_SCALE + 64;

// The 16 elements v[] of a thread (wave c, lane (i, g): elements 64 c + 16 g .. of row i of the row group)
// become the record `rec` of (row group, super-block).  256 threads.
// With SUB16 the I2 operand is over the 16 sub-blocks of 16 elements (Q2_K): g = 0 holds a0 of sub-blocks
// 0..7, g = 1 a0 of 8..15, g = 2 and 3 a1 of the same.
template <bool SUB16>
__device__ __forceinline__ void qi_prep_record(const float (&v)[16], uint8_t *__restrict__ rec) {
    __shared__ float amax_sh[4][16];
    __shared__ int xs_sh[16][SUB16 ? 16 : 8];
    const int tid = threadIdx.x, lane = tid & 63, c = tid >> 6, i = lane & 15, g = lane >> 4;
    float amax = 0.0f;
#pragma unroll
    for (int e = 0; e < 16; e++) amax = fmaxf(amax, mag_or_inf(v[e]));
    amax = max_xor32(max_xor16(amax));  // the four lane groups of this wave
    if (g == 0) amax_sh[c][i] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(amax_sh[0][i], amax_sh[1][i]), fmaxf(amax_sh[2][i], amax_sh[3][i]));
    const bool live = amax > 0.0f && amax < INFINITY;
    const float inv = live ? QD_RANGE / amax : 0.0f, s = fixed_scale(amax, QD_RANGE);
    uint32_t h[4] = {0, 0, 0, 0}, l[4] = {0, 0, 0, 0};
    int sum = 0;
#pragma unroll
    for (int e = 0; e < 16; e++) {
        const int Xq = __float2int_rn(v[e] * inv);
        l[e >> 2] |= (uint32_t)(Xq & 255) << (8 * (e & 3));
        h[e >> 2] |= (uint32_t)(((Xq + 128) >> 8) & 255) << (8 * (e & 3));
        sum += Xq;
    }
    if (SUB16) {
        xs_sh[i][4 * c + g] = sum;  // a lane's 16 elements are a sub-block
    } else {
        sum = isum_xor16(sum);  // the two lane groups of a sub-block
        if ((g & 1) == 0) xs_sh[i][2 * c + (g >> 1)] = sum;
    }
    // word w of chunk c at position (w + c) % 4, as in the weight tiles (qi_word)
    auto rotated = [&](const uint32_t (&v)[4]) {
        uint32_t a0 = v[0], a1 = v[1], a2 = v[2], a3 = v[3];
        if (c & 1) {
            const uint32_t t = a3;
            a3 = a2, a2 = a1, a1 = a0, a0 = t;
        }
        if (c & 2) {
            const uint32_t t0 = a0, t1 = a1;
            a0 = a2, a1 = a3, a2 = t0, a3 = t1;
        }
        return uint4{a0, a1, a2, a3};
    };
    *(uint4 *)(rec + ((size_t)(2 * c) * 64 + lane) * 16) = rotated(h);
    *(uint4 *)(rec + ((size_t)(2 * c + 1) * 64 + lane) * 16) = rotated(l);
    __syncthreads();
    if (tid < 64) {
        uint32_t w[4] = {0, 0, 0, 0};
        if (SUB16 || g < 2) {
#pragma unroll
            for (int j = 0; j < 8; j += 2) {
                qi_h2 pair;
#pragma unroll
                for (int e = 0; e < 2; e++) {
                    const int xs = xs_sh[i][(SUB16 ? 8 * (g & 1) : 0) + j + e], a1 = (xs + 512) >> 10, a0 = xs - 1024 * a1;
                    pair[e] = (_Float16)(float)((SUB16 ? g < 2 : g == 0) ? a0 : a1);
                }
                w[j >> 1] = __builtin_bit_cast(uint32_t, pair);
            }
        }
        *(uint4 *)(rec + QI_MIN + lane * 16) = uint4{w[0], w[1], w[2], w[3]};
    }
    if (tid < 16) ((float *)(rec + QI_SCALE))[tid] = s;
}

// grid (k / 256 super-blocks, groups of 16 activation rows), 256 threads.  Rows from m_rows on are zero
// operands.
// With PAIRS the activations are silu(gate) * up over rows of 2 k floats in which gate_j and up_j alternate
// (the result of a product with a row-paired gate|up matrix): the SwiGLU of a feed-forward block happens on the
// way into the down projection.
template <bool PAIRS, bool SUB16 = false>
__global__ __launch_bounds__(256) void q4k_gemm_i8_prep(const float *__restrict__ X, int m_rows, int k,
                                                         uint8_t *__restrict__ out) {
    const int tid = threadIdx.x, lane = tid & 63, c = tid >> 6, i = lane & 15, g = lane >> 4;
    const int b = blockIdx.x, row = 16 * (int)blockIdx.y + i;
    uint8_t *rec = out + ((size_t)blockIdx.y * gridDim.x + b) * QI_REC;
    float v[16];
    if (row < m_rows && PAIRS) {
        const float4 *src = (const float4 *)(X + 2 * ((size_t)row * k + 256 * b + 64 * c + 16 * g));
#pragma unroll
        for (int q = 0; q < 8; q++) {
            const float4 a = src[q];
            v[2 * q] = silu(a.x) * a.y, v[2 * q + 1] = silu(a.z) * a.w;
        }
    } else if (row < m_rows) {
        const float4 *src = (const float4 *)(X + (size_t)row * k + 256 * b + 64 * c + 16 * g);
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const float4 a = src[q];
            v[4 * q] = a.x, v[4 * q + 1] = a.y, v[4 * q + 2] = a.z, v[4 * q + 3] = a.w;
        }
    } else {
#pragma unroll
        for (int e = 0; e < 16; e++) v[e] = 0.0f;
    }
    qi_prep_record<SUB16>(v, rec);
}

// The grouped product (expert matmuls over (token, slot) pairs sorted by expert): pairs offsets[g] ..
// offsets[g + 1] - 1 of group g are laid out in row groups of 16 that never mix two experts, and the row
// groups of an expert in tiles of up to `tile_rgs` of them.  One workgroup of 256 threads writes the tables:
//   rg_pair[r], rg_cnt[r]   first pair and number of pairs (1..16) of row group r
//   mt_group[t], mt_rg0[t], mt_nrg[t]   group, first row group and number of row groups of tile t
//   counts[0], counts[1]    row groups and tiles in all
// for at most max_rg row groups and max_mt tiles (callers size them as pairs / 16 + groups and
// pairs / (16 tile_rgs) + groups, which always suffice).
// tile_rgs = 0, the mixed plan: an expert's row groups go eight to a tile while five or more are left (mt_*, counts[1]
// of them, at most row groups / 5) and the rest two to a tile (`small`'s mt_*, counts[2] of them, at most two an expert),
// for two launches: tiles whose waves share the rows where an expert has many pairs, tiles whose waves share the weight
// rows for the tails and for experts with few.  `small.counts` is counts + 1, so that either launch finds its tile count
// at counts[1].
struct QiGroupTables {
    int *rg_pair, *rg_cnt, *mt_group, *mt_rg0, *mt_nrg, *counts;
};
__global__ __launch_bounds__(256) void moe_gemm_i8_plan(const int *__restrict__ offsets, int groups, int tile_rgs,
                                                         QiGroupTables t, QiGroupTables small = QiGroupTables{}) {
    if (tile_rgs == 0) {
        __shared__ int base[3][257], run[3];
        if (threadIdx.x == 0) run[0] = run[1] = run[2] = 0;
        __syncthreads();
        for (int g0 = 0; g0 < groups; g0 += 256) {
            const int g = g0 + (int)threadIdx.x;
            const int cnt = g < groups ? offsets[g + 1] - offsets[g] : 0;
            const int nrg = (cnt + 15) >> 4;
            const int nbig = nrg / 8 + (nrg % 8 >= 5 ? 1 : 0), rest = max(nrg - 8 * nbig, 0), nsmall = (rest + 1) / 2;
            base[0][threadIdx.x] = nrg, base[1][threadIdx.x] = nbig, base[2][threadIdx.x] = nsmall;
            __syncthreads();
            if (threadIdx.x < 3) {
                int a = run[threadIdx.x];
                for (int i = 0; i < 256; i++) {
                    const int x = base[threadIdx.x][i];
                    base[threadIdx.x][i] = a;
                    a += x;
                }
                run[threadIdx.x] = a;
            }
            __syncthreads();
            if (g < groups) {
                const int first = offsets[g], rg0 = base[0][threadIdx.x];
                for (int r = 0; r < nrg; r++) {
                    t.rg_pair[rg0 + r] = first + 16 * r;
                    t.rg_cnt[rg0 + r] = min(16, cnt - 16 * r);
                }
                for (int q = 0; q < nbig; q++) {
                    const int at = base[1][threadIdx.x] + q;
                    t.mt_group[at] = g, t.mt_rg0[at] = rg0 + 8 * q, t.mt_nrg[at] = min(8, nrg - 8 * q);
                }
                for (int q = 0; q < nsmall; q++) {
                    const int at = base[2][threadIdx.x] + q;
                    small.mt_group[at] = g, small.mt_rg0[at] = rg0 + 8 * nbig + 2 * q, small.mt_nrg[at] = min(2, rest - 2 * q);
                }
            }
            __syncthreads();
        }
        if (threadIdx.x == 0) t.counts[0] = run[0], t.counts[1] = run[1], t.counts[2] = run[2];
        return;
    }
    __shared__ int rg_base[257], mt_base[257];
    // serial prefix over the groups in chunks of 256 (a few hundred groups at most)
    __shared__ int carry[2];
    if (threadIdx.x == 0) carry[0] = carry[1] = 0;
    __syncthreads();
    for (int g0 = 0; g0 < groups; g0 += 256) {
        const int g = g0 + (int)threadIdx.x;
        const int cnt = g < groups ? offsets[g + 1] - offsets[g] : 0;
        const int nrg = (cnt + 15) >> 4, nmt = (nrg + tile_rgs - 1) / tile_rgs;
        rg_base[threadIdx.x] = nrg, mt_base[threadIdx.x] = nmt;
        __syncthreads();
        if (threadIdx.x == 0) {
            int a = carry[0], b = carry[1];
            for (int i = 0; i < 256; i++) {
                const int x = rg_base[i], y = mt_base[i];
                rg_base[i] = a, mt_base[i] = b;
                a += x, b += y;
            }
            carry[0] = a, carry[1] = b;
        }
        __syncthreads();
        if (g < groups) {
            const int first = offsets[g];
            for (int r = 0; r < nrg; r++) {
                t.rg_pair[rg_base[threadIdx.x] + r] = first + 16 * r;
                t.rg_cnt[rg_base[threadIdx.x] + r] = min(16, cnt - 16 * r);
            }
            for (int q = 0; q < nmt; q++) {
                t.mt_group[mt_base[threadIdx.x] + q] = g;
                t.mt_rg0[mt_base[threadIdx.x] + q] = rg_base[threadIdx.x] + tile_rgs * q;
                t.mt_nrg[mt_base[threadIdx.x] + q] = min(tile_rgs, nrg - tile_rgs * q);
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) t.counts[0] = carry[0], t.counts[1] = carry[1];
}

// Prepared activations of the grouped product: grid (k / 256, max row groups); row i of row group r is
// X[xsel[rg_pair[r] + i]] (rows past rg_cnt[r] are zero operands; workgroups past counts[0] leave).
template <bool SUB16>
__global__ __launch_bounds__(256) void moe_gemm_i8_prep(const float *__restrict__ X, const int *__restrict__ xsel,
                                                         QiGroupTables t, int k, uint8_t *__restrict__ out) {
    const int r = (int)blockIdx.y;
    if (r >= t.counts[0]) return;
    const int tid = threadIdx.x, lane = tid & 63, c = tid >> 6, i = lane & 15, g = lane >> 4;
    const int b = blockIdx.x;
    uint8_t *rec = out + ((size_t)r * gridDim.x + b) * QI_REC;
    float v[16];
    if (i < t.rg_cnt[r]) {
        const float4 *src = (const float4 *)(X + (size_t)xsel[t.rg_pair[r] + i] * k + 256 * b + 64 * c + 16 * g);
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const float4 a = src[q];
            v[4 * q] = a.x, v[4 * q + 1] = a.y, v[4 * q + 2] = a.z, v[4 * q + 3] = a.w;
        }
    } else {
#pragma unroll
        for (int e = 0; e < 16; e++) v[e] = 0.0f;
    }
    qi_prep_record<SUB16>(v, rec);
}

// LDS per buffer: NG tiles of 16 weight rows x [chunk 4][plane 2 (Ph, Pl)][lane 64] x 16 bytes, then per
// weight row F::META bytes: the I2 operands of the lane groups (16 bytes each), d and dmin as floats in the
// last 16.  With eight sub-blocks (48 bytes): m_0..7 as halves, 1024 m_0..7 as halves; with sixteen (80
// bytes): m_0..7, m_8..15, 1024 m_0..7, 1024 m_8..15.
constexpr int QI_TILE = 4 * 2 * 64 * 16;
template <class F, int NG, bool SINGLE = false>
constexpr int qi_lds_bytes() { return (SINGLE ? 1 : 2) * (NG * QI_TILE + 16 * NG * F::META) + F::TABLE; }

typedef short qi_s2 __attribute__((ext_vector_type(2)));

// Where word wi (elements 4 wi .. + 3) of a lane's 16 operand bytes of chunk uc goes: rotated by the chunk
// number, in the weight tiles and in the activation records alike (the MFMA sums over a lane's 16 elements, so
// their order is free as long as both operands agree).  The four threads of a weight row unpack its four chunks
// at once, and unrotated their stores fall on the same LDS bank (the chunks are 2048 bytes apart).
__device__ __forceinline__ int qi_word(int uc, int wi) { return 4 * ((wi + uc) & 3); }

// A format's side of the GEMM.  A thread's unit is (weight row, 64-k chunk uc) of a super-block at `blk`:
// fetch() takes its bytes in three parts (0: the scales, into `next`, 1, 2: the halves of the chunk's
// packed bytes), take() makes the scales fetched ahead current (and builds what depends on them alone),
// piece(j) turns the bytes of elements
// 16 g + 4 (j % 4) .. + 3 of slices g = j / 4 and 2 + j / 4 into operand words (p + 128 = 256 Ph + L,
// Pl = L - 128; slice g of the chunk at tile + 256 g, plane Pl 1024 bytes further), meta() writes the
// row's 48 bytes.
struct QiQ4K {  // w = d sc q - dmin m, 6-bit sc and m, q in 0..15: p = sc q in 0..945
    static constexpr int BLOCK = 144, META = 48, ALIGN = 16, TABLE = 0;
    static constexpr bool HAS_MIN = true, ONE_PLANE = false, SUB16 = false;
    struct Hdr {
        uint4 h;
    };
    struct Raw {
        Hdr hdr;
        uint4 q0, q1;
    };
    __device__ __forceinline__ static void fetch(const uint8_t *blk, int uc, int part, Raw &raw, Hdr &next) {
        if (part == 0) next.h = *(const uint4 *)blk;
        if (part == 1) raw.q0 = *(const uint4 *)(blk + 16 + 32 * uc);
        if (part == 2) raw.q1 = *(const uint4 *)(blk + 32 + 32 * uc);
    }
    __device__ __forceinline__ static void take(Raw &raw, const Hdr &next, int uc, const uint8_t *) { raw.hdr = next; }
    __device__ __forceinline__ static void piece(const Raw &raw, int uc, int j, uint8_t *tile, const uint8_t *) {
        const uint4 hdr = raw.hdr.h;
        const uint32_t scl = hdr.y & 0x3F3F3F3Fu, sch = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
        const uint32_t s4 = (uc < 2 ? scl : sch) >> (16 * (uc & 1));
        const uint32_t sc[2] = {s4 & 0xFFu, (s4 >> 8) & 0xFFu};
        const uint4 qv = j < 4 ? raw.q0 : raw.q1;
        const uint32_t word = (j & 3) == 0 ? qv.x : (j & 3) == 1 ? qv.y : (j & 3) == 2 ? qv.z : qv.w;
#pragma unroll
        for (int nib = 0; nib < 2; nib++) {  // low nibbles: sub-block 2 uc, high nibbles: sub-block 2 uc + 1
            // two elements an instruction (v_mad_u32_u24): elements 0, 2 of the word in `even`, 1, 3 in `odd`
            const uint32_t w = nib ? word >> 4 : word;
            const uint32_t even = __umul24(w & 0x000F000Fu, sc[nib]) + 0x00800080u;
            const uint32_t odd = __umul24((w >> 8) & 0x000F000Fu, sc[nib]) + 0x00800080u;
            const int gg = 2 * nib + (j >> 2);
            *(uint32_t *)(tile + gg * 256 + qi_word(uc, j & 3)) = __builtin_amdgcn_perm(odd, even, 0x07030501u);
            *(uint32_t *)(tile + 1024 + gg * 256 + qi_word(uc, j & 3)) = __builtin_amdgcn_perm(odd, even, 0x06020400u) ^ 0x80808080u;
        }
    }
    __device__ __forceinline__ static void meta(const Raw &raw, int uc, uint8_t *meta) {  // the min scales, d and dmin
        const uint4 hdr = raw.hdr.h;
        const uint32_t mnl = hdr.z & 0x3F3F3F3Fu, mnh = ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u);
        const uint32_t m4 = (uc < 2 ? mnl : mnh) >> (16 * (uc & 1));
        const float mn[2] = {(float)(m4 & 0xFFu), (float)((m4 >> 8) & 0xFFu)};
        const qi_h2 m1 = {(_Float16)mn[0], (_Float16)mn[1]}, m1k = {(_Float16)(1024.0f * mn[0]), (_Float16)(1024.0f * mn[1])};
        *(uint32_t *)(meta + 4 * uc) = __builtin_bit_cast(uint32_t, m1);
        *(uint32_t *)(meta + 16 + 4 * uc) = __builtin_bit_cast(uint32_t, m1k);
        *(float2 *)(meta + 32) = float2{f16_bits(hdr.x), f16_bits(hdr.x >> 16)};  // the same from all four
    }
};

// Q6_K: ql[128] | qh[64] | scales[16] i8 | d, w = d sc (q - 32) with q in 0..63 (layout:
// vendor/candle-metal-kernels/src/metal_src/quantized.metal:198-203, 6673-6694): p = sc (q - 32) in
// -4096..3968, Ph in -16..15, no min term.  Chunk uc = 2 h + jj of the super-block is elements
// 128 h + 64 jj + e: e < 32 from ql[64 h + e] and qh[32 h + e] >> 4 jj, e >= 32 from ql[64 h + e] and
// qh[32 h + e - 32] >> (4 jj + 2), nibble jj of ql, scales[8 h + 4 jj + e / 16].  Blocks of 210 bytes sit at
// even addresses only: everything is read through aligned words.
struct QiQ6K {
    static constexpr int BLOCK = 210, META = 48, ALIGN = 2, TABLE = 0;
    static constexpr bool HAS_MIN = false, ONE_PLANE = false, SUB16 = false;
    struct Hdr {
        uint32_t sc4, d;
    };
    struct Raw {
        Hdr hdr;
        uint4 la[2], lb[2], hv[2];  // halves of ql[64 h ..+31], ql[64 h + 32 ..+31], qh[32 h ..+31]
    };
    __device__ __forceinline__ static void fetch(const uint8_t *blk, int uc, int part, Raw &raw, Hdr &next) {
        const int h = uc >> 1;
        if (part == 0) next.sc4 = ldw<uint32_t>(blk + 192 + 4 * uc), next.d = ld<uint16_t>(blk + 208);
        if (part == 1 || part == 2) {
            const int o = 16 * (part - 1);
            raw.la[part - 1] = ldw<uint4>(blk + 64 * h + o);
            raw.lb[part - 1] = ldw<uint4>(blk + 64 * h + 32 + o);
            raw.hv[part - 1] = ldw<uint4>(blk + 128 + 32 * h + o);
        }
    }
    __device__ __forceinline__ static void take(Raw &raw, const Hdr &next, int uc, const uint8_t *) { raw.hdr = next; }
    __device__ __forceinline__ static uint32_t word_of(const uint4 &v, int i) {
        return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w;
    }
    __device__ __forceinline__ static void piece(const Raw &raw, int uc, int j, uint8_t *tile, const uint8_t *) {
        const int sh = 4 * (uc & 1), half = j >> 2, wi = j & 3;
        const uint32_t qh = word_of(raw.hv[half], wi) >> sh;
        const uint32_t lo[2] = {word_of(raw.la[half], wi) >> sh, word_of(raw.lb[half], wi) >> sh};
#pragma unroll
        for (int e32 = 0; e32 < 2; e32++) {  // elements 16 half + 4 wi .. of the first and second 32 of the chunk
            const uint32_t q = (lo[e32] & 0x0F0F0F0Fu) | (((qh >> (2 * e32)) & 0x03030303u) << 4);
            const int gg = 2 * e32 + half;
            const short sc = (short)(int8_t)(raw.hdr.sc4 >> (8 * gg));
            const short bias = (short)(128 - 32 * sc);
            // two elements an instruction (v_pk_mad_i16): sc q + 128 - 32 sc in -3968..4096 as signed halfwords
            const qi_s2 even = __builtin_bit_cast(qi_s2, q & 0x00FF00FFu) * qi_s2{sc, sc} + qi_s2{bias, bias};
            const qi_s2 odd = __builtin_bit_cast(qi_s2, (q >> 8) & 0x00FF00FFu) * qi_s2{sc, sc} + qi_s2{bias, bias};
            const uint32_t ev = __builtin_bit_cast(uint32_t, even), od = __builtin_bit_cast(uint32_t, odd);
            *(uint32_t *)(tile + gg * 256 + qi_word(uc, wi)) = __builtin_amdgcn_perm(od, ev, 0x07030501u);
            *(uint32_t *)(tile + 1024 + gg * 256 + qi_word(uc, wi)) = __builtin_amdgcn_perm(od, ev, 0x06020400u) ^ 0x80808080u;
        }
    }
    __device__ __forceinline__ static void meta(const Raw &raw, int uc, uint8_t *meta) {
        *(float2 *)(meta + 32) = float2{f16_bits(raw.hdr.d), 0.0f};  // the same from all four
    }
};

// Q2_K: scales[16] (scale | min << 4) | qs[64] | d | dmin, w = d sc q - dmin m with q in 0..3 and 4-bit sc and m
// over sub-blocks of 16 elements (src/kquant_dot.rs:63-76, 345-385): element 128 sg + 32 f + 16 hf + i is
// field f of qs[32 sg + 16 hf + i] with the scale byte 8 sg + 2 f + hf.  p = sc q in 0..45 is a single signed
// byte: Ph = 0, so HH and half of MID vanish and a chunk costs two MFMAs instead of four.  Chunk uc is
// elements 64 uc ..: slice gg of 16 is sub-block 4 uc + gg, fields 2 (uc % 2) + gg / 2 of the 16 bytes
// qs[32 (uc / 2) + 16 (gg % 2) ..].  The four products of a byte come out of a register table (0, sc, 2 sc,
// 3 sc) with one v_perm_b32 per four elements.
struct QiQ2K {
    static constexpr int BLOCK = 84, META = 80, ALIGN = 4, TABLE = 0;
    static constexpr bool HAS_MIN = true, ONE_PLANE = true, SUB16 = true;
    struct Hdr {
        uint32_t sc4, dd;
    };
    struct Raw {
        Hdr hdr;
        uint32_t table[4];  // per slice: sc * (0, 1, 2, 3) as bytes
        uint4 q0, q1;
    };
    __device__ __forceinline__ static void fetch(const uint8_t *blk, int uc, int part, Raw &raw, Hdr &next) {
        if (part == 0) next.sc4 = ld<uint32_t>(blk + 4 * uc), next.dd = ld<uint32_t>(blk + 80);
        if (part == 1) raw.q0 = ld<uint4>(blk + 16 + 32 * (uc >> 1));
        if (part == 2) raw.q1 = ld<uint4>(blk + 32 + 32 * (uc >> 1));
    }
    __device__ __forceinline__ static void take(Raw &raw, const Hdr &next, int uc, const uint8_t *) {
        raw.hdr = next;
#pragma unroll
        for (int gg = 0; gg < 4; gg++) {
            const uint32_t sc = (next.sc4 >> (8 * gg)) & 0xFu;
            raw.table[gg] = (sc << 8) + (sc << 17) + ((sc + 2 * sc) << 24);
        }
    }
    __device__ __forceinline__ static void piece(const Raw &raw, int uc, int j, uint8_t *tile, const uint8_t *) {
        const int half = j >> 2, wi = j & 3;
        const uint4 qv = half ? raw.q1 : raw.q0;
        const uint32_t word = (wi == 0 ? qv.x : wi == 1 ? qv.y : wi == 2 ? qv.z : qv.w) >> (4 * (uc & 1));
#pragma unroll
        for (int e = 0; e < 2; e++) {  // slices half and 2 + half: the same bytes, the next field
            const int gg = 2 * e + half;
            const uint32_t q = (word >> (2 * e)) & 0x03030303u;
            *(uint32_t *)(tile + 1024 + gg * 256 + qi_word(uc, wi)) = __builtin_amdgcn_perm(0u, raw.table[gg], q);
        }
    }
    __device__ __forceinline__ static void meta(const Raw &raw, int uc, uint8_t *meta) {
        float mn[4];
#pragma unroll
        for (int gg = 0; gg < 4; gg++) mn[gg] = (float)((raw.hdr.sc4 >> (8 * gg + 4)) & 0xFu);
#pragma unroll
        for (int e = 0; e < 2; e++) {
            const qi_h2 m1 = {(_Float16)mn[2 * e], (_Float16)mn[2 * e + 1]};
            const qi_h2 m1k = {(_Float16)(1024.0f * mn[2 * e]), (_Float16)(1024.0f * mn[2 * e + 1])};
            *(uint32_t *)(meta + 8 * uc + 4 * e) = __builtin_bit_cast(uint32_t, m1);
            *(uint32_t *)(meta + 32 + 8 * uc + 4 * e) = __builtin_bit_cast(uint32_t, m1k);
        }
        *(float2 *)(meta + 64) = float2{f16_bits(raw.hdr.dd), f16_bits(raw.hdr.dd >> 16)};  // the same from all four
    }
};

// Q8_0: blocks of d (f16) | 32 signed bytes, w = d q (src/kquant_dot.rs:37-46); a "super-block" here is eight
// blocks, 272 bytes.  The scale of a block of 32 cannot ride in an integer operand exactly, so the eight
// blocks are put on one scale D / 256, D the largest |d| among them: p = round(256 q d / D) in
// -32512..32512, w ~ (D / 256) p.  That resolves every weight to 2^-16 of the largest magnitude its 256-run
// can hold -- what the activations' fixed point does on their side -- and is exact where the eight scales are
// equal.  Chunk uc is blocks 2 uc and 2 uc + 1; the four threads of a weight row are neighbouring lanes and
// agree on D with two quad permutes.  Blocks sit at even addresses only: read through aligned words.
struct QiQ8_0 {
    static constexpr int BLOCK = 272, META = 48, ALIGN = 2, TABLE = 0;
    static constexpr bool HAS_MIN = false, ONE_PLANE = false, SUB16 = false;
    struct Hdr {
        float d0, d1;
    };
    struct Raw {
        float r0, r1, unit;  // 256 d / D of the chunk's two blocks, and D / 256
        uint4 qa[2], qb[2];  // halves of the quants of block 2 uc and of block 2 uc + 1
    };
    __device__ __forceinline__ static void fetch(const uint8_t *blk, int uc, int part, Raw &raw, Hdr &next) {
        if (part == 0) next.d0 = f16_bits(ld<uint16_t>(blk + 68 * uc)), next.d1 = f16_bits(ld<uint16_t>(blk + 68 * uc + 34));
        if (part == 1 || part == 2) {
            raw.qa[part - 1] = ldw<uint4>(blk + 68 * uc + 2 + 16 * (part - 1));
            raw.qb[part - 1] = ldw<uint4>(blk + 68 * uc + 36 + 16 * (part - 1));
        }
    }
    __device__ __forceinline__ static void take(Raw &raw, const Hdr &next, int uc, const uint8_t *) {
        float D = fmaxf(mag_or_inf(next.d0), mag_or_inf(next.d1));
        D = fmaxf(D, dpp_f<0xB1>(D));  // quad_perm [1,0,3,2]
        D = fmaxf(D, dpp_f<0x4E>(D));  // quad_perm [2,3,0,1]
        const float inv = D > 0.0f ? 256.0f / D : 0.0f;
        raw.r0 = next.d0 * inv, raw.r1 = next.d1 * inv, raw.unit = D * (1.0f / 256.0f);
    }
    __device__ __forceinline__ static void piece(const Raw &raw, int uc, int j, uint8_t *tile, const uint8_t *) {
        const int half = j >> 2, wi = j & 3;
#pragma unroll
        for (int e32 = 0; e32 < 2; e32++) {
            const uint4 qv = e32 ? raw.qb[half] : raw.qa[half];
            const uint32_t word = wi == 0 ? qv.x : wi == 1 ? qv.y : wi == 2 ? qv.z : qv.w;
            const float ratio = e32 ? raw.r1 : raw.r0;
            // round(q ratio) + 128 in the low 16 bits of 1.5 * 2^23 + 128 + q ratio
            uint32_t t[4];
#pragma unroll
            for (int b = 0; b < 4; b++)
                t[b] = __builtin_bit_cast(uint32_t, fmaf((float)(int)(int8_t)(word >> (8 * b)), ratio, 12583040.0f));
            const uint32_t even = __builtin_amdgcn_perm(t[2], t[0], 0x05040100u), odd = __builtin_amdgcn_perm(t[3], t[1], 0x05040100u);
            const int gg = 2 * e32 + half;
            *(uint32_t *)(tile + gg * 256 + qi_word(uc, wi)) = __builtin_amdgcn_perm(odd, even, 0x07030501u);
            *(uint32_t *)(tile + 1024 + gg * 256 + qi_word(uc, wi)) = __builtin_amdgcn_perm(odd, even, 0x06020400u) ^ 0x80808080u;
        }
    }
    __device__ __forceinline__ static void meta(const Raw &raw, int uc, uint8_t *meta) {
        *(float2 *)(meta + 32) = float2{raw.unit, 0.0f};  // the same from all four
    }
};

// IQ2_XXS: d (f16) | 8 groups of (4 codebook indices, 4 x 7 sign bits + a 4-bit scale), w = d (2 s + 1) / 8 *
// (+-grid value), grid values 8, 25 and 43 (src/iq2xxs.rs:34-71, 349-380): p = +-(2 s + 1) grid in
// -1333..1333 is exact in two bytes, the scale of a super-block is d / 8 and there is no min term.  Chunk uc is
// groups 2 uc and 2 uc + 1.  The codebook sits in LDS behind the operand buffers (a read from global memory
// in the unpacking would wait for the weight bytes asked for ahead of it); grid value v is number v >> 4 of
// the three, so per group six products (three magnitudes, two signs) make two 8-byte tables a plane and one
// v_perm_b32 a plane looks four elements up with the selector (v >> 4) | sign << 2.  Blocks of 66 bytes sit
// at even addresses only: read through aligned words.
struct QiIQ2XXS {
    static constexpr int BLOCK = 66, META = 48, ALIGN = 2, TABLE = 2048;
    static constexpr bool HAS_MIN = false, ONE_PLANE = false, SUB16 = false;
    struct Hdr {
        uint32_t d;
    };
    struct Raw {
        float unit;
        uint32_t lo[2], signs[2];        // per group: the four codes; the four sign bytes (parity bit restored)
        uint32_t th[2][2], tl[2][2];     // per group: Ph and Pl of +p_0..2 (word 0) and -p_0..2 (word 1)
        uint4 q;                         // the bytes of the next super-block's chunk
    };
    __device__ __forceinline__ static void stage(uint8_t *lds) {
        for (int i = threadIdx.x; i < 256; i += blockDim.x) ((uint64_t *)lds)[i] = g_tables.iq2xxs_grid[i];
    }
    __device__ __forceinline__ static void fetch(const uint8_t *blk, int uc, int part, Raw &raw, Hdr &next) {
        if (part == 0) next.d = ld<uint16_t>(blk);
        if (part == 2) raw.q = ldw<uint4>(blk + 2 + 16 * uc);
    }
    __device__ __forceinline__ static void take(Raw &raw, const Hdr &next, int uc, const uint8_t *) {
        raw.unit = f16_bits(next.d) * 0.125f;
        const uint32_t w[4] = {raw.q.x, raw.q.y, raw.q.z, raw.q.w};
#pragma unroll
        for (int grp = 0; grp < 2; grp++) {
            const uint32_t hi = w[2 * grp + 1];
            raw.lo[grp] = w[2 * grp];
            uint32_t signs = 0;
#pragma unroll
            for (int l = 0; l < 4; l++) {
                const uint32_t s7 = (hi >> (7 * l)) & 127u;
                signs |= (s7 | ((__popc(s7) & 1u) << 7)) << (8 * l);
            }
            raw.signs[grp] = signs;
            const int sc = 2 * (int)(hi >> 28) + 1;
            uint32_t th[2] = {0, 0}, tl[2] = {0, 0};
#pragma unroll
            for (int i = 0; i < 3; i++) {
                const int p = sc * (i == 0 ? 8 : i == 1 ? 25 : 43);
#pragma unroll
                for (int neg = 0; neg < 2; neg++) {
                    const int v = (neg ? -p : p) + 128;  // 256 Ph + L
                    th[neg] |= (uint32_t)((v >> 8) & 255) << (8 * i);
                    tl[neg] |= (uint32_t)((v & 255) ^ 128) << (8 * i);
                }
            }
            raw.th[grp][0] = th[0], raw.th[grp][1] = th[1], raw.tl[grp][0] = tl[0], raw.tl[grp][1] = tl[1];
        }
    }
    __device__ __forceinline__ static void piece(const Raw &raw, int uc, int j, uint8_t *tile, const uint8_t *tab) {
        const int half = j >> 2, wi = j & 3, l = 2 * half + (wi >> 1), hf = wi & 1;
#pragma unroll
        for (int grp = 0; grp < 2; grp++) {  // elements 16 half + 4 wi .. + 3 of both groups
            const uint32_t code = (raw.lo[grp] >> (8 * l)) & 0xFFu;
            const uint32_t mag = *(const uint32_t *)(tab + 8 * code + 4 * hf);
            const uint32_t nib = (raw.signs[grp] >> (8 * l + 4 * hf)) & 15u;
            const uint32_t sel = ((mag >> 4) & 0x03030303u) | (((nib * 0x00204081u) & 0x01010101u) << 2);
            const int gg = 2 * grp + half;
            *(uint32_t *)(tile + gg * 256 + qi_word(uc, wi)) = __builtin_amdgcn_perm(raw.th[grp][1], raw.th[grp][0], sel);
            *(uint32_t *)(tile + 1024 + gg * 256 + qi_word(uc, wi)) = __builtin_amdgcn_perm(raw.tl[grp][1], raw.tl[grp][0], sel);
        }
    }
    __device__ __forceinline__ static void meta(const Raw &raw, int uc, uint8_t *meta) {
        *(float2 *)(meta + 32) = float2{raw.unit, 0.0f};  // the same from all four
    }
};

// Blocks of 32 elements as a scale and sixteen bytes of 4-bit codes, low nibbles elements 0..15, high nibbles
// 16..31, w = scale * value(code); a "super-block" here is eight blocks.  As for Q8_0 the eight blocks are put
// on one scale: with D the largest |scale| among them, p = round(2048 value scale / D), within +-24576 --
// exact for every block within seven octaves or more of the largest (eleven for MXFP4), rounded to 2^-12 of
// the run's largest element below that.  Per block the sixteen products make two 8-byte tables a plane (codes
// 0..7 and 8..15): four v_perm_b32 and two bit selects for four elements.  Runs whose largest scale is below
// 2^-100 count as zeros.  T gives the block: BYTES, HEAD (bytes in front of the codes), ALIGN, scale_of(block),
// value(code) and UNIT (the value of one unit of p over D).
//   MXFP4: e (E8M0) | codes, w = 2^(e - 127) * +-{0, .5, 1, 1.5, 2, 3, 4, 6}, e = 255 a block of zeros
//   (src/mxfp4.rs:45-94); value() is the doubled E2M1 value.  Blocks of 17 bytes sit at any byte.
//   Q4_0: d (f16) | codes, w = d (code - 8) (vendor/candle-metal-kernels/src/metal_src/quantized.metal:86-89).
struct QtMXFP4 {
    static constexpr int BYTES = 17, HEAD = 1, ALIGN = 1;
    static constexpr bool HAS_OFFSET = false;
    static constexpr float UNIT = 1.0f / 4096.0f;
    __device__ __forceinline__ static float offset_of(const uint8_t *) { return 0.0f; }
    __device__ __forceinline__ static float scale_of(const uint8_t *blk) {
        const uint32_t e = blk[0];
        return e == 0xFFu ? 0.0f : __uint_as_float(e == 0 ? 0x00400000u : (e << 23));
    }
    __device__ __forceinline__ static constexpr float value(int code) {
        const int i = code & 7, v = i < 5 ? i : i == 5 ? 6 : i == 6 ? 8 : 12;
        return (float)(code & 8 ? -v : v);
    }
};
struct QtQ4_0 {
    static constexpr int BYTES = 18, HEAD = 2, ALIGN = 2;
    static constexpr bool HAS_OFFSET = false;
    static constexpr float UNIT = 1.0f / 2048.0f;
    __device__ __forceinline__ static float scale_of(const uint8_t *blk) { return f16_bits(ld<uint16_t>(blk)); }
    __device__ __forceinline__ static float offset_of(const uint8_t *) { return 0.0f; }
    __device__ __forceinline__ static constexpr float value(int code) { return (float)(code - 8); }
};
//   Q4_1: d (f16) | m (f16) | codes, w = d code + m (quantized.metal:91-95): the offsets are the min term.
struct QtQ4_1 {
    static constexpr int BYTES = 20, HEAD = 4, ALIGN = 2;
    static constexpr bool HAS_OFFSET = true;
    static constexpr float UNIT = 1.0f / 2048.0f;
    __device__ __forceinline__ static float scale_of(const uint8_t *blk) { return f16_bits(ld<uint16_t>(blk)); }
    __device__ __forceinline__ static float offset_of(const uint8_t *blk) { return f16_bits(ld<uint16_t>(blk + 2)); }
    __device__ __forceinline__ static constexpr float value(int code) { return (float)code; }
};
template <class T>
struct QiNibbles32 {
    static constexpr int BLOCK = 8 * T::BYTES, META = 48, ALIGN = T::ALIGN, TABLE = 0;
    static constexpr bool HAS_MIN = T::HAS_OFFSET, MIN_F16 = T::HAS_OFFSET, ONE_PLANE = false, SUB16 = false;
    struct Hdr {
        float d0, d1, m0, m1;
    };
    struct Raw {
        float unit, m0, m1;
        uint32_t th[2][4], tl[2][4];  // per block: Ph / Pl of codes 0..7 (words 0, 1) and of codes 8..15 (words 2, 3)
        uint4 qa, qb;                 // the codes of block 2 uc and of block 2 uc + 1
        uint4 na, nb;                 // the same of the next super-block
    };
    __device__ __forceinline__ static void fetch(const uint8_t *blk, int uc, int part, Raw &raw, Hdr &next) {
        const uint8_t *pair = blk + 2 * T::BYTES * uc;
        if (part == 0) {
            next.d0 = T::scale_of(pair), next.d1 = T::scale_of(pair + T::BYTES);
            next.m0 = T::offset_of(pair), next.m1 = T::offset_of(pair + T::BYTES);
        }
        if (part == 1) raw.na = ldw<uint4>(pair + T::HEAD);
        if (part == 2) raw.nb = ldw<uint4>(pair + T::BYTES + T::HEAD);
    }
    __device__ __forceinline__ static void take(Raw &raw, const Hdr &next, int uc, const uint8_t *) {
        float D = fmaxf(mag_or_inf(next.d0), mag_or_inf(next.d1));
        D = fmaxf(D, dpp_f<0xB1>(D));  // quad_perm [1,0,3,2]
        D = fmaxf(D, dpp_f<0x4E>(D));  // quad_perm [2,3,0,1]
        const bool live = D >= 7.888609052210118e-31f;  // 2^-100
        const float inv = live ? 2048.0f / D : 0.0f;
        raw.unit = live ? D * T::UNIT : 0.0f;
        raw.m0 = next.m0, raw.m1 = next.m1;
        raw.qa = raw.na, raw.qb = raw.nb;
#pragma unroll
        for (int blk = 0; blk < 2; blk++) {
            const float ratio = (blk ? next.d1 : next.d0) * inv;
            uint32_t t[2][8];
#pragma unroll
            for (int i = 0; i < 8; i++) {  // round(value ratio) + 128 in the low 16 bits of 1.5 * 2^23 + 128 + value ratio
                t[0][i] = __builtin_bit_cast(uint32_t, fmaf(T::value(i), ratio, 12583040.0f));
                t[1][i] = __builtin_bit_cast(uint32_t, fmaf(T::value(8 + i), ratio, 12583040.0f));
            }
#pragma unroll
            for (int top = 0; top < 2; top++)
#pragma unroll
                for (int h4 = 0; h4 < 2; h4++) {
                    const uint32_t *q = &t[top][4 * h4];
                    const uint32_t a = __builtin_amdgcn_perm(q[1], q[0], 0x05010400u);  // L0 L1 H0 H1
                    const uint32_t b = __builtin_amdgcn_perm(q[3], q[2], 0x05010400u);  // L2 L3 H2 H3
                    raw.tl[blk][2 * top + h4] = __builtin_amdgcn_perm(b, a, 0x05040100u) ^ 0x80808080u;
                    raw.th[blk][2 * top + h4] = __builtin_amdgcn_perm(b, a, 0x07060302u);
                }
        }
    }
    __device__ __forceinline__ static void piece(const Raw &raw, int uc, int j, uint8_t *tile, const uint8_t *) {
        const int half = j >> 2, wi = j & 3;
#pragma unroll
        for (int blk = 0; blk < 2; blk++) {  // elements 16 half + 4 wi .. + 3 of both blocks
            const uint4 qv = blk ? raw.qb : raw.qa;
            const uint32_t word = (wi == 0 ? qv.x : wi == 1 ? qv.y : wi == 2 ? qv.z : qv.w) >> (4 * half);
            const uint32_t sel = word & 0x07070707u, top = ((word >> 3) & 0x01010101u) * 0xFFu;
            const uint32_t h0 = __builtin_amdgcn_perm(raw.th[blk][1], raw.th[blk][0], sel);
            const uint32_t h1 = __builtin_amdgcn_perm(raw.th[blk][3], raw.th[blk][2], sel);
            const uint32_t l0 = __builtin_amdgcn_perm(raw.tl[blk][1], raw.tl[blk][0], sel);
            const uint32_t l1 = __builtin_amdgcn_perm(raw.tl[blk][3], raw.tl[blk][2], sel);
            const int gg = 2 * blk + half;
            *(uint32_t *)(tile + gg * 256 + qi_word(uc, wi)) = (h1 & top) | (h0 & ~top);
            *(uint32_t *)(tile + 1024 + gg * 256 + qi_word(uc, wi)) = (l1 & top) | (l0 & ~top);
        }
    }
    __device__ __forceinline__ static void meta(const Raw &raw, int uc, uint8_t *meta) {
        if constexpr (T::HAS_OFFSET) {  // the chunk's two offsets among m_0..7, zeros in the second sixteen bytes
            const qi_h2 m = {(_Float16)raw.m0, (_Float16)raw.m1};
            *(uint32_t *)(meta + 4 * uc) = __builtin_bit_cast(uint32_t, m);
            *(uint32_t *)(meta + 16 + 4 * uc) = 0u;
            *(float2 *)(meta + 32) = float2{raw.unit, -1.0f};  // + sum m XS
        } else {
            *(float2 *)(meta + 32) = float2{raw.unit, 0.0f};  // the same from all four
        }
    }
};
using QiMXFP4 = QiNibbles32<QtMXFP4>;
using QiQ4_0 = QiNibbles32<QtQ4_0>;
using QiQ4_1 = QiNibbles32<QtQ4_1>;

// Q5_K: d | dmin | scales[12] | qh[32] | qs[128], w = d sc q - dmin m with q in 0..31: the nibble of Q4_K's
// layout and, for element l of sub-block j, bit j of qh[l] as the fifth bit
// (vendor/candle-metal-kernels/src/metal_src/quantized.metal:176-189, 6649-6670); scales and mins as in Q4_K.
// p = sc q in 0..1953.
struct QiQ5K {
    static constexpr int BLOCK = 176, META = 48, ALIGN = 16, TABLE = 0;
    static constexpr bool HAS_MIN = true, ONE_PLANE = false, SUB16 = false;
    using Hdr = QiQ4K::Hdr;
    struct Raw {
        Hdr hdr;
        uint4 q0, q1, h0, h1;
    };
    __device__ __forceinline__ static void fetch(const uint8_t *blk, int uc, int part, Raw &raw, Hdr &next) {
        if (part == 0) next.h = *(const uint4 *)blk;
        if (part == 1) raw.q0 = *(const uint4 *)(blk + 48 + 32 * uc), raw.h0 = *(const uint4 *)(blk + 16);
        if (part == 2) raw.q1 = *(const uint4 *)(blk + 64 + 32 * uc), raw.h1 = *(const uint4 *)(blk + 32);
    }
    __device__ __forceinline__ static void take(Raw &raw, const Hdr &next, int uc, const uint8_t *) { raw.hdr = next; }
    __device__ __forceinline__ static void piece(const Raw &raw, int uc, int j, uint8_t *tile, const uint8_t *) {
        const uint4 hdr = raw.hdr.h;
        const uint32_t scl = hdr.y & 0x3F3F3F3Fu, sch = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
        const uint32_t s4 = (uc < 2 ? scl : sch) >> (16 * (uc & 1));
        const uint32_t sc[2] = {s4 & 0xFFu, (s4 >> 8) & 0xFFu};
        const uint4 qv = j < 4 ? raw.q0 : raw.q1, hv = j < 4 ? raw.h0 : raw.h1;
        const uint32_t word = (j & 3) == 0 ? qv.x : (j & 3) == 1 ? qv.y : (j & 3) == 2 ? qv.z : qv.w;
        const uint32_t high = ((j & 3) == 0 ? hv.x : (j & 3) == 1 ? hv.y : (j & 3) == 2 ? hv.z : hv.w) >> (2 * uc);
#pragma unroll
        for (int nib = 0; nib < 2; nib++) {  // low nibbles: sub-block 2 uc, high nibbles: sub-block 2 uc + 1
            const uint32_t q = ((nib ? word >> 4 : word) & 0x0F0F0F0Fu) | (((high >> nib) & 0x01010101u) << 4);
            const uint32_t even = __umul24(q & 0x00FF00FFu, sc[nib]) + 0x00800080u;
            const uint32_t odd = __umul24((q >> 8) & 0x00FF00FFu, sc[nib]) + 0x00800080u;
            const int gg = 2 * nib + (j >> 2);
            *(uint32_t *)(tile + gg * 256 + qi_word(uc, j & 3)) = __builtin_amdgcn_perm(odd, even, 0x07030501u);
            *(uint32_t *)(tile + 1024 + gg * 256 + qi_word(uc, j & 3)) = __builtin_amdgcn_perm(odd, even, 0x06020400u) ^ 0x80808080u;
        }
    }
    __device__ __forceinline__ static void meta(const Raw &raw, int uc, uint8_t *meta) {
        QiQ4K::Raw as_q4k;
        as_q4k.hdr = raw.hdr;
        QiQ4K::meta(as_q4k, uc, meta);
    }
};

// Q5_0: blocks of d (f16) | qh (32 fifth bits) | 16 code bytes, w = d (q - 16) with q the nibble and bit j (low
// nibbles, elements 0..15) or 16 + j (high nibbles, elements 16..31) of qh as its fifth bit; Q5_1: d | m (f16) |
// qh | codes, w = d q + m (vendor/candle-metal-kernels/src/metal_src/quantized.metal:98-110).  A "super-block"
// here is eight blocks, put on one scale as for Q8_0: p = round(1024 (q - 16) d / D) or round(1024 q d / D),
// within +-31744 whatever the sign of d; Q5_1's offsets are the min term (MIN_F16).  The four fifth bits of a
// word are spread to bytes with a multiply, q - 16 becomes a signed byte without carries between bytes
// ((q | 0x80) - 0x10, then the top bit flipped back), and the product goes the way of Q8_0's.  Blocks sit at
// even addresses only: read through aligned words.
template <bool OFFSET>
struct QiQ5x {
    static constexpr int BYTES = OFFSET ? 24 : 22, HIGH = OFFSET ? 4 : 2, CODES = OFFSET ? 8 : 6;
    static constexpr int BLOCK = 8 * BYTES, META = 48, ALIGN = 2, TABLE = 0;
    static constexpr bool HAS_MIN = OFFSET, MIN_F16 = OFFSET, ONE_PLANE = false, SUB16 = false;
    struct Hdr {
        float d0, d1, m0, m1;
    };
    struct Raw {
        float r0, r1, unit;  // 1024 d / D of the chunk's two blocks, and D / 1024
        float m0, m1;
        uint32_t ha, hb;     // the fifth bits of block 2 uc and of block 2 uc + 1
        uint4 qa, qb;        // their code bytes
        uint32_t hna, hnb;   // the same of the next super-block (every piece reads all 16 bytes of a block, so the
        uint4 na, nb;        // bytes fetched ahead wait here until take())
    };
    __device__ __forceinline__ static void fetch(const uint8_t *blk, int uc, int part, Raw &raw, Hdr &next) {
        const uint8_t *pair = blk + 2 * BYTES * uc;
        if (part == 0) {
            next.d0 = f16_bits(ld<uint16_t>(pair)), next.d1 = f16_bits(ld<uint16_t>(pair + BYTES));
            next.m0 = OFFSET ? f16_bits(ld<uint16_t>(pair + 2)) : 0.0f;
            next.m1 = OFFSET ? f16_bits(ld<uint16_t>(pair + BYTES + 2)) : 0.0f;
        }
        if (part == 1) raw.hna = ldw<uint32_t>(pair + HIGH), raw.na = ldw<uint4>(pair + CODES);
        if (part == 2) raw.hnb = ldw<uint32_t>(pair + BYTES + HIGH), raw.nb = ldw<uint4>(pair + BYTES + CODES);
    }
    __device__ __forceinline__ static void take(Raw &raw, const Hdr &next, int uc, const uint8_t *) {
        float D = fmaxf(mag_or_inf(next.d0), mag_or_inf(next.d1));
        D = fmaxf(D, dpp_f<0xB1>(D));  // quad_perm [1,0,3,2]
        D = fmaxf(D, dpp_f<0x4E>(D));  // quad_perm [2,3,0,1]
        const float inv = D > 0.0f ? 1024.0f / D : 0.0f;
        raw.r0 = next.d0 * inv, raw.r1 = next.d1 * inv, raw.unit = D * (1.0f / 1024.0f);
        raw.m0 = next.m0, raw.m1 = next.m1;
        raw.ha = raw.hna, raw.hb = raw.hnb, raw.qa = raw.na, raw.qb = raw.nb;
    }
    __device__ __forceinline__ static void piece(const Raw &raw, int uc, int j, uint8_t *tile, const uint8_t *) {
        const int half = j >> 2, wi = j & 3;
#pragma unroll
        for (int blk = 0; blk < 2; blk++) {  // elements 16 half + 4 wi .. + 3 of both blocks
            const uint4 qv = blk ? raw.qb : raw.qa;
            const uint32_t word = (wi == 0 ? qv.x : wi == 1 ? qv.y : wi == 2 ? qv.z : qv.w) >> (4 * half);
            const uint32_t fifth = (((blk ? raw.hb : raw.ha) >> (16 * half + 4 * wi)) & 15u) * 0x00204081u & 0x01010101u;
            const uint32_t q = (word & 0x0F0F0F0Fu) | (fifth << 4);
            // Q5_0: q - 16 as signed bytes; Q5_1: q as it is (0..31)
            const uint32_t sb = OFFSET ? q : ((q | 0x80808080u) - 0x10101010u) ^ 0x80808080u;
            const float ratio = blk ? raw.r1 : raw.r0;
            uint32_t t[4];
#pragma unroll
            for (int b = 0; b < 4; b++)
                t[b] = __builtin_bit_cast(uint32_t, fmaf((float)(int)(int8_t)(sb >> (8 * b)), ratio, 12583040.0f));
            const uint32_t even = __builtin_amdgcn_perm(t[2], t[0], 0x05040100u), odd = __builtin_amdgcn_perm(t[3], t[1], 0x05040100u);
            const int gg = 2 * blk + half;
            *(uint32_t *)(tile + gg * 256 + qi_word(uc, wi)) = __builtin_amdgcn_perm(odd, even, 0x07030501u);
            *(uint32_t *)(tile + 1024 + gg * 256 + qi_word(uc, wi)) = __builtin_amdgcn_perm(odd, even, 0x06020400u) ^ 0x80808080u;
        }
    }
    __device__ __forceinline__ static void meta(const Raw &raw, int uc, uint8_t *meta) {
        if constexpr (OFFSET) {  // the chunk's two offsets among m_0..7, zeros in the second sixteen bytes
            const qi_h2 m = {(_Float16)raw.m0, (_Float16)raw.m1};
            *(uint32_t *)(meta + 4 * uc) = __builtin_bit_cast(uint32_t, m);
            *(uint32_t *)(meta + 16 + 4 * uc) = 0u;
            *(float2 *)(meta + 32) = float2{raw.unit, -1.0f};  // + sum m XS
        } else {
            *(float2 *)(meta + 32) = float2{raw.unit, 0.0f};  // the same from all four
        }
    }
};
using QiQ5_0 = QiQ5x<false>;
using QiQ5_1 = QiQ5x<true>;

// Q3_K: hmask[32] | qs[64] | scales[12] | d, w = d (sc - 32) (q - (hbit ? 0 : 4)) over sub-blocks of 16: element
// 128 h + 32 t + 16 hf + i is field t of qs[32 h + 16 hf + i] with bit 4 h + t of hmask[16 hf + i] as its
// third bit and the 6-bit scale number 8 h + 2 t + hf, low four bits in scales[0..7] (a nibble each, the first
// eight scales low, the next eight high), high two bits in scales[8..11]
// (vendor/candle-metal-kernels/src/metal_src/quantized.metal:151-156, 6597-6623).  With v = q + 4 hbit in
// 0..7 the weight is d s (v - 4), s = sc - 32 in -32..31: p = s (v - 4) in -124..128, two bytes (Ph is 0 or 1),
// no min term.  Chunk uc is half h = uc / 2, fields 2 (uc % 2) and 2 (uc % 2) + 1: slice gg of 16 is field
// 2 (uc % 2) + gg / 2 of bytes 16 (gg % 2) .., scale number 4 uc + gg.  Per slice the eight products make one
// 8-byte table a plane; one v_perm_b32 a plane looks four elements up with selector v.  Blocks of 110 bytes
// sit at even addresses only: read through aligned words.
struct QiQ3K {
    static constexpr int BLOCK = 110, META = 48, ALIGN = 2, TABLE = 0;
    static constexpr bool HAS_MIN = false, ONE_PLANE = false, SUB16 = false;
    struct Hdr {
        uint32_t s0, s1, s2, d;
    };
    struct Raw {
        float d;
        uint32_t th[4][2], tl[4][2];  // per slice: Ph and Pl of s (v - 4), v = 0..3 and 4..7
        uint4 q[2], m[2];             // qs[32 h + 16 hf ..] and hmask[16 hf ..], hf = 0, 1
    };
    __device__ __forceinline__ static void fetch(const uint8_t *blk, int uc, int part, Raw &raw, Hdr &next) {
        if (part == 0) {
            next.s0 = ldw<uint32_t>(blk + 96), next.s1 = ldw<uint32_t>(blk + 100), next.s2 = ldw<uint32_t>(blk + 104);
            next.d = ld<uint16_t>(blk + 108);
        }
        if (part == 1 || part == 2) {
            raw.q[part - 1] = ldw<uint4>(blk + 32 + 32 * (uc >> 1) + 16 * (part - 1));
            raw.m[part - 1] = ldw<uint4>(blk + 16 * (part - 1));
        }
    }
    __device__ __forceinline__ static void take(Raw &raw, const Hdr &hdr, int uc, const uint8_t *) {
        raw.d = f16_bits(hdr.d);
        const uint32_t lw = (uc & 1) ? hdr.s1 : hdr.s0;
        const uint32_t sc6 = ((uc < 2 ? lw : lw >> 4) & 0x0F0F0F0Fu) | (((hdr.s2 >> (2 * uc)) & 0x03030303u) << 4);
#pragma unroll
        for (int gg = 0; gg < 4; gg++) {
            const short sc = (short)((int)((sc6 >> (8 * gg)) & 0xFFu) - 32);
            // s (v - 4) + 128 for v = 0..7 as signed halfwords, two an instruction
            const qi_s2 step2 = {(short)(2 * sc), (short)(2 * sc)};
            const qi_s2 v01 = {(short)(128 - 4 * sc), (short)(128 - 3 * sc)};
            const qi_s2 v23 = v01 + step2, v45 = v23 + step2, v67 = v45 + step2;
            const uint32_t a = __builtin_bit_cast(uint32_t, v01), b = __builtin_bit_cast(uint32_t, v23);
            const uint32_t c = __builtin_bit_cast(uint32_t, v45), e = __builtin_bit_cast(uint32_t, v67);
            raw.tl[gg][0] = __builtin_amdgcn_perm(b, a, 0x06040200u) ^ 0x80808080u;
            raw.th[gg][0] = __builtin_amdgcn_perm(b, a, 0x07050301u);
            raw.tl[gg][1] = __builtin_amdgcn_perm(e, c, 0x06040200u) ^ 0x80808080u;
            raw.th[gg][1] = __builtin_amdgcn_perm(e, c, 0x07050301u);
        }
    }
    __device__ __forceinline__ static uint32_t word_of(const uint4 &v, int i) {
        return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w;
    }
    __device__ __forceinline__ static void piece(const Raw &raw, int uc, int j, uint8_t *tile, const uint8_t *) {
        const int hf = j >> 2, wi = j & 3;
        const uint32_t word = word_of(raw.q[hf], wi) >> (4 * (uc & 1));
        const uint32_t high = word_of(raw.m[hf], wi) >> (4 * (uc >> 1) + 2 * (uc & 1));
#pragma unroll
        for (int tt = 0; tt < 2; tt++) {  // slices hf and 2 + hf: the same bytes, the next field
            const int gg = 2 * tt + hf;
            const uint32_t v = ((word >> (2 * tt)) & 0x03030303u) | (((high >> tt) & 0x01010101u) << 2);
            *(uint32_t *)(tile + gg * 256 + qi_word(uc, wi)) = __builtin_amdgcn_perm(raw.th[gg][1], raw.th[gg][0], v);
            *(uint32_t *)(tile + 1024 + gg * 256 + qi_word(uc, wi)) = __builtin_amdgcn_perm(raw.tl[gg][1], raw.tl[gg][0], v);
        }
    }
    __device__ __forceinline__ static void meta(const Raw &raw, int uc, uint8_t *meta) {
        *(float2 *)(meta + 32) = float2{raw.d, 0.0f};  // the same from all four
    }
};

// Sides whose min term has an f16 factor per block of 32 (Q4_1, Q5_1: w = d q + m) say MIN_F16: the row meta
// holds m_0..7 as halves and sixteen bytes of zeros, and the term takes two f16 MFMAs, sum m a0 and sum m a1
// (1024 m, which the integer mins carry as a second operand, may not be an f16 value).
template <class F, class = void>
struct QiMinF16 : std::false_type {};
template <class F>
struct QiMinF16<F, std::void_t<decltype(F::MIN_F16)>> : std::bool_constant<F::MIN_F16> {};

// grid: 1-D; workgroup L takes tile (x, y) of tx x ty (weight-row tiles x activation-row tiles).  When ty
// divides 8 the eight XCDs (L % 8) each work on one activation-row tile, whose operands then stay in that
// XCD's L2; the grid is padded to a multiple of 8 and workgroups past the last tile leave at once.
// gridDim.y > 1 splits the product over k.
// GROUPED: the expert matmuls of a mixture-of-experts layer over pairs sorted by expert (tables of
// moe_gemm_i8_plan, activations of moe_gemm_i8_prep).  Workgroup L takes weight-row tile L % tx of activation
// tile L / tx (workgroups past the last tile leave at once): the weights are those of the tile's expert,
// gp.wptr[gp.gexp[group]], row i of the tile's row group j is pair rg_pair + i, stored at Y[gp.yrow[pair]].
// W, m_rows, groups, ty and the split arguments are unused.
struct QiGrouped {
    const uint8_t *const *wptr;
    const int *gexp, *yrow;
    QiGroupTables t;
};
// NSPLIT: few activation rows.  The tile is 32 activation rows (two row groups) against 16 NG weight rows, and
// the waves share the weight-row groups instead of the activation rows: wave w takes groups w NG / NW ..
// of them against both row groups, so that every wave has matrix work whatever the row count (with the rows
// split, a tile of one row group leaves all waves but one only the unpacking).
// SINGLE: one operand buffer instead of two.  A super-block is unpacked as a whole, then multiplied, with a barrier
// after either; half the LDS lets twice the workgroups share a compute unit, and while one unpacks the others
// multiply (for the tiles of few rows, whose two waves a workgroup leave the unpacking's lookups nothing to hide behind).
template <class F, int NW, int NG, bool GROUPED = false, bool NSPLIT = false, bool SINGLE = false>
__global__ __launch_bounds__(64 * NW) void kq_gemm_i8(const uint8_t *__restrict__ W, size_t row_bytes,
                                                      const uint8_t *__restrict__ acts, float *__restrict__ Y,
                                                      int m_rows, int n, int nb, int groups, int tx, int ty,
                                                      int nb_total, size_t split_stride, QiGrouped gp = QiGrouped{}) {
    constexpr int NT = 16 * NG, THREADS = 64 * NW, UNITS = 4 * NT, PER = (UNITS + THREADS - 1) / THREADS;
    constexpr int BUF = NG * QI_TILE + NT * F::META;
    constexpr int NGW = NSPLIT ? NG / NW : NG;  // weight-row groups a wave multiplies
    constexpr int MT = NSPLIT ? 32 : 32 * NW;   // activation rows a tile
    static_assert(!NSPLIT || (NG % NW == 0 && NGW >= 2), "two weight-row groups a wave or more");
    extern __shared__ __attribute__((aligned(16))) uint8_t qi_lds[];
    const uint8_t *tab = qi_lds + (SINGLE ? 1 : 2) * BUF;  // the format's lookup table, behind the buffers
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, g = lane >> 4;
    int bx, by;
    int rg0 = 0, nrg = 0;  // GROUPED: the tile's first row group and how many it has
    if (GROUPED) {
        by = (int)blockIdx.x / tx, bx = (int)blockIdx.x % tx;
        if (by >= gp.t.counts[1]) return;
        rg0 = gp.t.mt_rg0[by], nrg = gp.t.mt_nrg[by];
        W = gp.wptr[gp.gexp[gp.t.mt_group[by]]];
    } else if (8 % ty == 0) {
        const int xcd = (int)blockIdx.x & 7, slot = (int)blockIdx.x >> 3;
        by = xcd % ty, bx = slot * (8 / ty) + xcd / ty;
    } else {
        by = (int)blockIdx.x / tx, bx = (int)blockIdx.x % tx;
    }
    if (bx >= tx || (!GROUPED && by >= ty)) return;
    const int n0 = bx * NT, m0 = by * MT;
    const int cg0 = NSPLIT ? (tid >> 6) * NGW : 0;   // this wave's first weight-row group
    const int wrow = NSPLIT ? 0 : 2 * (tid >> 6);    // this wave's first row group within the tile
    // split over k: workgroups blockIdx.y = i take super-blocks i nb .. (i + 1) nb - 1 of the nb_total and store
    // their sums at Y + i split_stride (splitk_sum adds the parts in a fixed order)
    const int b_first = GROUPED ? 0 : (int)blockIdx.y * nb;
    if (!GROUPED) Y += (size_t)blockIdx.y * split_stride;

    // activation operands of this wave: row groups 2 wave, 2 wave + 1 of the tile (clamped: rows past m_rows
    // are computed and not stored)
    const uint8_t *arec[2];
#pragma unroll
    for (int mg = 0; mg < 2; mg++)
        arec[mg] = acts + ((size_t)(GROUPED ? rg0 + min(wrow + mg, nrg - 1) : min(m0 / 16 + wrow + mg, groups - 1)) * nb_total + b_first) * QI_REC;

    // unpack units of this thread: chunk c = tid % 4 of weight rows tid / 4 + (THREADS / 4) p
    const int uc = tid & 3;
    const uint8_t *wsrc[PER];
#pragma unroll
    for (int p = 0; p < PER; p++) {
        const int row = min((tid >> 2) + (THREADS / 4) * p, NT - 1);
        wsrc[p] = W + (size_t)min(n0 + row, n - 1) * row_bytes + (size_t)b_first * F::BLOCK;
    }
    typename F::Raw raw[PER];
    typename F::Hdr hdr_next[PER];
    auto fetch_part = [&](int b, int part) __attribute__((always_inline)) {  // 0: scales into hdr_next, 1, 2: the two halves of the chunk
#pragma unroll
        for (int p = 0; p < PER; p++) F::fetch(wsrc[p] + (size_t)b * F::BLOCK, uc, part, raw[p], hdr_next[p]);
    };
    // Piece j of 8: an eighth of this thread's chunk becomes two operand words of either plane.
    auto unpack_piece = [&](uint8_t *buf, int j) __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < PER; p++) {
            const int row = min((tid >> 2) + (THREADS / 4) * p, NT - 1);  // threads past the last unit repeat it
            F::piece(raw[p], uc, j, buf + (row >> 4) * QI_TILE + uc * 2048 + (row & 15) * 16, tab);
        }
    };
    auto unpack_meta = [&](uint8_t *buf) __attribute__((always_inline)) {  // the row's scales of the min term, d and dmin
#pragma unroll
        for (int p = 0; p < PER; p++) {
            const int row = min((tid >> 2) + (THREADS / 4) * p, NT - 1);
            F::meta(raw[p], uc, buf + NG * QI_TILE + row * F::META);
        }
    };
    auto take_header = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < PER; p++) F::take(raw[p], hdr_next[p], uc, tab);
    };

    fetch_part(0, 0), fetch_part(0, 1), fetch_part(0, 2);
    if constexpr (F::TABLE > 0) {  // every workgroup that got this far: no wave has left
        F::stage(qi_lds + (SINGLE ? 1 : 2) * BUF);
        __syncthreads();
    }
    take_header();
#pragma unroll
    for (int j = 0; j < 8; j++) unpack_piece(qi_lds, j);
    unpack_meta(qi_lds);
    fetch_part(min(1, nb - 1), 0), fetch_part(min(1, nb - 1), 1), fetch_part(min(1, nb - 1), 2);

    // The loop walks through quarters: (activation row group mg of this wave, 64-k chunk c) against all NG
    // groups of weight rows.  A[c] holds the operands of chunk c for the row group at work; once the quarter is
    // through with them, the same chunk of the other row group is asked for (of the next super-block when mg is
    // 1), three quarters before its turn.
    qm_i4 A[4][2];
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int P = 0; P < 2; P++) A[c][P] = *(const qm_i4 *)(arec[0] + ((size_t)(2 * c + P) * 64 + lane) * 16);

    qm_f4 acc[2][NGW];
#pragma unroll
    for (int mg = 0; mg < 2; mg++)
#pragma unroll
        for (int cg = 0; cg < NGW; cg++) acc[mg][cg] = qm_f4{0.0f, 0.0f, 0.0f, 0.0f};
    const qm_i4 zero_i = {0, 0, 0, 0};
    const qm_f4 zero_f = {0.0f, 0.0f, 0.0f, 0.0f};
    __syncthreads();

    for (int b = 0; b < nb; b++) {
        const uint8_t *buf = qi_lds + (SINGLE ? 0 : (b & 1) * BUF);
        const int b_next = min(b + 1, nb - 1), b_next2 = min(b + 2, nb - 1);
        if (SINGLE && b > 0) {
            // (every wave is through with super-block b - 1: the barrier that ended its iteration)
            take_header();
#pragma unroll
            for (int j = 0; j < 8; j++) unpack_piece(qi_lds, j);
            unpack_meta(qi_lds);
            fetch_part(b_next, 0), fetch_part(b_next, 1), fetch_part(b_next, 2);
            __syncthreads();
        }
#pragma unroll
        for (int mg = 0; mg < 2; mg++) {
            // scales and I2 operand of this row group: wanted in the last quarter
            const qm_f4 sx = *(const qm_f4 *)(arec[mg] + (size_t)b * QI_REC + QI_SCALE + 16 * g);
            const qi_h8 minA = *(const qi_h8 *)(arec[mg] + (size_t)b * QI_REC + QI_MIN + lane * 16);
            // The wave's weight-row groups in two sets (T0 and NGW - T0 of them), each taken through the four chunks: the
            // integer sums of one set are alive at a time.  Step s of a half = (set, chunk, group within the set).
            constexpr int T0 = (NGW + 1) / 2, STEPS = 4 * NGW;
            auto step_cg = [](int s) { return s < 4 * T0 ? s % T0 : T0 + (s - 4 * T0) % (NGW - T0); };
            auto step_c = [](int s) { return s < 4 * T0 ? s / T0 : (s - 4 * T0) / (NGW - T0); };
            qm_i4 HH[NGW], MID[NGW], LL[NGW];
            // the weight operands travel one step ahead of the MFMAs that use them, through two register sets
            qm_i4 Bh[2], Bl[2];
            if constexpr (!F::ONE_PLANE) Bh[0] = *(const qm_i4 *)(buf + 4 * cg0 * 2048 + lane * 16);
            Bl[0] = *(const qm_i4 *)(buf + 4 * cg0 * 2048 + 1024 + lane * 16);
            auto finish = [&](int cg) __attribute__((always_inline)) {  // the 16 x 16 results of weight-row group cg
                const uint8_t *meta = buf + NG * QI_TILE + (16 * (cg0 + cg) + r) * F::META;
                const float2 dd = *(const float2 *)(meta + F::META - 16);
                qm_f4 I2 = zero_f;
                if constexpr (QiMinF16<F>::value) {
                    // lane group 0 carries a0, group 1 a1: m against the one, zeros against the other
                    const qi_h8 m0 = *(const qi_h8 *)(meta + 16 * (g & 1)), m1 = *(const qi_h8 *)(meta + 16 * (~g & 1));
                    I2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(minA, m0, zero_f, 0, 0, 0);
                    const qm_f4 high = __builtin_amdgcn_mfma_f32_16x16x32_f16(minA, m1, zero_f, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; i++) I2[i] = fmaf(1024.0f, high[i], I2[i]);
                } else if constexpr (F::HAS_MIN) {
                    // eight sub-blocks: lane groups 2, 3 meet zeros in the activation operand, any finite halves
                    // will do for them
                    const qi_h8 mB = *(const qi_h8 *)(meta + 16 * (F::SUB16 ? g : g & 1));
                    I2 = __builtin_amdgcn_mfma_f32_16x16x32_f16(minA, mB, zero_f, 0, 0, 0);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float I1 = F::ONE_PLANE ? (float)(MID[cg][i] * 256 + LL[cg][i])
                                                  : fmaf((float)(HH[cg][i] * 256 + MID[cg][i]), 256.0f, (float)LL[cg][i]);
                    if constexpr (F::HAS_MIN) acc[mg][cg][i] = fmaf(sx[i], dd.x * I1 - dd.y * I2[i], acc[mg][cg][i]);
                    else acc[mg][cg][i] = fmaf(sx[i], dd.x * I1, acc[mg][cg][i]);
                }
            };
#pragma unroll
            for (int s = 0; s < STEPS; s++) {
                const int cg = step_cg(s), c = step_c(s), cur = s & 1, nxt = cur ^ 1;
                const bool first_of_pass = s < 4 * T0 ? s % T0 == 0 : (s - 4 * T0) % (NGW - T0) == 0;
                const bool last_of_pass = s < 4 * T0 ? s % T0 == T0 - 1 : (s - 4 * T0) % (NGW - T0) == NGW - T0 - 1;
                const int pass = s < 4 * T0 ? c : 4 + c;  // 0..7 within the half
                if (!SINGLE && first_of_pass) {
                    // An eighth of the next super-block's weights becomes operands in every pass, thinly spread
                    // among the MFMAs (its bytes were asked for half an iteration or more ago); the registers of
                    // a part are refilled with the super-block after that as soon as the part is used up.
                    const int piece = 4 * mg + (pass >> 1);
                    if (mg == 0 && pass == 0) take_header();
                    if ((pass & 1) == 0) unpack_piece(qi_lds + ((b + 1) & 1) * BUF, piece);
                    if (mg == 1 && pass == 0) fetch_part(b_next2, 1), fetch_part(b_next2, 0);
                    if (mg == 1 && pass == 7) unpack_meta(qi_lds + ((b + 1) & 1) * BUF);
                }
                if (c == 0) HH[cg] = zero_i, MID[cg] = zero_i, LL[cg] = zero_i;
                if (s + 1 < STEPS) {
                    const int cg1 = step_cg(s + 1), c1 = step_c(s + 1);
                    if constexpr (!F::ONE_PLANE) Bh[nxt] = *(const qm_i4 *)(buf + (4 * (cg0 + cg1) + c1) * 2048 + lane * 16);
                    Bl[nxt] = *(const qm_i4 *)(buf + (4 * (cg0 + cg1) + c1) * 2048 + 1024 + lane * 16);
                }
                __builtin_amdgcn_sched_barrier(0);
                MID[cg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[c][0], Bl[cur], MID[cg], 0, 0, 0);
                if constexpr (!F::ONE_PLANE) HH[cg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[c][0], Bh[cur], HH[cg], 0, 0, 0);
                LL[cg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[c][1], Bl[cur], LL[cg], 0, 0, 0);
                if constexpr (!F::ONE_PLANE) MID[cg] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[c][1], Bh[cur], MID[cg], 0, 0, 0);
                // one group behind the MFMAs, whose results it would otherwise wait for
                if (c == 3 && !first_of_pass) finish(cg - 1);
                if (last_of_pass && pass >= 4) {
                    // this chunk's operands have done their work in this half: the other row group's take their place
#pragma unroll
                    for (int P = 0; P < 2; P++)
                        A[c][P] = *(const qm_i4 *)(arec[mg ^ 1] + (size_t)(mg == 0 ? b : b_next) * QI_REC + ((size_t)(2 * c + P) * 64 + lane) * 16);
                }
                if (c == 3 && last_of_pass && pass < 4) finish(cg);
                __builtin_amdgcn_sched_barrier(0);
            }
            finish(NGW - 1);
            if (!SINGLE && mg == 1) fetch_part(b_next2, 2);
            __builtin_amdgcn_sched_barrier(0);
        }
        // every wave is done with the buffer the next super-block went into: it was read one iteration ago, in
        // front of the barrier that ended that iteration
        __syncthreads();
    }
#pragma unroll
    for (int mg = 0; mg < 2; mg++) {
        int first_pair = 0, pairs = 0;
        if (GROUPED && wrow + mg < nrg) first_pair = gp.t.rg_pair[rg0 + wrow + mg], pairs = gp.t.rg_cnt[rg0 + wrow + mg];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int row = m0 + 16 * (wrow + mg) + 4 * g + i;
            if (GROUPED) {
                if (4 * g + i >= pairs) continue;
                row = gp.yrow[first_pair + 4 * g + i];
            } else if (row >= m_rows) {
                continue;
            }
#pragma unroll
            for (int cg = 0; cg < NGW; cg++) {
                const int col = n0 + 16 * (cg0 + cg) + r;
                if (col < n) Y[(size_t)row * n + col] = acc[mg][cg][i];
            }
        }
    }
}

}  // namespace jq
