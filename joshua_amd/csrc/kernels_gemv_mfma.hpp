// GEMV for one activation row over weight rows of 4096 columns (16 super-blocks of 256) with the integer
// dot products on the int8 matrix cores: one kernel (gemv_mfma_lds<F>, at the end of the file) over a
// per-format policy F that says how a row's bytes are laid out, how a lane's operands are made from the
// wave's 256 activations and how a super-block is multiplied.  Policies: QvQ4K and QvQ2K.
//
// ---- Q4_K ----
//
// Per 32-element sub-block j of a weight row (reference arithmetic w = d sc q - dmin m,
// src/kquant_dot.rs:440-465):
//
//   sum_k x_k w_k = (d sc_j) s_j S_j - (dmin m_j) s_j XS_j,   S_j = sum_k q_k X_k,  XS_j = sum_k X_k
//
// with X = round(x / s_j), s_j = amax_j(x) / 32639: 16-bit fixed point per sub-block in two int8 planes
// X = 256 Xh + Xl, exactly the quantisation of q4k_gemv_dot4_lds.  Wave w owns super-block column w of
// the matrix; lane (r = lane % 16, c = lane / 16) reads row r's 16-byte header and the 32 bytes of chunk c
// (low nibbles: sub-block 2c, high nibbles: sub-block 2c + 1) from LDS.
//
// The sums S run on v_mfma_i32_16x16x64_i8 with the weights as the B operand (column = weight row r, the
// lane group c holds 16 bytes of chunk c) and the activations as a block-diagonal A operand held in 16
// registers for the whole kernel: row m = 4c + 2p + plane of A is non-zero only in lane group c, so that
// C[m][r] collects sub-block 2c + p, plane `plane`, of weight row r, and the lane (r, c) that loaded the
// bytes also receives the four sums it needs (C rows 4c .. 4c + 3).  Four MFMAs a tile and wave:
//   B = q & 0x0F0F0F0F  (low nibbles l)          against  X of sub-block 2c   and  -X' of sub-block 2c + 1
//   B = q ^ 0x80808080  (signed 16 h + l - 128)  against  X' of sub-block 2c + 1
// for bytes 0..15 and 16..31 of the chunk.  The high-nibble rows add up to 16 sum h X' - 128 XS': the low
// nibbles cancel, and the accumulator of those rows starts at 128 XS', so the unpacking costs two vector
// instructions a register instead of three, no shift, and every integer sum is exact.
#pragma once
#include "kernels_dot4_q4k.hpp"

namespace jq {

typedef int qv_i4 __attribute__((ext_vector_type(4)));

// What a lane keeps of its wave's 256 activations for the whole kernel.
struct QvActs {
    qv_i4 a_even[2], a_odd[2];  // A operands: [bytes 0..15 | 16..31 of the chunk]
    qv_i4 c_init;               // accumulator start: 128 XS of sub-block 2c + 1 in the low-plane row
    float s_e, s_o16, xs_e, xs_o;
};

// Quantises the wave's activation column (lane i holds elements 4i .. 4i+3, sub-block i / 8) and builds
// the lane's operands through `stage`, 1184 bytes of LDS that only this wave touches:
// words [0,64) Xl, [64,128) Xh, [128,192) and [192,256) the planes of -X, 8 words of zeros, then per
// sub-block {scale, scale x sum, 128 x sum (integer), scale / 16}.
__device__ __forceinline__ QvActs qv_prepare(const float4 v, uint32_t *stage, int lane) {
    const int r = lane & 15, c = lane >> 4;
    float4 *side = (float4 *)(stage + 264);
    {
        const QvQuant q = qv_quantise4(v);
        stage[lane] = q.wl, stage[64 + lane] = q.wh, stage[128 + lane] = q.nl, stage[192 + lane] = q.nh;
        if (lane < 8) stage[256 + lane] = 0;
        if ((lane & 7) == 0) side[lane >> 3] = float4{q.s, q.s * (float)q.sum, __builtin_bit_cast(float, 128 * q.sum), q.s * 0.0625f};
    }
    asm volatile("" ::: "memory");  // (written as scalars, read back as vectors: the compiler keeps the order only when told)
    QvActs a;
    {
        // A operands of lane (m = r, g = c): row m is sub-block m / 2, plane m % 2, and non-zero in lane group
        // (m / 2) / 2 only; p = 0: the low-nibble sub-block 2g, 1: the high-nibble sub-block 2g + 1.  The lanes
        // that hold zeros read them from the staging area's zero words, so no register is selected afterwards.
        const bool mine = (r >> 2) == c, odd = (r & 2) != 0;
        const uint32_t *pos = stage + 64 * (r & 1) + 16 * c + (odd ? 8 : 0);  // plane words of the sub-block's 32 elements
        const uint32_t *zero = stage + 256;
        const uint32_t *ev = mine ? (odd ? pos + 128 : pos) : zero, *od = mine && odd ? pos : zero;
        const uint4 e0 = *(const uint4 *)ev, e1 = *(const uint4 *)(ev + 4), o0 = *(const uint4 *)od, o1 = *(const uint4 *)(od + 4);
        a.a_even[0] = qv_i4{(int)e0.x, (int)e0.y, (int)e0.z, (int)e0.w};
        a.a_even[1] = qv_i4{(int)e1.x, (int)e1.y, (int)e1.z, (int)e1.w};
        a.a_odd[0] = qv_i4{(int)o0.x, (int)o0.y, (int)o0.z, (int)o0.w};
        a.a_odd[1] = qv_i4{(int)o1.x, (int)o1.y, (int)o1.z, (int)o1.w};
    }
    // what lane (r, c) needs of sub-blocks 2c and 2c + 1 after the MFMAs
    const float4 fe = side[2 * c], fo = side[2 * c + 1];
    a.s_e = fe.x, a.xs_e = fe.y, a.s_o16 = fo.w, a.xs_o = fo.y;
    a.c_init = qv_i4{0, 0, __builtin_bit_cast(int, fo.z), 0};
    asm volatile("" ::: "memory");  // (the next column's preparation writes the same words as another type)
    return a;
}

// The sum of chunk c of a super-block of weight row r against the wave's column.  blk: the row's 144-byte
// block in LDS.
__device__ __forceinline__ float qv_block_dot_lane(const uint8_t *blk, const QvActs &a, int c) {
    const uint4 hdr = *(const uint4 *)blk;
    const uint4 qa = *(const uint4 *)(blk + 16 + 32 * c), qb = *(const uint4 *)(blk + 32 + 32 * c);
    const qv_i4 la = qv_i4{(int)(qa.x & 0x0F0F0F0Fu), (int)(qa.y & 0x0F0F0F0Fu), (int)(qa.z & 0x0F0F0F0Fu), (int)(qa.w & 0x0F0F0F0Fu)};
    const qv_i4 lb = qv_i4{(int)(qb.x & 0x0F0F0F0Fu), (int)(qb.y & 0x0F0F0F0Fu), (int)(qb.z & 0x0F0F0F0Fu), (int)(qb.w & 0x0F0F0F0Fu)};
    const qv_i4 ha = qv_i4{(int)(qa.x ^ 0x80808080u), (int)(qa.y ^ 0x80808080u), (int)(qa.z ^ 0x80808080u), (int)(qa.w ^ 0x80808080u)};
    const qv_i4 hb = qv_i4{(int)(qb.x ^ 0x80808080u), (int)(qb.y ^ 0x80808080u), (int)(qb.z ^ 0x80808080u), (int)(qb.w ^ 0x80808080u)};
    qv_i4 C = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a_even[0], la, a.c_init, 0, 0, 0);
    C = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a_even[1], lb, C, 0, 0, 0);
    C = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a_odd[0], ha, C, 0, 0, 0);
    C = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a_odd[1], hb, C, 0, 0, 0);
    uint32_t scp, mnp;
    q4k_scale_min_pair(hdr.y, hdr.z, hdr.w, c, scp, mnp);
    const uint32_t sc_lo = scp & 0xFFu, sc_hi = (scp >> 8) & 0xFFu, mn_lo = mnp & 0xFFu, mn_hi = (mnp >> 8) & 0xFFu;
    const float d = f16_bits(hdr.x), dmin = f16_bits(hdr.x >> 16);
    const float f_e = (float)((C[1] << 8) + C[0]) * a.s_e, f_o = (float)((C[3] << 8) + C[2]) * a.s_o16;
    float acc = d * fmaf((float)sc_lo, f_e, (float)sc_hi * f_o);
    return fmaf(-dmin, fmaf((float)mn_lo, a.xs_e, (float)mn_hi * a.xs_o), acc);
}
// The same reduced over the four chunks: every lane of a row ends up with the block's sum.
__device__ __forceinline__ float qv_block_dot(const uint8_t *blk, const QvActs &a, int c) {
    return sum_xor32(sum_xor16(qv_block_dot_lane(blk, a, c)));
}

// The Q4_K policy.
struct QvQ4K {
    static constexpr int BLOCK = 144, ROW = 16 * BLOCK, ROW_LDS = QD_ROW_LDS;  // rows 16 bytes apart in banks
    static constexpr int STAGE_BYTES = 1184;  // what prepare() uses of `stage`
    static constexpr bool SIDE_LDS = false;
    static constexpr int COLS = 4096, SLOTS = 3;
    typedef QvActs Acts;
    // the activations times f: one factor onto everything that carries the activation scale
    __device__ static __forceinline__ void scale(Acts &a, float f) { a.s_e *= f, a.s_o16 *= f, a.xs_e *= f, a.xs_o *= f; }
    __device__ static __forceinline__ Acts prepare(const float4 v, uint32_t *stage, int lane) { return qv_prepare(v, stage, lane); }
    __device__ static __forceinline__ float block_dot(const uint8_t *blk, const Acts &a, int c) { return qv_block_dot(blk, a, c); }
    __device__ static __forceinline__ float block_dot_lane(const uint8_t *blk, const Acts &a, int c) { return qv_block_dot_lane(blk, a, c); }
};

// The same for the kernel that keeps the operands of four columns: the accumulator start as the one word
// that is not zero, and the four scale factors of a lane group in LDS (16 bytes a wave, column and lane group,
// read back once a tile), 18 registers a column instead of 24.
struct QvQ4KCompact {
    static constexpr int BLOCK = QvQ4K::BLOCK, ROW = QvQ4K::ROW, ROW_LDS = QvQ4K::ROW_LDS, STAGE_BYTES = QvQ4K::STAGE_BYTES;
    static constexpr bool SIDE_LDS = true;
    static constexpr int SLOTS = 3;
    struct Acts {
        qv_i4 a_even[2], a_odd[2];
        int c_init2;
        const float4 *side;  // s_e, s_o16, xs_e, xs_o
    };
    __device__ static __forceinline__ Acts prepare(const float4 v, uint32_t *stage, int lane, float4 *side) {
        const QvActs a = qv_prepare(v, stage, lane);
        *side = float4{a.s_e, a.s_o16, a.xs_e, a.xs_o};  // the same from the 16 lanes of a group
        return Acts{{a.a_even[0], a.a_even[1]}, {a.a_odd[0], a.a_odd[1]}, a.c_init[2], side};
    }
    __device__ static __forceinline__ float block_dot_lane(const uint8_t *blk, const Acts &a, int c) {
        const float4 f = *a.side;
        const QvActs full{{a.a_even[0], a.a_even[1]}, {a.a_odd[0], a.a_odd[1]}, qv_i4{0, 0, a.c_init2, 0}, f.x, f.y, f.z, f.w};
        return qv_block_dot_lane(blk, full, c);
    }
};

// ---- Q2_K ----
//
// Block of 84 bytes: scales[16] | qs[64] | d | dmin; element 128 sg + 32 f + l (l < 32) is the two-bit
// field f of byte qs[32 sg + l], and the 16 elements 128 sg + 32 f + 16 hf + [0, 16) share the scale byte
// scales[8 sg + 2 f + hf]: w = d (sc & 15) q - dmin (sc >> 4)  (reference: src/kquant_dot.rs:326-400).
// Lane (r, c) takes bytes 16c .. 16c+15 of the block's qs, i.e. super-group c / 2, byte half c % 2: one
// 16-element scale group per field.  Four MFMAs a block, one per field, with B = the field where it sits
// (q & 0x03, q & 0x0C = 4 f1, q & 0x30 = 16 f2; the top field shifted down) and the powers of four taken
// back through the activation scale; A row 4c + plane is non-zero in lane group c only, so a lane receives
// the two plane sums of its own group.  The activations are 16-bit fixed point per 32 elements, as for Q4_K;
// the min term needs their sums per 16.
struct Q2Acts {
    qv_i4 a[4];         // A operand per field
    float s[4], xs[4];  // per field: activation scale of its 32 elements (over 1, 4, 16, 1), scale x sum of the lane's 16
};

struct QvQ2K {
    static constexpr int BLOCK = 84, ROW = 16 * BLOCK, ROW_LDS = ROW + 16;  // 340 words: 16 rows x 4 words fill the 64 banks
    static constexpr int STAGE_BYTES = 640;
    static constexpr int COLS = 4096, SLOTS = 3;
    static constexpr bool SIDE_LDS = false;
    typedef Q2Acts Acts;
    __device__ static __forceinline__ void scale(Acts &a, float f) {
#pragma unroll
        for (int i = 0; i < 4; i++) a.s[i] *= f, a.xs[i] *= f;
    }
    __device__ static __forceinline__ Acts prepare(const float4 v, uint32_t *stage, int lane) {
        const int r = lane & 15, c = lane >> 4;
        float *stage_f = (float *)(stage + 128);  // [0,8) scales of the 32-element sub-blocks, [8,24) scale x sum per 16
        {
            float amax = fmaxf(fmaxf(mag_or_inf(v.x), mag_or_inf(v.y)), fmaxf(mag_or_inf(v.z), mag_or_inf(v.w)));
            amax = max_row8(amax);
            const bool live = amax > 0.0f && amax < INFINITY;
            const float inv = live ? QD_RANGE / amax : 0.0f, s = fixed_scale(amax, QD_RANGE);
            const int Xq[4] = {__float2int_rn(v.x * inv), __float2int_rn(v.y * inv), __float2int_rn(v.z * inv),
                               __float2int_rn(v.w * inv)};
            uint32_t wl = 0, wh = 0;
            int sum = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                wl |= (uint32_t)(Xq[i] & 255) << (8 * i);
                wh |= (uint32_t)(((Xq[i] + 128) >> 8) & 255) << (8 * i);
                sum += Xq[i];
            }
            stage[lane] = wl, stage[64 + lane] = wh;
            sum += dpp_i<0xB1>(sum);  // the four lanes of a 16-element group
            sum += dpp_i<0x4E>(sum);
            if ((lane & 7) == 0) stage_f[lane >> 3] = s;
            if ((lane & 3) == 0) stage_f[8 + (lane >> 2)] = s * (float)sum;
        }
        asm volatile("" ::: "memory");  // (written as scalars, read back as vectors: the compiler keeps the order only when told)
        Acts a;
        const int cm = r >> 2, pl = r & 3;  // A row m = 4 cm + plane
        const bool mine = cm == c && pl < 2;
        const uint4 z = uint4{0, 0, 0, 0};
#pragma unroll
        for (int f = 0; f < 4; f++) {
            // elements 128 (c / 2) + 32 f + 16 (c % 2) + [0, 16): words 32 (c / 2) + 8 f + 4 (c % 2) of the plane
            const uint4 w = mine ? *(const uint4 *)(stage + 64 * (pl & 1) + 32 * (c >> 1) + 8 * f + 4 * (c & 1)) : z;
            a.a[f] = qv_i4{(int)w.x, (int)w.y, (int)w.z, (int)w.w};
            const float pw = f == 1 ? 0.25f : (f == 2 ? 0.0625f : 1.0f);
            a.s[f] = stage_f[4 * (c >> 1) + f] * pw;
            a.xs[f] = stage_f[8 + 8 * (c >> 1) + 2 * f + (c & 1)];
        }
        asm volatile("" ::: "memory");  // (the next column's preparation writes the same words as another type)
        return a;
    }
    __device__ static __forceinline__ float block_dot(const uint8_t *blk, const Acts &a, int c) {
        return sum_xor32(sum_xor16(block_dot_lane(blk, a, c)));
    }
    __device__ static __forceinline__ float block_dot_lane(const uint8_t *blk, const Acts &a, int c) {
        // blocks sit at multiples of 84 bytes: everything is read as aligned 32-bit words
        const uint32_t *w32 = (const uint32_t *)blk;
        const uint32_t sc0 = w32[2 * (c >> 1)] >> (8 * (c & 1)), sc1 = w32[2 * (c >> 1) + 1] >> (8 * (c & 1));
        const uint32_t q[4] = {w32[4 + 4 * c], w32[5 + 4 * c], w32[6 + 4 * c], w32[7 + 4 * c]};
        const uint32_t dd = w32[20];
        const qv_i4 zero = qv_i4{0, 0, 0, 0};
        const qv_i4 b0 = qv_i4{(int)(q[0] & 0x03030303u), (int)(q[1] & 0x03030303u), (int)(q[2] & 0x03030303u), (int)(q[3] & 0x03030303u)};
        const qv_i4 b1 = qv_i4{(int)(q[0] & 0x0C0C0C0Cu), (int)(q[1] & 0x0C0C0C0Cu), (int)(q[2] & 0x0C0C0C0Cu), (int)(q[3] & 0x0C0C0C0Cu)};
        const qv_i4 b2 = qv_i4{(int)(q[0] & 0x30303030u), (int)(q[1] & 0x30303030u), (int)(q[2] & 0x30303030u), (int)(q[3] & 0x30303030u)};
        const qv_i4 b3 = qv_i4{(int)((q[0] >> 6) & 0x03030303u), (int)((q[1] >> 6) & 0x03030303u), (int)((q[2] >> 6) & 0x03030303u),
                               (int)((q[3] >> 6) & 0x03030303u)};
        const qv_i4 C0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a[0], b0, zero, 0, 0, 0);
        const qv_i4 C1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a[1], b1, zero, 0, 0, 0);
        const qv_i4 C2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a[2], b2, zero, 0, 0, 0);
        const qv_i4 C3 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a[3], b3, zero, 0, 0, 0);
        // scale bytes of the lane's four groups: bytes 0 and 2 of sc0 (fields 0, 1) and of sc1 (fields 2, 3)
        const float t0 = (float)((C0[1] << 8) + C0[0]) * a.s[0], t1 = (float)((C1[1] << 8) + C1[0]) * a.s[1];
        const float t2 = (float)((C2[1] << 8) + C2[0]) * a.s[2], t3 = (float)((C3[1] << 8) + C3[0]) * a.s[3];
        float sd = (float)(sc0 & 0xFu) * t0;
        sd = fmaf((float)((sc0 >> 16) & 0xFu), t1, sd);
        sd = fmaf((float)(sc1 & 0xFu), t2, sd);
        sd = fmaf((float)((sc1 >> 16) & 0xFu), t3, sd);
        float sm = (float)((sc0 >> 4) & 0xFu) * a.xs[0];
        sm = fmaf((float)((sc0 >> 20) & 0xFu), a.xs[1], sm);
        sm = fmaf((float)((sc1 >> 4) & 0xFu), a.xs[2], sm);
        sm = fmaf((float)((sc1 >> 20) & 0xFu), a.xs[3], sm);
        return fmaf(-f16_bits(dd >> 16), sm, f16_bits(dd) * sd);
    }
};

// ---- Q6_K ----
//
// Block of 210 bytes: ql[128] | qh[64] | scales[16] (int8) | d; element 128 h + 32 t + l (l < 32) is the low (t < 2) or
// high nibble of ql[64 h + 32 (t & 1) + l] with bits 2t, 2t + 1 of qh[32 h + l] above it, and the 16 elements
// 128 h + 32 t + 16 lh + [0, 16) share scales[8 h + 2 t + lh]: w = d sc (q - 32)  (the reference decodes the
// format through candle's to_float, src/quant_matmul.rs:228-248; layout as in
// vendor/candle-metal-kernels/src/metal_src/quantized.metal:198-203,6673-6694).
// Lane (r, c = 2 h + lh) takes the 16 values of l in [16 lh, 16 lh + 16) of half h in all four quarters t: 16
// bytes of each of ql's two runs and of qh, four MFMAs (one a quarter: B = the sixteen 6-bit values q, 0..63, of
// one scale group; A row 4c + 2 (t & 1) + plane non-zero in lane group c only, so the quarters (0, 1) share one
// accumulator and (2, 3) another), and the accumulators start at -32 sum X of the group, which turns sum q X
// into sum (q - 32) X.  The blocks sit at multiples of 210 bytes: every field is read as aligned words and
// shifted into place (ldw).
struct Q6Acts {
    qv_i4 a[4];     // A operand per quarter
    qv_i4 init[2];  // accumulator starts of quarters (0, 1) and (2, 3): -32 sum X in the low-plane rows
    float s[4];     // activation scale of the quarter's 32-element block
};

struct QvQ6K {
    static constexpr int BLOCK = 210, ROW = 16 * BLOCK, ROW_LDS = ROW + 16;  // rows 48 bytes apart in a bank row: 8 rows, 8 slots
    static constexpr int STAGE_BYTES = 640;
    static constexpr int COLS = 4096, SLOTS = 2;  // a tile is 54 KB: two of them, and one more barrier a tile
    static constexpr bool SIDE_LDS = false;
    typedef Q6Acts Acts;
    __device__ static __forceinline__ void scale(Acts &a, float f) {
#pragma unroll
        for (int t = 0; t < 4; t++) a.s[t] *= f;
    }
    // stage: words [0,64) Xl, [64,128) Xh, 8 words of zeros, 8 block scales, 16 sums of X per 16 elements
    __device__ static __forceinline__ Acts prepare(const float4 v, uint32_t *stage, int lane) {
        const int r = lane & 15, c = lane >> 4, h = c >> 1, lh = c & 1;
        float *sf = (float *)(stage + 136);
        int *xs16 = (int *)(stage + 144);
        {
            const QvQuant q = qv_quantise4(v);
            stage[lane] = q.wl, stage[64 + lane] = q.wh;
            if (lane < 8) stage[128 + lane] = 0;
            int s4 = q.sum4;
            s4 += dpp_i<0xB1>(s4);  // the four lanes of a 16-element group
            s4 += dpp_i<0x4E>(s4);
            if ((lane & 7) == 0) sf[lane >> 3] = q.s;
            if ((lane & 3) == 0) xs16[lane >> 2] = s4;
        }
        asm volatile("" ::: "memory");  // (written as scalars, read back as vectors: the compiler keeps the order only when told)
        Acts a;
        const bool mine = (r >> 2) == c;
        const int p = (r >> 1) & 1, pl = r & 1;
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const uint32_t *src = mine && p == (t & 1) ? stage + 64 * pl + 32 * h + 8 * t + 4 * lh : stage + 128;
            const uint4 w = *(const uint4 *)src;
            a.a[t] = qv_i4{(int)w.x, (int)w.y, (int)w.z, (int)w.w};
            a.s[t] = sf[4 * h + t];
        }
        a.init[0] = qv_i4{-32 * xs16[8 * h + lh], 0, -32 * xs16[8 * h + 2 + lh], 0};
        a.init[1] = qv_i4{-32 * xs16[8 * h + 4 + lh], 0, -32 * xs16[8 * h + 6 + lh], 0};
        asm volatile("" ::: "memory");  // (the next column's preparation writes the same words as another type)
        return a;
    }
    __device__ static __forceinline__ float block_dot_lane(const uint8_t *blk, const Acts &a, int c) {
        const int h = c >> 1, lh = c & 1;
        const uint4 qa = ldw<uint4>(blk + 64 * h + 16 * lh), qb = ldw<uint4>(blk + 64 * h + 32 + 16 * lh);
        const uint4 qh = ldw<uint4>(blk + 128 + 32 * h + 16 * lh);
        const uint2 sc8 = ldw<uint2>(blk + 192 + 8 * h);
        const float d = f16_bits(ld<uint16_t>(blk + 208));
        const uint32_t A[4] = {qa.x, qa.y, qa.z, qa.w}, B[4] = {qb.x, qb.y, qb.z, qb.w}, H[4] = {qh.x, qh.y, qh.z, qh.w};
        qv_i4 b0, b1, b2, b3;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            b0[j] = (int)((A[j] & 0x0F0F0F0Fu) | ((H[j] << 4) & 0x30303030u));
            b1[j] = (int)((B[j] & 0x0F0F0F0Fu) | ((H[j] << 2) & 0x30303030u));
            b2[j] = (int)(((A[j] >> 4) & 0x0F0F0F0Fu) | (H[j] & 0x30303030u));
            b3[j] = (int)(((B[j] >> 4) & 0x0F0F0F0Fu) | ((H[j] >> 2) & 0x30303030u));
        }
        qv_i4 C1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a[0], b0, a.init[0], 0, 0, 0);
        qv_i4 C2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a[2], b2, a.init[1], 0, 0, 0);
        C1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a[1], b1, C1, 0, 0, 0);
        C2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a[3], b3, C2, 0, 0, 0);
        // the lane's four scale bytes: scales[8 h + 2 t + lh], bytes lh and 2 + lh of each word
        const int o = 8 * lh;
        const float s0 = (float)(int8_t)(sc8.x >> o), s1 = (float)(int8_t)(sc8.x >> (16 + o));
        const float s2 = (float)(int8_t)(sc8.y >> o), s3 = (float)(int8_t)(sc8.y >> (16 + o));
        float f = s0 * ((float)((C1[1] << 8) + C1[0]) * a.s[0]);
        f = fmaf(s1, (float)((C1[3] << 8) + C1[2]) * a.s[1], f);
        f = fmaf(s2, (float)((C2[1] << 8) + C2[0]) * a.s[2], f);
        f = fmaf(s3, (float)((C2[3] << 8) + C2[2]) * a.s[3], f);
        return d * f;
    }
};

// Work of workgroup b (of G): tiles b, b + G, b + 2 G, ... of 16 rows each; there are rounds G + extra tiles,
// so the first `extra` workgroups take one more than the others.  The kernels take the four numbers as
// arguments of their own: scalars among the leading arguments arrive preloaded in registers, a struct is
// fetched by a scalar load in front of the first global load.  (Tiles of 14 rows, which give each of 256
// workgroups four tiles of a 14336-row matrix where tiles of 16 rows leave 32 compute units idle, measured
// 1.5 % slower for Q4_K: 7.49 against 7.39 us.)
struct QvWork {
    int n, G, rounds, extra;
};

// An asynchronous 16-byte load a lane whose global address is a scalar base (the wave's row) plus the lane's own
// byte offset: no vector instruction goes into the address.
__device__ __forceinline__ void async_load16_s(const uint8_t *sbase, uint32_t voff, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase),
                 "s"(__builtin_amdgcn_readfirstlane(lds_base))
                 : "memory");
}

// Wave w copies row w of a tile into a ring of three tiles in LDS (contiguous asynchronous loads, two tiles
// ahead of the arithmetic) and multiplies column w of all 16 rows, so a tile is published by a barrier.
//   * A tile's arithmetic comes first, the request for the tile after next behind it: a load instruction holds its
//     wave until the compute unit's memory pipeline accepts it, which with a tile in flight takes until most of
//     that tile has landed, and a wave that waits there multiplies late.
//   * A lane keeps its chunk's sum; the four chunk sums of a (row, wave) pair and the 16 waves' sums of a row are
//     added when the rows are stored, once per four tiles and behind one more barrier.  The partial sums sit in
//     LDS as [tile][row][4 wave + chunk] with rows 16 bytes longer than their 64 words: the writes of a wave
//     (lane (r, c) -> row r) and the 16-byte reads of the flush (lane (tile, wave) of row w) both touch every
//     bank once.  (As [tile][wave][row] the flush's reads fell on two banks: 0.5 us of the launch's end.)
//   * Stores go out only behind the last tile of four: a store between the tiles' loads costs 0.15 us each.
//   * NORM puts a residual add and an RMSNorm in front of the product (QdNorm: x += res; hn = x / rms(x) * w;
//     y = W hn as one launch): every workgroup normalises the row for itself and quantises (x + res) w; the
//     1 / rms, one factor for the whole row, goes onto the sub-block scales behind the barrier that publishes
//     tile 0, where the waves' sums of squares have met anyway.  Workgroup 0 stores x + res (into a buffer other
//     than X: the others are still reading X) and, when asked, the normalised row.  The norm's operands are
//     arguments of their own so that the leading ones arrive preloaded.
//   * SWIGLU: the matrix holds gate and up rows alternately (row 2j gate_j, row 2j + 1 up_j) and
//     Y[j] = silu(gate_j . x) * (up_j . x), n / 2 values (reference: src/quantized_qwen3_moe.rs:397-401).
// The kernel's LDS, one block of bytes so that a launch which runs two kernels' bodies side by side can give both the
// same block: the ring, the partial sums [FL][16][68], the waves' staging areas where the ring has no room for
// them, the waves' sums of squares.
template <class F>
struct GemvMfmaLds {
    static constexpr int FL = 4;                     // tiles a flush
    static constexpr int STAGE = F::STAGE_BYTES + 1024;
    static constexpr bool STAGE_IN_RING = STAGE <= F::ROW_LDS;
    static constexpr int RING = F::SLOTS * 16 * F::ROW_LDS, PART = FL * 16 * 68 * 4;
    static constexpr int STAGE_AT = RING + PART, SS_AT = STAGE_AT + (STAGE_IN_RING ? 16 : 16 * ((STAGE + 15) / 16 * 16));
    static constexpr int BYTES = SS_AT + 64;
};

// `b`: the workgroup's number among the G of this product.
template <class F, bool NORM, bool SWIGLU>
__device__ __forceinline__ void gemv_mfma_lds_body(uint8_t *lds, int b, const uint8_t *__restrict__ W,
                                                   const float *__restrict__ X, float *__restrict__ Y, int n, int G,
                                                   int rounds, int extra, const float *nm_res, const float *nm_w,
                                                   float nm_eps, float *nm_x_out, float *nm_hn_out) {
    typedef GemvMfmaLds<F> L;
    constexpr int SLOTS = F::SLOTS, FL = L::FL;      // ring slots (three: two tiles in flight); tiles a flush
    static_assert(!NORM || (2048 <= F::ROW_LDS && F::SLOTS == 3), "the norm's operands wait in a wave's row of ring slot 1");
    constexpr int FULL = F::ROW / 1024, REST = (F::ROW - 1024 * FULL) / 16, LOADS = FULL + (REST ? 1 : 0);
    constexpr int SLOT_BYTES = 16 * F::ROW_LDS;
    uint8_t *ring = lds;                             // [SLOTS][16 * ROW_LDS]
    float *part = (float *)(lds + L::RING);          // [FL][16][68]
    float *ss_lds = (float *)(lds + L::SS_AT);       // [16]
    // a wave's staging area (what prepare() needs, then its 256 raw activations): its own row of the last ring
    // slot when that is long enough, which no load targets before tile 2 is asked for in the main loop; else
    // memory of its own
    constexpr int STAGE = (L::STAGE + 15) / 16 * 16;
    constexpr bool STAGE_IN_RING = L::STAGE_IN_RING;
    uint8_t *stage_mem = lds + L::STAGE_AT;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, c = lane >> 4;
    const int nt = rounds + (b < extra ? 1 : 0);  // tiles of this workgroup (no division in front of the first loads)
    if (nt <= 0) return;
    auto tile_row0 = [&](int i) __attribute__((always_inline)) { return 16 * (b + i * G); };
    const uint32_t voff = 16 * lane, ring0 = lds_offset_of(ring);
    // fetch(i) asks for tile min(i, nt - 1) into slot i % 3 (the fetches in front of the main loop are
    // unconditional, so that every wave counts the same loads); the row's address is scalar arithmetic
    auto fetch = [&](int slot_i) __attribute__((always_inline)) {
        const int i = min(slot_i, nt - 1);
        const int row = min(tile_row0(i) + wave, n - 1);
        const uint8_t *src = W + (size_t)row * F::ROW;
        const uint32_t dst = ring0 + (uint32_t)(slot_i % SLOTS) * (16 * F::ROW_LDS) + (uint32_t)wave * F::ROW_LDS;
#pragma unroll
        for (int j = 0; j < FULL; j++) async_load16_s(src + 1024 * j, voff, dst + 1024 * j);
        if (REST && lane < REST) async_load16_s(src + 1024 * FULL, voff, dst + 1024 * FULL);
    };
    // the raw activations travel like the tiles (every global read of this kernel is an asynchronous load
    // counted by hand)
    uint32_t *stage = (uint32_t *)(STAGE_IN_RING ? ring + (SLOTS - 1) * SLOT_BYTES + wave * F::ROW_LDS : stage_mem + wave * STAGE);
    float *x_raw = (float *)((uint8_t *)stage + F::STAGE_BYTES);
    async_load16(X + 256 * wave + 4 * lane, lds_offset_of(x_raw));
    // norm weight and residual columns wait in the wave's row of ring slot 1, which no tile enters before the
    // activations are prepared
    float *w_raw = (float *)(ring + SLOT_BYTES + wave * F::ROW_LDS), *r_raw = w_raw + 256;
    if (NORM) {
        async_load16(nm_w + 256 * wave + 4 * lane, lds_offset_of(w_raw));
        if (nm_res) async_load16(nm_res + 256 * wave + 4 * lane, lds_offset_of(r_raw));
    }
    // every wave's activations are asked for before anybody's tile: the memory pipeline takes a compute
    // unit's requests in the order they were issued, and a wave whose activations queue behind the other
    // waves' tile loads starts its preparation late
    __builtin_amdgcn_s_barrier();
    // tile 0 is asked for alone and lands while the activations are prepared; tile 1 follows the preparation
    // (asked for in front of it, tile 1 delays the preparation: a wave stands at a load until the memory
    // pipeline accepts it; measured slower both on a resident activation row and behind another kernel)
    fetch(0);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOADS) : "memory");
    float4 v = *(const float4 *)&x_raw[4 * lane];
    if (NORM) {
        if (nm_res) {
            const float4 rr = *(const float4 *)&r_raw[4 * lane];
            v.x += rr.x, v.y += rr.y, v.z += rr.z, v.w += rr.w;
        }
        float ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, v.w * v.w)));
        ss = wave_sum(ss);
        if (lane == 0) ss_lds[wave] = ss;
        const float4 g = *(const float4 *)&w_raw[4 * lane];
        if (b == 0) *(float4 *)(nm_x_out + 256 * wave + 4 * lane) = v;
        v = float4{v.x * g.x, v.y * g.y, v.z * g.z, v.w * g.w};
    }
    typename F::Acts acts = F::prepare(v, stage, lane);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    // (the store of x + res counts among the wave's memory operations until it is acknowledged: the waits
    // below then hold a little longer in workgroup 0, never too short)
    fetch(1);

    for (int t = 0; t < nt; t++) {
        // tile t has landed when only tile t + 1's loads are out (nothing behind the last tile)
        if (t + 1 < nt) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOADS) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (NORM && t == 0) {  // the waves' sums of squares are all written
            float tot = 0.0f;
#pragma unroll
            for (int i = 0; i < 16; i++) tot += ss_lds[i];
            const float inv = 1.0f / sqrtf(tot / (float)F::COLS + nm_eps);
            F::scale(acts, inv);
            if (b == 0 && nm_hn_out) *(float4 *)(nm_hn_out + 256 * wave + 4 * lane) = float4{v.x * inv, v.y * inv, v.z * inv, v.w * inv};
        }
        part[((t & (FL - 1)) * 16 + r) * 68 + 4 * wave + c] =
            F::block_dot_lane(ring + (t % SLOTS) * SLOT_BYTES + r * F::ROW_LDS + wave * F::BLOCK, acts, c);
        // every wave is done with tile t - 1, whose slot tile t + 2 takes; with two slots it takes tile t's own,
        // once every wave has read it
        if (t + 2 < nt) {
            if (SLOTS == 2) __builtin_amdgcn_s_barrier();
            fetch(t + 2);
        }
        if ((t & (FL - 1)) == FL - 1 || t == nt - 1) {
            // the partial sums of this group's tiles are written: lane (tt = lane / 16, ww = lane % 16) takes wave
            // ww's four chunk sums of row `wave` in tile tt of the group
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            const int tt = (t & ~(FL - 1)) + c;
            const float4 p = *(const float4 *)&part[(c * 16 + wave) * 68 + 4 * r];
            float sum = (p.x + p.y) + (p.z + p.w);
            sum = sum_row16(sum);
            if (!SWIGLU) {
                if (r == 0 && tt <= t) {
                    const int row = tile_row0(tt) + wave;
                    if (row < n) Y[row] = sum;
                }
            } else if ((wave & 1) == 0) {  // an even wave takes its gate row and the up row behind it
                const float4 q = *(const float4 *)&part[(c * 16 + wave + 1) * 68 + 4 * r];
                float up = (q.x + q.y) + (q.z + q.w);
                up = sum_row16(up);
                if (r == 0 && tt <= t) {
                    const int row = tile_row0(tt) + wave;
                    if (row + 1 < n) Y[row >> 1] = silu(sum) * up;
                }
            }
        }
    }
}

template <class F, bool NORM = false, bool SWIGLU = false>
__global__ __launch_bounds__(1024) void gemv_mfma_lds(const uint8_t *__restrict__ W, const float *__restrict__ X,
                                                      float *__restrict__ Y, int n, int G, int rounds, int extra,
                                                      const float *nm_res, const float *nm_w, float nm_eps,
                                                      float *nm_x_out, float *nm_hn_out) {
    __shared__ __attribute__((aligned(16))) uint8_t lds[GemvMfmaLds<F>::BYTES];
    gemv_mfma_lds_body<F, NORM, SWIGLU>(lds, (int)blockIdx.x, W, X, Y, n, G, rounds, extra, nm_res, nm_w, nm_eps, nm_x_out,
                                        nm_hn_out);
}

// The same kernel for rows of more than 16 super-blocks (up to 16 NG): a tile is 16 rows x one pass of 16
// columns (the last pass may hold fewer), tile i of a workgroup = (row tile i / NG, pass i % NG), and wave w
// keeps the operands of its column of every pass.  A lane adds its chunk sums of a row tile's passes in a
// register.  nb = super-blocks a row (contiguous rows of nb blocks); rounds / extra count row tiles.
struct QvColsWork {
    int n, G, rounds, extra, nb;
};

template <class F, int NG>
__global__ __launch_bounds__(1024) void gemv_mfma_cols(const uint8_t *__restrict__ W, const float *__restrict__ X,
                                                       float *__restrict__ Y, int n, int G, int rounds, int extra, int nb) {
    static_assert(NG >= 2 && NG <= 4, "two to four passes a row");
    // ring slots (two tiles in flight; a fourth slot only where the staging of four passes needs it) and row
    // tiles a flush
    constexpr int SLOTS = F::SLOTS == 2 ? 2 : (NG == 4 ? 4 : 3), FL = NG == 4 ? 2 : 4;
    static_assert(SLOTS > 2 || NG <= 3, "two slots: the staging below holds three passes");
    constexpr int LOADS = (F::ROW + 1023) / 1024;
    // the raw activations of the passes wait in the wave's own rows of the last ring slot (behind what prepare()
    // uses), of the one in front of it and of slot 1, which no load targets before the wave itself has prepared
    // its activations and asks for tile 1
    static_assert(F::STAGE_BYTES + 1024 <= F::ROW_LDS && 2048 <= F::ROW_LDS && (F::SLOTS > 2 || F::STAGE_BYTES + 2048 <= F::ROW_LDS), "staging in the ring");
    __shared__ __attribute__((aligned(16))) uint8_t ring[SLOTS][16 * F::ROW_LDS];
    __shared__ __attribute__((aligned(16))) float part[FL][16][68];  // [row tile][row][4 wave + chunk], as in gemv_mfma_lds
    __shared__ float4 side[F::SIDE_LDS ? 16 * NG * 4 : 1];  // [wave][pass][lane group], for the policies that want it
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, c = lane >> 4, b = (int)blockIdx.x;
    const size_t row_bytes = (size_t)nb * F::BLOCK;
    const int nrt = rounds + (b < extra ? 1 : 0), nt = NG * nrt;  // row tiles, tiles (row tile, pass) of this workgroup
    if (nt <= 0) return;
    const uint32_t ring0 = lds_offset_of(&ring[0][0]);
    // every fetch is LOADS instructions with at least one lane at work, so that every wave counts the same
    // loads; a short last pass repeats its last 16 bytes into LDS bytes nobody reads
    auto fetch = [&](int slot_i) __attribute__((always_inline)) {
        const int i = min(slot_i, nt - 1), rt = i / NG, cg = i - rt * NG;
        const int row = min(16 * (b + rt * G) + wave, n - 1);
        const int len = min(16, nb - 16 * cg) * F::BLOCK;
        const uint8_t *src = W + (size_t)row * row_bytes + (size_t)cg * F::ROW;
        const uint32_t dst = ring0 + (uint32_t)(slot_i % SLOTS) * (16 * F::ROW_LDS) + (uint32_t)wave * F::ROW_LDS;
#pragma unroll
        for (int j = 0; j < LOADS; j++) {
            const int lanes = max(1, min(64, (min(len, F::ROW) - 1024 * j) / 16));
            if (lane < lanes) async_load16_s(src, (uint32_t)min(1024 * j + 16 * lane, len - 16), dst + 1024 * j);
        }
    };
    uint32_t *stage = (uint32_t *)&ring[SLOTS - 1][wave * F::ROW_LDS];
    auto x_raw = [&](int cg) __attribute__((always_inline)) {
        if (SLOTS == 2)  // two passes behind the staging area in the wave's row of slot 1, a third in the partial sums' memory
            return cg < 2 ? (float *)((uint8_t *)stage + F::STAGE_BYTES + 1024 * cg) : (float *)&part[0][0][0] + 256 * wave;
        return cg == 0   ? (float *)((uint8_t *)stage + F::STAGE_BYTES)
               : cg == 3 ? (float *)&ring[1][wave * F::ROW_LDS]
                         : (float *)&ring[SLOTS > 2 ? SLOTS - 2 : 0][wave * F::ROW_LDS + 1024 * (cg - 1)];
    };
#pragma unroll
    for (int cg = 0; cg < NG; cg++)  // a column past the row's last block reads the last one's and is not used
        async_load16(X + 256 * min(16 * cg + wave, nb - 1) + 4 * lane, lds_offset_of(x_raw(cg)));
    __builtin_amdgcn_s_barrier();
    fetch(0);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOADS) : "memory");
    typename F::Acts acts[NG];
#pragma unroll
    for (int cg = 0; cg < NG; cg++) {
        const float4 v = *(const float4 *)&x_raw(cg)[4 * lane];
        if constexpr (F::SIDE_LDS) acts[cg] = F::prepare(v, stage, lane, &side[(wave * NG + cg) * 4 + c]);
        else acts[cg] = F::prepare(v, stage, lane);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    fetch(1);

    for (int rt = 0; rt < nrt; rt++) {
        float acc = 0.0f;  // a lane's chunk sums of the row tile's passes
#pragma unroll
        for (int cg = 0; cg < NG; cg++) {
            const int t = NG * rt + cg;
            if (t + 1 < nt) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LOADS) : "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (16 * cg + wave < nb)
                acc += F::block_dot_lane(&ring[t % SLOTS][r * F::ROW_LDS + wave * F::BLOCK], acts[cg], c);
            // every wave is done with tile t - 1, whose slot tile t + 2 takes (with four slots: tile t - 2's; with
            // two: tile t's own, once every wave has read it)
            if (t + 2 < nt) {
                if (SLOTS == 2) __builtin_amdgcn_s_barrier();
                fetch(t + 2);
            }
        }
        part[rt & (FL - 1)][r][4 * wave + c] = acc;
        if ((rt & (FL - 1)) == FL - 1 || rt == nrt - 1) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            // lane (tt = lane / 16, ww = lane % 16) takes wave ww's four chunk sums of row `wave` in row tile tt of
            // the group
            const int tt = (rt & ~(FL - 1)) + c;
            const float4 p = *(const float4 *)&part[c & (FL - 1)][wave][4 * r];
            float sum = (p.x + p.y) + (p.z + p.w);
            sum = sum_row16(sum);
            if (r == 0 && c < FL && tt <= rt) {
                const int row = 16 * (b + tt * G) + wave;
                if (row < n) Y[row] = sum;
            }
        }
    }
}

}  // namespace jq
