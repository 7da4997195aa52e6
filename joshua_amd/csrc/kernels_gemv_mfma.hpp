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

constexpr int QV_SLOTS = 4;  // ring slots

typedef int qv_i4 __attribute__((ext_vector_type(4)));

// What a lane keeps of its wave's 256 activations for the whole kernel.
struct QvActs {
    qv_i4 a_even[2], a_odd[2];  // A operands: [bytes 0..15 | 16..31 of the chunk]
    qv_i4 c_init;               // accumulator start: 128 XS of sub-block 2c + 1 in the low-plane row
    float s_e, s_o16, xs_e, xs_o;
};

// Quantises the wave's activation column (lane i holds elements 4i .. 4i+3, sub-block i / 8) and builds
// the lane's operands through `stage`, 1152 bytes of LDS that only this wave touches:
// words [0,64) Xl, [64,128) Xh, [128,192) and [192,256) the planes of -X, then 8 scales, 8 scaled sums, 8
// integer sums.
__device__ __forceinline__ QvActs qv_prepare(const float4 v, uint32_t *stage, int lane) {
    const int r = lane & 15, c = lane >> 4;
    float *stage_f = (float *)(stage + 256);
    {
        float amax = fmaxf(fmaxf(mag_or_inf(v.x), mag_or_inf(v.y)), fmaxf(mag_or_inf(v.z), mag_or_inf(v.w)));
        amax = max_row8(amax);
        const bool live = amax > 0.0f && amax < INFINITY;
        const float inv = live ? QD_RANGE / amax : 0.0f, s = fixed_scale(amax, QD_RANGE);
        const int Xq[4] = {__float2int_rn(v.x * inv), __float2int_rn(v.y * inv), __float2int_rn(v.z * inv),
                           __float2int_rn(v.w * inv)};
        uint32_t wl = 0, wh = 0, nl = 0, nh = 0;
        int sum = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // balanced planes: the low byte read as signed, the rest above it
            wl |= (uint32_t)(Xq[i] & 255) << (8 * i);
            wh |= (uint32_t)(((Xq[i] + 128) >> 8) & 255) << (8 * i);
            nl |= (uint32_t)(-Xq[i] & 255) << (8 * i);
            nh |= (uint32_t)(((-Xq[i] + 128) >> 8) & 255) << (8 * i);
            sum += Xq[i];
        }
        stage[lane] = wl, stage[64 + lane] = wh, stage[128 + lane] = nl, stage[192 + lane] = nh;
        sum = isum_row8(sum);
        if ((lane & 7) == 0) {
            stage_f[lane >> 3] = s;
            stage_f[8 + (lane >> 3)] = s * (float)sum;
            ((int *)stage_f)[16 + (lane >> 3)] = sum;
        }
    }
    QvActs a;
    {
        // A operands of lane (m = r, g = c): sub-block jm = m / 2, plane m % 2; non-zero when jm is 2g or 2g + 1
        const int jm = r >> 1, pl = r & 1, p = jm - 2 * c;  // p: 0 low-nibble sub-block, 1 high-nibble sub-block
        const bool mine = p == 0 || p == 1;
        const uint32_t *pos = stage + 64 * pl + 16 * c + 8 * (p & 1);  // plane words of the sub-block's 32 elements
        const uint32_t *neg = pos + 128;
        const uint4 z = uint4{0, 0, 0, 0};
        const uint4 p0 = mine ? *(const uint4 *)pos : z, p1 = mine ? *(const uint4 *)(pos + 4) : z;
        const uint4 n0 = mine ? *(const uint4 *)neg : z, n1 = mine ? *(const uint4 *)(neg + 4) : z;
        const bool odd = p == 1;
        const uint4 e0 = odd ? n0 : p0, e1 = odd ? n1 : p1, o0 = odd ? p0 : z, o1 = odd ? p1 : z;
        a.a_even[0] = qv_i4{(int)e0.x, (int)e0.y, (int)e0.z, (int)e0.w};
        a.a_even[1] = qv_i4{(int)e1.x, (int)e1.y, (int)e1.z, (int)e1.w};
        a.a_odd[0] = qv_i4{(int)o0.x, (int)o0.y, (int)o0.z, (int)o0.w};
        a.a_odd[1] = qv_i4{(int)o1.x, (int)o1.y, (int)o1.z, (int)o1.w};
    }
    // what lane (r, c) needs of sub-blocks 2c and 2c + 1 after the MFMAs
    a.s_e = stage_f[2 * c], a.s_o16 = stage_f[2 * c + 1] * 0.0625f;
    a.xs_e = stage_f[8 + 2 * c], a.xs_o = stage_f[8 + 2 * c + 1];
    a.c_init = qv_i4{0, 0, 128 * ((const int *)stage_f)[16 + 2 * c + 1], 0};
    return a;
}

// The sum of a super-block of weight row r against the wave's column, over chunk c, reduced over the four
// chunks: every lane of a row ends up with the block's sum.  blk: the row's 144-byte block in LDS.
__device__ __forceinline__ float qv_block_dot(const uint8_t *blk, const QvActs &a, int c) {
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
    acc = fmaf(-dmin, fmaf((float)mn_lo, a.xs_e, (float)mn_hi * a.xs_o), acc);
    acc = sum_xor16(acc);
    return sum_xor32(acc);
}

// The Q4_K policy.
struct QvQ4K {
    static constexpr int BLOCK = 144, ROW = 16 * BLOCK, ROW_LDS = QD_ROW_LDS;  // rows 16 bytes apart in banks
    static constexpr int STAGE_BYTES = 1152;  // what prepare() uses of `stage`
    static constexpr bool SIDE_LDS = false;
    typedef QvActs Acts;
    __device__ static __forceinline__ Acts prepare(const float4 v, uint32_t *stage, int lane) { return qv_prepare(v, stage, lane); }
    __device__ static __forceinline__ float block_dot(const uint8_t *blk, const Acts &a, int c) { return qv_block_dot(blk, a, c); }
};

// The same for the kernel that keeps the operands of four columns: the accumulator start as the one word
// that is not zero, and the four scale factors of a lane group in LDS (16 bytes a wave, column and lane group,
// read back once a tile), 18 registers a column instead of 24.
struct QvQ4KCompact {
    static constexpr int BLOCK = QvQ4K::BLOCK, ROW = QvQ4K::ROW, ROW_LDS = QvQ4K::ROW_LDS, STAGE_BYTES = QvQ4K::STAGE_BYTES;
    static constexpr bool SIDE_LDS = true;
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
    __device__ static __forceinline__ float block_dot(const uint8_t *blk, const Acts &a, int c) {
        const float4 f = *a.side;
        const QvActs full{{a.a_even[0], a.a_even[1]}, {a.a_odd[0], a.a_odd[1]}, qv_i4{0, 0, a.c_init2, 0}, f.x, f.y, f.z, f.w};
        return qv_block_dot(blk, full, c);
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
    typedef Q2Acts Acts;
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
        return a;
    }
    __device__ static __forceinline__ float block_dot(const uint8_t *blk, const Acts &a, int c) {
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
        float acc = fmaf(-f16_bits(dd >> 16), sm, f16_bits(dd) * sd);
        acc = sum_xor16(acc);
        return sum_xor32(acc);
    }
};

// Work of workgroup b (of G): tiles b, b + G, b + 2 G, ... of 16 rows each; there are rounds G + extra tiles,
// so the first `extra` workgroups take one more than the others.  (Tiles of 14 rows, which give each of 256
// workgroups four tiles of a 14336-row matrix where tiles of 16 rows leave 32 compute units idle, measured
// 1.5 % slower for Q4_K: 7.49 against 7.39 us.)
struct QvWork {
    int n, G, rounds, extra;
};

// Wave w copies row w of a tile into a ring of four tiles in LDS (contiguous asynchronous loads, two tiles
// ahead of the arithmetic) and multiplies column w of all 16 rows, so a tile is published by a barrier.
// The waves' partial sums of up to four tiles wait in LDS and are added, stored and forgotten behind one
// more barrier.
template <class F>
__global__ __launch_bounds__(1024) void gemv_mfma_lds(const uint8_t *__restrict__ W, const float *__restrict__ X,
                                                      float *__restrict__ Y, QvWork wk) {
    constexpr int D = 2;  // tiles asked for ahead of the one being multiplied (3 measured slower)
    constexpr int LOADS = (F::ROW + 1023) / 1024;  // asynchronous loads a wave and tile
    __shared__ __attribute__((aligned(16))) uint8_t ring[QV_SLOTS][16 * F::ROW_LDS];
    __shared__ float part[QV_SLOTS][16][16];  // [tile % 4][wave][row]
    // a wave's staging area (what prepare() needs, then its 256 raw activations): its own row of ring slot 3
    // when that is long enough, which no load targets before tile 3 is asked for in the main loop; else
    // memory of its own
    constexpr int STAGE = F::STAGE_BYTES + 1024;
    constexpr bool STAGE_IN_RING = STAGE <= F::ROW_LDS;
    __shared__ __attribute__((aligned(16))) uint8_t stage_mem[STAGE_IN_RING ? 16 : 16 * STAGE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, c = lane >> 4, b = (int)blockIdx.x;
    const int n = wk.n, G = wk.G;
    const int nt = wk.rounds + (b < wk.extra ? 1 : 0);  // tiles of this workgroup (no division in front of the first loads)
    if (nt <= 0) return;
    auto tile_row0 = [&](int i) __attribute__((always_inline)) { return 16 * (b + i * G); };
    // fetch(i) asks for tile min(i, nt - 1) into slot i % 4 (the fetches in front of the main loop are
    // unconditional, so that every wave counts the same loads)
    auto fetch = [&](int slot_i) __attribute__((always_inline)) {
        const int i = min(slot_i, nt - 1);
        const int row = min(tile_row0(i) + wave, n - 1);
        const uint8_t *src = W + (size_t)row * F::ROW + 16 * lane;
        const uint32_t dst = lds_offset_of(&ring[slot_i & (QV_SLOTS - 1)][wave * F::ROW_LDS]);
#pragma unroll
        for (int j = 0; j < LOADS; j++) {
            constexpr int full = F::ROW / 1024;
            if (j < full) async_load16(src + 1024 * j, dst + 1024 * j);
            else if (lane < (F::ROW - 1024 * full) / 16) async_load16(src + 1024 * j, dst + 1024 * j);
        }
    };
    // the raw activations travel like the tiles (every global read of this kernel is an asynchronous load
    // counted by hand)
    uint32_t *stage = (uint32_t *)(STAGE_IN_RING ? &ring[QV_SLOTS - 1][wave * F::ROW_LDS] : &stage_mem[wave * STAGE]);
    float *x_raw = (float *)((uint8_t *)stage + F::STAGE_BYTES);
    async_load16(X + 256 * wave + 4 * lane, lds_offset_of(x_raw));
    // every wave's activations are asked for before anybody's tile: the memory pipeline takes a compute
    // unit's requests in the order they were issued, and a wave whose activations queue behind the other
    // waves' tile loads starts its preparation a microsecond late
    __builtin_amdgcn_s_barrier();
    // tile 0 is asked for alone: it has the memory system to itself and lands while the activations are
    // prepared; the next D - 1 tiles follow the preparation
    fetch(0);
    if (LOADS == 3) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
    const float4 v = *(const float4 *)&x_raw[4 * lane];
    const typename F::Acts acts = F::prepare(v, stage, lane);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    fetch(1);
    if (D == 3) fetch(2);

    const int n_groups = (nt + QV_SLOTS - 1) / QV_SLOTS;
    for (int grp = 0; grp < n_groups; grp++) {
        const int t_end = min(nt, QV_SLOTS * (grp + 1));
        for (int t = QV_SLOTS * grp; t < t_end; t++) {
            // tile t has landed; tiles up to max(D - 1, min(nt - 1, t + D - 1)) have been asked for and may be
            // in flight, nothing behind the last tile
            const int ahead = t == nt - 1 ? 0 : max(D - 1, min(nt - 1, t + D - 1)) - t;
            if (LOADS == 3) {
                if (ahead >= 2) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
                else if (ahead == 1) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            } else {
                if (ahead >= 2) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
                else if (ahead == 1) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            // every wave is done with tile t - 1, so the slot of tile t + D - 4 is free
            if (t + D < nt) fetch(t + D);
            const float acc = F::block_dot(&ring[t & (QV_SLOTS - 1)][r * F::ROW_LDS + wave * F::BLOCK], acts, c);
            if (lane < 16) part[t & (QV_SLOTS - 1)][wave][lane] = acc;
        }
        // the waves' partial sums of this group's tiles are written: lane (tt = lane / 16, ww = lane % 16)
        // takes wave ww's sum of row `wave` in tile tt of the group
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const int t = QV_SLOTS * grp + c;
        float sum = part[c][r][wave];
        sum = sum_row16(sum);
        if (r == 0 && t < t_end) {
            const int row = tile_row0(t) + wave;
            if (row < n) Y[row] = sum;
        }
    }
}

// The same kernel for rows of more than 16 super-blocks (up to 16 NG): a tile is 16 rows x one pass of 16
// columns (the last pass may hold fewer), tile i of a workgroup = (row tile i / NG, pass i % NG), and wave w
// keeps the operands of its column of every pass.  The partial sums of a row tile's passes are added when the
// tile is flushed.  nb = super-blocks a row (contiguous rows of nb blocks); rounds / extra count row tiles.
struct QvColsWork {
    int n, G, rounds, extra, nb;
};

template <class F, int NG>
__global__ __launch_bounds__(1024) void gemv_mfma_cols(const uint8_t *__restrict__ W, const float *__restrict__ X,
                                                       float *__restrict__ Y, QvColsWork wk) {
    static_assert(NG >= 2 && NG <= 4, "two to four passes a row");
    constexpr int D = 2, LOADS = (F::ROW + 1023) / 1024, TG = NG == 3 ? 3 : 4;  // tiles a flush: whole row tiles
    // the raw activations of the passes wait in the wave's own rows of ring slots 3 (behind what prepare()
    // uses), 2 and 1, which no load targets before the wave itself asks for tiles 1, 2 and 3
    static_assert(F::STAGE_BYTES + 1024 <= F::ROW_LDS && 2048 <= F::ROW_LDS, "staging in the ring");
    __shared__ __attribute__((aligned(16))) uint8_t ring[QV_SLOTS][16 * F::ROW_LDS];
    __shared__ float part[TG][16][16];  // [tile of the flush group][wave][row]
    __shared__ float4 side[F::SIDE_LDS ? 16 * NG * 4 : 1];  // [wave][pass][lane group], for the policies that want it
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, c = lane >> 4, b = (int)blockIdx.x;
    const int n = wk.n, G = wk.G, nb = wk.nb;
    const size_t row_bytes = (size_t)nb * F::BLOCK;
    const int nt = NG * (wk.rounds + (b < wk.extra ? 1 : 0));
    if (nt <= 0) return;
    // every fetch is LOADS instructions with at least one lane at work, so that every wave counts the same
    // loads; a short last pass repeats its last 16 bytes into LDS bytes nobody reads
    auto fetch = [&](int slot_i) __attribute__((always_inline)) {
        const int i = min(slot_i, nt - 1), rt = i / NG, cg = i - rt * NG;
        const int row = min(16 * (b + rt * G) + wave, n - 1);
        const int len = min(16, nb - 16 * cg) * F::BLOCK;
        const uint8_t *src = W + (size_t)row * row_bytes + (size_t)cg * F::ROW;
        const uint32_t dst = lds_offset_of(&ring[slot_i & (QV_SLOTS - 1)][wave * F::ROW_LDS]);
#pragma unroll
        for (int j = 0; j < LOADS; j++) {
            const int lanes = max(1, min(64, (min(len, F::ROW) - 1024 * j) / 16));
            if (lane < lanes) async_load16(src + min(1024 * j + 16 * lane, len - 16), dst + 1024 * j);
        }
    };
    uint32_t *stage = (uint32_t *)&ring[3][wave * F::ROW_LDS];
    auto x_raw = [&](int cg) __attribute__((always_inline)) {
        return cg == 0   ? (float *)((uint8_t *)stage + F::STAGE_BYTES)
               : cg == 3 ? (float *)&ring[1][wave * F::ROW_LDS]
                         : (float *)&ring[2][wave * F::ROW_LDS + 1024 * (cg - 1)];
    };
#pragma unroll
    for (int cg = 0; cg < NG; cg++)  // a column past the row's last block reads the last one's and is not used
        async_load16(X + 256 * min(16 * cg + wave, nb - 1) + 4 * lane, lds_offset_of(x_raw(cg)));
    __builtin_amdgcn_s_barrier();
    fetch(0);
    if (LOADS == 3) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
    typename F::Acts acts[NG];
#pragma unroll
    for (int cg = 0; cg < NG; cg++) {
        const float4 v = *(const float4 *)&x_raw(cg)[4 * lane];
        if constexpr (F::SIDE_LDS) acts[cg] = F::prepare(v, stage, lane, &side[(wave * NG + cg) * 4 + c]);
        else acts[cg] = F::prepare(v, stage, lane);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    fetch(1);

    const int n_groups = (nt + TG - 1) / TG;
    for (int grp = 0; grp < n_groups; grp++) {
        const int t0 = TG * grp, t_end = min(nt, t0 + TG);
#pragma unroll
        for (int u = 0; u < TG; u++) {
            const int t = t0 + u;
            if (t >= t_end) break;  // the same for the whole workgroup
            const int ahead = t == nt - 1 ? 0 : max(D - 1, min(nt - 1, t + D - 1)) - t;
            if (LOADS == 3) {
                if (ahead >= 2) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
                else if (ahead == 1) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            } else {
                if (ahead >= 2) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
                else if (ahead == 1) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            }
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (t + D < nt) fetch(t + D);
            const int cg = u % NG;  // t0 is a multiple of NG
            float acc = 0.0f;
            if (16 * cg + wave < nb)
                acc = F::block_dot(&ring[t & (QV_SLOTS - 1)][r * F::ROW_LDS + wave * F::BLOCK], acts[cg], c);
            if (lane < 16) part[u][wave][lane] = acc;
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // lane (tt = lane / 16, ww = lane % 16) takes wave ww's sum of row `wave` in tile tt of the group, the
        // 16 lanes of a tile add up, then the tiles that are passes of one row tile
        float sum = t0 + c < t_end ? part[c < TG ? c : 0][r][wave] : 0.0f;
        sum = sum_row16(sum);
        if (NG == 2) sum = sum_xor16(sum);
        else sum = sum_xor32(sum_xor16(sum));
        if (r == 0 && c % NG == 0 && t0 + c < t_end) {
            const int row = 16 * (b + ((t0 + c) / NG) * G) + wave;
            if (row < n) Y[row] = sum;
        }
    }
}

}  // namespace jq
