// Q4_K GEMV for one activation row over weight rows of 4096 columns with the integer dot products on the
// int8 matrix cores.
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

// Work of workgroup b (of G): tiles b, b + G, b + 2 G, ... of 16 rows each; there are rounds G + extra tiles,
// so the first `extra` workgroups take one more than the others.  (Tiles of 14 rows, which give each of 256
// workgroups four tiles of a 14336-row matrix where tiles of 16 rows leave 32 compute units idle, measured
// 1.5 % slower: 7.49 against 7.39 us.)
struct QvWork {
    int n, G, rounds, extra;
};

// Wave w copies row w of a tile into a ring of four tiles in LDS (three contiguous asynchronous loads, two
// tiles ahead of the arithmetic) and multiplies column w of all 16 rows, so a tile is published by a
// barrier.  The waves' partial sums of up to four tiles wait in LDS and are added, stored and forgotten
// behind one more barrier.
__global__ __launch_bounds__(1024) void q4k_gemv_mfma_lds(const uint8_t *__restrict__ W, const float *__restrict__ X,
                                                          float *__restrict__ Y, QvWork wk) {
    constexpr int D = 2;  // tiles asked for ahead of the one being multiplied (3 measured slower)
    __shared__ __attribute__((aligned(16))) uint8_t ring[QV_SLOTS][QD_TILE_LDS];
    __shared__ float part[QV_SLOTS][16][16];  // [tile % 4][wave][row]
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
        const uint8_t *src = W + (size_t)row * QD_ROW + 16 * lane;
        const uint32_t dst = lds_offset_of(&ring[slot_i & (QV_SLOTS - 1)][wave * QD_ROW_LDS]);
        async_load16(src, dst);
        async_load16(src + 1024, dst + 1024);
        if (lane < 16) async_load16(src + 2048, dst + 2048);
    };
    // staging area of this wave: its own row of ring slot 3, which no load targets before tile 3 is asked
    // for in the main loop; from byte 1152 the wave's 256 raw activations, which travel like the tiles
    // (every global read of this kernel is an asynchronous load counted by hand)
    uint32_t *stage = (uint32_t *)&ring[QV_SLOTS - 1][wave * QD_ROW_LDS];
    float *x_raw = (float *)(stage + 288);
    async_load16(X + 256 * wave + 4 * lane, lds_offset_of(x_raw));
    // every wave's activations are asked for before anybody's tile: the memory pipeline takes a compute
    // unit's requests in the order they were issued, and a wave whose activations queue behind the other
    // waves' tile loads starts its preparation a microsecond late
    __builtin_amdgcn_s_barrier();
    // tile 0 is asked for alone: it has the memory system to itself and lands while the activations are
    // prepared; the next D - 1 tiles follow the preparation
    fetch(0);
    asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
    const float4 v = *(const float4 *)&x_raw[4 * lane];
    const QvActs acts = qv_prepare(v, stage, lane);
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
            if (ahead >= 2) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
            else if (ahead == 1) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            // every wave is done with tile t - 1, so the slot of tile t + D - 4 is free
            if (t + D < nt) fetch(t + D);
            const float acc = qv_block_dot(&ring[t & (QV_SLOTS - 1)][r * QD_ROW_LDS + wave * 144], acts, c);
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

}  // namespace jq
