// Q4_K GEMV for one activation row: integer dot products on the vector ALU (v_dot4_i32_i8),
// weights streamed once from HBM straight into registers, nothing but a 16-float reduction per
// row tile in LDS.
//
// Per 32-element sub-block j of a weight row (reference arithmetic w = d sc q - dmin m,
// src/kquant_dot.rs:440-465):
//
//   sum_k x_k w_k = (d sc_j) s_j S_j - (dmin m_j) s_j XS_j,   S_j = sum_k q_k X_k,  XS_j = sum_k X_k
//
// with X = round(x / s_j), s_j = amax_j(x) / 32639, the activation in 16-bit fixed point PER
// SUB-BLOCK, split into two balanced byte planes X = 256 Xh + Xl.  S_j = 256 Sh + Sl with Sh, Sl
// exact int32 sums of four-element dot products, so the integer dot product of a sub-block is
// bit-exact; rounding the activation to 2^-16 of its own sub-block's maximum is far below the f32
// accumulation noise of the reference and inside the 1e-3 bound on the results.
//
// Work split: a workgroup has one wave per 256-element super-block column of the weight matrix
// (at most 16); lane (r = lane % 16, c = lane / 16) owns row r of the current 16-row tile and the
// 64-element chunk c of the wave's block: 32 bytes whose low nibbles are sub-block 2c and whose high
// nibbles are sub-block 2c+1, so a lane never shares a scale with another.  The activation planes of
// that chunk (32 registers) are prepared once per workgroup and stay in registers; per tile a lane
// loads its row's 16-byte block header and its 32 nibble bytes (the wave's loads cover the tile's
// 16 x 144 bytes exactly once), two tiles ahead of use.  Each workgroup walks an equal share of the rows.
#pragma once
#include "kernels_valu.hpp"

namespace jq {

constexpr int QD_MAX_WAVES = 16;
constexpr float QD_RANGE = 32639.0f;  // 127 * 256 + 127

// A lane's four activations (elements 4i .. 4i+3 of a 32-element sub-block held by 8 lanes) as 16-bit fixed
// point against the sub-block's maximum, in as few vector instructions as the arithmetic allows: every
// workgroup repeats this for the whole activation row in front of its first product, four waves a SIMD, so
// an instruction here costs sixteen cycles of the launch's start.  (The one-row kernels of every format use it.)
//   * the maximum is taken over the magnitudes' bit patterns as unsigned integers: NaN > inf > finite, so a
//     non-finite element needs no test of its own;
//   * the scale amax / 32639 by a multiplication with one correction step, which is exact whenever the
//     quotient is a float; its inverse by the hardware reciprocal (a relative error of 2^-22 moves X by less
//     than 0.02, so an activation that is an integer multiple of the scale still quantises to that integer);
//   * X = round(x inv) as the mantissa of fma(x, inv, 1.5 * 2^23 + 128): bits 0..15 of the result are X + 128,
//     byte 1 the high plane, byte 0 the low plane with its top bit flipped; four v_perm_b32 gather the planes.
// Returns the plane words of X (wl, wh) and of -X (nl, nh), the scale (NaN for a sub-block with a non-finite
// element, 0 for one of zeros) and the sum of the sub-block's X in every lane of the sub-block.
struct QvQuant {
    uint32_t wl, wh, nl, nh;
    float s;
    int sum;   // of the sub-block's 32 values
    int sum4;  // of the lane's own four
};
__device__ __forceinline__ QvQuant qv_quantise4(const float4 v) {
    const uint32_t b0 = __builtin_bit_cast(uint32_t, v.x) & 0x7FFFFFFFu, b1 = __builtin_bit_cast(uint32_t, v.y) & 0x7FFFFFFFu;
    const uint32_t b2 = __builtin_bit_cast(uint32_t, v.z) & 0x7FFFFFFFu, b3 = __builtin_bit_cast(uint32_t, v.w) & 0x7FFFFFFFu;
    uint32_t m = max(max(b0, b1), max(b2, b3));
    m = max(m, (uint32_t)dpp_i<0x141>((int)m));
    m = max(m, (uint32_t)dpp_i<0xB1>((int)m));
    m = max(m, (uint32_t)dpp_i<0x4E>((int)m));
    const float amax = __builtin_bit_cast(float, m);
    constexpr float RC = 1.0f / QD_RANGE;
    float s = amax * RC;
    s = fmaf(fmaf(-s, QD_RANGE, amax), RC, s);
    const float inv = __builtin_amdgcn_rcpf(fmaxf(s, 1e-35f));  // of the scale: a normal number for every finite amax
    s = m >= 0x7F800000u ? NAN : s;
    constexpr float MAGIC = 12582912.0f + 128.0f;
    const float ninv = -inv;
    const uint32_t t0 = __builtin_bit_cast(uint32_t, fmaf(v.x, inv, MAGIC)), t1 = __builtin_bit_cast(uint32_t, fmaf(v.y, inv, MAGIC));
    const uint32_t t2 = __builtin_bit_cast(uint32_t, fmaf(v.z, inv, MAGIC)), t3 = __builtin_bit_cast(uint32_t, fmaf(v.w, inv, MAGIC));
    const uint32_t u0 = __builtin_bit_cast(uint32_t, fmaf(v.x, ninv, MAGIC)), u1 = __builtin_bit_cast(uint32_t, fmaf(v.y, ninv, MAGIC));
    const uint32_t u2 = __builtin_bit_cast(uint32_t, fmaf(v.z, ninv, MAGIC)), u3 = __builtin_bit_cast(uint32_t, fmaf(v.w, ninv, MAGIC));
    // v_perm_b32(a, b, sel): selector 0..3 takes byte 0..3 of b, 4..7 of a
    const uint32_t p01 = __builtin_amdgcn_perm(t1, t0, 0x05010400u), p23 = __builtin_amdgcn_perm(t3, t2, 0x05010400u);
    const uint32_t n01 = __builtin_amdgcn_perm(u1, u0, 0x05010400u), n23 = __builtin_amdgcn_perm(u3, u2, 0x05010400u);
    QvQuant q;
    q.wl = __builtin_amdgcn_perm(p23, p01, 0x05040100u) ^ 0x80808080u, q.wh = __builtin_amdgcn_perm(p23, p01, 0x07060302u);
    q.nl = __builtin_amdgcn_perm(n23, n01, 0x05040100u) ^ 0x80808080u, q.nh = __builtin_amdgcn_perm(n23, n01, 0x07060302u);
    q.s = s;
    constexpr uint32_t BASE4 = 4u * 0x4B400080u;  // four times the bit pattern of MAGIC, modulo 2^32
    q.sum4 = (int)(t0 + t1 + t2 + t3 - BASE4);
    q.sum = isum_row8(q.sum4);
    return q;
}


struct QdTile {  // what a lane holds of one 16-row tile
    uint4 hdr, qa, qb;
};

__global__ __launch_bounds__(64 * QD_MAX_WAVES) void q4k_gemv_dot4(const uint8_t *__restrict__ W, size_t row_bytes,
                                                                    const float *__restrict__ X,
                                                                    float *__restrict__ Y, int k, int n) {
    __shared__ uint32_t xl_lds[QD_MAX_WAVES][64], xh_lds[QD_MAX_WAVES][64];  // byte planes, 4 elements a word
    __shared__ float s_lds[QD_MAX_WAVES][8], xs_lds[QD_MAX_WAVES][8];        // per sub-block: scale, s * XS
    __shared__ float red[2][QD_MAX_WAVES][16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
    const int r = lane & 15, c = lane >> 4;
    // this workgroup's share of the rows: an equal, contiguous range (not a whole number of tiles,
    // so that every workgroup streams the same number of bytes); its last tile may be partial
    const int G = (int)gridDim.x;
    const int row_beg = (int)((long long)blockIdx.x * n / G), row_end = (int)((long long)(blockIdx.x + 1) * n / G);
    const int n_tiles = (row_end - row_beg + 15) >> 4;
    if (n_tiles == 0) return;

    // loads are unconditional (tile and row indices are clamped into the range) so that every step
    // issues the same number of loads and the compiler can wait for exactly the ones it needs
    auto load_tile = [&](int i, QdTile &q) __attribute__((always_inline)) {
        const int row = min(row_beg + 16 * min(i, n_tiles - 1) + r, row_end - 1);
        const uint8_t *blk = W + (size_t)row * row_bytes + (size_t)wave * 144;
        q.hdr = *(const uint4 *)blk;
        q.qa = *(const uint4 *)(blk + 16 + 32 * c);
        q.qb = *(const uint4 *)(blk + 32 + 32 * c);
    };

    // a ring of three register sets: tile i of this workgroup lives in set i % 3 and is loaded two
    // steps before its use; the first two are on their way while the activation is prepared
    QdTile ring0, ring1, ring2;
    int t = 0;
    load_tile(0, ring0);
    load_tile(1, ring1);

    // ---- activation of this wave's super-block: lane i quantises elements 4i .. 4i+3 ----
    {
        const float4 v = *(const float4 *)(X + 256 * wave + 4 * lane);
        float amax = fmaxf(fmaxf(mag_or_inf(v.x), mag_or_inf(v.y)), fmaxf(mag_or_inf(v.z), mag_or_inf(v.w)));
        amax = max_row8(amax);  // the 8 lanes of a sub-block
        const bool live = amax > 0.0f && amax < INFINITY;
        const float inv = live ? QD_RANGE / amax : 0.0f, s = fixed_scale(amax, QD_RANGE);
        const int Xq[4] = {__float2int_rn(v.x * inv), __float2int_rn(v.y * inv), __float2int_rn(v.z * inv),
                           __float2int_rn(v.w * inv)};
        uint32_t wl = 0, wh = 0;
        int sum = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int lo = ((Xq[i] + 128) & 255) - 128, hi = (Xq[i] - lo) >> 8;
            wl |= (uint32_t)(lo & 255) << (8 * i);
            wh |= (uint32_t)(hi & 255) << (8 * i);
            sum += Xq[i];
        }
        xl_lds[wave][lane] = wl;
        xh_lds[wave][lane] = wh;
        sum = isum_row8(sum);
        if ((lane & 7) == 0) {
            s_lds[wave][lane >> 3] = s;
            xs_lds[wave][lane >> 3] = s * (float)sum;
        }
    }
    __syncthreads();
    // chunk c: elements 64c .. 64c+31 ride on the low nibbles, 64c+32 .. 64c+63 on the high nibbles
    uint32_t xl_lo[8], xh_lo[8], xl_hi[8], xh_hi[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        xl_lo[i] = xl_lds[wave][16 * c + i], xh_lo[i] = xh_lds[wave][16 * c + i];
        xl_hi[i] = xl_lds[wave][16 * c + 8 + i], xh_hi[i] = xh_lds[wave][16 * c + 8 + i];
    }
    const float s_lo = s_lds[wave][2 * c], s_hi = s_lds[wave][2 * c + 1];
    const float xs_lo = xs_lds[wave][2 * c], xs_hi = xs_lds[wave][2 * c + 1];

    auto step = [&](QdTile &cur, QdTile &fill) __attribute__((always_inline)) {
        load_tile(t + 2, fill);

        uint32_t scp, mnp;
        q4k_scale_min_pair(cur.hdr.y, cur.hdr.z, cur.hdr.w, c, scp, mnp);
        const uint32_t sc_lo = scp & 0xFFu, sc_hi = (scp >> 8) & 0xFFu, mn_lo = mnp & 0xFFu, mn_hi = (mnp >> 8) & 0xFFu;
        const uint32_t q[8] = {cur.qa.x, cur.qa.y, cur.qa.z, cur.qa.w, cur.qb.x, cur.qb.y, cur.qb.z, cur.qb.w};
        int sl_lo = 0, sh_lo = 0, sl_hi = 0, sh_hi = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int lo4 = (int)(q[i] & 0x0F0F0F0Fu), hi4 = (int)((q[i] >> 4) & 0x0F0F0F0Fu);
            sl_lo = __builtin_amdgcn_sdot4(lo4, (int)xl_lo[i], sl_lo, false);
            sh_lo = __builtin_amdgcn_sdot4(lo4, (int)xh_lo[i], sh_lo, false);
            sl_hi = __builtin_amdgcn_sdot4(hi4, (int)xl_hi[i], sl_hi, false);
            sh_hi = __builtin_amdgcn_sdot4(hi4, (int)xh_hi[i], sh_hi, false);
        }
        const float d = f16_bits(cur.hdr.x), dmin = f16_bits(cur.hdr.x >> 16);
        const float f_lo = (float)((sh_lo << 8) + sl_lo) * s_lo, f_hi = (float)((sh_hi << 8) + sl_hi) * s_hi;
        float acc = d * fmaf((float)sc_lo, f_lo, (float)sc_hi * f_hi);
        acc = fmaf(-dmin, fmaf((float)mn_lo, xs_lo, (float)mn_hi * xs_hi), acc);
        acc = sum_xor16(acc);
        acc = sum_xor32(acc);  // the four chunks of the block

        // the waves' partial sums of the 16 rows meet in LDS; wave w then sums rows w, w + waves, ...
        // over the waves (16 lanes, one partial each, a fixed tree), so no wave carries the whole reduction
        const int buf = t & 1;
        if (lane < 16) red[buf][wave][lane] = acc;
        __syncthreads();
        for (int rr = wave; rr < 16; rr += waves) {
            float v = (lane < waves) ? red[buf][lane & 15][rr] : 0.0f;
            v = sum_row16(v);
            const int row = row_beg + 16 * t + rr;
            if (lane == 0 && row < row_end) Y[row] = v;
        }
        t++;
    };
    while (t < n_tiles) {
        step(ring0, ring2);
        if (t >= n_tiles) break;
        step(ring1, ring0);
        if (t >= n_tiles) break;
        step(ring2, ring1);
    }
}

// The same GEMV with the weights travelling HBM -> LDS as asynchronous, fully coalesced loads: wave w
// copies row w of every 16-row tile (its whole packed row: three instructions of up to 1 KB) into a
// ring of three tiles in LDS, two tiles ahead of the arithmetic; the lanes then read their header and
// 32 nibble bytes from LDS.  Rows are padded by 16 bytes in LDS so that the 16 rows a wave reads in one
// instruction fall into different banks.  No vector register is spent on prefetching, and every global
// access is a contiguous kilobyte.  Needs exactly 16 super-blocks a row (one wave per row of a tile).
constexpr int QD_ROW = 16 * 144, QD_ROW_LDS = QD_ROW + 16, QD_TILE_LDS = 16 * QD_ROW_LDS;

// NORM puts a residual add and an RMSNorm in front of the product (a decoder layer's
// x += res; hn = x / sqrt(mean(x^2) + eps) * w; y = W hn as one launch): every workgroup normalises
// the 4096-wide row for itself, workgroup 0 also stores x + res (into a buffer other than X: the
// others are still reading X) and, when asked, the normalised row.
struct QdNorm {
    const float *res;  // added to X first (null: nothing to add)
    const float *w;    // norm weight
    float eps;
    float *x_out;      // X + res
    float *hn_out;     // the normalised row (null: not wanted)
};

// SWIGLU: the matrix holds the rows of a gate and an up projection alternately (row 2j gate_j, row
// 2j + 1 up_j) and the result is Y[j] = silu(gate_j . x) * (up_j . x), n / 2 values
// (reference: src/quantized_qwen3_moe.rs:397-401).
template <bool NORM, bool SWIGLU>
__global__ __launch_bounds__(1024) void q4k_gemv_dot4_lds(const uint8_t *__restrict__ W, const float *__restrict__ X,
                                                          float *__restrict__ Y, int n, int G, const float *nm_res,
                                                          const float *nm_w, float nm_eps, float *nm_x_out,
                                                          float *nm_hn_out) {
    // the norm's operands are arguments of their own, not a struct: scalars and pointers at the head of
    // the argument list arrive preloaded in registers, a struct is fetched by a scalar load first
    const QdNorm nm{nm_res, nm_w, nm_eps, nm_x_out, nm_hn_out};
    __shared__ __attribute__((aligned(16))) uint8_t ring[3][QD_TILE_LDS];
    __shared__ float ss_lds[16];
    __shared__ uint32_t xl_lds[16][64], xh_lds[16][64];
    __shared__ float s_lds[16][8], xs_lds[16][8];
    __shared__ float red[2][16][16];
    __shared__ __attribute__((aligned(16))) float x_raw[16][256];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, c = lane >> 4;
    // tiles blockIdx.x, blockIdx.x + G, ...: at any moment the chip reads one contiguous stretch of the
    // matrix (measured 5.4 TB/s against 5.1 TB/s for one contiguous range per workgroup).  G, the number of
    // workgroups, is an argument: with the leading arguments preloaded into scalar registers the first
    // loads go out 0.4 us after the wave starts, where gridDim.x costs a scalar load from memory first.
    const int n_tiles = (((n + 15) >> 4) - (int)blockIdx.x + G - 1) / G;
    if (n_tiles <= 0) return;

    // 3 asynchronous loads per wave and tile: row `wave` of tile i (clamped into the range) -> ring slot
    auto fetch = [&](int i, int slot) __attribute__((always_inline)) {
        const int row = min(16 * ((int)blockIdx.x + min(i, n_tiles - 1) * G) + wave, n - 1);
        const uint8_t *src = W + (size_t)row * QD_ROW + 16 * lane;
        const uint32_t dst = lds_offset_of(&ring[slot][wave * QD_ROW_LDS]);
        async_load16(src, dst);
        async_load16(src + 1024, dst + 1024);
        if (lane < 16) async_load16(src + 2048, dst + 2048);
    };
    // the activation column of this wave travels the same way, first (every global read of this kernel
    // is an asynchronous load, counted by hand)
    async_load16(X + 256 * wave + 4 * lane, lds_offset_of(&x_raw[wave][0]));
    // norm weight and residual columns wait in the third ring slot, which no tile enters before the main loop
    float *w_raw = (float *)&ring[2][0] + 256 * wave, *r_raw = (float *)&ring[2][16384] + 256 * wave;
    if (NORM) {
        async_load16(nm.w + 256 * wave + 4 * lane, lds_offset_of(w_raw));
        if (nm.res) async_load16(nm.res + 256 * wave + 4 * lane, lds_offset_of(r_raw));
    }
    fetch(0, 0);
    // Tile 1 is asked for only after the activation has been prepared: every workgroup's tile 0 then has
    // the memory system to itself and lands sooner, and the arithmetic, which is what the kernel waits
    // for in the end, starts sooner.  A workgroup with one tile (4096 rows over 256 workgroups) fetches
    // nothing more.
    const bool two = n_tiles > 1;
    asm volatile("s_waitcnt vmcnt(3)" ::: "memory");  // the activation landed (own wave's data: no barrier needed)

    // With NORM the row that is multiplied is (x + res) g / rms: the 1 / rms is a factor of the whole row, so
    // the activation is quantised as (x + res) g and the sub-block scales take the factor afterwards, once
    // the waves' sums of squares have met at the barrier that publishes tile 0 anyway (a barrier of its own
    // in front of the quantisation cost 0.9 us a launch).
    float4 v;
    {
        v = *(const float4 *)&x_raw[wave][4 * lane];
        if (NORM) {
            if (nm.res) {
                const float4 r = *(const float4 *)&r_raw[4 * lane];
                v.x += r.x, v.y += r.y, v.z += r.z, v.w += r.w;
            }
            float ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, v.w * v.w)));
            ss = wave_sum(ss);
            if (lane == 0) ss_lds[wave] = ss;
            const float4 g = *(const float4 *)&w_raw[4 * lane];
            if (blockIdx.x == 0) *(float4 *)(nm.x_out + 256 * wave + 4 * lane) = v;
            v = float4{v.x * g.x, v.y * g.y, v.z * g.z, v.w * g.w};
        }
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
            const int lo = ((Xq[i] + 128) & 255) - 128, hi = (Xq[i] - lo) >> 8;
            wl |= (uint32_t)(lo & 255) << (8 * i);
            wh |= (uint32_t)(hi & 255) << (8 * i);
            sum += Xq[i];
        }
        xl_lds[wave][lane] = wl;
        xh_lds[wave][lane] = wh;
        sum = isum_row8(sum);
        if ((lane & 7) == 0) {
            s_lds[wave][lane >> 3] = s;
            xs_lds[wave][lane >> 3] = s * (float)sum;
        }
    }
    // tile 0 landed (tile 1 may be in flight), planes written
    if (two) {
        fetch(1, 1);
        asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory");
    } else {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    uint32_t xl_lo[8], xh_lo[8], xl_hi[8], xh_hi[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        xl_lo[i] = xl_lds[wave][16 * c + i], xh_lo[i] = xh_lds[wave][16 * c + i];
        xl_hi[i] = xl_lds[wave][16 * c + 8 + i], xh_hi[i] = xh_lds[wave][16 * c + 8 + i];
    }
    float s_lo = s_lds[wave][2 * c], s_hi = s_lds[wave][2 * c + 1];
    float xs_lo = xs_lds[wave][2 * c], xs_hi = xs_lds[wave][2 * c + 1];
    if (NORM) {
        float tot = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) tot += ss_lds[i];
        const float inv = 1.0f / sqrtf(tot / 4096.0f + nm.eps);
        s_lo *= inv, s_hi *= inv, xs_lo *= inv, xs_hi *= inv;
        if (blockIdx.x == 0 && nm.hn_out)
            *(float4 *)(nm.hn_out + 256 * wave + 4 * lane) = float4{v.x * inv, v.y * inv, v.z * inv, v.w * inv};
    }

    // on entry to step t: tile t is in LDS and visible (the barrier just passed), tile t+1 in flight
    for (int t = 0; t < n_tiles; t++) {
        const int slot = t % 3;
        const bool more = t + 2 < n_tiles;
        if (more) fetch(t + 2, (t + 2) % 3);  // the slot of tile t-1, which every wave finished reading before that barrier

        const uint8_t *blk = &ring[slot][r * QD_ROW_LDS + wave * 144];
        const uint4 hdr = *(const uint4 *)blk;
        const uint4 qa = *(const uint4 *)(blk + 16 + 32 * c), qb = *(const uint4 *)(blk + 32 + 32 * c);
        uint32_t scp, mnp;
        q4k_scale_min_pair(hdr.y, hdr.z, hdr.w, c, scp, mnp);
        const uint32_t sc_lo = scp & 0xFFu, sc_hi = (scp >> 8) & 0xFFu, mn_lo = mnp & 0xFFu, mn_hi = (mnp >> 8) & 0xFFu;
        const uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        int sl_lo = 0, sh_lo = 0, sl_hi = 0, sh_hi = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int lo4 = (int)(q[i] & 0x0F0F0F0Fu), hi4 = (int)((q[i] >> 4) & 0x0F0F0F0Fu);
            sl_lo = __builtin_amdgcn_sdot4(lo4, (int)xl_lo[i], sl_lo, false);
            sh_lo = __builtin_amdgcn_sdot4(lo4, (int)xh_lo[i], sh_lo, false);
            sl_hi = __builtin_amdgcn_sdot4(hi4, (int)xl_hi[i], sl_hi, false);
            sh_hi = __builtin_amdgcn_sdot4(hi4, (int)xh_hi[i], sh_hi, false);
        }
        const float d = f16_bits(hdr.x), dmin = f16_bits(hdr.x >> 16);
        const float f_lo = (float)((sh_lo << 8) + sl_lo) * s_lo, f_hi = (float)((sh_hi << 8) + sl_hi) * s_hi;
        float acc = d * fmaf((float)sc_lo, f_lo, (float)sc_hi * f_hi);
        acc = fmaf(-dmin, fmaf((float)mn_lo, xs_lo, (float)mn_hi * xs_hi), acc);
        acc = sum_xor16(acc);
        acc = sum_xor32(acc);

        const int buf = t & 1;
        if (lane < 16) red[buf][wave][lane] = acc;
        // the partial sums are written and tile t+1 has landed: at most this step's 3 loads stay in flight
        if (more) asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (!SWIGLU) {  // wave w sums row w of the tile over the 16 waves
            float v = (lane < 16) ? red[buf][lane][wave] : 0.0f;
            v = sum_row16(v);
            const int row = 16 * ((int)blockIdx.x + t * G) + wave;
            if (lane == 0 && row < n) Y[row] = v;
        } else if (wave < 8) {  // wave w sums rows 2w (lanes 0..15) and 2w + 1 (lanes 16..31): a gate / up pair
            float v = (lane < 32) ? red[buf][lane & 15][2 * wave + (lane >> 4)] : 0.0f;
            v = sum_row16(v);
            const float up = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
            const int row = 16 * ((int)blockIdx.x + t * G) + 2 * wave;
            if (lane == 0 && row + 1 < n) Y[row >> 1] = silu(v) * up;
        }
    }
}

}  // namespace jq
