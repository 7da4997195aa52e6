// Q4_K times one activation row on v_dot4 for rows of 16 * NG super-blocks (k = 4096 NG), in steps of
// 8 weight rows x 16 super-blocks.
//
// The road of q4k_gemv_dot4_lds with a finer grain: the 16 waves of a workgroup copy the 8 row slices
// of a step (2304 B each, half a slice a wave, two instructions) into a ring of four steps in LDS,
// three steps ahead of the arithmetic; wave w then works on super-block w of the slice, 8 lanes a
// row: lane (row r = lane % 8, sub-block j = lane / 8) multiplies the 32 four-bit values of its
// sub-block (the low or the high nibbles of 32 bytes, shifted into place by a per-lane amount) with
// v_dot4_i32_i8 against the activations, which every wave keeps in registers as 15-bit fixed point
// per 32-element block (two int8 planes, X = 256 hi + lo; 16 registers a column group).  The integer
// sum of a sub-block is exact.  Result per row: sum over sub-blocks of d sc s_x S - dmin m s_x XS, over
// the NG steps of a row tile (in a register), the 8 lanes of a row and the 16 waves (through LDS).
#pragma once
#include "kernels_dot4_q4k.hpp"

namespace jq {

constexpr int QR8_ROWS = 8, QR8_ROW_LDS = QD_ROW + 16, QR8_STEP_LDS = QR8_ROWS * QR8_ROW_LDS, QR8_RING = 4;

template <int NG>
__global__ __launch_bounds__(1024) void q4k_gemv_dot4_r8(const uint8_t *__restrict__ W, const float *__restrict__ X,
                                                         float *__restrict__ Y, int n, int G) {
    __shared__ __attribute__((aligned(16))) uint8_t ring[QR8_RING][QR8_STEP_LDS];
    __shared__ __attribute__((aligned(16))) float x_raw[NG][16][256];
    __shared__ uint32_t xl_lds[NG][16][64], xh_lds[NG][16][64];
    __shared__ float s_lds[NG][16][8], xs_lds[NG][16][8];
    __shared__ float red[2][16][QR8_ROWS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 7, j = lane >> 3, c = j >> 1;  // row of the step, sub-block of the super-block, its 64-element chunk
    const int n_tiles = (((n + QR8_ROWS - 1) / QR8_ROWS) - (int)blockIdx.x + G - 1) / G;  // row tiles blockIdx.x, + G, ...
    if (n_tiles <= 0) return;
    const int n_steps = NG * n_tiles;
    constexpr size_t row_bytes = (size_t)NG * QD_ROW;

    // step i = (row tile i / NG, column group i % NG); 2 asynchronous loads per wave: half a row slice (72 pieces of 16 bytes)
    auto fetch = [&](int i) __attribute__((always_inline)) {
        const int row = min(QR8_ROWS * ((int)blockIdx.x + (i / NG) * G) + (wave >> 1), n - 1);
        const uint8_t *src = W + (size_t)row * row_bytes + (size_t)(i % NG) * QD_ROW + (wave & 1) * 1152 + 16 * lane;
        const uint32_t dst = lds_offset_of(&ring[i % QR8_RING][(wave >> 1) * QR8_ROW_LDS + (wave & 1) * 1152]);
        async_load16(src, dst);
        if (lane < 8) async_load16(src + 1024, dst + 1024);
    };
    // every global read of this kernel is an asynchronous load counted by hand: the activation columns
    // first, then step 0; steps 1 and 2 are asked for once the activations are prepared
#pragma unroll
    for (int g = 0; g < NG; g++)
        async_load16(X + (size_t)(16 * g + wave) * 256 + 4 * lane, lds_offset_of(&x_raw[g][wave][0]));
    fetch(0);
    asm volatile("s_waitcnt vmcnt(2)" ::: "memory");  // the activations landed (own wave's data: no barrier needed)

    // activations of super-block 16 g + wave: 4 elements a lane, one scale per 32
#pragma unroll
    for (int g = 0; g < NG; g++) {
        const float4 v = *(const float4 *)&x_raw[g][wave][4 * lane];
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
        xl_lds[g][wave][lane] = wl;
        xh_lds[g][wave][lane] = wh;
        sum = isum_row8(sum);
        if ((lane & 7) == 0) {
            s_lds[g][wave][lane >> 3] = s;
            xs_lds[g][wave][lane >> 3] = s * (float)sum;
        }
    }
    // step 0 landed (steps 1 and 2 may be in flight), planes written
    if (n_steps > 2) {
        fetch(1);
        fetch(2);
        asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory");
    } else if (n_steps > 1) {
        fetch(1);
        asm volatile("s_waitcnt vmcnt(2) lgkmcnt(0)" ::: "memory");
    } else {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    uint32_t xl[NG][8], xh[NG][8];
    float sx[NG], xs[NG];
#pragma unroll
    for (int g = 0; g < NG; g++) {
#pragma unroll
        for (int i = 0; i < 8; i++) xl[g][i] = xl_lds[g][wave][8 * j + i], xh[g][i] = xh_lds[g][wave][8 * j + i];
        sx[g] = s_lds[g][wave][j], xs[g] = xs_lds[g][wave][j];
    }
    const int nib_shift = 4 * (j & 1), byte_shift = 8 * (j & 3);

    // on entry to step st: step st is in LDS and visible (the barrier just passed), steps st+1, st+2 in flight
    float acc = 0.0f;
    for (int i = 0, tile = 0; i < n_steps; i += NG, tile++) {
#pragma unroll
        for (int g = 0; g < NG; g++) {
            const int st = i + g;
            if (st + 3 < n_steps) fetch(st + 3);  // the slot of step st-1, which every wave finished reading before that barrier

            const uint8_t *blk = &ring[st % QR8_RING][r * QR8_ROW_LDS + wave * 144];
            const uint4 hdr = *(const uint4 *)blk;
            const uint4 qa = *(const uint4 *)(blk + 16 + 32 * c), qb = *(const uint4 *)(blk + 32 + 32 * c);
            // 6-bit (scale, min) pair j without a branch (reference: src/kquant_dot.rs:108-118)
            const uint32_t a = hdr.y >> byte_shift, b = hdr.z >> byte_shift, h = hdr.w >> byte_shift;
            const uint32_t sc_a = a & 63u, mn_a = b & 63u;
            const uint32_t sc_b = (h & 0xFu) | ((a >> 2) & 0x30u), mn_b = ((h >> 4) & 0xFu) | ((b >> 2) & 0x30u);
            const uint32_t sc = j < 4 ? sc_a : sc_b, mn = j < 4 ? mn_a : mn_b;
            const uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
            int sl = 0, sh = 0;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int v = (int)((q[e] >> nib_shift) & 0x0F0F0F0Fu);
                sl = __builtin_amdgcn_sdot4(v, (int)xl[g][e], sl, false);
                sh = __builtin_amdgcn_sdot4(v, (int)xh[g][e], sh, false);
            }
            const float d = f16_bits(hdr.x), dmin = f16_bits(hdr.x >> 16);
            acc = fmaf(d * (float)sc, (float)((sh << 8) + sl) * sx[g], acc);
            acc = fmaf(-dmin * (float)mn, xs[g], acc);

            const int buf = tile & 1;
            if (g == NG - 1) {  // the row tile is complete: the 8 lanes of a row, then the waves through LDS
                acc += dpp_f<0x128>(acc);  // row_ror:8: lane ^ 8
                acc = sum_xor16(acc);
                acc = sum_xor32(acc);
                if (lane < QR8_ROWS) red[buf][wave][lane] = acc;
                acc = 0.0f;
            }
            // step st+1 has landed (and the partial sums are written): the loads of steps st+2, st+3 may stay in flight
            const int ahead = min(st + 3, n_steps - 1) - (st + 1);
            if (ahead >= 2) asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory");
            else if (ahead == 1) asm volatile("s_waitcnt vmcnt(2) lgkmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (g == NG - 1 && wave < QR8_ROWS) {  // wave w sums row w of the tile over the 16 waves
                float v = (lane < 16) ? red[buf][lane][wave] : 0.0f;
                v = sum_row16(v);
                const int row = QR8_ROWS * ((int)blockIdx.x + tile * G) + wave;
                if (lane == 0 && row < n) Y[row] = v;
            }
        }
    }
}

// The same rows (k = 4096 NG) on the 16-row tiles of q4k_gemv_dot4_lds: a step is 16 weight rows x one
// column group of 16 super-blocks, wave w owns super-block w of the group, lane (row, 64-element chunk)
// as there; the partial sum of a row tile rides in a register over its NG steps.  The activation planes
// of all groups wait in LDS and a lane reloads its 32 plane registers for the group of each step (they
// do not fit in registers for three groups); they take the place of the raw activation columns in LDS.
// 4096 x 12288: 8.8 us against 9.1 us for the 8-row steps above (4096 x 8192: 6.4 against 6.8 us), when
// the row count gives every compute unit one tile; with fewer tiles, or a ragged number of them per
// workgroup, the 8-row steps are ahead (2048 x 12288: 6.9 against 7.5 us).
template <int NG>
__global__ __launch_bounds__(1024) void q4k_gemv_dot4_cols(const uint8_t *__restrict__ W, const float *__restrict__ X,
                                                           float *__restrict__ Y, int n, int G) {
    static_assert(NG == 2 || NG == 3, "two or three column groups");
    __shared__ __attribute__((aligned(16))) uint8_t ring[3][QD_TILE_LDS];
    // a wave's 256 raw activations of a group (1 KB), overwritten by the wave with what it makes of them:
    // words 0..63 low plane, 64..127 high plane, 128..135 scales, 136..143 scale * sum of the sub-blocks
    __shared__ __attribute__((aligned(16))) uint32_t xbuf[NG][16][256];
    __shared__ float red[2][16][16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, c = lane >> 4;
    const int n_tiles = (((n + 15) >> 4) - (int)blockIdx.x + G - 1) / G;  // row tiles blockIdx.x, + G, ...
    if (n_tiles <= 0) return;
    const int n_steps = NG * n_tiles;
    constexpr size_t row_bytes = (size_t)NG * QD_ROW;

    // step i = (row tile i / NG, column group i % NG); 3 asynchronous loads per wave: row `wave` of the step
    auto fetch = [&](int i) __attribute__((always_inline)) {
        const int row = min(16 * ((int)blockIdx.x + (i / NG) * G) + wave, n - 1);
        const uint8_t *src = W + (size_t)row * row_bytes + (size_t)(i % NG) * QD_ROW + 16 * lane;
        const uint32_t dst = lds_offset_of(&ring[i % 3][wave * QD_ROW_LDS]);
        async_load16(src, dst);
        async_load16(src + 1024, dst + 1024);
        if (lane < 16) async_load16(src + 2048, dst + 2048);
    };
#pragma unroll
    for (int g = 0; g < NG; g++) async_load16(X + (size_t)(16 * g + wave) * 256 + 4 * lane, lds_offset_of(&xbuf[g][wave][0]));
    fetch(0);
    asm volatile("s_waitcnt vmcnt(3)" ::: "memory");  // the activations landed (own wave's data: no barrier needed)
    float4 raw[NG];
#pragma unroll
    for (int g = 0; g < NG; g++) raw[g] = *(const float4 *)&xbuf[g][wave][4 * lane];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // every lane holds its raw values: the planes may take their place
#pragma unroll
    for (int g = 0; g < NG; g++) {
        const float4 v = raw[g];
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
        xbuf[g][wave][lane] = wl;
        xbuf[g][wave][64 + lane] = wh;
        sum = isum_row8(sum);
        if ((lane & 7) == 0) {
            xbuf[g][wave][128 + (lane >> 3)] = __float_as_uint(s);
            xbuf[g][wave][136 + (lane >> 3)] = __float_as_uint(s * (float)sum);
        }
    }
    // step 0 landed (steps 1 and 2 may be in flight), planes written; n_steps >= 2
    fetch(1);
    if (n_steps > 2) {
        fetch(2);
        asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)" ::: "memory");
    } else {
        asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory");
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    // on entry to step st: step st is in LDS and visible (the barrier just passed), step st+1 in flight
    float acc = 0.0f;
    for (int i = 0, tile = 0; i < n_steps; i += NG, tile++) {
#pragma unroll
        for (int g = 0; g < NG; g++) {
            const int st = i + g;
            const bool more = st + 2 < n_steps;
            if (more && st > 0) fetch(st + 2);  // the slot of step st-1, which every wave finished reading before that barrier

            uint32_t xl_lo[8], xh_lo[8], xl_hi[8], xh_hi[8];
#pragma unroll
            for (int e = 0; e < 8; e += 4) {
                const uint4 a = *(const uint4 *)&xbuf[g][wave][16 * c + e], b = *(const uint4 *)&xbuf[g][wave][64 + 16 * c + e];
                const uint4 a2 = *(const uint4 *)&xbuf[g][wave][16 * c + 8 + e], b2 = *(const uint4 *)&xbuf[g][wave][64 + 16 * c + 8 + e];
                xl_lo[e] = a.x, xl_lo[e + 1] = a.y, xl_lo[e + 2] = a.z, xl_lo[e + 3] = a.w;
                xh_lo[e] = b.x, xh_lo[e + 1] = b.y, xh_lo[e + 2] = b.z, xh_lo[e + 3] = b.w;
                xl_hi[e] = a2.x, xl_hi[e + 1] = a2.y, xl_hi[e + 2] = a2.z, xl_hi[e + 3] = a2.w;
                xh_hi[e] = b2.x, xh_hi[e + 1] = b2.y, xh_hi[e + 2] = b2.z, xh_hi[e + 3] = b2.w;
            }
            const float s_lo = __uint_as_float(xbuf[g][wave][128 + 2 * c]), s_hi = __uint_as_float(xbuf[g][wave][129 + 2 * c]);
            const float xs_lo = __uint_as_float(xbuf[g][wave][136 + 2 * c]), xs_hi = __uint_as_float(xbuf[g][wave][137 + 2 * c]);

            const uint8_t *blk = &ring[st % 3][r * QD_ROW_LDS + wave * 144];
            const uint4 hdr = *(const uint4 *)blk;
            const uint4 qa = *(const uint4 *)(blk + 16 + 32 * c), qb = *(const uint4 *)(blk + 32 + 32 * c);
            uint32_t scp, mnp;
            q4k_scale_min_pair(hdr.y, hdr.z, hdr.w, c, scp, mnp);
            const uint32_t sc_lo = scp & 0xFFu, sc_hi = (scp >> 8) & 0xFFu, mn_lo = mnp & 0xFFu, mn_hi = (mnp >> 8) & 0xFFu;
            const uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
            int sl_lo = 0, sh_lo = 0, sl_hi = 0, sh_hi = 0;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int lo4 = (int)(q[e] & 0x0F0F0F0Fu), hi4 = (int)((q[e] >> 4) & 0x0F0F0F0Fu);
                sl_lo = __builtin_amdgcn_sdot4(lo4, (int)xl_lo[e], sl_lo, false);
                sh_lo = __builtin_amdgcn_sdot4(lo4, (int)xh_lo[e], sh_lo, false);
                sl_hi = __builtin_amdgcn_sdot4(hi4, (int)xl_hi[e], sl_hi, false);
                sh_hi = __builtin_amdgcn_sdot4(hi4, (int)xh_hi[e], sh_hi, false);
            }
            const float d = f16_bits(hdr.x), dmin = f16_bits(hdr.x >> 16);
            const float f_lo = (float)((sh_lo << 8) + sl_lo) * s_lo, f_hi = (float)((sh_hi << 8) + sl_hi) * s_hi;
            acc = fmaf(d, fmaf((float)sc_lo, f_lo, (float)sc_hi * f_hi), acc);
            acc = fmaf(-dmin, fmaf((float)mn_lo, xs_lo, (float)mn_hi * xs_hi), acc);

            const int buf = tile & 1;
            if (g == NG - 1) {  // the row tile is complete: the four chunks of a row, then the waves through LDS
                acc = sum_xor16(acc);
                acc = sum_xor32(acc);
                if (lane < 16) red[buf][wave][lane] = acc;
                acc = 0.0f;
            }
            // step st+1 has landed (and the partial sums are written): at most this step's 3 loads stay in flight
            if (more) asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (g == NG - 1) {  // wave w sums row w of the tile over the 16 waves
                float v = (lane < 16) ? red[buf][lane][wave] : 0.0f;
                v = sum_row16(v);
                const int row = 16 * ((int)blockIdx.x + tile * G) + wave;
                if (lane == 0 && row < n) Y[row] = v;
            }
        }
    }
}

}  // namespace jq
