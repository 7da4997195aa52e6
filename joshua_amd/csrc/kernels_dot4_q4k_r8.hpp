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

}  // namespace jq
