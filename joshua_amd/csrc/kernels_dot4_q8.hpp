// Q8_0 times one activation row on v_dot4, the weights travelling HBM -> LDS as asynchronous, fully
// coalesced loads (the road of q4k_gemv_dot4_lds and q6k_gemv_dot4_lds, for the 34-byte Q8_0 blocks).
//
// Rows of 128 * NG blocks (k = 4096 NG).  A step is 8 weight rows x 128 blocks: the 16 waves of a
// workgroup copy the 8 row slices (4352 B each, half a slice a wave, three instructions) into a ring
// of three steps in LDS, two steps ahead of the arithmetic; wave w then works on blocks 8w .. 8w + 7
// of the slice, one block a lane: its 32 int8 weights go to v_dot4_i32_i8 against the block's
// activations, which the lane keeps in registers as 15-bit fixed point (two int8 planes,
// X = 256 hi + lo, one scale per block).  The integer sum of a block is exact; result per row:
// sum_blocks d * s_x * (integer), summed over the lanes of a row, the waves of a workgroup (through
// LDS) and the NG steps of a row tile (in a register).
#pragma once
#include "kernels_dot4_q4k.hpp"

namespace jq {

constexpr int Q8D_SLICE = 128 * 34, Q8D_SLICE_LDS = Q8D_SLICE + 16, Q8D_ROWS = 8, Q8D_STEP_LDS = Q8D_ROWS * Q8D_SLICE_LDS;

template <int NG>
__global__ __launch_bounds__(1024) void q8_0_gemv_dot4_lds(const uint8_t *__restrict__ W, const float *__restrict__ X,
                                                           float *__restrict__ Y, int n, int G) {
    __shared__ __attribute__((aligned(16))) uint8_t ring[3][Q8D_STEP_LDS];
    __shared__ uint32_t xl_lds[NG][16][64], xh_lds[NG][16][64];
    __shared__ float s_lds[NG][16][8];
    __shared__ float red[2][Q8D_ROWS][17];   // [tile % 2][row][wave]: a wave's writes and a row's reads each touch a bank once
    __shared__ float out_lds[8][Q8D_ROWS];  // the rows of up to eight tiles wait here: a store between the steps' loads costs 0.15 us
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane >> 3, j = lane & 7;  // row of the step, block of the wave's eight
    const int n_tiles = (((n + Q8D_ROWS - 1) / Q8D_ROWS) - (int)blockIdx.x + G - 1) / G;  // row tiles blockIdx.x, + G, ...
    if (n_tiles <= 0) return;
    const int n_steps = NG * n_tiles;
    constexpr size_t row_bytes = (size_t)NG * Q8D_SLICE;

    // step i = (row tile i / NG, column group i % NG); 3 asynchronous loads per wave: half a row slice
    auto fetch = [&](int i, int slot) __attribute__((always_inline)) {
        const int ii = min(i, n_steps - 1);
        const int row = min(Q8D_ROWS * ((int)blockIdx.x + (ii / NG) * G) + (wave >> 1), n - 1);
        const uint8_t *src = W + (size_t)row * row_bytes + (size_t)(ii % NG) * Q8D_SLICE + (wave & 1) * 2176 + 16 * lane;
        const uint32_t dst = lds_offset_of(&ring[slot][(wave >> 1) * Q8D_SLICE_LDS + (wave & 1) * 2176]);
        async_load16(src, dst);
        async_load16(src + 1024, dst + 1024);
        if (lane < 8) async_load16(src + 2048, dst + 2048);  // 136 pieces of 16 bytes per half slice
    };
    // Up to two column groups (LDS has room for their raw activations): every global read is an
    // asynchronous load counted by hand, the activation columns first, then step 0, and step 1 once the
    // activations are prepared, so that every workgroup's step 0 has the memory system to itself.  With
    // three groups the activations are plain loads behind both steps (the compiler's wait for them then
    // covers the steps as well).
    constexpr bool STAGED_X = NG <= 2;
    __shared__ __attribute__((aligned(16))) float x_raw[STAGED_X ? NG : 1][16][256];
    if constexpr (STAGED_X) {
#pragma unroll
        for (int g = 0; g < NG; g++)
            async_load16(X + (size_t)(16 * g + wave) * 256 + 4 * lane, lds_offset_of(&x_raw[g][wave][0]));
        fetch(0, 0);
        asm volatile("s_waitcnt vmcnt(3)" ::: "memory");  // the activations landed (own wave's data: no barrier needed)
    } else {
        fetch(0, 0);
        fetch(1, 1);  // (a clamped copy of step 0 when there is one step only)
    }

    // activations of blocks 128 g + 8 wave .. + 7: 4 elements a lane, one scale per block of 32
#pragma unroll
    for (int g = 0; g < NG; g++) {
        float4 v;
        if constexpr (STAGED_X) v = *(const float4 *)&x_raw[g][wave][4 * lane];
        else v = *(const float4 *)(X + (size_t)(16 * g + wave) * 256 + 4 * lane);
        const QvQuant qx = qv_quantise4(v);
        xl_lds[g][wave][lane] = qx.wl;
        xh_lds[g][wave][lane] = qx.wh;
        const float s = qx.s;
        if ((lane & 7) == 0) s_lds[g][wave][lane >> 3] = s;
    }
    // step 0 landed (step 1 may be in flight), planes written
    if (STAGED_X && n_steps == 1) {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    } else {
        if constexpr (STAGED_X) fetch(1, 1);
        asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory");
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    uint32_t xl[NG][8], xh[NG][8];  // this lane's block: elements 32 j .. 32 j + 31 of the wave's 256
    float sx[NG];
#pragma unroll
    for (int g = 0; g < NG; g++) {
#pragma unroll
        for (int i = 0; i < 8; i++) xl[g][i] = xl_lds[g][wave][8 * j + i], xh[g][i] = xh_lds[g][wave][8 * j + i];
        sx[g] = s_lds[g][wave][j];
    }

    // on entry to step i: step i is in LDS and visible (the barrier just passed), step i+1 in flight
    float acc = 0.0f;
    for (int i = 0, tile = 0; i < n_steps; i += NG, tile++) {
#pragma unroll
        for (int g = 0; g < NG; g++) {
            const int st = i + g;
            const bool more = st + 2 < n_steps;
            if (more) fetch(st + 2, (st + 2) % 3);  // the slot of step st-1, which every wave finished reading before that barrier

            const uint8_t *blk = &ring[st % 3][r * Q8D_SLICE_LDS + (8 * wave + j) * 34];
            const float d = f16_bits(ld<uint16_t>(blk));
            const uint4 qa = ldw<uint4>(blk + 2), qb = ldw<uint4>(blk + 18);  // 34-byte blocks: odd word offsets
            const uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
            int sl = 0, sh = 0;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                sl = __builtin_amdgcn_sdot4((int)q[e], (int)xl[g][e], sl, false);
                sh = __builtin_amdgcn_sdot4((int)q[e], (int)xh[g][e], sh, false);
            }
            acc = fmaf(d * sx[g], (float)((sh << 8) + sl), acc);

            const int buf = tile & 1;
            if (g == NG - 1) {  // the row tile is complete: the lanes of a row, then the waves through LDS
                acc = sum_row8(acc);
                if (j == 0) red[buf][r][wave] = acc;
                acc = 0.0f;
            }
            // step st+1 has landed (and the partial sums are written): at most this step's 3 loads stay in flight
            if (more) asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (g == NG - 1) {
                if (wave < Q8D_ROWS) {  // wave w sums row w of the tile over the 16 waves
                    float v = (lane < 16) ? red[buf][wave][lane] : 0.0f;
                    v = sum_row16(v);
                    if (lane == 0) out_lds[tile & 7][wave] = v;
                }
                if ((tile & 7) == 7 || tile == n_tiles - 1) {  // wave 0 stores the rows of the last (up to) eight tiles
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    const int tt = (tile & ~7) + (lane >> 3), row = Q8D_ROWS * ((int)blockIdx.x + tt * G) + (lane & 7);
                    if (wave == 0 && tt <= tile && row < n) Y[row] = out_lds[lane >> 3][lane & 7];
                }
            }
        }
    }
}

}  // namespace jq
