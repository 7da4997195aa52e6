// Q6_K times one activation row on v_dot4, the weights travelling HBM -> LDS as asynchronous, fully
// coalesced loads (the road of q4k_gemv_dot4_lds, for the 210-byte Q6_K blocks).
//
// Rows of 16 * NG super-blocks (k = 4096 NG).  A step is 8 weight rows x 16 super-blocks: the 16
// waves of a workgroup copy the 8 row slices (3360 B each, half a slice a wave, two instructions)
// into a ring of three steps in LDS, two steps ahead of the arithmetic; wave w then works on
// super-block w of the slice, 8 lanes a row: lane (half h, eighth e) takes l in [8e, 8e + 8) of the
// half's four 32-element quarters (24 bytes of ql and qh), builds the 6-bit values four to a
// register and multiplies them with v_dot4_i32_i8 against the activations, which every wave keeps
// in registers as 15-bit fixed point per 32-element block (two int8 planes, X = 256 hi + lo).  The
// per-quarter integer sums are exact; sum (q - 32) X = sum q X - 32 sum X with the lanes' sums of X
// prepared once.  Result per row: d * sum_quarters sc * s_x * (integer), summed over the lanes of a
// row, the waves of a workgroup (through LDS) and the NG steps of a row tile (in a register).
#pragma once
#include "kernels_dot4_q4k.hpp"

namespace jq {

constexpr int Q6D_SLICE = 16 * 210, Q6D_SLICE_LDS = Q6D_SLICE + 16, Q6D_ROWS = 8, Q6D_STEP_LDS = Q6D_ROWS * Q6D_SLICE_LDS;

template <int NG>
__global__ __launch_bounds__(1024) void q6k_gemv_dot4_lds(const uint8_t *__restrict__ W, const float *__restrict__ X,
                                                          float *__restrict__ Y, int n, int G) {
    __shared__ __attribute__((aligned(16))) uint8_t ring[3][Q6D_STEP_LDS];
    __shared__ uint32_t xl_lds[NG][16][64], xh_lds[NG][16][64];
    __shared__ float s_lds[NG][16][8];
    __shared__ float red[2][Q6D_ROWS][17];   // [tile % 2][row][wave]: a wave's writes and a row's reads each touch a bank once
    __shared__ float out_lds[8][Q6D_ROWS];  // the rows of up to eight tiles wait here: a store between the steps' loads costs 0.15 us
    __shared__ __attribute__((aligned(16))) float x_raw[NG][16][256];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane >> 3, h = (lane >> 2) & 1, e = lane & 3;  // row of the step, half of the super-block, eighth
    const int n_tiles = (((n + Q6D_ROWS - 1) / Q6D_ROWS) - (int)blockIdx.x + G - 1) / G;  // row tiles blockIdx.x, + G, ...
    if (n_tiles <= 0) return;
    const int n_steps = NG * n_tiles;
    constexpr size_t row_bytes = (size_t)NG * Q6D_SLICE;

    // step i = (row tile i / NG, column group i % NG); 2 asynchronous loads per wave: half a row slice
    auto fetch = [&](int i, int slot) __attribute__((always_inline)) {
        const int ii = min(i, n_steps - 1);
        const int row = min(Q6D_ROWS * ((int)blockIdx.x + (ii / NG) * G) + (wave >> 1), n - 1);
        const uint8_t *src = W + (size_t)row * row_bytes + (size_t)(ii % NG) * Q6D_SLICE + (wave & 1) * 1680 + 16 * lane;
        const uint32_t dst = lds_offset_of(&ring[slot][(wave >> 1) * Q6D_SLICE_LDS + (wave & 1) * 1680]);
        async_load16(src, dst);
        if (lane < 41) async_load16(src + 1024, dst + 1024);  // 105 pieces of 16 bytes per half slice
    };
    // every global read of this kernel is an asynchronous load counted by hand: the activation columns
    // first, then step 0; step 1 is asked for once the activations are prepared, so that every
    // workgroup's step 0 has the memory system to itself and the arithmetic starts sooner
#pragma unroll
    for (int g = 0; g < NG; g++)
        async_load16(X + (size_t)(16 * g + wave) * 256 + 4 * lane, lds_offset_of(&x_raw[g][wave][0]));
    fetch(0, 0);
    asm volatile("s_waitcnt vmcnt(2)" ::: "memory");  // the activations landed (own wave's data: no barrier needed)

    // activations of super-block 16 g + wave: 4 elements a lane, one scale per 32
#pragma unroll
    for (int g = 0; g < NG; g++) {
        const float4 v = *(const float4 *)&x_raw[g][wave][4 * lane];
        const QvQuant qx = qv_quantise4(v);
        xl_lds[g][wave][lane] = qx.wl;
        xh_lds[g][wave][lane] = qx.wh;
        const float s = qx.s;
        if ((lane & 7) == 0) s_lds[g][wave][lane >> 3] = s;
    }
    // step 0 landed (step 1 may be in flight), planes written
    if (n_steps > 1) {
        fetch(1, 1);
        asm volatile("s_waitcnt vmcnt(2) lgkmcnt(0)" ::: "memory");
    } else {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    // this lane's share: quarter t of half h covers elements 128 h + 32 t + 8 e .. + 7 (two registers a plane)
    uint32_t xl[NG][4][2], xh[NG][4][2];
    float sx[NG][4];   // activation scale of the quarter's 32-element block
    int xs32[NG][4];   // 32 * (sum of the lane's 8 fixed-point activations of the quarter)
#pragma unroll
    for (int g = 0; g < NG; g++) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int dw = 32 * h + 8 * t + 2 * e;
            xl[g][t][0] = xl_lds[g][wave][dw], xl[g][t][1] = xl_lds[g][wave][dw + 1];
            xh[g][t][0] = xh_lds[g][wave][dw], xh[g][t][1] = xh_lds[g][wave][dw + 1];
            sx[g][t] = s_lds[g][wave][4 * h + t];
            const int ones = 0x01010101;
            const int sl = __builtin_amdgcn_sdot4(ones, (int)xl[g][t][0], __builtin_amdgcn_sdot4(ones, (int)xl[g][t][1], 0, false), false);
            const int sh = __builtin_amdgcn_sdot4(ones, (int)xh[g][t][0], __builtin_amdgcn_sdot4(ones, (int)xh[g][t][1], 0, false), false);
            xs32[g][t] = 32 * ((sh << 8) + sl);
        }
    }

    // on entry to step i: step i is in LDS and visible (the barrier just passed), step i+1 in flight
    float acc = 0.0f;
    for (int i = 0, tile = 0; i < n_steps; i += NG, tile++) {
#pragma unroll
        for (int g = 0; g < NG; g++) {
            const int st = i + g;
            const bool more = st + 2 < n_steps;
            if (more) fetch(st + 2, (st + 2) % 3);  // the slot of step st-1, which every wave finished reading before that barrier

            // Block `wave` of a row starts 210 * wave bytes into the slice: a multiple of four for even
            // waves, two bytes past one for odd waves.  LDS reads that are not naturally aligned run at
            // a fraction of the aligned rate (the 151936 x 4096 output head: 130 us with 8-byte reads
            // at these addresses, 82 us with every read on a word boundary), so each 8-byte field is
            // read as the three aligned words that hold it and shifted into place; the shift is the
            // same for the whole wave.
            const uint8_t *blk = &ring[st % 3][r * Q6D_SLICE_LDS + wave * 210];
            const uint32_t *blk4 = (const uint32_t *)(blk - 2 * (wave & 1));
            const uint32_t mis = 16 * (wave & 1);
            auto field = [&](int off) __attribute__((always_inline)) {   // off: a multiple of 4
                const uint32_t d0 = blk4[off / 4], d1 = blk4[off / 4 + 1], d2 = blk4[off / 4 + 2];
                return uint2{__builtin_amdgcn_alignbit(d1, d0, mis), __builtin_amdgcn_alignbit(d2, d1, mis)};
            };
            const uint2 qa = field(64 * h + 8 * e);         // ql[64h + l]
            const uint2 qb = field(64 * h + 32 + 8 * e);    // ql[64h + 32 + l]
            const uint2 qh = field(128 + 32 * h + 8 * e);   // qh[32h + l]
            const float d = f16_bits(ld<uint16_t>(blk + 208));
            const uint32_t a[2] = {qa.x, qa.y}, b[2] = {qb.x, qb.y}, hh[2] = {qh.x, qh.y};
            float f = 0.0f;
#pragma unroll
            for (int t = 0; t < 4; t++) {
                int sl = 0, sh = 0;
#pragma unroll
                for (int j = 0; j < 2; j++) {
                    const uint32_t lo = (t & 1) ? b[j] : a[j];
                    const uint32_t nib = (t < 2) ? (lo & 0x0F0F0F0Fu) : ((lo >> 4) & 0x0F0F0F0Fu);
                    const uint32_t two = t == 0 ? hh[j] << 4 : t == 1 ? hh[j] << 2 : t == 2 ? hh[j] : hh[j] >> 2;
                    const int q = (int)(nib | (two & 0x30303030u));  // four 6-bit values, 0..63
                    sl = __builtin_amdgcn_sdot4(q, (int)xl[g][t][j], sl, false);
                    sh = __builtin_amdgcn_sdot4(q, (int)xh[g][t][j], sh, false);
                }
                const float sc = (float)(int8_t)blk[192 + 8 * h + 2 * t + (e >> 1)];
                f = fmaf(sc * sx[g][t], (float)((sh << 8) + sl - xs32[g][t]), f);
            }
            acc = fmaf(d, f, acc);

            const int buf = tile & 1;
            if (g == NG - 1) {  // the row tile is complete: the lanes of a row, then the waves through LDS
                acc = sum_row8(acc);
                if ((lane & 7) == 0) red[buf][r][wave] = acc;
                acc = 0.0f;
            }
            // step st+1 has landed (and the partial sums are written): at most this step's 2 loads stay in flight
            if (more) asm volatile("s_waitcnt vmcnt(2) lgkmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (g == NG - 1) {
                if (wave < Q6D_ROWS) {  // wave w sums row w of the tile over the 16 waves
                    float v = (lane < 16) ? red[buf][wave][lane] : 0.0f;
                    v = sum_row16(v);
                    if (lane == 0) out_lds[tile & 7][wave] = v;
                }
                if ((tile & 7) == 7 || tile == n_tiles - 1) {  // wave 0 stores the rows of the last (up to) eight tiles
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    const int tt = (tile & ~7) + (lane >> 3), row = Q6D_ROWS * ((int)blockIdx.x + tt * G) + (lane & 7);
                    if (wave == 0 && tt <= tile && row < n) Y[row] = out_lds[lane >> 3][lane & 7];
                }
            }
        }
    }
}

}  // namespace jq
