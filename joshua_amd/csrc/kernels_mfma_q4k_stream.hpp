// Q4_K decode matmul (1 to 16 activation rows) as a weight-streaming kernel on the matrix cores.
//
// The arithmetic is that of the prefill GEMM (kernels_mfma_q4k_gemm.hpp): per 256-element
// super-block, activations in 23-bit fixed point X = 2048 Xh + Xl with scale s, weights as the exact
// f16 integers sc*q, products on v_mfma_f32_16x16x32_f16, the min term as one more MFMA over the
// sub-block sums, one f32 combination  s (d (2048 Ph + Pl) - 4096 dmin MM)  per super-block.
//
// What differs is where the operands live.  The weights are read once from HBM and never touch
// LDS: a wave owns CPW super-block columns of the weight matrix and, for each tile of 16 weight
// rows, every lane loads the 16-byte header of its row and the 8 nibble bytes of its k group of
// each 64-element chunk straight into registers (the four loads of a row together cover its
// 128 nibble bytes), unpacks them, and feeds them to the MFMAs as the A operand.  The activations
// of those columns are quantised ONCE per wave, at kernel start, directly into MFMA B-operand
// registers (64 registers per column), so the main loop reads neither LDS nor global memory for
// them.  A workgroup's waves cover all columns of a row; their 16x16 partial results meet in LDS
// (8 KB per tile, double buffered: one barrier per tile) and are summed in a fixed order.
// Workgroups are persistent: each walks the row tiles blockIdx.x, blockIdx.x + gridDim.x, ...
#pragma once
#include "kernels_mfma_q4k_gemm.hpp"

namespace jq {

constexpr int QS_MAX_WAVES = 8;

struct QsTileRegs {  // one 16-row tile of one column, as loaded
    qg_u4 hdr;       // d, dmin, 12 scale bytes of this lane's row
    uint2 nib[4];    // bytes 8*kg .. 8*kg+7 of each chunk's 32 nibble bytes
};

template <int CPW>
__global__ __launch_bounds__(64 * QS_MAX_WAVES) void q4k_stream_mfma(const uint8_t *__restrict__ W, size_t row_bytes,
                                                                      const float *__restrict__ X,
                                                                      float *__restrict__ Y, int m, int k, int n) {
    __shared__ qg_f4 red[2][QS_MAX_WAVES][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
    const int col = lane & 15, kg = lane >> 4;
    const int n_tiles = (n + 15) >> 4;

    // ---- activations of this wave's columns -> B operand registers ----
    qg_u4 Bh[CPW][8], Bl[CPW][8], Bm[CPW];
    float sx[CPW];
#pragma unroll
    for (int j = 0; j < CPW; j++) {
        const int b = wave * CPW + j;
        float xv[8][8];
        float amax = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            float4 a = float4{0.f, 0.f, 0.f, 0.f}, c = a;
            if (col < m) {
                const float *xp = X + (size_t)col * k + 256 * b + 32 * ks + 8 * kg;
                a = *(const float4 *)xp, c = *(const float4 *)(xp + 4);
            }
            xv[ks][0] = a.x, xv[ks][1] = a.y, xv[ks][2] = a.z, xv[ks][3] = a.w;
            xv[ks][4] = c.x, xv[ks][5] = c.y, xv[ks][6] = c.z, xv[ks][7] = c.w;
#pragma unroll
            for (int i = 0; i < 8; i++) amax = fmaxf(amax, fabsf(xv[ks][i]));
        }
        amax = fmaxf(amax, __shfl_xor(amax, 16, 64));
        amax = fmaxf(amax, __shfl_xor(amax, 32, 64));
        const bool live = amax > 0.0f && amax < INFINITY;
        const float inv = live ? QG_RANGE / amax : 0.0f;
        sx[j] = live ? amax / QG_RANGE : 0.0f;
        int xs[8];
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            int lo[8], hi[8], sum = 0;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int Xi = __float2int_rn(xv[ks][i] * inv);
                lo[i] = ((Xi + 1024) & 2047) - 1024;
                hi[i] = (Xi - lo[i]) >> 11;
                sum += Xi;
            }
            // operand order within the 8 k of a lane: 0,2,1,3,4,6,5,7 (what the weight unpack produces)
            Bh[j][ks] = qg_u4{qg_pack_h2(hi[0], hi[2]), qg_pack_h2(hi[1], hi[3]), qg_pack_h2(hi[4], hi[6]), qg_pack_h2(hi[5], hi[7])};
            Bl[j][ks] = qg_u4{qg_pack_h2(lo[0], lo[2]), qg_pack_h2(lo[1], lo[3]), qg_pack_h2(lo[4], lo[6]), qg_pack_h2(lo[5], lo[7])};
            sum += __shfl_xor(sum, 16, 64);
            sum += __shfl_xor(sum, 32, 64);
            xs[ks] = sum;  // the whole sub-block's sum, in all four lanes of the column
        }
        // k group g of the min operand: part g of XS_j / 4096 split three ways into f16, j = 0..7
        _Float16 part[8];
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            _Float16 p0, p1, p2;
            qg_split_sum(xs[ks], p0, p1, p2);
            part[ks] = kg == 0 ? p0 : kg == 1 ? p1 : kg == 2 ? p2 : (_Float16)0.0f;
        }
        const qg_h8 pm = qg_h8{part[0], part[1], part[2], part[3], part[4], part[5], part[6], part[7]};
        Bm[j] = __builtin_bit_cast(qg_u4, pm);
    }

    auto load_tile = [&](int t, QsTileRegs(&r)[CPW]) __attribute__((always_inline)) {
        const int row = min(16 * t + col, n - 1);
        const uint8_t *rp = W + (size_t)row * row_bytes + (size_t)(wave * CPW) * 144;
#pragma unroll
        for (int j = 0; j < CPW; j++) {
            const uint8_t *blk = rp + 144 * j;
            r[j].hdr = *(const qg_u4 *)blk;
#pragma unroll
            for (int c = 0; c < 4; c++) r[j].nib[c] = *(const uint2 *)(blk + 16 + 32 * c + 8 * kg);
        }
    };

    QsTileRegs cur[CPW], nxt[CPW];
    int t = blockIdx.x;
    if (t < n_tiles) load_tile(t, cur);
    for (int it = 0; t < n_tiles; t += gridDim.x, it++) {
        const int tn = t + gridDim.x;
        if (tn < n_tiles) load_tile(tn, nxt);

        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < CPW; j++) {
            const qg_u4 h = cur[j].hdr;
            uint32_t sc[8], mn[8];
#pragma unroll
            for (int q = 0; q < 8; q++) q4k_scale_min(h.y, h.z, h.w, q, sc[q], mn[q]);
            qg_f4 Ph = qg_f4{0.f, 0.f, 0.f, 0.f}, Pl = Ph;
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const uint32_t w0 = cur[j].nib[c].x, w1 = cur[j].nib[c].y;
                const qg_u4 lo = qg_u4{qg_scaled_h2(w0 & 0x000F000Fu, sc[2 * c]), qg_scaled_h2((w0 >> 8) & 0x000F000Fu, sc[2 * c]),
                                       qg_scaled_h2(w1 & 0x000F000Fu, sc[2 * c]), qg_scaled_h2((w1 >> 8) & 0x000F000Fu, sc[2 * c])};
                const qg_u4 hi = qg_u4{qg_scaled_h2((w0 >> 4) & 0x000F000Fu, sc[2 * c + 1]), qg_scaled_h2((w0 >> 12) & 0x000F000Fu, sc[2 * c + 1]),
                                       qg_scaled_h2((w1 >> 4) & 0x000F000Fu, sc[2 * c + 1]), qg_scaled_h2((w1 >> 12) & 0x000F000Fu, sc[2 * c + 1])};
                const qg_h8 alo = __builtin_bit_cast(qg_h8, lo), ahi = __builtin_bit_cast(qg_h8, hi);
                Ph = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, __builtin_bit_cast(qg_h8, Bh[j][2 * c]), Ph, 0, 0, 0);
                Pl = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, __builtin_bit_cast(qg_h8, Bl[j][2 * c]), Pl, 0, 0, 0);
                Ph = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, __builtin_bit_cast(qg_h8, Bh[j][2 * c + 1]), Ph, 0, 0, 0);
                Pl = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, __builtin_bit_cast(qg_h8, Bl[j][2 * c + 1]), Pl, 0, 0, 0);
            }
            qg_u4 am = qg_u4{0, 0, 0, 0};
            if (kg < 3)
                am = qg_u4{qg_pack_h2((int)mn[0], (int)mn[1]), qg_pack_h2((int)mn[2], (int)mn[3]),
                           qg_pack_h2((int)mn[4], (int)mn[5]), qg_pack_h2((int)mn[6], (int)mn[7])};
            const qg_f4 MM = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(qg_h8, am), __builtin_bit_cast(qg_h8, Bm[j]),
                                                                    qg_f4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
            // results: weight rows 4*kg + jj of the tile, activation row `col`; d and dmin of those rows
            // sit in lanes 4*kg + jj (lanes 0..15 hold the headers of rows 0..15)
            const float d = f16_bits(h.x), dmin = f16_bits(h.x >> 16);
#pragma unroll
            for (int jj = 0; jj < 4; jj++) {
                const float dr = __shfl(d, 4 * kg + jj, 64), mr = __shfl(dmin, 4 * kg + jj, 64);
                const float f = fmaf(Ph[jj], 2048.0f, Pl[jj]);
                const float tt = fmaf(-4096.0f * mr, MM[jj], dr * f);
                acc[jj] = fmaf(sx[j], tt, acc[jj]);
            }
        }

        // ---- the waves' partial tiles meet in LDS ----
        const int buf = it & 1;
        red[buf][wave][lane] = qg_f4{acc[0], acc[1], acc[2], acc[3]};
        __syncthreads();
        for (int e = tid; e < 256; e += blockDim.x) {
            const int src_lane = e >> 2, jj = e & 3;
            float s = 0.0f;
            for (int w = 0; w < waves; w++) s += red[buf][w][src_lane][jj];
            const int nn = 16 * t + 4 * (src_lane >> 4) + jj, mm = src_lane & 15;
            if (mm < m && nn < n) Y[(size_t)mm * n + nn] = s;
        }
#pragma unroll
        for (int j = 0; j < CPW; j++) cur[j] = nxt[j];
    }
}

}  // namespace jq
