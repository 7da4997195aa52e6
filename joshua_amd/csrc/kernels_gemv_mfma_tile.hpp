// One activation row against a matrix whose rows are fewer than 16 super-blocks long (a 2048-wide hidden size:
// 8), on the int8 matrix cores: the one-row kernel of kernels_gemv_mfma.hpp keeps 16 waves on the 16 columns of a
// tile and streams tiles through a ring; here a tile of 16 rows is a few KB, so a workgroup of NB waves takes ONE
// tile, wave w its column w, and every byte of the launch is asked for in its first microsecond (the shape of the
// expert kernel moe_gate_up_mfma, kernels_moe_mfma.hpp).  The arithmetic is the policies' of the one-row kernel:
// activations as 15-bit fixed point a 32-element sub-block in a block-diagonal A operand, exact integer sums
// (reference arithmetic: src/kquant_dot.rs:407-483 for Q4_K; the row-by-row schedule it replaces:
// src/quant_matmul.rs:110-249).
//
// NORM puts the decoder's residual add and RMSNorm in front (src/quantized_qwen3_moe.rs:792-805): every workgroup
// adds res to X and normalises the row itself, the 1 / rms goes onto the sub-block scales, workgroup 0 stores
// x + res to x_out (a buffer other than X: the others are still reading X) and, when asked, the normalised row.
#pragma once

#include "kernels_moe_mfma.hpp"

namespace jq {

template <class F, int NB>
constexpr int gemv_mfma_tile_stage() { return (F::STAGE_BYTES + 15) / 16 * 16 + 3 * 1024; }  // prepare()'s words, then x, norm weight, res

template <class F, int NB>
constexpr int gemv_mfma_tile_lds() {
    return qv_table_bytes<F>() + 16 * moe_mfma_row_lds(NB * F::BLOCK) + NB * gemv_mfma_tile_stage<F, NB>() + 16 * 68 * 4 + 64;
}

// `b`: the tile's number; `first`: this workgroup stores x + res and the normalised row.
template <class F, int NB, bool NORM>
__device__ __forceinline__ void gemv_mfma_tile_body(uint8_t *gemv_tile_lds, int b, bool first, const uint8_t *__restrict__ W,
                                                    const float *__restrict__ X, float *__restrict__ Y, int n,
                                                    const float *nm_res, const float *nm_w, float nm_eps, float *nm_x_out,
                                                    float *nm_hn_out) {
    static_assert(NB == 2 || NB == 4 || NB == 8 || NB == 16, "a row of 2, 4, 8 or 16 super-blocks");
    constexpr int RB = NB * F::BLOCK, ROW_LDS = moe_mfma_row_lds(RB), LOADS = (RB + 1023) / 1024;
    constexpr int STG = gemv_mfma_tile_stage<F, NB>(), RPW = 16 / NB;  // tile rows a wave copies
    static_assert(RB % 16 == 0, "rows are copied 16 bytes a lane");
    const uint64_t *table = qv_stage_table<F>(gemv_tile_lds);
    uint8_t *tile = gemv_tile_lds + qv_table_bytes<F>();  // [16][ROW_LDS]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, c = lane >> 4;
    uint32_t *stage = (uint32_t *)(tile + 16 * ROW_LDS + wave * STG);
    float *x_raw = (float *)((uint8_t *)stage + (STG - 3 * 1024)), *w_raw = x_raw + 256, *r_raw = x_raw + 512;
    float *part = (float *)(tile + 16 * ROW_LDS + NB * STG);  // [16][68]
    float *ss_lds = part + 16 * 68;                           // [NB]
    async_load16(X + 256 * wave + 4 * lane, lds_offset_of(x_raw));
    if (NORM) {
        async_load16(nm_w + 256 * wave + 4 * lane, lds_offset_of(w_raw));
        if (nm_res) async_load16(nm_res + 256 * wave + 4 * lane, lds_offset_of(r_raw));
    }
    const int row0 = 16 * b;
    const uint32_t tile0 = lds_offset_of(tile);
#pragma unroll
    for (int i = 0; i < RPW; i++) {
        const int rr = wave + NB * i;
        const uint8_t *src = W + (size_t)min(row0 + rr, n - 1) * RB;
        const uint32_t dst = tile0 + (uint32_t)rr * ROW_LDS;
#pragma unroll
        for (int l = 0; l < LOADS; l++) {
            const int lanes = (RB - 1024 * l) / 16 < 64 ? (RB - 1024 * l) / 16 : 64;
            if (lane < lanes) async_load16_s(src + 1024 * l, 16 * lane, dst + 1024 * l);
        }
    }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(RPW * LOADS) : "memory");  // the activations (and the norm's operands) are in
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
        if (first) *(float4 *)(nm_x_out + 256 * wave + 4 * lane) = v;
        v = float4{v.x * g.x, v.y * g.y, v.z * g.z, v.w * g.w};
    }
    typename F::Acts acts = F::prepare(v, stage, lane);
    asm volatile("s_waitcnt vmcnt(0)\n\ts_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (NORM) {
        float tot = 0.0f;
#pragma unroll
        for (int i = 0; i < NB; i++) tot += ss_lds[i];
        const float inv = 1.0f / sqrtf(tot / (float)(256 * NB) + nm_eps);
        F::scale(acts, inv);
        if (first && nm_hn_out)
            *(float4 *)(nm_hn_out + 256 * wave + 4 * lane) = float4{v.x * inv, v.y * inv, v.z * inv, v.w * inv};
    }
    part[r * 68 + 4 * wave + c] = qv_dot<F>(tile + r * ROW_LDS + wave * F::BLOCK, acts, c, table);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    // wave w adds the 4 NB chunk sums of rows w, w + NB, ..
#pragma unroll
    for (int q = 0; q < RPW; q++) {
        const int rr = wave + NB * q;
        float sum = lane < 4 * NB ? part[rr * 68 + lane] : 0.0f;
        sum = wave_sum(sum);
        if (lane == 0 && row0 + rr < n) Y[row0 + rr] = sum;
    }
}

template <class F, int NB, bool NORM>
__global__ __launch_bounds__(64 * NB) void gemv_mfma_tile(const uint8_t *__restrict__ W, const float *__restrict__ X,
                                                          float *__restrict__ Y, int n, const float *nm_res,
                                                          const float *nm_w, float nm_eps, float *nm_x_out,
                                                          float *nm_hn_out) {
    extern __shared__ __attribute__((aligned(16))) uint8_t gemv_tile_lds[];
    gemv_mfma_tile_body<F, NB, NORM>(gemv_tile_lds, (int)blockIdx.x, blockIdx.x == 0, W, X, Y, n, nm_res, nm_w, nm_eps, nm_x_out,
                                     nm_hn_out);
}

// Two products over the same normalised activation row in one launch: Y1 = W1 hn on the streaming kernel
// (gemv_mfma_lds, workgroups 0 .. G - 1) and Y2 = W2 hn, a smaller matrix of another format, one tile of 16 rows a
// workgroup behind them (the decoder's q|k product of Q4_K beside an attn_v kept as Q6_K or Q8_0: a launch less).
// Rows of 4096 columns.  Workgroup 0 stores x + res.
template <class F1, class F2>
constexpr int gemv_mfma_norm_pair_lds() {
    return GemvMfmaLds<F1>::BYTES > gemv_mfma_tile_lds<F2, 16>() ? GemvMfmaLds<F1>::BYTES : gemv_mfma_tile_lds<F2, 16>();
}

template <class F1, class F2>
__global__ __launch_bounds__(1024) void gemv_mfma_norm_pair(const uint8_t *__restrict__ W1, const float *__restrict__ X,
                                                            float *__restrict__ Y1, int n1, int G, int rounds, int extra,
                                                            const float *nm_res, const float *nm_w, float nm_eps,
                                                            float *nm_x_out, const uint8_t *__restrict__ W2,
                                                            float *__restrict__ Y2, int n2) {
    extern __shared__ __attribute__((aligned(16))) uint8_t gemv_tile_lds[];
    const int b = (int)blockIdx.x;
    if (b < G)
        gemv_mfma_lds_body<F1, true, false>(gemv_tile_lds, b, W1, X, Y1, n1, G, rounds, extra, nm_res, nm_w, nm_eps, nm_x_out, nullptr);
    else
        gemv_mfma_tile_body<F2, 16, true>(gemv_tile_lds, b - G, false, W2, X, Y2, n2, nm_res, nm_w, nm_eps, nullptr, nullptr);
}

// The same for rows of NB super-blocks: both products a tile of 16 rows a workgroup of NB waves, the tiles of W2 behind
// those of W1.
template <class F1, class F2, int NB>
constexpr int gemv_mfma_tile_pair_lds() {
    return gemv_mfma_tile_lds<F1, NB>() > gemv_mfma_tile_lds<F2, NB>() ? gemv_mfma_tile_lds<F1, NB>() : gemv_mfma_tile_lds<F2, NB>();
}

template <class F1, class F2, int NB>
__global__ __launch_bounds__(64 * NB) void gemv_mfma_tile_norm_pair(const uint8_t *__restrict__ W1, const float *__restrict__ X,
                                                                    float *__restrict__ Y1, int n1, const float *nm_res,
                                                                    const float *nm_w, float nm_eps, float *nm_x_out,
                                                                    const uint8_t *__restrict__ W2, float *__restrict__ Y2,
                                                                    int n2) {
    extern __shared__ __attribute__((aligned(16))) uint8_t gemv_tile_lds[];
    const int b = (int)blockIdx.x, t1 = (n1 + 15) / 16;
    if (b < t1)
        gemv_mfma_tile_body<F1, NB, true>(gemv_tile_lds, b, b == 0, W1, X, Y1, n1, nm_res, nm_w, nm_eps, nm_x_out, nullptr);
    else
        gemv_mfma_tile_body<F2, NB, true>(gemv_tile_lds, b - t1, false, W2, X, Y2, n2, nm_res, nm_w, nm_eps, nullptr, nullptr);
}

}  // namespace jq
