// Q4_K experts with a few tokens each on the int8 matrix cores.
//
// A mixture-of-experts layer at batch 64 sends four tokens to an expert on average: the group's weights are
// read once for a handful of activation rows, and the work per byte decides the speed.  Here a wave owns a
// 256-element column of the weight matrix (as in q4k_ring_mfma, whose road for the weights this kernel
// shares: whole 16-row tiles copied HBM -> LDS by asynchronous loads, a ring of three, two tiles ahead) and
// multiplies 16 weight rows by FOUR activation rows with one v_mfma_i32_16x16x64_i8 per 64-element chunk:
//
//   A operand row m = 4 i + 2 p + plane: activation row i of the quad, sub-block p of the chunk (the chunk's 32
//   bytes hold sub-block 2t in their low nibbles and 2t + 1 in their high nibbles), plane Xl or Xh of the
//   16-bit fixed-point activation X = 256 Xh + Xl (ActsI8: one scale per 32 elements, as the one-row kernels);
//   lane group g of the operand holds bytes 16 (g % 2) .. of nibble g / 2, so row m is zero where g / 2 != p.
//   B operand: the weight nibbles of the same 16 bytes, masked in place.
//   Result: lane (n, g) holds (S_lo, S_hi of sub-block 2t; S_lo, S_hi of 2t + 1) of weight row n against
//   activation row g of the quad: exact int32 sums, then y += d sc s S - dmin m s XS in f32
//   (reference arithmetic w = d sc q - dmin m: src/kquant_dot.rs:440-465).
//
// Against the f16 form of q4k_ring_mfma a wave issues about 6 to 9 vector instructions a block instead of 20.
// A pass takes up to 8 rows of a group (two quads; the second is skipped when the group has four or fewer);
// longer groups take more passes and re-read the weights from L2, so the dispatcher sends layers with many
// tokens an expert to q4k_ring_mfma.
//
// GROUPED as there: blockIdx.y walks (expert, token list) groups, rows gathered through `xsel`, results
// scattered through `yrow`; DUAL: tiles alternate between the same rows of two tables (gate, up) and the
// result is silu(gate . x) * (up . x)  (reference: src/quantized_qwen3_moe.rs:397-401).
#pragma once
#include "kernels_mfma_q4k_ring.hpp"

namespace jq {

typedef int mq_i4 __attribute__((ext_vector_type(4)));

constexpr int MQ_ROWS = 8;  // activation rows a pass

template <int MAXNB, bool DUAL>
// (register budget of 128: two workgroups of eight waves share a compute unit; the kernel lives on waves in flight)
__global__ __launch_bounds__(64 * MAXNB, 4) void moe_q4k_quads_mfma(const uint8_t *const *__restrict__ Wa,
                                                                 const uint8_t *const *__restrict__ Wb, ActsI8 xq,
                                                                 const int *__restrict__ gexp,
                                                                 const int *__restrict__ offsets,
                                                                 const int *__restrict__ xsel,
                                                                 const int *__restrict__ yrow, float *__restrict__ Y,
                                                                 int k, int n, MoeClamp cl) {
    __shared__ __attribute__((aligned(16))) uint8_t ring[3][16 * qr_row_lds(MAXNB)];
    __shared__ __attribute__((aligned(16))) float red[2][MAXNB][2][64];  // [step % 2][wave][quad][lane]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;  // waves == k / 256
    const int nrow = lane & 15, g = lane >> 4;
    const int row_bytes = waves * 144, row_lds = row_bytes + 16;
    const int G = (int)gridDim.x;
    const int n_row_tiles = (n + 15) >> 4;
    const int n_rt_mine = (n_row_tiles - (int)blockIdx.x + G - 1) / G;
    const int n_mine = DUAL ? 2 * n_rt_mine : n_rt_mine;  // steps
    if (n_mine <= 0) return;
    auto row_tile_of = [&](int i) __attribute__((always_inline)) { return (int)blockIdx.x + (DUAL ? i >> 1 : i) * G; };

    const int grp = blockIdx.y;
    const int beg = offsets[grp], cnt = offsets[grp + 1] - beg;
    if (cnt == 0) return;  // the whole workgroup leaves together
    const int e = gexp[grp];
    const uint8_t *wa = Wa[e], *wb = DUAL ? Wb[e] : wa;
    const float limit = e >= cl.n_routed ? cl.shared : cl.routed;  // the expert's SwiGLU clamp

    // a row is 9 * waves pieces of 16 bytes: `full` whole instructions and one of `rem` lanes; every
    // wave copies rows wave, wave + waves, ... (clamped to 15: the same bytes to the same place)
    const int pieces = 9 * waves, full = pieces >> 6, rem = pieces & 63;
    const int rows_per_wave = (16 + waves - 1) / waves;
    const int loads_per_tile = rows_per_wave * (full + (rem ? 1 : 0));
    auto fetch = [&](int i, int slot) __attribute__((always_inline)) {
        const int ii = min(i, n_mine - 1);
        const uint8_t *base = (DUAL && (ii & 1)) ? wb : wa;
        const int row0 = 16 * row_tile_of(ii);
        for (int j = 0; j < rows_per_wave; j++) {
            const int r = min(wave + j * waves, 15);
            const uint8_t *src = base + (size_t)min(row0 + r, n - 1) * row_bytes + 16 * lane;
            const uint32_t dst = lds_offset_of(&ring[slot][r * row_lds]);
            for (int f = 0; f < full; f++) async_load16(src + 1024 * f, dst + 1024 * f);
            if (lane < rem) async_load16(src + 1024 * full, dst + 1024 * full);
        }
    };

    const int kw = k >> 2, kb = k >> 5;  // words a plane row, 32-element blocks a row
    const int shift = 4 * (g >> 1);       // this lane group's nibble
    int it = 0;                            // steps so far: the reduction buffers alternate with it
    float gate_keep = 0.0f;
    for (int m0 = 0; m0 < cnt; m0 += MQ_ROWS) {
        const int mc = min(MQ_ROWS, cnt - m0);
        const bool two = mc > 4;  // the same for the whole workgroup
        fetch(0, 0);
        fetch(1, 1);  // (a clamped copy of the first tile when the workgroup has one step only)
        // The A operands of this wave's column for the pass: lane (m, g) with m = 4 i + 2 p + plane.
        mq_i4 A[2][4];
        // and what lane (n, g) needs of activation row g of each quad afterwards: the eight scales and scaled sums
        float sx[2][8], xs[2][8];
        {
            const int i = nrow >> 2, p = (nrow >> 1) & 1, plane = nrow & 1;
            const bool mine = (g >> 1) == p;
#pragma unroll
            for (int q = 0; q < 2; q++) {
                const int ra = 4 * q + i, rs = 4 * q + g;
                const bool has_a = mine && ra < mc && (q == 0 || two), has_s = rs < mc && (q == 0 || two);
                const size_t xa = has_a ? (size_t)xsel[beg + m0 + ra] : 0, xr = has_s ? (size_t)xsel[beg + m0 + rs] : 0;
                const uint32_t *pl = (plane ? xq.xh : xq.xl) + xa * kw + 64 * wave + 8 * p + 4 * (g & 1);
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    const uint4 v = has_a ? *(const uint4 *)(pl + 16 * t) : uint4{0, 0, 0, 0};
                    A[q][t] = mq_i4{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
                }
                const float4 *sp = (const float4 *)(xq.sx + xr * kb + 8 * wave), *xp = (const float4 *)(xq.sxs + xr * kb + 8 * wave);
                const float4 z = float4{0.0f, 0.0f, 0.0f, 0.0f};
                const float4 s0 = has_s ? sp[0] : z, s1 = has_s ? sp[1] : z, x0 = has_s ? xp[0] : z, x1 = has_s ? xp[1] : z;
                sx[q][0] = s0.x, sx[q][1] = s0.y, sx[q][2] = s0.z, sx[q][3] = s0.w;
                sx[q][4] = s1.x, sx[q][5] = s1.y, sx[q][6] = s1.z, sx[q][7] = s1.w;
                xs[q][0] = x0.x, xs[q][1] = x0.y, xs[q][2] = x0.z, xs[q][3] = x0.w;
                xs[q][4] = x1.x, xs[q][5] = x1.y, xs[q][6] = x1.z, xs[q][7] = x1.w;
            }
        }
        qr_wait_loads(loads_per_tile);  // the first tile landed; the second may be in flight
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");

        // on entry to step i: tile i is in LDS and visible (the barrier just passed), tile i+1 in flight
        for (int i = 0; i < n_mine; i++, it++) {
            const bool more = i + 2 < n_mine;
            if (more) fetch(i + 2, (i + 2) % 3);  // the slot of tile i-1, which every wave finished reading before that barrier

            const uint8_t *blk = &ring[i % 3][nrow * row_lds + wave * 144];
            const uint4 hdr = *(const uint4 *)blk;
            // the eight scales and mins of the row's block as bytes, four to a word
            const uint32_t sc4[2] = {hdr.y & 0x3F3F3F3Fu, (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u)};
            const uint32_t mn4[2] = {hdr.z & 0x3F3F3F3Fu, ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u)};
            float accd[2] = {0.0f, 0.0f}, accm[2] = {0.0f, 0.0f};
            const mq_i4 zero = {0, 0, 0, 0};
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const uint4 qv = *(const uint4 *)(blk + 16 + 32 * t + 16 * (g & 1));
                const mq_i4 B = mq_i4{(int)((qv.x >> shift) & 0x0F0F0F0Fu), (int)((qv.y >> shift) & 0x0F0F0F0Fu),
                                      (int)((qv.z >> shift) & 0x0F0F0F0Fu), (int)((qv.w >> shift) & 0x0F0F0F0Fu)};
                const float sc0 = (float)((sc4[t >> 1] >> (16 * (t & 1))) & 0xFFu), sc1 = (float)((sc4[t >> 1] >> (16 * (t & 1) + 8)) & 0xFFu);
                const float mn0 = (float)((mn4[t >> 1] >> (16 * (t & 1))) & 0xFFu), mn1 = (float)((mn4[t >> 1] >> (16 * (t & 1) + 8)) & 0xFFu);
#pragma unroll
                for (int q = 0; q < 2; q++) {
                    if (q == 1 && !two) continue;
                    const mq_i4 C = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[q][t], B, zero, 0, 0, 0);
                    const float f0 = (float)((C[1] << 8) + C[0]) * sx[q][2 * t], f1 = (float)((C[3] << 8) + C[2]) * sx[q][2 * t + 1];
                    accd[q] = fmaf(sc0, f0, fmaf(sc1, f1, accd[q]));
                    accm[q] = fmaf(mn0, xs[q][2 * t], fmaf(mn1, xs[q][2 * t + 1], accm[q]));
                }
            }
            const float d = f16_bits(hdr.x), dmin = f16_bits(hdr.x >> 16);
            const int buf = it & 1;
            red[buf][wave][0][lane] = fmaf(d, accd[0], -dmin * accm[0]);
            if (two) red[buf][wave][1][lane] = fmaf(d, accd[1], -dmin * accm[1]);
            // the partial sums are written and tile i+1 has landed: at most this step's loads stay in flight
            qr_wait_loads(more ? loads_per_tile : 0);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            // thread o < 128 takes output (quad o / 64, lane o % 64): weight row o % 16 of the tile, activation row
            // 4 (o / 64) + (o % 64) / 16; the same outputs in every step
            if (tid < (two ? 128 : 64)) {
                const int q = tid >> 6, ol = tid & 63;
                float s = 0.0f;
                for (int w = 0; w < waves; w++) s += red[buf][w][q][ol];
                const int nn = 16 * row_tile_of(i) + (ol & 15), mm = 4 * q + (ol >> 4);
                if (DUAL && !(i & 1)) {
                    gate_keep = s;  // the same rows of the second table are the next step
                } else if (mm < mc && nn < n) {
                    Y[(size_t)yrow[beg + m0 + mm] * n + nn] = DUAL ? swiglu(gate_keep, s, limit) : s;
                }
            }
        }
    }
}

}  // namespace jq
