// Q4_K times 1 to 16 activation rows on the matrix cores, the weights travelling HBM -> LDS as
// asynchronous, fully coalesced loads.
//
// Arithmetic and register layout are those of kernels_mfma_q4k_stream.hpp (23-bit fixed-point
// activations as MFMA B operands in registers, weights as the exact f16 integers sc*q, one wave per
// 256-element column of the weight matrix).  What differs is the road the weights take: the waves
// of a workgroup copy every 16-row tile whole (rows of up to 16 super-blocks, 16-byte pieces, each
// instruction a contiguous stretch of a row) into a ring of three tiles in LDS, two tiles ahead of
// the arithmetic, and read their header and nibble bytes from there.  No vector register is spent
// on prefetching, which leaves room for 16 waves of a workgroup on a compute unit.  The
// activations arrive already quantised, as the records q4k_acts_prep writes (quantising them in
// every workgroup costs a compute unit about 10 us for 16 rows of 4096).
//
// GROUPED: blockIdx.y walks (expert, token list) groups of a mixture-of-experts layer; up to 16 of
// the group's activation rows at a time are gathered through `xsel`, results scatter through `yrow`.
// DUAL (grouped only): tiles alternate between the same rows of two tables (gate, up) and the
// result is silu(gate . x) * (up . x)  (reference: src/quantized_qwen3_moe.rs:397-401).
#pragma once
#include "kernels_mfma_q4k_stream.hpp"
#include "kernels_moe.hpp"

namespace jq {

__device__ __forceinline__ void qr_wait_loads(int n) {  // at most n vector memory loads stay in flight; LDS traffic done
    switch (n) {
#define JQ_W(N) case N: asm volatile("s_waitcnt vmcnt(" #N ") lgkmcnt(0)" ::: "memory"); break;
        JQ_W(1) JQ_W(2) JQ_W(3) JQ_W(4) JQ_W(5) JQ_W(6) JQ_W(7) JQ_W(8) JQ_W(9) JQ_W(10) JQ_W(11) JQ_W(12)
        JQ_W(13) JQ_W(14) JQ_W(15) JQ_W(16)
#undef JQ_W
    default: asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); break;
    }
}

// Bytes a row takes in LDS: padded by 16 so that the 16 rows one instruction reads spread over the banks.
__host__ __device__ constexpr int qr_row_lds(int nb) { return nb * 144 + 16; }

constexpr int QR_RED_STRIDE = 264;

template <int MAXNB, bool GROUPED, bool DUAL>
__global__ __launch_bounds__(1024) void q4k_ring_mfma(const uint8_t *__restrict__ W,
                                                      const uint8_t *const *__restrict__ Wa,
                                                      const uint8_t *const *__restrict__ Wb,
                                                      const uint8_t *__restrict__ acts, const int *__restrict__ gexp,
                                                      const int *__restrict__ offsets,
                                                      const int *__restrict__ xsel, const int *__restrict__ yrow,
                                                      float *__restrict__ Y, int m, int n, MoeClamp cl) {
    static_assert(!DUAL || GROUPED, "two tables only in the grouped form");
    __shared__ __attribute__((aligned(16))) uint8_t ring[3][16 * qr_row_lds(MAXNB)];
    // the waves' partial tiles; 264 floats a wave (256 + 8) so that lanes summing different waves'
    // partials of neighbouring outputs fall into different banks
    __shared__ __attribute__((aligned(16))) float red[2][MAXNB][QR_RED_STRIDE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;  // waves == k / 256
    const int col = lane & 15, kg = lane >> 4;
    const int row_bytes = waves * 144, row_lds = row_bytes + 16;
    const int G = (int)gridDim.x;
    // Row tiles blockIdx.x, blockIdx.x + G, ... are this workgroup's; with two tables every row tile
    // is two steps, table 0 then table 1.
    const int n_row_tiles = (n + 15) >> 4;
    const int n_rt_mine = (n_row_tiles - (int)blockIdx.x + G - 1) / G;
    const int n_mine = DUAL ? 2 * n_rt_mine : n_rt_mine;  // steps
    if (n_mine <= 0) return;
    auto row_tile_of = [&](int i) __attribute__((always_inline)) { return (int)blockIdx.x + (DUAL ? i >> 1 : i) * G; };

    int beg = 0, cnt = m;
    const uint8_t *wa = W, *wb = W;
    float limit = 0.0f;  // the expert's SwiGLU clamp
    if (GROUPED) {
        const int grp = blockIdx.y;
        beg = offsets[grp], cnt = offsets[grp + 1] - beg;
        if (cnt == 0) return;  // the whole workgroup leaves together
        const int e = gexp[grp];
        wa = Wa[e], wb = DUAL ? Wb[e] : wa;
        limit = e >= cl.n_routed ? cl.shared : cl.routed;
    }

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

    const int parts = waves >= 16 ? 4 : waves >= 8 ? 2 : 1, pshift = parts == 4 ? 2 : parts == 2 ? 1 : 0;
    int it = 0;  // tiles processed so far: the reduction buffers alternate with it
    float gate_keep[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int m0 = 0; m0 < cnt; m0 += 16) {
        const int mc = min(16, cnt - m0);
        fetch(0, 0);
        fetch(1, 1);  // (a clamped copy of the first tile when the workgroup has one tile only)
        // the prepared activations (q4k_acts_prep) come in while those tiles are on their way
        QsActs<1> A;
        const uint8_t *base = nullptr;  // this lane group's piece of slot 0 of its row's record
        if (col < mc) base = acts + ((size_t)(GROUPED ? xsel[beg + m0 + col] : col) * waves + wave) * QS_REC + kg * 16;
        qs_load_acts(base, kg, A);
        qr_wait_loads(loads_per_tile);  // the first tile landed; the second may be in flight
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");

        // on entry to step i: tile i is in LDS and visible (the barrier just passed), tile i+1 in flight
        for (int i = 0; i < n_mine; i++, it++) {
            const bool more = i + 2 < n_mine;
            if (more) fetch(i + 2, (i + 2) % 3);  // the slot of tile i-1, which every wave finished reading before that barrier

            QsTileRegs cur[1];
            const uint8_t *blk = &ring[i % 3][col * row_lds + wave * 144];
            cur[0].hdr = *(const qg_u4 *)blk;
#pragma unroll
            for (int c = 0; c < 4; c++) cur[0].nib[c] = *(const uint2 *)(blk + 16 + 32 * c + 8 * kg);
#pragma unroll
            for (int jj = 0; jj < 4; jj++)
                cur[0].dm[jj] = *(const uint32_t *)&ring[i % 3][(4 * kg + jj) * row_lds + wave * 144];
            float acc[4];
            qs_tile_partial<1>(cur, A, kg, acc);

            const int buf = it & 1;
            *(qg_f4 *)&red[buf][wave][4 * lane] = qg_f4{acc[0], acc[1], acc[2], acc[3]};
            // the partial tile is written and tile i+1 has landed: at most this step's loads stay in flight
            qr_wait_loads(more ? loads_per_tile : 0);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            // output o of the tile's 256: weight row 4 * (o / 64) + o % 4, activation row (o / 4) % 16.
            // `parts` neighbouring lanes share an output, each summing every parts-th wave's partial;
            // a thread takes the same outputs in every step.
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int idx = tid + q * (int)blockDim.x;
                if (idx < 256 * parts && (q == 0 || blockDim.x < 256)) {  // whole waves pass (or fail) this test
                    const int o = idx >> pshift, p = idx & (parts - 1);
                    float s = 0.0f;
                    for (int w = p; w < waves; w += parts) s += red[buf][w][o];
                    if (parts >= 2) s += dpp_f<0xB1>(s);  // the neighbour: quad_perm [1,0,3,2]
                    if (parts == 4) s += dpp_f<0x4E>(s);  // the other pair: quad_perm [2,3,0,1]
                    const int src_lane = o >> 2, jj = o & 3;
                    const int nn = 16 * row_tile_of(i) + 4 * (src_lane >> 4) + jj, mm = src_lane & 15;
                    if (DUAL && !(i & 1)) {
                        gate_keep[q] = s;  // the same rows of the second table are the next step
                    } else if (p == 0 && mm < mc && nn < n) {
                        const size_t yr = GROUPED ? (size_t)yrow[beg + m0 + mm] : (size_t)mm;
                        Y[yr * n + nn] = DUAL ? swiglu(gate_keep[q], s, limit) : s;
                    }
                }
            }
        }
    }
}

}  // namespace jq
