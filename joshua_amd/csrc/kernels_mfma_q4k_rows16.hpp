// Q4_K matmul for 2..16 activation rows over weight rows of 4096 columns (longer rows: one launch per
// group of 4096 columns, the later ones adding to the result): the weight stream of the one-row
// GEMV (q4k_gemv_dot4_lds: asynchronous loads into a ring of three 16-row tiles in LDS, one wave per
// super-block column) with the integer dot products on the int8 matrix cores.
//
// Per 32-element sub-block j of a weight row and activation row i (reference arithmetic
// w = d sc q - dmin m, src/kquant_dot.rs:440-465):
//
//   sum_k x_ik w_k = (d sc_j) s_ij S_ij - (dmin m_j) s_ij XS_ij,  S_ij = sum_k q_k X_ik,  XS_ij = sum_k X_ik
//
// with X = round(x / s_ij), s_ij = amax_j(x_i) / 32639: 16-bit fixed point per (activation row, sub-block),
// two byte planes X = 256 Xh + Xl, exactly the one-row kernel's quantisation.  One
// v_mfma_i32_16x16x32_i8 per plane gives the 16 x 16 sums S over a sub-block's 32 elements (activation
// rows x weight rows), exact in int32; the min term is an f32 MFMA over the eight sub-blocks of a
// super-block (16x16x4, twice).  The activations arrive prepared as MFMA operands by q4k_acts16_prep
// (one small launch), so the 256 workgroups do not each repeat that work.
#pragma once
#include "kernels_dot4_q4k.hpp"

namespace jq {

// Per 256-element column of the activations: 8 sub-blocks x 64 lanes x 16 bytes of plane operands
// (lane (i = lane % 16, g = lane / 16): elements 8g .. 8g+7 of sub-block j in row i; high plane, then
// low plane), then the scales s[i][j] and the scaled sums s[i][j] XS[i][j] as 16 x 8 floats each.
constexpr int QM_PLANES = 8 * 64 * 16, QM_REC = QM_PLANES + 2 * 512;
constexpr int QM_RED_STRIDE = 260;  // floats a wave in the reduction buffer: the four quarter-sums a lane group reads fall into different banks

typedef int qm_i4 __attribute__((ext_vector_type(4)));
typedef float qm_f4 __attribute__((ext_vector_type(4)));

// grid (8 sub-blocks, k / 256 columns, groups of 16 activation rows), one wave.  Rows from m_rows on
// are zero operands.
__global__ __launch_bounds__(64) void q4k_acts16_prep(const float *__restrict__ X, int m_rows, int k,
                                                       uint8_t *__restrict__ out) {
    const int lane = threadIdx.x, i = lane & 15, g = lane >> 4, j = blockIdx.x, col = blockIdx.y;
    const int row = 16 * (int)blockIdx.z + i;
    uint8_t *rec = out + ((size_t)blockIdx.z * gridDim.y + col) * QM_REC;
    float v[8];
    if (row < m_rows) {
        const float4 a = *(const float4 *)(X + (size_t)row * k + 256 * col + 32 * j + 8 * g);
        const float4 b = *(const float4 *)(X + (size_t)row * k + 256 * col + 32 * j + 8 * g + 4);
        v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = 0.0f;
    }
    float amax = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; e++) amax = fmaxf(amax, mag_or_inf(v[e]));
    amax = max_xor32(max_xor16(amax));  // the four lanes that share (row, sub-block)
    const bool live = amax > 0.0f && amax < INFINITY;
    const float inv = live ? QD_RANGE / amax : 0.0f, s = fixed_scale(amax, QD_RANGE);
    uint32_t h[2] = {0, 0}, l[2] = {0, 0};
    int sum = 0;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        const int Xq = __float2int_rn(v[e] * inv);
        const int lo = ((Xq + 128) & 255) - 128, hi = (Xq - lo) >> 8;
        l[e >> 2] |= (uint32_t)(lo & 255) << (8 * (e & 3));
        h[e >> 2] |= (uint32_t)(hi & 255) << (8 * (e & 3));
        sum += Xq;
    }
    sum = isum_xor32(isum_xor16(sum));
    *(uint4 *)(rec + ((size_t)j * 64 + lane) * 16) = uint4{h[0], h[1], l[0], l[1]};
    if (g == 0) {
        ((float *)(rec + QM_PLANES))[i * 8 + j] = s;
        ((float *)(rec + QM_PLANES + 512))[i * 8 + j] = s * (float)sum;
    }
}

// grid G workgroups of 16 waves; tiles blockIdx.x, blockIdx.x + G, ... of 16 weight rows.  Wave w owns
// super-block column w.  In the MFMAs the activations are the A operand and the weights the B operand, so
// a lane ends up with weight row lane % 16 (whose eight sub-block scales it decodes for itself, four
// bytes at a time) and activation rows 4 (lane / 16) .. + 3.  Y is m_rows x n.
// W points at the first of the 16 super-blocks this launch covers in row 0, rows are row_bytes apart; with
// `accumulate` the sums are added to what Y holds (rows longer than 4096: one launch per group of 4096
// columns, in column order).
__global__ __launch_bounds__(1024) void q4k_rows16_mfma(const uint8_t *__restrict__ W, const uint8_t *__restrict__ acts,
                                                        float *__restrict__ Y, int m_rows, int n, int G,
                                                        size_t row_bytes, int accumulate) {
    __shared__ __attribute__((aligned(16))) uint8_t ring[3][QD_TILE_LDS];
    __shared__ float red[2][16 * QM_RED_STRIDE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, g = lane >> 4;
    const int n_tiles = (((n + 15) >> 4) - (int)blockIdx.x + G - 1) / G;
    if (n_tiles <= 0) return;

    auto fetch = [&](int i, int slot) __attribute__((always_inline)) {
        const int row = min(16 * ((int)blockIdx.x + min(i, n_tiles - 1) * G) + wave, n - 1);
        const uint8_t *src = W + (size_t)row * row_bytes + 16 * lane;
        const uint32_t dst = lds_offset_of(&ring[slot][wave * QD_ROW_LDS]);
        async_load16(src, dst);
        async_load16(src + 1024, dst + 1024);
        if (lane < 16) async_load16(src + 2048, dst + 2048);
    };
    fetch(0, 0);

    // this wave's activation operands (plain loads: the compiler waits for them, and with them for tile 0,
    // in front of the empty statements below, which read the registers)
    const uint8_t *rec = acts + (size_t)wave * QM_REC;
    uint4 ap[8];
#pragma unroll
    for (int j = 0; j < 8; j++) ap[j] = *(const uint4 *)(rec + ((size_t)j * 64 + lane) * 16);
    float4 sxa[4], sxb[4];  // s[4g + rr][0..3], s[4g + rr][4..7]
#pragma unroll
    for (int rr = 0; rr < 4; rr++) {
        sxa[rr] = *(const float4 *)(rec + QM_PLANES + ((4 * g + rr) * 8) * 4);
        sxb[rr] = *(const float4 *)(rec + QM_PLANES + ((4 * g + rr) * 8 + 4) * 4);
    }
    float xs0 = ((const float *)(rec + QM_PLANES + 512))[r * 8 + g], xs1 = ((const float *)(rec + QM_PLANES + 512))[r * 8 + g + 4];
#pragma unroll
    for (int j = 0; j < 8; j++) asm volatile("" : "+v"(ap[j].x), "+v"(ap[j].y), "+v"(ap[j].z), "+v"(ap[j].w));
#pragma unroll
    for (int rr = 0; rr < 4; rr++) {
        asm volatile("" : "+v"(sxa[rr].x), "+v"(sxa[rr].y), "+v"(sxa[rr].z), "+v"(sxa[rr].w));
        asm volatile("" : "+v"(sxb[rr].x), "+v"(sxb[rr].y), "+v"(sxb[rr].z), "+v"(sxb[rr].w));
    }
    asm volatile("" : "+v"(xs0), "+v"(xs1));
    // tile 1 is asked for once tile 0 has landed, as in the one-row kernel
    if (n_tiles > 1) {
        fetch(1, 1);
        asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory");
    } else {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");

    const float sx[4][8] = {{sxa[0].x, sxa[0].y, sxa[0].z, sxa[0].w, sxb[0].x, sxb[0].y, sxb[0].z, sxb[0].w},
                            {sxa[1].x, sxa[1].y, sxa[1].z, sxa[1].w, sxb[1].x, sxb[1].y, sxb[1].z, sxb[1].w},
                            {sxa[2].x, sxa[2].y, sxa[2].z, sxa[2].w, sxb[2].x, sxb[2].y, sxb[2].z, sxb[2].w},
                            {sxa[3].x, sxa[3].y, sxa[3].z, sxa[3].w, sxb[3].x, sxb[3].y, sxb[3].z, sxb[3].w}};
    const qm_i4 zero_i = {0, 0, 0, 0};
    const qm_f4 zero_f = {0.0f, 0.0f, 0.0f, 0.0f};
    auto as_long = [](uint32_t lo, uint32_t hi) __attribute__((always_inline)) { return (long)(((uint64_t)hi << 32) | lo); };

    for (int t = 0; t < n_tiles; t++) {
        const int slot = t % 3;
        const bool more = t + 2 < n_tiles;
        if (more) fetch(t + 2, (t + 2) % 3);

        const uint8_t *blk = &ring[slot][r * QD_ROW_LDS + wave * 144];
        const uint4 hdr = *(const uint4 *)blk;
        uint2 qq[4];
#pragma unroll
        for (int i = 0; i < 4; i++) qq[i] = *(const uint2 *)(blk + 16 + 32 * i + 8 * g);

        // the eight 6-bit scales and mins of this lane's weight row, four to a register
        const uint32_t sc4[2] = {hdr.y & 0x3F3F3F3Fu, (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u)};
        const uint32_t mn4[2] = {hdr.z & 0x3F3F3F3Fu, ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u)};
        // min term: sum_j (s XS)[i][j] m_j over the eight sub-blocks, k = lane / 16 (sub-blocks g and g + 4)
        const float mn_a = (float)((mn4[0] >> (8 * g)) & 0xFFu), mn_b = (float)((mn4[1] >> (8 * g)) & 0xFFu);
        qm_f4 msum = __builtin_amdgcn_mfma_f32_16x16x4f32(xs0, mn_a, zero_f, 0, 0, 0);
        msum = __builtin_amdgcn_mfma_f32_16x16x4f32(xs1, mn_b, msum, 0, 0, 0);

        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int hl = 0; hl < 2; hl++) {
                const int j = 2 * i + hl;
                const uint32_t b0 = hl ? (qq[i].x >> 4) & 0x0F0F0F0Fu : qq[i].x & 0x0F0F0F0Fu;
                const uint32_t b1 = hl ? (qq[i].y >> 4) & 0x0F0F0F0Fu : qq[i].y & 0x0F0F0F0Fu;
                const long b = as_long(b0, b1);
                const qm_i4 Sh = __builtin_amdgcn_mfma_i32_16x16x32_i8(as_long(ap[j].x, ap[j].y), b, zero_i, 0, 0, 0);
                const qm_i4 Sl = __builtin_amdgcn_mfma_i32_16x16x32_i8(as_long(ap[j].z, ap[j].w), b, zero_i, 0, 0, 0);
                const float sc = (float)((sc4[j >> 2] >> (8 * (j & 3))) & 0xFFu);
#pragma unroll
                for (int rr = 0; rr < 4; rr++)
                    acc[rr] = fmaf((float)((Sh[rr] << 8) + Sl[rr]) * sx[rr][j], sc, acc[rr]);
            }
        }
        const float d = f16_bits(hdr.x), dmin = f16_bits(hdr.x >> 16);
        const int buf = t & 1;
#pragma unroll
        for (int rr = 0; rr < 4; rr++) red[buf][wave * QM_RED_STRIDE + rr * 64 + lane] = fmaf(-dmin, msum[rr], d * acc[rr]);

        if (more) asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // wave w sums activation row w over the 16 waves: lane (o = lane % 16, p = lane / 16) takes weight
        // row o and waves 4p .. 4p + 3
        {
            const float *src = &red[buf][(wave & 3) * 64 + 16 * (wave >> 2) + r];
            float v = (src[(4 * g) * QM_RED_STRIDE] + src[(4 * g + 1) * QM_RED_STRIDE]) +
                      (src[(4 * g + 2) * QM_RED_STRIDE] + src[(4 * g + 3) * QM_RED_STRIDE]);
            v = sum_xor16(v);
            v = sum_xor32(v);
            const int row = 16 * ((int)blockIdx.x + t * G) + r;
            if (lane < 16 && wave < m_rows && row < n) {
                float *yp = Y + (size_t)wave * n + row;
                *yp = accumulate ? *yp + v : v;
            }
        }
    }
}

// The same product for rows of 4096 columns as one launch: every workgroup quantises the activations itself (wave w
// its column of all 16 rows, while the first two tiles travel), the weight rows come by scalar-base asynchronous
// loads with a tile's arithmetic in front of the request for the tile after next, one barrier a tile (the sums of
// tile t - 1 are added over the waves behind tile t's barrier), and a wave stores its activation row's results once
// per four tiles.  rounds / extra: tiles a workgroup, and how many workgroups take one more.
// OWN_PREP false: the operands come prepared by q4k_acts16_prep (`acts`), as for q4k_rows16_mfma.
template <bool OWN_PREP>
__global__ __launch_bounds__(1024) void q4k_rows16_lds(const uint8_t *__restrict__ W, const float *__restrict__ X,
                                                       const uint8_t *__restrict__ acts, float *__restrict__ Y, int m_rows,
                                                       int n, int G, int rounds, int extra, int k) {
    constexpr int LOADS = 3;
    __shared__ __attribute__((aligned(16))) uint8_t ring[3][QD_TILE_LDS];
    __shared__ __attribute__((aligned(16))) float red[2][16 * QM_RED_STRIDE];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4, b = (int)blockIdx.x;
    const int nt = rounds + (b < extra ? 1 : 0);
    if (nt <= 0) return;
    // this lane's share of the activations: row r, elements 8g .. 8g + 7 of each sub-block of column `wave`
    float4 xa[8], xb[8];
    uint4 ap[8];
    float sx[4][8], xs0, xs1;
    if (OWN_PREP) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            if (r < m_rows) {
                const float *src = X + (size_t)r * k + 256 * wave + 32 * j + 8 * g;
                xa[j] = *(const float4 *)src, xb[j] = *(const float4 *)(src + 4);
            } else {
                xa[j] = xb[j] = float4{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
    } else {
        const uint8_t *rec = acts + (size_t)wave * QM_REC;
#pragma unroll
        for (int j = 0; j < 8; j++) ap[j] = *(const uint4 *)(rec + ((size_t)j * 64 + lane) * 16);
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
            const float4 a = *(const float4 *)(rec + QM_PLANES + ((4 * g + rr) * 8) * 4);
            const float4 c = *(const float4 *)(rec + QM_PLANES + ((4 * g + rr) * 8 + 4) * 4);
            sx[rr][0] = a.x, sx[rr][1] = a.y, sx[rr][2] = a.z, sx[rr][3] = a.w;
            sx[rr][4] = c.x, sx[rr][5] = c.y, sx[rr][6] = c.z, sx[rr][7] = c.w;
        }
        xs0 = ((const float *)(rec + QM_PLANES + 512))[r * 8 + g], xs1 = ((const float *)(rec + QM_PLANES + 512))[r * 8 + g + 4];
    }
    const uint32_t ring0 = lds_offset_of(&ring[0][0]);
    auto fetch = [&](int slot_i) __attribute__((always_inline)) {
        const int i = min(slot_i, nt - 1);
        const int row = min(16 * (b + i * G) + wave, n - 1);
        const uint8_t *src = W + (size_t)row * QD_ROW;
        const uint32_t dst = ring0 + (uint32_t)(slot_i % 3) * QD_TILE_LDS + (uint32_t)wave * QD_ROW_LDS;
        async_load16_s(src, 16 * lane, dst);
        async_load16_s(src + 1024, 16 * lane, dst + 1024);
        if (lane < 16) async_load16_s(src + 2048, 16 * lane, dst + 2048);
    };
    fetch(0);
    fetch(1);
    // operands: per sub-block the high and the low plane of the lane's eight elements; the (row, sub-block) scales
    // and scaled sums go through this wave's kilobyte of the partial-sum buffer, which nobody writes before the
    // first tile's barrier
    if (OWN_PREP) {
        float *side_s = &red[0][wave * 256], *side_xs = side_s + 128;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float v[8] = {xa[j].x, xa[j].y, xa[j].z, xa[j].w, xb[j].x, xb[j].y, xb[j].z, xb[j].w};
            float amax = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; e++) amax = fmaxf(amax, mag_or_inf(v[e]));
            amax = max_xor32(max_xor16(amax));  // the four lanes that share (row, sub-block)
            const bool live = amax > 0.0f && amax < INFINITY;
            const float inv = live ? QD_RANGE / amax : 0.0f, sc = fixed_scale(amax, QD_RANGE);
            uint32_t h[2] = {0, 0}, l[2] = {0, 0};
            int sum = 0;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int Xq = __float2int_rn(v[e] * inv);
                const int lo = ((Xq + 128) & 255) - 128, hi = (Xq - lo) >> 8;
                l[e >> 2] |= (uint32_t)(lo & 255) << (8 * (e & 3));
                h[e >> 2] |= (uint32_t)(hi & 255) << (8 * (e & 3));
                sum += Xq;
            }
            sum = isum_xor32(isum_xor16(sum));
            ap[j] = uint4{h[0], h[1], l[0], l[1]};
            if (g == 0) side_s[r * 8 + j] = sc, side_xs[r * 8 + j] = sc * (float)sum;
        }
        asm volatile("" ::: "memory");
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
            const float4 a = *(const float4 *)&side_s[(4 * g + rr) * 8], c = *(const float4 *)&side_s[(4 * g + rr) * 8 + 4];
            sx[rr][0] = a.x, sx[rr][1] = a.y, sx[rr][2] = a.z, sx[rr][3] = a.w;
            sx[rr][4] = c.x, sx[rr][5] = c.y, sx[rr][6] = c.z, sx[rr][7] = c.w;
        }
        xs0 = side_xs[r * 8 + g], xs1 = side_xs[r * 8 + g + 4];
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }

    const qm_i4 zero_i = {0, 0, 0, 0};
    const qm_f4 zero_f = {0.0f, 0.0f, 0.0f, 0.0f};
    auto as_long = [](uint32_t lo, uint32_t hi) __attribute__((always_inline)) { return (long)(((uint64_t)hi << 32) | lo); };
    float keep = 0.0f;
    // wave w adds activation row w's sums of tile tt over the 16 waves (lane (o, p): weight row o, waves 4p .. 4p + 3),
    // keeps them in lane group tt % 4 and stores four tiles' worth at once
    auto reduce = [&](int tt) __attribute__((always_inline)) {
        const float *src = &red[tt & 1][(wave & 3) * 64 + 16 * (wave >> 2) + r];
        float v = (src[(4 * g) * QM_RED_STRIDE] + src[(4 * g + 1) * QM_RED_STRIDE]) +
                  (src[(4 * g + 2) * QM_RED_STRIDE] + src[(4 * g + 3) * QM_RED_STRIDE]);
        v = sum_xor16(v);
        v = sum_xor32(v);
        if (g == (tt & 3)) keep = v;
        if ((tt & 3) == 3 || tt == nt - 1) {
            const int mine = (tt & ~3) + g, row = 16 * (b + mine * G) + r;
            if (mine <= tt && wave < m_rows && row < n) Y[(size_t)wave * n + row] = keep;
        }
    };
    for (int t = 0; t < nt; t++) {
        if (t + 1 < nt) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(LOADS) : "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (t > 0) reduce(t - 1);
        const uint8_t *blk = &ring[t % 3][r * QD_ROW_LDS + wave * 144];
        const uint4 hdr = *(const uint4 *)blk;
        uint2 qq[4];
#pragma unroll
        for (int i = 0; i < 4; i++) qq[i] = *(const uint2 *)(blk + 16 + 32 * i + 8 * g);
        const uint32_t sc4[2] = {hdr.y & 0x3F3F3F3Fu, (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u)};
        const uint32_t mn4[2] = {hdr.z & 0x3F3F3F3Fu, ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u)};
        const float mn_a = (float)((mn4[0] >> (8 * g)) & 0xFFu), mn_b = (float)((mn4[1] >> (8 * g)) & 0xFFu);
        qm_f4 msum = __builtin_amdgcn_mfma_f32_16x16x4f32(xs0, mn_a, zero_f, 0, 0, 0);
        msum = __builtin_amdgcn_mfma_f32_16x16x4f32(xs1, mn_b, msum, 0, 0, 0);
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int hl = 0; hl < 2; hl++) {
                const int j = 2 * i + hl;
                const uint32_t b0 = hl ? (qq[i].x >> 4) & 0x0F0F0F0Fu : qq[i].x & 0x0F0F0F0Fu;
                const uint32_t b1 = hl ? (qq[i].y >> 4) & 0x0F0F0F0Fu : qq[i].y & 0x0F0F0F0Fu;
                const long bq = as_long(b0, b1);
                const qm_i4 Sh = __builtin_amdgcn_mfma_i32_16x16x32_i8(as_long(ap[j].x, ap[j].y), bq, zero_i, 0, 0, 0);
                const qm_i4 Sl = __builtin_amdgcn_mfma_i32_16x16x32_i8(as_long(ap[j].z, ap[j].w), bq, zero_i, 0, 0, 0);
                const float sc = (float)((sc4[j >> 2] >> (8 * (j & 3))) & 0xFFu);
#pragma unroll
                for (int rr = 0; rr < 4; rr++) acc[rr] = fmaf((float)((Sh[rr] << 8) + Sl[rr]) * sx[rr][j], sc, acc[rr]);
            }
        }
        const float d = f16_bits(hdr.x), dmin = f16_bits(hdr.x >> 16);
#pragma unroll
        for (int rr = 0; rr < 4; rr++) red[t & 1][wave * QM_RED_STRIDE + rr * 64 + lane] = fmaf(-dmin, msum[rr], d * acc[rr]);
        // every wave has passed this tile's barrier: all are done with tile t - 1, whose slot tile t + 2 takes
        if (t + 2 < nt) fetch(t + 2);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    reduce(nt - 1);
}

}  // namespace jq
