// Q4_K prefill GEMM (more than 16 activation rows) on the matrix cores.
//
// Per 256-element super-block B of a weight row n and an activation row m
//
//   sum_k x_k w_k = s (d I1 - dmin I2)
//   I1 = sum_k (sc_j(k) q_k) X_k          I2 = sum_j m_j XS_j,  XS_j = sum_{k in j} X_k
//
// where X = round(x / s), s = amax_B(x) / 4193279, is the activation in 23-bit fixed
// point per (row, super-block), and (sc_j, m_j) are the 6-bit sub-block scale and
// min of Q4_K (reference arithmetic: w = d sc q - dmin m, src/kquant_dot.rs:440-465).
//
// The factors go to v_mfma_f32_16x16x32_f16 as exactly representable f16 integers:
// sc q <= 945, and X = 2048 Xh + Xl with |Xh| <= 2047, -1024 <= Xl < 1024, so every
// product is exact and I1 = 2048 Ph + Pl with f32 accumulation over the 256 k of one
// super-block.  A single int8 activation plane (error 2^-8 of the group maximum)
// cannot meet the 1e-3 bound on the results, and int8 planes of equal accuracy need
// six MFMAs per tile and k step (two for sc q, three for X) against four here.
// I2 is one more MFMA per tile and super-block over XS / 4096 split three ways into
// f16.  One f32 combination per super-block applies d, dmin and s.
//
// Workgroup: 128 weight rows x 64*MI activation rows, 8 waves = 2 (weight rows) x 4
// (activation rows); a wave owns 64 x 16*MI outputs.  Weight nibbles are unpacked,
// multiplied by their sub-block scale and converted while being staged into LDS in
// MFMA operand order; the activation planes come prepared in operand order from
// q4k_gemm_prep and are copied global -> registers -> LDS.  LDS is double buffered
// by 64-k chunk and staged one chunk ahead; even and odd waves run their staging
// and MFMA phases in opposite order so the two waves of a SIMD overlap them.
#pragma once
#include "kernels_mfma_q4k.hpp"

namespace jq {

constexpr int QG_NT = 128;                 // weight rows per workgroup
constexpr float QG_RANGE = 4193279.0f;     // 2047 * 2048 + 1023

typedef _Float16 qg_h2 __attribute__((ext_vector_type(2)));
typedef _Float16 qg_h8 __attribute__((ext_vector_type(8)));
typedef float qg_f4 __attribute__((ext_vector_type(4)));
typedef uint32_t qg_u4 __attribute__((ext_vector_type(4)));

// Prepared activations, m_pad = a whole number of workgroup tiles, rows >= m zero.
//   planes: [m_pad/16][k/64][kstep 2][plane 2 (Xh, Xl)][lane 64][8 halves]; lane = m%16 + 16*((k%32)/8),
//           the 8 k of a lane stored in the order 0,2,1,3,4,6,5,7 (the order the weight unpack produces)
//   mins:   [m_pad/16][k/256][lane 64][8 halves]; lane = m%16 + 16*g, g = 0,1,2: the three f16 parts of
//           XS_j / 4096 for j = 0..7, g = 3: zeros
//   scale:  [m_pad][k/256]
struct Q4kGemmActs {
    _Float16 *planes;
    _Float16 *mins;
    float *scale;
};

__device__ __forceinline__ uint32_t qg_pack_h2(int a, int b) {  // two small integers as f16
    const qg_h2 v = qg_h2{(_Float16)(float)a, (_Float16)(float)b};
    return __builtin_bit_cast(uint32_t, v);
}

// One wave per (activation row, super-block).
__global__ __launch_bounds__(256) void q4k_gemm_prep(const float *__restrict__ x, int m, int m_pad, int k,
                                                      Q4kGemmActs a) {
    const int nb = k >> 8, nch = k >> 6;
    const size_t unit = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (unit >= (size_t)m_pad * nb) return;
    const int row = (int)(unit / nb), b = (int)(unit % nb), lane = threadIdx.x & 63;
    float4 v = float4{0.0f, 0.0f, 0.0f, 0.0f};
    if (row < m) v = *(const float4 *)(x + (size_t)row * k + 256 * b + 4 * lane);
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    const bool live = amax > 0.0f && amax < INFINITY;
    const float inv = live ? QG_RANGE / amax : 0.0f;
    int X[4] = {__float2int_rn(v.x * inv), __float2int_rn(v.y * inv), __float2int_rn(v.z * inv), __float2int_rn(v.w * inv)};
    int lo[4], hi[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        lo[i] = ((X[i] + 1024) & 2047) - 1024;
        hi[i] = (X[i] - lo[i]) >> 11;
    }
    // element k = 256 b + 4 lane + i
    const int kk = 4 * lane;                       // within the super-block
    const int chunk = 4 * b + (kk >> 6), kstep = (kk >> 5) & 1, g = (kk >> 3) & 3, pos = kk & 7;  // pos 0 or 4
    const int mt = row >> 4, ol = (row & 15) + 16 * g;
    const size_t base = ((((size_t)mt * nch + chunk) * 2 + kstep) * 2) * 64;  // in lanes, plane 0
    uint2 *ph = (uint2 *)(a.planes + ((base + ol) * 8 + pos));
    uint2 *pl = (uint2 *)(a.planes + ((base + 64 + ol) * 8 + pos));
    *ph = uint2{qg_pack_h2(hi[0], hi[2]), qg_pack_h2(hi[1], hi[3])};
    *pl = uint2{qg_pack_h2(lo[0], lo[2]), qg_pack_h2(lo[1], lo[3])};
    int xs = X[0] + X[1] + X[2] + X[3];  // sub-block j = lanes 8j .. 8j+7
    xs += __shfl_xor(xs, 1, 64), xs += __shfl_xor(xs, 2, 64), xs += __shfl_xor(xs, 4, 64);
    if ((lane & 7) == 0) {
        const int j = lane >> 3;
        const double val = (double)xs * (1.0 / 4096.0);
        const _Float16 p0 = (_Float16)val;
        const double r1 = val - (double)p0;
        const _Float16 p1 = (_Float16)r1;
        const _Float16 p2 = (_Float16)(r1 - (double)p1);
        _Float16 *o = a.mins + (((size_t)mt * nb + b) * 64 + (row & 15)) * 8 + j;
        o[0] = p0, o[16 * 8] = p1, o[32 * 8] = p2, o[48 * 8] = (_Float16)0.0f;
    }
    if (lane == 0) a.scale[(size_t)row * nb + b] = live ? amax / QG_RANGE : 0.0f;
}

// (sc * q) of the nibbles sitting in bits 0-3 and 16-19 of `two`, as two f16.
__device__ __forceinline__ uint32_t qg_scaled_h2(uint32_t two, uint32_t sc) {
    const uint32_t bits = (two * sc) | 0x64006400u;  // f16 of 1024 + sc q, sc q <= 945
    const qg_h2 v = __builtin_bit_cast(qg_h2, bits) - qg_h2{(_Float16)1024.0f, (_Float16)1024.0f};
    return __builtin_bit_cast(uint32_t, v);
}

template <int MI>  // 16-row activation tiles per wave
__global__ __launch_bounds__(512) void q4k_gemm_mfma(const uint8_t *__restrict__ W, size_t row_bytes, Q4kGemmActs acts,
                                                      float *__restrict__ Y, int m, int m_pad, int k, int n,
                                                      int m_tiles, int total_tiles) {
    constexpr int MT = 64 * MI;          // activation rows per workgroup
    constexpr int MT16 = 4 * MI;         // 16-row activation tiles per workgroup
    constexpr int A_U4 = 2 * 8 * 64;     // uint4 per A buffer:  [kstep][ntile 8][lane]
    constexpr int B_U4 = 2 * 2 * MT16 * 64;  // [kstep][plane][mtile][lane]
    extern __shared__ uint4 qg_lds[];
    uint4 *a_lds = qg_lds;                    // 2 buffers
    uint4 *b_lds = qg_lds + 2 * A_U4;         // 2 buffers
    uint4 *min_lds = b_lds + 2 * B_U4;        // [2 (super-block parity)][128 rows]: the eight mins as f16
    float *d_lds = (float *)(min_lds + 2 * QG_NT);  // [2][128]
    float *dmin_lds = d_lds + 2 * QG_NT;            // [2][128]

    // XCD-aware order: consecutive workgroup ids go round-robin over the 8 XCDs; make the tiles
    // an XCD works on consecutive, so the activation tiles of one weight tile share an L2.
    const int per_xcd = (total_tiles + 7) >> 3;
    const int logical = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (logical >= total_tiles) return;
    const int mt = logical % m_tiles, nt = logical / m_tiles;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave & 1, wm = wave >> 1;
    const int nb = k >> 8, nch = k >> 6;
    const int col = lane & 15, kg = lane >> 4;
    const int m0 = mt * MT + wm * 16 * MI;       // first activation row of this wave
    const bool wave_live = m0 < m;

    // staging roles
    const int ar = tid >> 2, aq = tid & 3;        // weight row of the tile, 8-byte piece of the chunk's 32 nibble bytes
    const uint8_t *wrow = W + (size_t)min(nt * QG_NT + ar, n - 1) * row_bytes;
    const qg_u4 *bsrc = (const qg_u4 *)acts.planes + (size_t)(mt * MT16) * nch * 256;  // + (mtile*nch + chunk)*256 + idx

    uint2 a_reg;
    uint4 h_reg;
    qg_u4 b_reg[2 * MI];

    auto load_chunk = [&](int c) __attribute__((always_inline)) {
        const uint8_t *blk = wrow + (size_t)(c >> 2) * 144;
        h_reg = *(const uint4 *)blk;
        a_reg = *(const uint2 *)(blk + 16 + 32 * (c & 3) + 8 * aq);
#pragma unroll
        for (int i = 0; i < 2 * MI; i++) {
            const int idx = tid + 512 * i;  // of MT16 * 256 uint4
            b_reg[i] = bsrc[((size_t)(idx >> 8) * nch + c) * 256 + (idx & 255)];
        }
    };
    auto store_chunk = [&](int c) __attribute__((always_inline)) {
        const int buf = c & 1, cc = c & 3;
        uint32_t sc_lo, mn_lo, sc_hi, mn_hi;
        q4k_scale_min(h_reg.y, h_reg.z, h_reg.w, 2 * cc, sc_lo, mn_lo);
        q4k_scale_min(h_reg.y, h_reg.z, h_reg.w, 2 * cc + 1, sc_hi, mn_hi);
        const uint32_t w0 = a_reg.x, w1 = a_reg.y;
        // operand order within the 8 k of a lane: 0,2,1,3,4,6,5,7
        const uint4 lo = uint4{qg_scaled_h2(w0 & 0x000F000Fu, sc_lo), qg_scaled_h2((w0 >> 8) & 0x000F000Fu, sc_lo),
                               qg_scaled_h2(w1 & 0x000F000Fu, sc_lo), qg_scaled_h2((w1 >> 8) & 0x000F000Fu, sc_lo)};
        const uint4 hi = uint4{qg_scaled_h2((w0 >> 4) & 0x000F000Fu, sc_hi), qg_scaled_h2((w0 >> 12) & 0x000F000Fu, sc_hi),
                               qg_scaled_h2((w1 >> 4) & 0x000F000Fu, sc_hi), qg_scaled_h2((w1 >> 12) & 0x000F000Fu, sc_hi)};
        uint4 *ab = a_lds + buf * A_U4;
        const int tile = ar >> 4, ol = (ar & 15) + 16 * aq;
        ab[(0 * 8 + tile) * 64 + ol] = lo;   // sub-block 2cc   -> k step 0
        ab[(1 * 8 + tile) * 64 + ol] = hi;   // sub-block 2cc+1 -> k step 1
        if (cc == 0 && aq == 0) {
            const int par = (c >> 2) & 1;
            d_lds[par * QG_NT + ar] = f16_bits(h_reg.x);
            dmin_lds[par * QG_NT + ar] = f16_bits(h_reg.x >> 16);
            uint32_t mm[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                uint32_t s_;
                q4k_scale_min(h_reg.y, h_reg.z, h_reg.w, j, s_, mm[j]);
            }
            min_lds[par * QG_NT + ar] = uint4{qg_pack_h2((int)mm[0], (int)mm[1]), qg_pack_h2((int)mm[2], (int)mm[3]),
                                              qg_pack_h2((int)mm[4], (int)mm[5]), qg_pack_h2((int)mm[6], (int)mm[7])};
        }
        uint4 *bb = b_lds + buf * B_U4;
#pragma unroll
        for (int i = 0; i < 2 * MI; i++) {
            const int idx = tid + 512 * i, mtile = idx >> 8, rest = idx & 255;  // rest = (kstep*2 + plane)*64 + lane
            *(qg_u4 *)(bb + ((rest >> 6) * MT16 + mtile) * 64 + (rest & 63)) = b_reg[i];
        }
    };

    qg_f4 Ph[4][MI], Pl[4][MI];
    float acc[4][MI][4];
#pragma unroll
    for (int ni = 0; ni < 4; ni++)
#pragma unroll
        for (int mi = 0; mi < MI; mi++) {
            Ph[ni][mi] = Pl[ni][mi] = qg_f4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int j = 0; j < 4; j++) acc[ni][mi][j] = 0.0f;
        }

    auto compute_chunk = [&](int c) __attribute__((always_inline)) {
        if (!wave_live) return;
        const uint4 *ab = a_lds + (c & 1) * A_U4, *bb = b_lds + (c & 1) * B_U4;
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            qg_h8 bh[MI], bl[MI];
#pragma unroll
            for (int mi = 0; mi < MI; mi++) {
                bh[mi] = __builtin_bit_cast(qg_h8, bb[((ks * 2 + 0) * MT16 + wm * MI + mi) * 64 + lane]);
                bl[mi] = __builtin_bit_cast(qg_h8, bb[((ks * 2 + 1) * MT16 + wm * MI + mi) * 64 + lane]);
            }
#pragma unroll
            for (int ni = 0; ni < 4; ni++) {
                const qg_h8 av = __builtin_bit_cast(qg_h8, ab[(ks * 8 + wn * 4 + ni) * 64 + lane]);
#pragma unroll
                for (int mi = 0; mi < MI; mi++) {
                    Ph[ni][mi] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bh[mi], Ph[ni][mi], 0, 0, 0);
                    Pl[ni][mi] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bl[mi], Pl[ni][mi], 0, 0, 0);
                }
            }
        }
    };

    float s_reg[MI];
    uint4 xs_reg[MI];
    auto close_block = [&](int b) __attribute__((always_inline)) {
        if (!wave_live) return;
        const int par = b & 1;
#pragma unroll
        for (int mi = 0; mi < MI; mi++) {
            const qg_h8 xm = __builtin_bit_cast(qg_h8, xs_reg[mi]);
            const float s = s_reg[mi];
#pragma unroll
            for (int ni = 0; ni < 4; ni++) {
                const int r0 = par * QG_NT + wn * 64 + 16 * ni;
                const uint4 mraw = kg < 3 ? min_lds[r0 + col] : uint4{0, 0, 0, 0};
                const qg_f4 MM = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(qg_h8, mraw), xm,
                                                                        qg_f4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
                const float4 dv = *(const float4 *)(d_lds + r0 + 4 * kg);
                const float4 mv = *(const float4 *)(dmin_lds + r0 + 4 * kg);
                const float dj[4] = {dv.x, dv.y, dv.z, dv.w}, mj[4] = {mv.x, mv.y, mv.z, mv.w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float f = fmaf(Ph[ni][mi][j], 2048.0f, Pl[ni][mi][j]);
                    const float t = fmaf(-4096.0f * mj[j], MM[j], dj[j] * f);
                    acc[ni][mi][j] = fmaf(s, t, acc[ni][mi][j]);
                }
                Ph[ni][mi] = Pl[ni][mi] = qg_f4{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
    };
    auto load_block_acts = [&](int b) __attribute__((always_inline)) {
        if (!wave_live) return;
#pragma unroll
        for (int mi = 0; mi < MI; mi++) {
            s_reg[mi] = acts.scale[(size_t)(m0 + 16 * mi + col) * nb + b];
            xs_reg[mi] = ((const uint4 *)acts.mins)[((size_t)((m0 >> 4) + mi) * nb + b) * 64 + lane];
        }
    };

    load_chunk(0);
    store_chunk(0);
    if (nch > 1) load_chunk(1);
    __syncthreads();
    const bool stage_first = (wave & 4) == 0;  // waves 0-3 and 4-7 share SIMDs pairwise
    for (int c = 0; c < nch; c++) {
        if ((c & 3) == 0) load_block_acts(c >> 2);
        if (stage_first) {
            if (c + 1 < nch) store_chunk(c + 1);
            if (c + 2 < nch) load_chunk(c + 2);
            compute_chunk(c);
        } else {
            compute_chunk(c);
            if (c + 1 < nch) store_chunk(c + 1);
            if (c + 2 < nch) load_chunk(c + 2);
        }
        if ((c & 3) == 3) close_block(c >> 2);
        __syncthreads();
    }

    if (!wave_live) return;
#pragma unroll
    for (int mi = 0; mi < MI; mi++) {
        const int row = m0 + 16 * mi + col;
        if (row >= m) continue;
#pragma unroll
        for (int ni = 0; ni < 4; ni++) {
            const int nn = nt * QG_NT + wn * 64 + 16 * ni + 4 * kg;
            float *yp = Y + (size_t)row * n + nn;
            if (nn + 3 < n && (n & 3) == 0) {
                *(float4 *)yp = float4{acc[ni][mi][0], acc[ni][mi][1], acc[ni][mi][2], acc[ni][mi][3]};
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (nn + j < n) yp[j] = acc[ni][mi][j];
            }
        }
    }
}

template <int MI>
constexpr size_t q4k_gemm_lds_bytes() {
    return (size_t)(2 * (2 * 8 * 64) + 2 * (2 * 2 * 4 * MI * 64) + 2 * QG_NT) * 16 + 4 * QG_NT * sizeof(float);
}

}  // namespace jq
