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
// I2 is one more MFMA per tile and super-block over XS / 4096 split exactly three ways
// into f16.  One f32 combination per super-block applies d, dmin and s.
//
// Workgroup: 128 weight rows x 64*MI activation rows, 8 waves = 2 (weight rows) x 4
// (activation rows); a wave owns 64 x 16*MI outputs.  Weight nibbles are unpacked,
// multiplied by their sub-block scale and converted while being staged into LDS in
// MFMA operand order; the activation planes come prepared in operand order from
// q4k_gemm_prep.  Everything the main loop reads from global memory travels as
// asynchronous global -> LDS loads through rings of three 64-k chunks, two chunks
// ahead of the MFMAs; the packed nibbles are then unpacked LDS -> LDS.
#pragma once
#include <type_traits>

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
//           XS_j / 4096 for j = 0..7; g = 3: the f32 scale s of row m in the first four bytes
struct Q4kGemmActs {
    _Float16 *planes;
    _Float16 *mins;
};

__device__ __forceinline__ uint32_t qg_pack_h2(int a, int b) {  // two small integers as f16
    const qg_h2 v = qg_h2{(_Float16)(float)a, (_Float16)(float)b};
    return __builtin_bit_cast(uint32_t, v);
}

// A sub-block sum XS (|XS| < 2^27) over 4096 as three f16 values that add up to it exactly: its
// balanced base-512 digits a0 + 512 a1 + 2^18 a2, scaled (a0 / 4096, a1 / 8, 64 a2).
__device__ __forceinline__ void qg_split_sum(int xs, _Float16 &p0, _Float16 &p1, _Float16 &p2) {
    const int a0 = ((xs + 256) & 511) - 256, r = (xs - a0) >> 9;
    const int a1 = ((r + 256) & 511) - 256, a2 = (r - a1) >> 9;
    p0 = (_Float16)((float)a0 * (1.0f / 4096.0f));
    p1 = (_Float16)((float)a1 * 0.125f);
    p2 = (_Float16)((float)a2 * 64.0f);
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
    float amax = fmaxf(fmaxf(mag_or_inf(v.x), mag_or_inf(v.y)), fmaxf(mag_or_inf(v.z), mag_or_inf(v.w)));
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
        _Float16 p0, p1, p2;
        qg_split_sum(xs, p0, p1, p2);
        _Float16 *o = a.mins + (((size_t)mt * nb + b) * 64 + (row & 15)) * 8 + j;
        o[0] = p0, o[16 * 8] = p1, o[32 * 8] = p2;
    }
    if (lane == 0) {  // lane 48 + m%16 of the block: the scale in its first dword, zeros behind it
        uint32_t *o = (uint32_t *)(a.mins + (((size_t)mt * nb + b) * 64 + 48 + (row & 15)) * 8);
        o[0] = __float_as_uint(fixed_scale(amax, QG_RANGE));
        o[1] = o[2] = o[3] = 0;
    }
}

// sc * q of two nibbles of `word`, as two exact f16, in two instructions and without moving the
// nibbles: OR-ing the f16 exponent of 16 over the masked word makes a nibble in bits 0-3 (16-19)
// the f16 16 + q/64, one in bits 4-7 (20-23) the f16 16 + q/4; a packed fused multiply-add with
// (64 sc, -1024 sc), respectively (4 sc, -64 sc), leaves sc q (at most 945; every operand is an f16
// integer, the exact result is representable, the fma rounds once).
struct QgScaleOps {
    qg_h2 lo, hi;  // for the nibbles in bits 0-3 / 4-7 of the bytes
};

__device__ __forceinline__ qg_h2 qg_scale_operand(uint32_t sc, float mul, float add) {
    const _Float16 s = (_Float16)(unsigned short)sc;
    return qg_h2{s * (_Float16)mul, s * (_Float16)add};
}
__device__ __forceinline__ qg_h2 qg_scale_operand_lo(uint32_t sc) { return qg_scale_operand(sc, 64.0f, -1024.0f); }
__device__ __forceinline__ qg_h2 qg_scale_operand_hi(uint32_t sc) { return qg_scale_operand(sc, 4.0f, -64.0f); }

// (word & mask) | 0x4C004C00 in one instruction: the mask in a vector register, the constant in a scalar one
__device__ __forceinline__ uint32_t qg_mask_exp(uint32_t word, uint32_t mask) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(word), "v"(mask), "s"(0x4C004C00u));
    return r;
}

__device__ __forceinline__ uint32_t qg_scaled_h2(uint32_t word, uint32_t mask, qg_h2 op) {
    const qg_h2 h = __builtin_bit_cast(qg_h2, qg_mask_exp(word, mask));
    const qg_h2 v = __builtin_elementwise_fma(h, qg_h2{op.x, op.x}, qg_h2{op.y, op.y});
    return __builtin_bit_cast(uint32_t, v);
}

// The 8 nibble bytes w0, w1 of a lane -> the MFMA A operands of the low-nibble and high-nibble
// sub-block, element order 0,2,1,3,4,6,5,7.
__device__ __forceinline__ void qg_unpack_words(uint32_t w0, uint32_t w1, qg_h2 op_lo, qg_h2 op_hi, qg_u4 &lo, qg_u4 &hi) {
    const uint32_t s0 = w0 >> 8, s1 = w1 >> 8;
    const uint32_t ml = 0x000F000Fu, mh = 0x00F000F0u;
    lo = qg_u4{qg_scaled_h2(w0, ml, op_lo), qg_scaled_h2(s0, ml, op_lo), qg_scaled_h2(w1, ml, op_lo), qg_scaled_h2(s1, ml, op_lo)};
    hi = qg_u4{qg_scaled_h2(w0, mh, op_hi), qg_scaled_h2(s0, mh, op_hi), qg_scaled_h2(w1, mh, op_hi), qg_scaled_h2(s1, mh, op_hi)};
}

// Asynchronous global -> LDS load: every active lane fetches `bytes` (4 or 16) from its own global
// address, and the wave's data lands contiguously at lds_base + lane * bytes (lds_base wave-uniform).
// Written as inline assembly so that the compiler neither tracks these loads nor inserts waits of
// its own for them: the kernel below orders and awaits them by hand with s_waitcnt vmcnt(n).
// M0 (the LDS base of such a load) is written here and used by nothing else in these kernels.
__device__ __forceinline__ uint32_t qg_lds_offset(const void *p) {
    return (uint32_t)(uintptr_t)((__attribute__((address_space(3))) const void *)p);
}
__device__ __forceinline__ void qg_async_load16(const void *gptr, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_base)) : "memory");
}
__device__ __forceinline__ void qg_async_load4(const void *gptr, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(gptr), "s"(__builtin_amdgcn_readfirstlane(lds_base)) : "memory");
}

// 16-row activation tiles per wave: 2 (the LDS budget below is sized for it)
constexpr int QG_MI = 2;
constexpr int QG_MT = 64 * QG_MI;        // activation rows per workgroup
constexpr int QG_MT16 = 4 * QG_MI;       // 16-row activation tiles per workgroup = waves per workgroup
constexpr int QG_A_U4 = 2 * 8 * 64;      // 16-byte slots of an unpacked A chunk: [kstep][ntile 8][lane]
constexpr int QG_B_U4 = 2 * 2 * QG_MT16 * 64;  // of a B chunk: [kstep][plane][mtile][lane]

// Every global read of the main loop is an asynchronous global->LDS load (no register in
// between), ordered and awaited by hand: the vmcnt arithmetic in step() relies on each
// wave issuing exactly the operations listed there, youngest last.
//
// Split over k: the grid is `splits` copies of the tile list (base_grid workgroups each, a multiple of 8
// so that the XCD of a workgroup does not change); copy i takes the i-th of `splits` contiguous runs of
// super-blocks and stores its m x n partial sums at Y + i * split_stride (splitk_sum adds them up in a
// fixed order).  With splits == 1 and split_stride == 0, Y is the result.
__global__ __launch_bounds__(512) void q4k_gemm_mfma(const uint8_t *__restrict__ W, size_t row_bytes, Q4kGemmActs acts,
                                                      float *__restrict__ Y, int m, int m_pad, int k, int n,
                                                      int m_tiles, int total_tiles, int splits, int base_grid,
                                                      size_t split_stride) {
    constexpr int MI = QG_MI, MT = QG_MT, MT16 = QG_MT16;
    static_assert(MT16 == 8, "one activation tile of mins per wave");
    // Rings of 64-k chunks.  The slots are separate arrays so that the compiler can tell a
    // read of one slot from the asynchronous loads in flight into another.
    __shared__ qg_u4 b_s0[QG_B_U4], b_s1[QG_B_U4], b_s2[QG_B_U4];   // activation planes, 3 x 32 KB
    __shared__ uint32_t r_s0[1024], r_s1[1024], r_s2[1024];         // packed nibbles [row 128][8 dwords], 3 x 4 KB
    __shared__ qg_u4 h_s0[QG_NT], h_s1[QG_NT], h_s2[QG_NT];          // block header of each row, per chunk slot
    __shared__ qg_u4 x_s[QG_MT16 * 64];                              // mins operand + scales of the super-block
    __shared__ qg_u4 a_lds[2 * QG_A_U4];                             // unpacked weights, by chunk parity
    __shared__ qg_u4 min_lds[2 * QG_NT];   // [super-block parity][row]: the eight mins as f16
    __shared__ float d_lds[2 * QG_NT], dmin_lds[2 * QG_NT];

    // XCD-aware order.  Consecutive workgroup ids go round-robin over the 8 XCDs, each with its own
    // L2.  The activation planes are the heavy operand (4 bytes per element against 0.5 for the
    // weights), so an XCD works on as few activation tiles as possible and keeps them in its L2,
    // while a weight tile is fetched by the XCDs that share it.
    const int split = (int)blockIdx.x / base_grid, bid = (int)blockIdx.x - split * base_grid;
    const int xcd = bid & 7, slot = bid >> 3;
    int mt, nt;
    if (m_tiles >= 8 || (8 % m_tiles) != 0) {
        // activation tiles xcd, xcd + 8, ... (or plain round-robin when the counts do not divide)
        const int per_xcd = (total_tiles + 7) >> 3;
        const int logical = m_tiles >= 8 ? slot : xcd * per_xcd + slot;
        if (m_tiles >= 8) {
            const int n_tiles = total_tiles / m_tiles;
            mt = xcd + 8 * (logical / n_tiles), nt = logical % n_tiles;
            if (mt >= m_tiles) return;
        } else {
            if (logical >= total_tiles) return;
            mt = logical % m_tiles, nt = logical / m_tiles;
        }
    } else {
        const int g = 8 / m_tiles, n_tiles = total_tiles / m_tiles;   // g XCDs share one activation tile
        mt = xcd % m_tiles;
        nt = xcd / m_tiles + g * slot;
        if (nt >= n_tiles) return;
    }

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wn = wave & 1, wm = wave >> 1;
    const int nb_all = k >> 8, nch_all = k >> 6;
    const int b_begin = (int)((long)split * nb_all / splits), b_end = (int)((long)(split + 1) * nb_all / splits);
    const int nb = b_end - b_begin, nch = 4 * nb;   // this workgroup's super-blocks and 64-k chunks, numbered from 0
    const int col = lane & 15, kg = lane >> 4;
    const int m0 = mt * MT + wm * 16 * MI;       // first activation row of this wave
    const bool wave_live = m0 < m;

    const int ar = tid >> 2, aq = tid & 3;        // unpack role: weight row of the tile, 8-byte piece of its 32 nibble bytes
    const qg_u4 *bsrc = (const qg_u4 *)acts.planes + ((size_t)(mt * MT16) * nch_all + 4 * b_begin) * 256;
    // asynchronous-load roles: nibble rows 16 wave + 8 j + lane/8 (dword lane%8), header row 16 wave + lane/4
    const uint8_t *nib_src[2];
#pragma unroll
    for (int j = 0; j < 2; j++)
        nib_src[j] = W + (size_t)min(nt * QG_NT + 16 * wave + 8 * j + (lane >> 3), n - 1) * row_bytes + (size_t)b_begin * 144 + 16 + 4 * (lane & 7);
    const uint8_t *hdr_src = W + (size_t)min(nt * QG_NT + 16 * wave + (lane >> 2), n - 1) * row_bytes + (size_t)b_begin * 144 + 4 * (lane & 3);
    const qg_u4 *xs_src = (const qg_u4 *)acts.mins + ((size_t)(mt * MT16 + wave) * nb_all + b_begin) * 64 + lane;

    auto b_slot = [&](auto S) __attribute__((always_inline)) -> qg_u4 * {
        if constexpr (decltype(S)::value == 0) return b_s0;
        else if constexpr (decltype(S)::value == 1) return b_s1;
        else return b_s2;
    };
    auto r_slot = [&](auto S) __attribute__((always_inline)) -> uint32_t * {
        if constexpr (decltype(S)::value == 0) return r_s0;
        else if constexpr (decltype(S)::value == 1) return r_s1;
        else return r_s2;
    };

    // 2 operations: packed nibbles of chunk c
    auto dma_nibbles = [&](auto S, int c) __attribute__((always_inline)) {
        uint32_t *rr = r_slot(S);
        const size_t off = (size_t)(c >> 2) * 144 + 32 * (c & 3);
#pragma unroll
        for (int j = 0; j < 2; j++)
            qg_async_load4(nib_src[j] + off, qg_lds_offset(rr + (wave * 2 + j) * 64));
    };
    auto h_slot = [&](auto S) __attribute__((always_inline)) -> qg_u4 * {
        if constexpr (decltype(S)::value == 0) return h_s0;
        else if constexpr (decltype(S)::value == 1) return h_s1;
        else return h_s2;
    };
    // 1 operation: the 16-byte block headers of chunk c's super-block (fetched with every chunk so
    // that the slot read by unpack_a is known at compile time)
    auto dma_header = [&](auto S, int c) __attribute__((always_inline)) {
        qg_async_load4(hdr_src + (size_t)(c >> 2) * 144, qg_lds_offset((uint32_t *)h_slot(S) + wave * 64));
    };
    auto dma_block_acts = [&](int b) __attribute__((always_inline)) {
        qg_async_load16(xs_src + (size_t)b * 64, qg_lds_offset(x_s + wave * 64));
    };
    // 4 operations: activation planes of chunk c, four 1 KB blocks per wave
    auto dma_b = [&](auto S, int c) __attribute__((always_inline)) {
        qg_u4 *bb = b_slot(S);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int blk = wave * 4 + i;                       // LDS block = ksp * MT16 + mtile
            const int ksp = blk / MT16, mtile = blk % MT16;
            const qg_u4 *src = bsrc + ((size_t)mtile * nch_all + c) * 256 + ksp * 64 + lane;
            qg_async_load16(src, qg_lds_offset(bb + blk * 64));
        }
    };
    // packed nibbles of chunk c (slot S) -> scaled f16 in the A buffer of its parity
    auto unpack_a = [&](auto S, int c) __attribute__((always_inline)) {
        const int cc = c & 3, par = (c >> 2) & 1;
        const qg_u4 h = h_slot(S)[ar];
        uint32_t sc_lo, mn_lo, sc_hi, mn_hi;
        q4k_scale_min(h.y, h.z, h.w, 2 * cc, sc_lo, mn_lo);
        q4k_scale_min(h.y, h.z, h.w, 2 * cc + 1, sc_hi, mn_hi);
        const uint2 raw = *(const uint2 *)(r_slot(S) + ar * 8 + aq * 2);
        const uint32_t w0 = raw.x, w1 = raw.y;
        // operand order within the 8 k of a lane: 0,2,1,3,4,6,5,7
        qg_u4 lo, hi;
        qg_unpack_words(w0, w1, qg_scale_operand_lo(sc_lo), qg_scale_operand_hi(sc_hi), lo, hi);
        qg_u4 *ab = a_lds + (c & 1) * QG_A_U4;
        const int tile = ar >> 4, ol = (ar & 15) + 16 * aq;
        ab[(0 * 8 + tile) * 64 + ol] = lo;   // sub-block 2cc   -> k step 0
        ab[(1 * 8 + tile) * 64 + ol] = hi;   // sub-block 2cc+1 -> k step 1
        if (cc == 0 && aq == 0) {
            d_lds[par * QG_NT + ar] = f16_bits(h.x);
            dmin_lds[par * QG_NT + ar] = f16_bits(h.x >> 16);
            uint32_t mm[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                uint32_t s_;
                q4k_scale_min(h.y, h.z, h.w, j, s_, mm[j]);
            }
            min_lds[par * QG_NT + ar] = qg_u4{qg_pack_h2((int)mm[0], (int)mm[1]), qg_pack_h2((int)mm[2], (int)mm[3]),
                                              qg_pack_h2((int)mm[4], (int)mm[5]), qg_pack_h2((int)mm[6], (int)mm[7])};
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

    auto compute = [&](auto S, int c) __attribute__((always_inline)) {
        if (!wave_live) return;
        const qg_u4 *ab = a_lds + (c & 1) * QG_A_U4, *bb = b_slot(S);
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

    auto close_block = [&](int b) __attribute__((always_inline)) {
        if (!wave_live) return;
        const int par = b & 1;
#pragma unroll
        for (int mi = 0; mi < MI; mi++) {
            const qg_u4 *xt = x_s + (wm * MI + mi) * 64;
            const qg_u4 xraw = kg < 3 ? xt[lane] : qg_u4{0, 0, 0, 0};
            const qg_h8 xm = __builtin_bit_cast(qg_h8, xraw);
            const float s = __uint_as_float(xt[48 + col].x);
#pragma unroll
            for (int ni = 0; ni < 4; ni++) {
                const int r0 = par * QG_NT + wn * 64 + 16 * ni;
                const qg_u4 mraw = kg < 3 ? min_lds[r0 + col] : qg_u4{0, 0, 0, 0};
                const qg_f4 MM = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(qg_h8, mraw), xm,
                                                                        qg_f4{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0);
                const qg_f4 dv = *(const qg_f4 *)(d_lds + r0 + 4 * kg);
                const qg_f4 mv = *(const qg_f4 *)(dmin_lds + r0 + 4 * kg);
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float f = fmaf(Ph[ni][mi][j], 2048.0f, Pl[ni][mi][j]);
                    const float t = fmaf(-4096.0f * mv[j], MM[j], dv[j] * f);
                    acc[ni][mi][j] = fmaf(s, t, acc[ni][mi][j]);
                }
                Ph[ni][mi] = Pl[ni][mi] = qg_f4{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
    };

    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;

    // One pipeline step: chunk c, activation planes in slot S.
    //   on entry, in flight and oldest first: [group of step c-2], [group of step c-1]
    //   group of step c = nibbles(c+3) x2, header(c+3), mins(c/4) if c%4 == 0, planes(c+2) x4;
    //                     at least 7 operations while c + 3 < nch
    //   needed now: planes(c), nibbles and header (c+1), mins issued at step c-2 or earlier
    //   => at most the 7 youngest operations (all from step c-1) may still be in flight.
    auto step = [&](auto S, auto S1, auto S2, int c) __attribute__((always_inline)) {
        if (c + 4 < nch) asm volatile("s_waitcnt vmcnt(7) lgkmcnt(0)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (c + 3 < nch) {
            dma_nibbles(S, c + 3);                              // slot S held chunk c, unpacked during step c-1
            dma_header(S, c + 3);
        }
        if (c > 0 && (c & 3) == 0) dma_block_acts(c >> 2);      // x_s last read by close_block at step c-1; needed at c+3
        if (c + 2 < nch) dma_b(S2, c + 2);                      // slot S2 last read by compute(c-1)
        asm volatile("" ::: "memory");
        compute(S, c);
        if (c + 1 < nch) unpack_a(S1, c + 1);                   // A buffer (c+1)&1 last read by compute(c-1)
        if ((c & 3) == 3) close_block(c >> 2);
    };

    // prologue: chunks 0..2 of nibbles, headers and mins of super-block 0, planes of chunks 0 and 1
    dma_block_acts(0);
    dma_nibbles(I0{}, 0), dma_header(I0{}, 0);
    if (nch > 1) dma_nibbles(I1{}, 1), dma_header(I1{}, 1);
    if (nch > 2) dma_nibbles(I2{}, 2), dma_header(I2{}, 2);
    dma_b(I0{}, 0);
    if (nch > 1) dma_b(I1{}, 1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    unpack_a(I0{}, 0);
    for (int c = 0; c < nch; c += 3) {
        step(I0{}, I1{}, I2{}, c);
        if (c + 1 < nch) step(I1{}, I2{}, I0{}, c + 1);
        if (c + 2 < nch) step(I2{}, I0{}, I1{}, c + 2);
    }

    if (!wave_live) return;
#pragma unroll
    for (int mi = 0; mi < MI; mi++) {
        const int row = m0 + 16 * mi + col;
        if (row >= m) continue;
#pragma unroll
        for (int ni = 0; ni < 4; ni++) {
            const int nn = nt * QG_NT + wn * 64 + 16 * ni + 4 * kg;
            float *yp = Y + (size_t)split * split_stride + (size_t)row * n + nn;
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

// Y[i] = P[0][i] + P[1][i] + ... + P[splits - 1][i], in that order, four elements a thread.
__global__ __launch_bounds__(256) void splitk_sum(const float *__restrict__ P, float *__restrict__ Y, size_t count,
                                                   int splits) {
    const size_t i = 4 * ((size_t)blockIdx.x * 256 + threadIdx.x);
    if (i >= count) return;
    if (i + 3 < count && (count & 3) == 0) {
        float4 a = *(const float4 *)(P + i);
        for (int sp = 1; sp < splits; sp++) {
            const float4 b = *(const float4 *)(P + (size_t)sp * count + i);
            a.x += b.x, a.y += b.y, a.z += b.z, a.w += b.w;
        }
        *(float4 *)(Y + i) = a;
    } else {
        for (size_t j = i; j < count && j < i + 4; j++) {
            float a = P[j];
            for (int sp = 1; sp < splits; sp++) a += P[(size_t)sp * count + j];
            Y[j] = a;
        }
    }
}

}  // namespace jq
