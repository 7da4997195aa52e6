// GGUF block formats decoded in registers (gfx950 device code).
//
// A block is cut into "units": the piece one lane decodes at a time, chosen
// so that a unit reads 16-byte runs of packed values and covers 32 or 64
// consecutive-ish elements.  Every decoder writes the same f32 weights the
// reference's fused CPU kernels build in registers, with the same rounding
// steps (products d*sc and dmin*m rounded to f32 first, then one fused
// multiply-subtract per element).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "iq2xxs_grid_codes.h"

namespace jq {

// |x|, or +inf when x is not finite (a NaN fails the comparison): the fixed-point quantisers take the
// block maximum of these and give a block with a non-finite activation the scale NaN (fixed_scale), so
// that the results say so instead of reading the block as zeros.
__device__ __forceinline__ float mag_or_inf(float x) {
    const float a = fabsf(x);
    return a <= 3.402823466e38f ? a : INFINITY;
}
__device__ __forceinline__ float fixed_scale(float amax, float range) {
    return amax > 0.0f ? (amax < INFINITY ? amax / range : NAN) : 0.0f;
}

// Sums over the aligned 16 (8) lanes around a lane, in every lane of the group, on the data-parallel
// primitives (row rotations, half-row mirror, quad permutes): four (three) instructions with no trip
// through LDS, where __shfl_xor costs a ds_bpermute each.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    const int u = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, u, CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float sum_row16(float v) {
    v += dpp_f<0x128>(v);  // row_ror:8
    v += dpp_f<0x124>(v);  // row_ror:4
    v += dpp_f<0x122>(v);  // row_ror:2
    v += dpp_f<0x121>(v);  // row_ror:1
    return v;
}
__device__ __forceinline__ float sum_row8(float v) {
    v += dpp_f<0x141>(v);  // row_half_mirror
    v += dpp_f<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_f<0x4E>(v);   // quad_perm [2,3,0,1]
    return v;
}

__device__ __forceinline__ float max_row16(float v) {
    v = fmaxf(v, dpp_f<0x128>(v));
    v = fmaxf(v, dpp_f<0x124>(v));
    v = fmaxf(v, dpp_f<0x122>(v));
    v = fmaxf(v, dpp_f<0x121>(v));
    return v;
}
__device__ __forceinline__ float max_row8(float v) {
    v = fmaxf(v, dpp_f<0x141>(v));
    v = fmaxf(v, dpp_f<0xB1>(v));
    v = fmaxf(v, dpp_f<0x4E>(v));
    return v;
}
template <int CTRL>
__device__ __forceinline__ int dpp_i(int u) { return __builtin_amdgcn_update_dpp(0, u, CTRL, 0xF, 0xF, true); }
__device__ __forceinline__ int isum_row8(int v) {
    v += dpp_i<0x141>(v);
    v += dpp_i<0xB1>(v);
    v += dpp_i<0x4E>(v);
    return v;
}

// v[lane] + v[lane ^ 16] and v[lane] + v[lane ^ 32] in every lane, as one row-swap instruction and
// one add (v_permlane16_swap / v_permlane32_swap exchange the odd rows of one operand with the even
// rows of the other; with v in both, the two results hold the pair's values) instead of a trip
// through LDS.
__device__ __forceinline__ float sum_xor16(float v) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
}
__device__ __forceinline__ float sum_xor32(float v) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
}
__device__ __forceinline__ int isum_xor16(int v) {
    const auto r = __builtin_amdgcn_permlane16_swap((unsigned)v, (unsigned)v, false, false);
    return (int)r[0] + (int)r[1];
}
__device__ __forceinline__ int isum_xor32(int v) {
    const auto r = __builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false);
    return (int)r[0] + (int)r[1];
}
__device__ __forceinline__ float max_xor16(float v) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return fmaxf(__builtin_bit_cast(float, (unsigned)r[0]), __builtin_bit_cast(float, (unsigned)r[1]));
}
__device__ __forceinline__ float max_xor32(float v) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__builtin_bit_cast(float, (unsigned)r[0]), __builtin_bit_cast(float, (unsigned)r[1]));
}
// The maximum over the wave, in every lane.
__device__ __forceinline__ float wave_max(float v) {
    const unsigned u = __builtin_bit_cast(unsigned, v);
    const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    v = fmaxf(__builtin_bit_cast(float, (unsigned)a[0]), __builtin_bit_cast(float, (unsigned)a[1]));
    const unsigned w = __builtin_bit_cast(unsigned, v);
    const auto b = __builtin_amdgcn_permlane16_swap(w, w, false, false);
    v = fmaxf(__builtin_bit_cast(float, (unsigned)b[0]), __builtin_bit_cast(float, (unsigned)b[1]));
    return max_row16(v);
}


template <class T>
__device__ __forceinline__ T ld(const uint8_t *p) {
    T v;
    __builtin_memcpy(&v, p, sizeof(T));
    return v;
}

// 4, 8 or 16 bytes at any address, taken from the aligned 32-bit words that hold them and shifted into
// place.  For blocks whose size is not a multiple of four (Q8_0 34, Q6_K 210, IQ2_XXS 66, MXFP4 17,
// Q5_0 22 bytes) a plain wide read lands on odd addresses, and in LDS a read that is not naturally aligned
// runs at a fraction of the aligned rate (the Q6_K output head: 130 us with 8-byte reads at 2-byte
// aligned LDS addresses, 88 us through aligned words).  The word past the field is only read when the
// field reaches into it, so nothing is touched beyond the bytes asked for.
template <class T>
__device__ __forceinline__ T ldw(const uint8_t *p) {
    constexpr int N = sizeof(T) / 4;
    static_assert(sizeof(T) % 4 == 0 && N >= 1 && N <= 4, "ldw reads 4, 8 or 16 bytes");
    const uint32_t mis = (uint32_t)(uintptr_t)p & 3u;
    const uint32_t *q = (const uint32_t *)(p - mis);
    uint32_t w[N + 1], o[N];
#pragma unroll
    for (int i = 0; i < N; i++) w[i] = q[i];
    w[N] = q[mis ? N : N - 1];
#pragma unroll
    for (int i = 0; i < N; i++) o[i] = __builtin_amdgcn_alignbyte(w[i + 1], w[i], mis);
    T v;
    __builtin_memcpy(&v, o, sizeof(T));
    return v;
}

__device__ __forceinline__ float f16_bits(uint32_t h) {
    return __half2float(__ushort_as_half((unsigned short)(h & 0xFFFFu)));
}

// byte i (0..11) of the 12 packed Q4_K scale bytes held in three dwords
__device__ __forceinline__ uint32_t q4k_byte(uint32_t s0, uint32_t s1, uint32_t s2, int i) {
    uint32_t w = i < 4 ? s0 : (i < 8 ? s1 : s2);
    return (w >> (8 * (i & 3))) & 0xFFu;
}

// 6-bit (scale, min) pair j of a Q4_K block (reference: src/kquant_dot.rs:108-118)
__device__ __forceinline__ void q4k_scale_min(uint32_t s0, uint32_t s1, uint32_t s2, int j, uint32_t &sc,
                                              uint32_t &mn) {
    if (j < 4) {
        sc = q4k_byte(s0, s1, s2, j) & 63u;
        mn = q4k_byte(s0, s1, s2, j + 4) & 63u;
    } else {
        uint32_t hi = q4k_byte(s0, s1, s2, j + 4);
        sc = (hi & 0xFu) | ((q4k_byte(s0, s1, s2, j - 4) >> 6) << 4);
        mn = (hi >> 4) | ((q4k_byte(s0, s1, s2, j) >> 6) << 4);
    }
}

// The (scale, min) pairs of sub-blocks 2c and 2c + 1 of a Q4_K block at once and without a branch, for
// lanes whose c differs: sc and mn hold the two 6-bit values as bytes 0 and 1 (the bits above are junk
// when c is even), so that `(float)(sc & 0xFF)` and `(float)((sc >> 8) & 0xFF)` are one byte-to-float
// conversion each.  Same values as q4k_scale_min(.., 2c, ..) and (.., 2c + 1, ..).
__device__ __forceinline__ void q4k_scale_min_pair(uint32_t s0, uint32_t s1, uint32_t s2, int c, uint32_t &sc,
                                                   uint32_t &mn) {
    const int sh = 16 * (c & 1);
    const uint32_t a = s0 >> sh, b = s1 >> sh, h = s2 >> sh;  // bytes (2c', 2c'+1) of each word, c' = c & 1
    const uint32_t sc_lo = a & 0x3F3Fu, mn_lo = b & 0x3F3Fu;
    const uint32_t sc_hi = (h & 0x0F0Fu) | ((a >> 2) & 0x3030u), mn_hi = ((h >> 4) & 0x0F0Fu) | ((b >> 2) & 0x3030u);
    sc = c < 2 ? sc_lo : sc_hi;
    mn = c < 2 ? mn_lo : mn_hi;
}

// IQ2_XXS codebook expanded at compile time to 256 x 8 bytes (value j of entry
// c in byte j), from the base-3 packed form in iq2xxs_grid_codes.h, followed by the
// 128 sign patterns of a group of eight as byte masks: entry 256 + s holds 0xFF in
// byte j where element j is negative, for the seven stored sign bits s and the
// eighth that makes their number even (reference: src/iq2xxs.rs:349-380).
struct Tables {
    uint64_t iq2xxs_grid[384];
    constexpr Tables() : iq2xxs_grid{} {
        for (int i = 0; i < 256; i++) {
            unsigned c = JQ_IQ2XXS_GRID_TRITS[i];
            uint64_t v = 0;
            for (int j = 0; j < 8; j++) {
                unsigned t = c % 3;
                c /= 3;
                v |= (uint64_t)(8 + 17 * t + (t >> 1)) << (8 * j);
            }
            iq2xxs_grid[i] = v;
        }
        for (unsigned s = 0; s < 128; s++) {
            unsigned ones = 0;
            for (int j = 0; j < 7; j++) ones += (s >> j) & 1u;
            const unsigned signs = s | ((ones & 1u) << 7);
            uint64_t v = 0;
            for (int j = 0; j < 8; j++)
                if ((signs >> j) & 1u) v |= (uint64_t)0xFF << (8 * j);
            iq2xxs_grid[256 + s] = v;
        }
    }
};
__device__ const Tables g_tables{};

// ---------------------------------------------------------------------------
// Every format exposes:
//   BLOCK_ELEMS, BLOCK_BYTES  geometry of one block
//   UNITS                     units per block
//   SEGS, SEGLEN, SEG_STRIDE  a unit covers SEGS runs of SEGLEN consecutive
//                             elements, SEG_STRIDE elements apart
//   elem_base(u)              first element (within the block) of unit u
//   decode(blk, u, w)         w[s*SEGLEN + i] = weight of element
//                             elem_base(u) + s*SEG_STRIDE + i
// ---------------------------------------------------------------------------

struct Q8_0 {  // d:f16 | qs[32] i8   (reference: src/kquant_dot.rs:53-61,287-302)
    static constexpr int BLOCK_ELEMS = 32, BLOCK_BYTES = 34, UNITS = 1;
    static constexpr int SEGS = 1, SEGLEN = 32, SEG_STRIDE = 0;
    __device__ static int elem_base(int) { return 0; }
    __device__ static void decode(const uint8_t *blk, int, float *w) {
        float d = f16_bits(ld<uint16_t>(blk));
        const uint4 qa = ldw<uint4>(blk + 2), qb = ldw<uint4>(blk + 18);
        const uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
#pragma unroll
            for (int b = 0; b < 4; b++) w[4 * i + b] = (float)(int8_t)(q[i] >> (8 * b)) * d;
        }
    }
    // The block as eight words of int8: the codes as they are, w = scale code.
    static constexpr bool HAS_DECODE_I8 = true, I8_HAS_MIN = false;
    static constexpr int I8_UNITS = 1, I8_EXTRA_ENTRIES = 0;
    __device__ static uint64_t i8_extra_entry(int) { return 0; }
    __device__ static void decode_i8(const uint64_t *, const uint8_t *blk, int, int *w, float &scale, float &offset) {
        const uint4 qa = ldw<uint4>(blk + 2), qb = ldw<uint4>(blk + 18);
        w[0] = (int)qa.x, w[1] = (int)qa.y, w[2] = (int)qa.z, w[3] = (int)qa.w;
        w[4] = (int)qb.x, w[5] = (int)qb.y, w[6] = (int)qb.z, w[7] = (int)qb.w;
        scale = f16_bits(ld<uint16_t>(blk));
        offset = 0.0f;
    }
};

// Bits 0..3 of b as bit 4 of bytes 0..3: the fifth bits of four 5-bit codes beside their nibbles.
__device__ __forceinline__ uint32_t fifth_bits(uint32_t b) { return (((b & 0xFu) * 0x00204081u) & 0x01010101u) << 4; }

// The 32-element formats with 4 or 5 bits a weight.  The reference has no kernel of its own for them:
// they run through the canonical decode plus the 8-lane dot (reference: src/quant_matmul.rs:228-248);
// the layouts are those of vendor/candle-metal-kernels/src/metal_src/quantized.metal:21-61 and the
// element maps those of its dequantize_q4_0 .. dequantize_q5_1 (:6482-6567): byte j of qs holds
// element j in its low and element j + 16 in its high nibble, bit e of qh is the fifth bit of element e.
// Every product below is exact in f32 and each weight has at most one rounding, so the order of the
// operations does not matter.
struct Q4_0 {  // d:f16 | qs[16]        w = d (q - 8)
    static constexpr int BLOCK_ELEMS = 32, BLOCK_BYTES = 18, UNITS = 1;
    static constexpr int SEGS = 1, SEGLEN = 32, SEG_STRIDE = 0;
    __device__ static int elem_base(int) { return 0; }
    __device__ static void decode(const uint8_t *blk, int, float *w) {
        const float d = f16_bits(ld<uint16_t>(blk));
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const int b = blk[2 + j];
            w[j] = d * (float)((b & 0xF) - 8);
            w[j + 16] = d * (float)((b >> 4) - 8);
        }
    }
    // The block as eight words of int8 (elements 4i .. 4i+3 in word i: the low nibbles' sixteen first), the codes as they
    // are; w = scale code - offset.
    static constexpr bool HAS_DECODE_I8 = true, I8_HAS_MIN = true;
    static constexpr int I8_UNITS = 1, I8_EXTRA_ENTRIES = 0;
    __device__ static uint64_t i8_extra_entry(int) { return 0; }
    __device__ static void decode_i8(const uint64_t *, const uint8_t *blk, int, int *w, float &scale, float &offset) {
        const uint4 qv = ldw<uint4>(blk + 2);
        const uint32_t q[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (int)(q[i] & 0x0F0F0F0Fu), w[4 + i] = (int)((q[i] >> 4) & 0x0F0F0F0Fu);
        scale = f16_bits(ld<uint16_t>(blk));
        offset = 8.0f * scale;
    }
};

struct Q4_1 {  // d:f16 | m:f16 | qs[16]        w = d q + m
    static constexpr int BLOCK_ELEMS = 32, BLOCK_BYTES = 20, UNITS = 1;
    static constexpr int SEGS = 1, SEGLEN = 32, SEG_STRIDE = 0;
    __device__ static int elem_base(int) { return 0; }
    __device__ static void decode(const uint8_t *blk, int, float *w) {
        const float d = f16_bits(ld<uint16_t>(blk)), m = f16_bits(ld<uint16_t>(blk + 2));
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const int b = blk[4 + j];
            w[j] = fmaf(d, (float)(b & 0xF), m);
            w[j + 16] = fmaf(d, (float)(b >> 4), m);
        }
    }
    // The block as eight words of int8 (elements 4i .. 4i+3 in word i: the low nibbles' sixteen first), the codes as they
    // are; w = scale code - offset.
    static constexpr bool HAS_DECODE_I8 = true, I8_HAS_MIN = true;
    static constexpr int I8_UNITS = 1, I8_EXTRA_ENTRIES = 0;
    __device__ static uint64_t i8_extra_entry(int) { return 0; }
    __device__ static void decode_i8(const uint64_t *, const uint8_t *blk, int, int *w, float &scale, float &offset) {
        const uint4 qv = ldw<uint4>(blk + 4);
        const uint32_t q[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
        for (int i = 0; i < 4; i++) w[i] = (int)(q[i] & 0x0F0F0F0Fu), w[4 + i] = (int)((q[i] >> 4) & 0x0F0F0F0Fu);
        scale = f16_bits(ld<uint16_t>(blk));
        offset = -f16_bits(ld<uint16_t>(blk + 2));
    }
};

struct Q5_0 {  // d:f16 | qh:u32 | qs[16]        w = d (q - 16)
    static constexpr int BLOCK_ELEMS = 32, BLOCK_BYTES = 22, UNITS = 1;
    static constexpr int SEGS = 1, SEGLEN = 32, SEG_STRIDE = 0;
    __device__ static int elem_base(int) { return 0; }
    __device__ static void decode(const uint8_t *blk, int, float *w) {
        const float d = f16_bits(ld<uint16_t>(blk));
        const uint32_t qh = ldw<uint32_t>(blk + 2);
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const int b = blk[6 + j];
            w[j] = d * (float)(((b & 0xF) | (int)(((qh >> j) & 1u) << 4)) - 16);
            w[j + 16] = d * (float)(((b >> 4) | (int)(((qh >> (j + 16)) & 1u) << 4)) - 16);
        }
    }
    // The block as eight words of int8 (elements 4i .. 4i+3 in word i: the low nibbles' sixteen first), the codes as they
    // are; w = scale code - offset.
    static constexpr bool HAS_DECODE_I8 = true, I8_HAS_MIN = true;
    static constexpr int I8_UNITS = 1, I8_EXTRA_ENTRIES = 0;
    __device__ static uint64_t i8_extra_entry(int) { return 0; }
    __device__ static void decode_i8(const uint64_t *, const uint8_t *blk, int, int *w, float &scale, float &offset) {
        const uint32_t qh = ldw<uint32_t>(blk + 2);
        const uint4 qv = ldw<uint4>(blk + 6);
        const uint32_t q[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w[i] = (int)((q[i] & 0x0F0F0F0Fu) | fifth_bits(qh >> (4 * i)));
            w[4 + i] = (int)(((q[i] >> 4) & 0x0F0F0F0Fu) | fifth_bits(qh >> (16 + 4 * i)));
        }
        scale = f16_bits(ld<uint16_t>(blk));
        offset = 16.0f * scale;
    }
};

struct Q5_1 {  // d:f16 | m:f16 | qh:u32 | qs[16]        w = d q + m
    static constexpr int BLOCK_ELEMS = 32, BLOCK_BYTES = 24, UNITS = 1;
    static constexpr int SEGS = 1, SEGLEN = 32, SEG_STRIDE = 0;
    __device__ static int elem_base(int) { return 0; }
    __device__ static void decode(const uint8_t *blk, int, float *w) {
        const float d = f16_bits(ld<uint16_t>(blk)), m = f16_bits(ld<uint16_t>(blk + 2));
        const uint32_t qh = ld<uint32_t>(blk + 4);
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const int b = blk[8 + j];
            w[j] = fmaf(d, (float)((b & 0xF) | (int)(((qh >> j) & 1u) << 4)), m);
            w[j + 16] = fmaf(d, (float)((b >> 4) | (int)(((qh >> (j + 16)) & 1u) << 4)), m);
        }
    }
    // The block as eight words of int8 (elements 4i .. 4i+3 in word i: the low nibbles' sixteen first), the codes as they
    // are; w = scale code - offset.
    static constexpr bool HAS_DECODE_I8 = true, I8_HAS_MIN = true;
    static constexpr int I8_UNITS = 1, I8_EXTRA_ENTRIES = 0;
    __device__ static uint64_t i8_extra_entry(int) { return 0; }
    __device__ static void decode_i8(const uint64_t *, const uint8_t *blk, int, int *w, float &scale, float &offset) {
        const uint32_t qh = ldw<uint32_t>(blk + 4);
        const uint4 qv = ldw<uint4>(blk + 8);
        const uint32_t q[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w[i] = (int)((q[i] & 0x0F0F0F0Fu) | fifth_bits(qh >> (4 * i)));
            w[4 + i] = (int)(((q[i] >> 4) & 0x0F0F0F0Fu) | fifth_bits(qh >> (16 + 4 * i)));
        }
        scale = f16_bits(ld<uint16_t>(blk));
        offset = -f16_bits(ld<uint16_t>(blk + 2));
    }
};

struct Q4_K {  // d | dmin | scales[12] | qs[128]   (reference: src/kquant_dot.rs:78-93,426-466)
    static constexpr int BLOCK_ELEMS = 256, BLOCK_BYTES = 144, UNITS = 4;
    static constexpr int SEGS = 1, SEGLEN = 64, SEG_STRIDE = 0;
    __device__ static int elem_base(int u) { return 64 * u; }
    __device__ static void decode(const uint8_t *blk, int c, float *w) {
        uint4 hdr = ld<uint4>(blk);
        float d = f16_bits(hdr.x), dmin = f16_bits(hdr.x >> 16);
        uint32_t sc0, mn0, sc1, mn1;
        q4k_scale_min(hdr.y, hdr.z, hdr.w, 2 * c, sc0, mn0);
        q4k_scale_min(hdr.y, hdr.z, hdr.w, 2 * c + 1, sc1, mn1);
        float d0 = d * (float)sc0, m0 = dmin * (float)mn0;
        float d1 = d * (float)sc1, m1 = dmin * (float)mn1;
        uint4 qa = ld<uint4>(blk + 16 + 32 * c), qb = ld<uint4>(blk + 32 + 32 * c);
        uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t lo = q[i] & 0x0F0F0F0Fu, hi = (q[i] >> 4) & 0x0F0F0F0Fu;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                w[4 * i + b] = fmaf((float)((lo >> (8 * b)) & 0xFFu), d0, -m0);
                w[32 + 4 * i + b] = fmaf((float)((hi >> (8 * b)) & 0xFFu), d1, -m1);
            }
        }
    }
    // Unit c (64 elements: the low and the high nibbles of 32 bytes) against its activations as two
    // int8 planes, 16 registers a plane; sx, sxs: scale and scale * sum X of the two 32-element blocks.
    static constexpr bool HAS_DOT8 = true;
    __device__ static float dot8(const uint64_t *, const uint8_t *blk, int c, const uint32_t *xl, const uint32_t *xh,
                                 const float *sx, const float *sxs) {
        const uint4 hdr = ld<uint4>(blk);
        uint32_t scp, mnp;
        q4k_scale_min_pair(hdr.y, hdr.z, hdr.w, c, scp, mnp);
        const uint32_t sc0 = scp & 0xFFu, sc1 = (scp >> 8) & 0xFFu, mn0 = mnp & 0xFFu, mn1 = (mnp >> 8) & 0xFFu;
        const uint4 qa = ld<uint4>(blk + 16 + 32 * c), qb = ld<uint4>(blk + 32 + 32 * c);
        const uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        int l0 = 0, h0 = 0, l1 = 0, h1 = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int lo4 = (int)(q[i] & 0x0F0F0F0Fu), hi4 = (int)((q[i] >> 4) & 0x0F0F0F0Fu);
            l0 = __builtin_amdgcn_sdot4(lo4, (int)xl[i], l0, false);
            h0 = __builtin_amdgcn_sdot4(lo4, (int)xh[i], h0, false);
            l1 = __builtin_amdgcn_sdot4(hi4, (int)xl[8 + i], l1, false);
            h1 = __builtin_amdgcn_sdot4(hi4, (int)xh[8 + i], h1, false);
        }
        const float d = f16_bits(hdr.x), dmin = f16_bits(hdr.x >> 16);
        const float f0 = (float)((h0 << 8) + l0) * sx[0], f1 = (float)((h1 << 8) + l1) * sx[1];
        const float acc = d * fmaf((float)sc0, f0, (float)sc1 * f1);
        return fmaf(-dmin, fmaf((float)mn0, sxs[0], (float)mn1 * sxs[1]), acc);
    }
    // Sub-block u (32 elements, eight a block) as eight words of int8: its nibbles 0..15 as they are, the
    // scale d * sc_u that goes with their sum and the offset dmin * m_u that goes with the activations' sum.
    static constexpr bool HAS_DECODE_I8 = true, I8_HAS_MIN = true;
    static constexpr int I8_UNITS = 8, I8_EXTRA_ENTRIES = 0;
    __device__ static uint64_t i8_extra_entry(int) { return 0; }
    __device__ static void decode_i8(const uint64_t *, const uint8_t *blk, int u, int *w, float &scale, float &offset) {
        const uint4 hdr = ld<uint4>(blk);
        uint32_t sc, mn;
        q4k_scale_min(hdr.y, hdr.z, hdr.w, u, sc, mn);
        const uint4 qa = ld<uint4>(blk + 16 + 32 * (u >> 1)), qb = ld<uint4>(blk + 32 + 32 * (u >> 1));
        const uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
#pragma unroll
        for (int i = 0; i < 8; i++) w[i] = (int)((q[i] >> (4 * (u & 1))) & 0x0F0F0F0Fu);
        scale = f16_bits(hdr.x) * (float)sc;
        offset = f16_bits(hdr.x >> 16) * (float)mn;
    }
};

struct Q2_K {  // scales[16] | qs[64] | d | dmin   (reference: src/kquant_dot.rs:63-76,345-385)
    // unit u = (super-group sg = u/2, byte half hf = u%2): 16 bytes, four
    // 2-bit fields -> elements 128*sg + 32*f + 16*hf + [0,16), f = 0..3,
    // scale byte scales[8*sg + 2*f + hf].
    static constexpr int BLOCK_ELEMS = 256, BLOCK_BYTES = 84, UNITS = 4;
    static constexpr int SEGS = 4, SEGLEN = 16, SEG_STRIDE = 32;
    __device__ static int elem_base(int u) { return 128 * (u >> 1) + 16 * (u & 1); }
    __device__ static void decode(const uint8_t *blk, int u, float *w) {
        int sg = u >> 1, hf = u & 1;
        uint32_t dd = ld<uint32_t>(blk + 80);
        float d = f16_bits(dd), dmin = f16_bits(dd >> 16);
        uint4 qv = ld<uint4>(blk + 16 + 32 * sg + 16 * hf);
        uint32_t q[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
        for (int f = 0; f < 4; f++) {
            uint32_t s = blk[8 * sg + 2 * f + hf];
            float d1 = d * (float)(s & 0xFu), m1 = dmin * (float)(s >> 4);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                uint32_t v = (q[i] >> (2 * f)) & 0x03030303u;
#pragma unroll
                for (int b = 0; b < 4; b++) w[16 * f + 4 * i + b] = fmaf((float)((v >> (8 * b)) & 0xFFu), d1, -m1);
            }
        }
    }
};

struct Q3_K {  // hmask[32] | qs[64] | scales[12] | d        w = d (sc - 32) (q - (hbit ? 0 : 4))
    // (layout and element map: vendor/candle-metal-kernels/src/metal_src/quantized.metal:151-156,6597-6623)
    // unit u = (half h = u/2, byte half hf = u%2): 16 bytes of qs, four 2-bit fields t -> elements
    // 128 h + 32 t + 16 hf + [0,16); their third bit is bit 4 h + t of hmask[16 hf + i]; the 6-bit scale
    // of the 16 elements is number 8 h + 2 t + hf: low four bits in scales[0..7] (a nibble each, the
    // first eight scales low, the next eight high), high two bits in scales[8..11].
    static constexpr int BLOCK_ELEMS = 256, BLOCK_BYTES = 110, UNITS = 4;
    static constexpr int SEGS = 4, SEGLEN = 16, SEG_STRIDE = 32;
    __device__ static int elem_base(int u) { return 128 * (u >> 1) + 16 * (u & 1); }
    __device__ static void decode(const uint8_t *blk, int u, float *w) {
        const int h = u >> 1, hf = u & 1;
        const float d = f16_bits(ld<uint16_t>(blk + 108));
        const uint8_t *q = blk + 32 + 32 * h + 16 * hf, *hm = blk + 16 * hf, *sc = blk + 96;
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int is = 8 * h + 2 * t + hf;
            const int low4 = is < 8 ? (sc[is] & 0xF) : (sc[is - 8] >> 4);
            const int high2 = (sc[8 + (is & 3)] >> (2 * (is >> 2))) & 3;
            const float dl = d * (float)((low4 | (high2 << 4)) - 32);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int v = ((q[i] >> (2 * t)) & 3) - (((hm[i] >> (4 * h + t)) & 1) ? 0 : 4);
                w[16 * t + i] = dl * (float)v;
            }
        }
    }
};

struct Q5_K {  // d | dmin | scales[12] | qh[32] | qs[128]        w = d sc q - dmin m
    // (layout and element map: vendor/candle-metal-kernels/src/metal_src/quantized.metal:176-189,6649-6670)
    // unit c: 64 elements, sub-blocks 2c (low nibbles of qs[32c + l]) and 2c + 1 (high nibbles); the
    // fifth bit of element l of sub-block j is bit j of qh[l]; scales and mins are packed as in Q4_K.
    static constexpr int BLOCK_ELEMS = 256, BLOCK_BYTES = 176, UNITS = 4;
    static constexpr int SEGS = 1, SEGLEN = 64, SEG_STRIDE = 0;
    __device__ static int elem_base(int u) { return 64 * u; }
    __device__ static void decode(const uint8_t *blk, int c, float *w) {
        const uint4 hdr = ld<uint4>(blk);
        const float d = f16_bits(hdr.x), dmin = f16_bits(hdr.x >> 16);
        uint32_t sc0, mn0, sc1, mn1;
        q4k_scale_min(hdr.y, hdr.z, hdr.w, 2 * c, sc0, mn0);
        q4k_scale_min(hdr.y, hdr.z, hdr.w, 2 * c + 1, sc1, mn1);
        const float d0 = d * (float)sc0, m0 = dmin * (float)mn0, d1 = d * (float)sc1, m1 = dmin * (float)mn1;
#pragma unroll
        for (int l = 0; l < 32; l++) {
            const int b = blk[48 + 32 * c + l], hb = blk[16 + l];
            w[l] = fmaf((float)((b & 0xF) | (((hb >> (2 * c)) & 1) << 4)), d0, -m0);
            w[32 + l] = fmaf((float)((b >> 4) | (((hb >> (2 * c + 1)) & 1) << 4)), d1, -m1);
        }
    }
    // Sub-block u (32 elements, eight a block) as eight words of int8: its 5-bit codes as they are, the scale d sc_u that
    // goes with their sum and the offset dmin m_u that goes with the activations' sum.
    static constexpr bool HAS_DECODE_I8 = true, I8_HAS_MIN = true;
    static constexpr int I8_UNITS = 8, I8_EXTRA_ENTRIES = 0;
    __device__ static uint64_t i8_extra_entry(int) { return 0; }
    __device__ static void decode_i8(const uint64_t *, const uint8_t *blk, int u, int *w, float &scale, float &offset) {
        const uint4 hdr = ld<uint4>(blk);
        uint32_t sc, mn;
        q4k_scale_min(hdr.y, hdr.z, hdr.w, u, sc, mn);
        const uint4 qa = ld<uint4>(blk + 48 + 32 * (u >> 1)), qb = ld<uint4>(blk + 64 + 32 * (u >> 1));
        const uint4 ha = ld<uint4>(blk + 16), hb = ld<uint4>(blk + 32);
        const uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        const uint32_t h[8] = {ha.x, ha.y, ha.z, ha.w, hb.x, hb.y, hb.z, hb.w};
#pragma unroll
        for (int i = 0; i < 8; i++) w[i] = (int)(((q[i] >> (4 * (u & 1))) & 0x0F0F0F0Fu) | (((h[i] >> u) & 0x01010101u) << 4));
        scale = f16_bits(hdr.x) * (float)sc;
        offset = f16_bits(hdr.x >> 16) * (float)mn;
    }
};

struct Q6_K {  // ql[128] | qh[64] | scales[16] i8 | d
    // (reference: vendor/candle-metal-kernels/src/metal_src/quantized.metal:198-203,6673-6694;
    //  the reference decodes it through candle's to_float, src/quant_matmul.rs:228-248)
    // unit u = (half h = u/2, lq = u%2): l in [16*lq, 16*lq+16); quarter t
    // covers elements 128*h + 32*t + l, scale scales[8*h + 2*t + lq].
    static constexpr int BLOCK_ELEMS = 256, BLOCK_BYTES = 210, UNITS = 4;
    static constexpr int SEGS = 4, SEGLEN = 16, SEG_STRIDE = 32;
    __device__ static int elem_base(int u) { return 128 * (u >> 1) + 16 * (u & 1); }
    __device__ static void decode(const uint8_t *blk, int u, float *w) {
        int h = u >> 1, lq = u & 1;
        float d = f16_bits(ld<uint16_t>(blk + 208));
        uint4 la = ldw<uint4>(blk + 64 * h + 16 * lq);        // ql[64h + l]
        uint4 lb = ldw<uint4>(blk + 64 * h + 32 + 16 * lq);   // ql[64h + 32 + l]
        uint4 hv = ldw<uint4>(blk + 128 + 32 * h + 16 * lq);  // qh[32h + l]
        uint32_t a[4] = {la.x, la.y, la.z, la.w}, b[4] = {lb.x, lb.y, lb.z, lb.w}, hh[4] = {hv.x, hv.y, hv.z, hv.w};
#pragma unroll
        for (int t = 0; t < 4; t++) {
            float ds = d * (float)(int8_t)blk[192 + 8 * h + 2 * t + lq];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                uint32_t lo = (t & 1) ? b[i] : a[i];
                uint32_t nib = (t < 2) ? (lo & 0x0F0F0F0Fu) : ((lo >> 4) & 0x0F0F0F0Fu);
                uint32_t q = nib | (((hh[i] >> (2 * t)) & 0x03030303u) << 4);
#pragma unroll
                for (int bb = 0; bb < 4; bb++)
                    w[16 * t + 4 * i + bb] = ds * (float)((int)((q >> (8 * bb)) & 0xFFu) - 32);
            }
        }
    }
};

struct IQ2_XXS {  // d | 8 x (lo:u32 codes, hi:u32 signs+scale)   (reference: src/iq2xxs.rs:34-71,349-380)
    static constexpr int BLOCK_ELEMS = 256, BLOCK_BYTES = 66, UNITS = 8;
    static constexpr int SEGS = 1, SEGLEN = 32, SEG_STRIDE = 0;
    __device__ static int elem_base(int u) { return 32 * u; }
    // `grid` is the 256-entry codebook: the constant table, or a workgroup's copy of it in LDS
    // (TABLE_BYTES), where the four lookups of a group cost LDS instead of vector-memory latency.
    static constexpr int TABLE_BYTES = 3072;  // the codebook and the sign masks behind it
    __device__ static const uint64_t *table() { return g_tables.iq2xxs_grid; }
    __device__ static void decode_with(const uint64_t *grid_table, const uint8_t *blk, int u, float *w) {
        float d = f16_bits(ld<uint16_t>(blk));
        uint2 g = ldw<uint2>(blk + 2 + 8 * u);
        uint32_t lo = g.x, hi = g.y;
        float db = d * (0.5f + (float)(hi >> 28)) * 0.25f;
#pragma unroll
        for (int l = 0; l < 4; l++) {
            uint64_t grid = grid_table[(lo >> (8 * l)) & 0xFFu];
            uint32_t s7 = (hi >> (7 * l)) & 127u;
            uint32_t signs = s7 | ((__popc(s7) & 1u) << 7);
#pragma unroll
            for (int j = 0; j < 8; j++) {
                float gv = (float)(uint32_t)((grid >> (8 * j)) & 0xFFu);
                w[8 * l + j] = ((signs >> j) & 1u ? -gv : gv) * db;
            }
        }
    }
    __device__ static void decode(const uint8_t *blk, int u, float *w) { decode_with(g_tables.iq2xxs_grid, blk, u, w); }
    // Unit u (32 elements) against its activations as two int8 planes: the codebook's magnitudes 8, 25, 43 are
    // negated byte by byte where the group's sign mask (table entry 256 + s) says so ((m ^ 0xFF) + 1 = 256 - m
    // never carries for m >= 8) and go to v_dot4 as signed bytes, so the integer arithmetic is exact.
    static constexpr bool HAS_DOT8 = true;
    __device__ static float dot8(const uint64_t *grid_table, const uint8_t *blk, int u, const uint32_t *xl,
                                 const uint32_t *xh, const float *sx, const float *) {
        const float d = f16_bits(ld<uint16_t>(blk));
        const uint2 g = ldw<uint2>(blk + 2 + 8 * u);
        const uint32_t lo = g.x, hi = g.y;
        int pl = 0, ph = 0;
#pragma unroll
        for (int l = 0; l < 4; l++) {
            const uint64_t grid = grid_table[(lo >> (8 * l)) & 0xFFu];
            const uint64_t neg = grid_table[256 + ((hi >> (7 * l)) & 127u)];
#pragma unroll
            for (int hf = 0; hf < 2; hf++) {  // elements 8l + 4hf .. + 3
                const uint32_t mag = (uint32_t)(grid >> (32 * hf)), mask = (uint32_t)(neg >> (32 * hf));
                const int w = (int)((mag ^ mask) + (mask & 0x01010101u));
                pl = __builtin_amdgcn_sdot4(w, (int)xl[2 * l + hf], pl, false);
                ph = __builtin_amdgcn_sdot4(w, (int)xh[2 * l + hf], ph, false);
            }
        }
        const float db = d * (0.5f + (float)(hi >> 28)) * 0.25f;
        return sx[0] * db * (float)((ph << 8) + pl);
    }
    // Unit u as eight words of signed int8 (elements 4i .. 4i+3 in word i) and its scale, the same way.
    static constexpr bool HAS_DECODE_I8 = true, I8_HAS_MIN = false;
    static constexpr int I8_UNITS = 8, I8_EXTRA_ENTRIES = 0;
    __device__ static uint64_t i8_extra_entry(int) { return 0; }
    __device__ static void decode_i8(const uint64_t *grid_table, const uint8_t *blk, int u, int *w, float &scale, float &offset) {
        offset = 0.0f;
        const float d = f16_bits(ld<uint16_t>(blk));
        const uint2 g = ldw<uint2>(blk + 2 + 8 * u);
        const uint32_t lo = g.x, hi = g.y;
#pragma unroll
        for (int l = 0; l < 4; l++) {
            const uint64_t grid = grid_table[(lo >> (8 * l)) & 0xFFu];
            const uint64_t neg = grid_table[256 + ((hi >> (7 * l)) & 127u)];
#pragma unroll
            for (int hf = 0; hf < 2; hf++) {
                const uint32_t mag = (uint32_t)(grid >> (32 * hf)), mask = (uint32_t)(neg >> (32 * hf));
                w[2 * l + hf] = (int)((mag ^ mask) + (mask & 0x01010101u));
            }
        }
        scale = d * (0.5f + (float)(hi >> 28)) * 0.25f;
    }
};

struct MXFP4 {  // e:u8 | qs[16]   (reference: src/mxfp4.rs:45-94)
    static constexpr int BLOCK_ELEMS = 32, BLOCK_BYTES = 17, UNITS = 1;
    static constexpr int SEGS = 1, SEGLEN = 32, SEG_STRIDE = 0;
    __device__ static int elem_base(int) { return 0; }
    // E2M1 code c -> its value: the code's three magnitude bits placed at bit 22 of an f32 word read as
    // (1 + mant/2) * 2^(exp - 127), or as the denormal mant * 2^-127 when exp == 0, which is 2^-126
    // times the E2M1 value in both cases (1 exponent bit of bias against 127); the sign bit moves to
    // bit 31.  One multiply by 2^126 then gives +-{0, .5, 1, 1.5, 2, 3, 4, 6} exactly.
    __device__ static float e2m1(uint32_t c) {
        return __uint_as_float(((c & 7u) << 22) | ((c & 8u) << 28)) * 8.507059173023462e37f;  // 2^126
    }
    // The block against its 32 activations given as 15-bit fixed point in two int8 planes (X = 256 hi +
    // lo, eight registers a plane): v_perm_b32 looks four magnitude codes up at once in the table of
    // doubled E2M1 values {0,1,2,3,4,6,8,12} and once more in the table of their negatives, the sign bits
    // pick between the two byte by byte, and the signed bytes go to v_dot4, so the integer arithmetic is exact.
    // Returns sum w_i x_i over the block: sx is the activations' scale, x = sx X.
    static constexpr bool HAS_DOT8 = true;
    __device__ static float dot8(const uint64_t *, const uint8_t *blk, int, const uint32_t *xl, const uint32_t *xh,
                                 const float *sx, const float *) {
        const uint32_t e = blk[0];
        if (e == 0xFFu) return 0.0f;
        const float d = __uint_as_float(e == 0 ? 0x00400000u : (e << 23));
        int pl = 0, ph = 0;
        const uint4 qv = ldw<uint4>(blk + 1);
        const uint32_t qw[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int hi = 0; hi < 2; hi++) {  // low nibbles: elements 4i .. 4i+3; high nibbles: 16 + 4i ..
                const uint32_t v = hi ? qw[i] >> 4 : qw[i];
                const uint32_t sel = v & 0x07070707u;
                const uint32_t pos = __builtin_amdgcn_perm(0x0C080604u, 0x03020100u, sel);
                const uint32_t neg = __builtin_amdgcn_perm(0xF4F8FAFCu, 0xFDFEFF00u, sel);
                const uint32_t mask = ((v >> 3) & 0x01010101u) * 0xFFu;
                const int w = (int)((pos & ~mask) | (neg & mask));
                pl = __builtin_amdgcn_sdot4(w, (int)xl[4 * hi + i], pl, false);
                ph = __builtin_amdgcn_sdot4(w, (int)xh[4 * hi + i], ph, false);
            }
        }
        const int s2 = (ph << 8) + pl;  // twice the sum: the table holds doubled values
        return sx[0] * d * (0.5f * (float)s2);
    }
    // The block as eight words of signed int8, twice the E2M1 values (elements 4i .. 4i+3 in word i, the low
    // nibbles first), and the scale that goes with them (half the block's): two lookups, of the doubled
    // magnitudes and of their negatives, and the sign bit picks between them byte by byte.
    static constexpr bool HAS_DECODE_I8 = true, I8_HAS_MIN = false;
    static constexpr int I8_UNITS = 1, I8_EXTRA_ENTRIES = 0;
    __device__ static uint64_t i8_extra_entry(int) { return 0; }
    __device__ static void decode_i8(const uint64_t *, const uint8_t *blk, int, int *w, float &scale, float &offset) {
        offset = 0.0f;
        const uint32_t e = blk[0];
        const uint4 qv = ldw<uint4>(blk + 1);
        const uint32_t qw[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int hi = 0; hi < 2; hi++) {
                const uint32_t v = hi ? qw[i] >> 4 : qw[i];
                const uint32_t sel = v & 0x07070707u;
                const uint32_t pos = __builtin_amdgcn_perm(0x0C080604u, 0x03020100u, sel);
                const uint32_t neg = __builtin_amdgcn_perm(0xF4F8FAFCu, 0xFDFEFF00u, sel);
                const uint32_t mask = ((v >> 3) & 0x01010101u) * 0xFFu;
                w[4 * hi + i] = (int)((pos & ~mask) | (neg & mask));
            }
        }
        // 2^(e-127) / 2; e == 0 is the f32 denormal 2^-127; 0xFF (reserved) decodes the block to zeros
        scale = e == 0xFFu ? 0.0f : 0.5f * __uint_as_float(e == 0 ? 0x00400000u : (e << 23));
    }
    __device__ static void decode(const uint8_t *blk, int, float *w) {
        uint32_t e = blk[0];
        // 2^(e-127); e == 0 is the f32 denormal 2^-127; 0xFF (reserved) decodes the block to zeros
        float d = __uint_as_float(e == 0 ? 0x00400000u : (e << 23));
        const bool dead = e == 0xFFu;
        const uint4 qv = ldw<uint4>(blk + 1);
        const uint32_t qw[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t v = qw[i];
#pragma unroll
            for (int b = 0; b < 4; b++) {
                uint32_t byte = (v >> (8 * b)) & 0xFFu;
                w[4 * i + b] = dead ? 0.0f : d * e2m1(byte & 0xFu);
                w[16 + 4 * i + b] = dead ? 0.0f : d * e2m1(byte >> 4);
            }
        }
    }
};

}  // namespace jq
