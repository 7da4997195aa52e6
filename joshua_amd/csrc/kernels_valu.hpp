// Row-per-wavefront fused dequant+dot kernels on the vector ALU, plus the
// decode-only kernels (dequantize, embedding).  One wave64 owns one weight
// row: its lanes take the row's units in turn, decode each unit in registers
// and multiply-accumulate it against up to MT activation rows; a cross-lane
// butterfly finishes the sum.  Per element the arithmetic is the reference's
// (decode with one fused multiply-subtract, then one fused multiply-add into
// the running sum; reference: src/kquant_dot.rs:426-476); only the order in
// which a row's products are added differs from the 8-lane CPU order.
//
// These kernels serve every format and every m.  They are the general path;
// the MFMA kernels take over where they apply.
#pragma once
#include <type_traits>
#include "blocks.hpp"

namespace jq {

__device__ __forceinline__ float silu(float v) { return v / (1.0f + expf(-v)); }

// The optional clamp in front of an expert's SwiGLU: gate from above, up on both sides
// (reference: src/quantized_deepseek4.rs:445-462; limit <= 0: none).  An expert whose id is at or past
// `n_routed` is a shared expert and has a limit of its own (:2419-2448).  A NaN stays a NaN.
struct MoeClamp {
    float routed, shared;
    int n_routed;
};
__device__ __forceinline__ float swiglu(float g, float u, float limit) {
    if (limit > 0.0f) {
        g = g > limit ? limit : g;
        u = u > limit ? limit : (u < -limit ? -limit : u);
    }
    return silu(g) * u;
}
__device__ __forceinline__ float swiglu(float g, float u, const MoeClamp &cl, int expert) {
    return swiglu(g, u, expert >= cl.n_routed ? cl.shared : cl.routed);
}

__device__ __forceinline__ float wave_sum(float v) {
    v = sum_xor32(v);
    v = sum_xor16(v);
    return sum_row16(v);
}

constexpr int ROWS_PER_WG = 4;  // one wave per row, 256 threads

template <class Q, int MT>
__global__ __launch_bounds__(64 * ROWS_PER_WG) void matmul_rows_valu(const uint8_t *__restrict__ W, size_t row_bytes,
                                                                      const float *__restrict__ X,
                                                                      float *__restrict__ Y, int m, int k, int n) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * ROWS_PER_WG + (threadIdx.x >> 6);
    if (row >= n) return;  // wave-uniform
    const uint8_t *rp = W + (size_t)row * row_bytes;
    const int units = (k / Q::BLOCK_ELEMS) * Q::UNITS;
    constexpr int UE = Q::SEGS * Q::SEGLEN;
    for (int m0 = 0; m0 < m; m0 += MT) {
        float acc[MT];
#pragma unroll
        for (int i = 0; i < MT; i++) acc[i] = 0.0f;
        for (int u = lane; u < units; u += 64) {
            const int b = u / Q::UNITS, ub = u % Q::UNITS;
            float w[UE];
            Q::decode(rp + (size_t)b * Q::BLOCK_BYTES, ub, w);
            const int xoff = b * Q::BLOCK_ELEMS + Q::elem_base(ub);
#pragma unroll
            for (int i = 0; i < MT; i++) {
                if (m0 + i < m) {
                    const float *xp = X + (size_t)(m0 + i) * k + xoff;
#pragma unroll
                    for (int s = 0; s < Q::SEGS; s++) {
#pragma unroll
                        for (int e = 0; e < Q::SEGLEN; e += 4) {
                            float4 xv = ld<float4>((const uint8_t *)(xp + s * Q::SEG_STRIDE + e));
                            acc[i] = fmaf(xv.x, w[s * Q::SEGLEN + e + 0], acc[i]);
                            acc[i] = fmaf(xv.y, w[s * Q::SEGLEN + e + 1], acc[i]);
                            acc[i] = fmaf(xv.z, w[s * Q::SEGLEN + e + 2], acc[i]);
                            acc[i] = fmaf(xv.w, w[s * Q::SEGLEN + e + 3], acc[i]);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < MT; i++) {
            float s = wave_sum(acc[i]);
            if (lane == 0 && m0 + i < m) Y[(size_t)(m0 + i) * n + row] = s;
        }
    }
}

// Asynchronous global -> LDS load of `bytes` (4 or 16) per active lane; the wave's data lands
// contiguously at lds_base + lane * bytes (lds_base wave-uniform, carried in M0, which nothing else
// in these kernels uses).  Inline assembly: the caller awaits the loads itself with s_waitcnt vmcnt.
__device__ __forceinline__ uint32_t lds_offset_of(const void *p) {
    return (uint32_t)(uintptr_t)((__attribute__((address_space(3))) const void *)p);
}
__device__ __forceinline__ void async_load16(const void *gptr, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr),
                 "s"(__builtin_amdgcn_readfirstlane(lds_base))
                 : "memory");
}
__device__ __forceinline__ void async_load4(const void *gptr, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(gptr),
                 "s"(__builtin_amdgcn_readfirstlane(lds_base))
                 : "memory");
}

// Formats that decode through a lookup table keep a copy of it at the start of the workgroup's
// dynamic LDS (table_bytes<Q>() bytes, 0 for the others).
template <class Q, class = void>
struct HasTable : std::false_type {};
template <class Q>
struct HasTable<Q, std::void_t<decltype(Q::TABLE_BYTES)>> : std::true_type {};

template <class Q>
__host__ __device__ constexpr int table_bytes() {
    if constexpr (HasTable<Q>::value) return Q::TABLE_BYTES;
    else return 0;
}
template <class Q>
__device__ __forceinline__ const uint64_t *stage_table(uint8_t *lds) {
    if constexpr (HasTable<Q>::value) {
        for (int i = threadIdx.x; i < Q::TABLE_BYTES / 8; i += blockDim.x) ((uint64_t *)lds)[i] = Q::table()[i];
        __syncthreads();
        return (const uint64_t *)lds;
    } else {
        return nullptr;
    }
}
template <class Q>
__device__ __forceinline__ void decode_staged(const uint64_t *table, const uint8_t *blk, int u, float *w) {
    if constexpr (HasTable<Q>::value) Q::decode_with(table, blk, u, w);
    else Q::decode(blk, u, w);
}

// The same arithmetic as matmul_rows_valu with the weight row staged through LDS: each wave first
// pulls its whole packed row into LDS with fully coalesced asynchronous loads of G bytes per lane
// (the whole row in flight at once, whatever the block size), then decodes blocks out of LDS.  A
// block-strided global read (34-, 66-, 210-byte blocks) touches every cache line many times; this
// touches each once.  Needs row starts and row_bytes that are multiples of G; LDS = 4 rows.
template <class Q, int MT, int G>
__global__ __launch_bounds__(64 * ROWS_PER_WG) void matmul_rows_staged(const uint8_t *__restrict__ W, size_t row_bytes,
                                                                        const float *__restrict__ X,
                                                                        float *__restrict__ Y, int m, int k, int n,
                                                                        int lds_stride) {
    extern __shared__ __attribute__((aligned(16))) uint8_t staged_rows[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const auto *table = stage_table<Q>(staged_rows);  // before any wave leaves: it holds a barrier
    const int row = blockIdx.x * ROWS_PER_WG + wave;
    if (row >= n) return;  // wave-uniform
    uint8_t *rp = staged_rows + table_bytes<Q>() + (size_t)wave * lds_stride;
    {
        const uint8_t *src = W + (size_t)row * row_bytes;
        const int pieces = (int)(row_bytes / G);
        for (int p0 = 0; p0 < pieces; p0 += 64) {
            if (p0 + lane < pieces) {
                if (G == 16) async_load16(src + (size_t)(p0 + lane) * 16, lds_offset_of(rp + (size_t)p0 * 16));
                else async_load4(src + (size_t)(p0 + lane) * 4, lds_offset_of(rp + (size_t)p0 * 4));
            }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    const int units = (k / Q::BLOCK_ELEMS) * Q::UNITS;
    constexpr int UE = Q::SEGS * Q::SEGLEN;
    for (int m0 = 0; m0 < m; m0 += MT) {
        float acc[MT];
#pragma unroll
        for (int i = 0; i < MT; i++) acc[i] = 0.0f;
        for (int u = lane; u < units; u += 64) {
            const int b = u / Q::UNITS, ub = u % Q::UNITS;
            float w[UE];
            decode_staged<Q>(table, rp + (size_t)b * Q::BLOCK_BYTES, ub, w);
            const int xoff = b * Q::BLOCK_ELEMS + Q::elem_base(ub);
#pragma unroll
            for (int i = 0; i < MT; i++) {
                if (m0 + i < m) {
                    const float *xp = X + (size_t)(m0 + i) * k + xoff;
#pragma unroll
                    for (int s = 0; s < Q::SEGS; s++) {
#pragma unroll
                        for (int e = 0; e < Q::SEGLEN; e += 4) {
                            float4 xv = ld<float4>((const uint8_t *)(xp + s * Q::SEG_STRIDE + e));
                            acc[i] = fmaf(xv.x, w[s * Q::SEGLEN + e + 0], acc[i]);
                            acc[i] = fmaf(xv.y, w[s * Q::SEGLEN + e + 1], acc[i]);
                            acc[i] = fmaf(xv.z, w[s * Q::SEGLEN + e + 2], acc[i]);
                            acc[i] = fmaf(xv.w, w[s * Q::SEGLEN + e + 3], acc[i]);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < MT; i++) {
            float s = wave_sum(acc[i]);
            if (lane == 0 && m0 + i < m) Y[(size_t)(m0 + i) * n + row] = s;
        }
    }
}

// Canonical decode ("to_float"): differs from the in-dot decode only for the
// formats whose to_float uses two rounded operations instead of one fused
// multiply-subtract (Q2_K, Q4_K; reference: src/kquant_dot.rs:258-260).
template <class Q>
struct ToFloat {
    __device__ static void decode(const uint8_t *blk, int u, float *w) { Q::decode(blk, u, w); }
};

template <>
struct ToFloat<Q4_K> {
    __device__ static void decode(const uint8_t *blk, int c, float *w) {
        uint4 hdr = ld<uint4>(blk);
        float d = f16_bits(hdr.x), dmin = f16_bits(hdr.x >> 16);
        uint32_t sc0, mn0, sc1, mn1;
        q4k_scale_min(hdr.y, hdr.z, hdr.w, 2 * c, sc0, mn0);
        q4k_scale_min(hdr.y, hdr.z, hdr.w, 2 * c + 1, sc1, mn1);
        float d0 = d * (float)sc0, m0 = dmin * (float)mn0;
        float d1 = d * (float)sc1, m1 = dmin * (float)mn1;
        for (int i = 0; i < 32; i++) {
            uint32_t byte = blk[16 + 32 * c + i];
            w[i] = __fsub_rn(__fmul_rn(d0, (float)(byte & 0xFu)), m0);
            w[32 + i] = __fsub_rn(__fmul_rn(d1, (float)(byte >> 4)), m1);
        }
    }
};

template <>
struct ToFloat<Q2_K> {
    __device__ static void decode(const uint8_t *blk, int u, float *w) {
        int sg = u >> 1, hf = u & 1;
        float d = f16_bits(ld<uint16_t>(blk + 80)), dmin = f16_bits(ld<uint16_t>(blk + 82));
        for (int f = 0; f < 4; f++) {
            uint32_t s = blk[8 * sg + 2 * f + hf];
            float dl = d * (float)(s & 0xFu), ml = dmin * (float)(s >> 4);
            for (int i = 0; i < 16; i++) {
                uint32_t q = (blk[16 + 32 * sg + 16 * hf + i] >> (2 * f)) & 3u;
                w[16 * f + i] = __fsub_rn(__fmul_rn(dl, (float)q), ml);
            }
        }
    }
};

// out[r*k + ...] = decode(row ids[r]) (ids == nullptr: row r itself).
template <class Q>
__global__ __launch_bounds__(256) void decode_rows(const uint8_t *__restrict__ W, size_t row_bytes,
                                                    const uint32_t *__restrict__ ids, float *__restrict__ out,
                                                    size_t n_out_rows, int k) {
    const int units_per_row = (k / Q::BLOCK_ELEMS) * Q::UNITS;
    const size_t total = n_out_rows * (size_t)units_per_row;
    constexpr int UE = Q::SEGS * Q::SEGLEN;
    for (size_t g = (size_t)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += (size_t)gridDim.x * blockDim.x) {
        const size_t r = g / units_per_row;
        const int u = (int)(g % units_per_row);
        const size_t src_row = ids ? ids[r] : r;
        const int b = u / Q::UNITS, ub = u % Q::UNITS;
        float w[UE];
        ToFloat<Q>::decode(W + src_row * row_bytes + (size_t)b * Q::BLOCK_BYTES, ub, w);
        float *o = out + r * (size_t)k + (size_t)b * Q::BLOCK_ELEMS + Q::elem_base(ub);
#pragma unroll
        for (int s = 0; s < Q::SEGS; s++)
#pragma unroll
            for (int e = 0; e < Q::SEGLEN; e++) o[s * Q::SEG_STRIDE + e] = w[s * Q::SEGLEN + e];
    }
}

// Raw tensor bytes that are no weight format of the matmuls, to f32 (reference: src/quant_matmul.rs:36-103
// decode_raw_to_f32): KIND 1 = F16 elements, 9 = Q8_1 blocks (f16 d, f16 s, 32 int8: d * q, the published ggml
// layout), 15 = Q8_K blocks (f32 d, 256 int8, 16 int16 sums: d * q).  One element a thread.
template <int KIND>
__global__ __launch_bounds__(256) void decode_plain(const uint8_t *__restrict__ raw, float *__restrict__ out, size_t elems) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < elems; i += (size_t)gridDim.x * blockDim.x) {
        if (KIND == 1) {
            out[i] = f16_bits((uint32_t)raw[2 * i] | ((uint32_t)raw[2 * i + 1] << 8));
        } else {
            constexpr size_t BLCK = KIND == 9 ? 32 : 256, BB = KIND == 9 ? 36 : 292;
            const uint8_t *blk = raw + (i / BLCK) * BB;
            float d;
            if (KIND == 9) d = f16_bits((uint32_t)blk[0] | ((uint32_t)blk[1] << 8));
            else d = __builtin_bit_cast(float, (uint32_t)blk[0] | ((uint32_t)blk[1] << 8) | ((uint32_t)blk[2] << 16) | ((uint32_t)blk[3] << 24));
            out[i] = d * (float)(int8_t)blk[4 + i % BLCK];
        }
    }
}

// f32 -> f16 (round to nearest even, overflow to infinity: half::f16::from_f32), one element a thread.
__global__ __launch_bounds__(256) void f32_to_f16(const float *__restrict__ in, uint16_t *__restrict__ out, size_t elems) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < elems; i += (size_t)gridDim.x * blockDim.x)
        out[i] = __builtin_bit_cast(uint16_t, (_Float16)in[i]);
}

}  // namespace jq
