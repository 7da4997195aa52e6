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
    uint32_t dm[4];  // d | dmin of rows 4*kg .. 4*kg+3: the rows this lane holds results of
};

// The activations of a wave's CPW columns as MFMA B operands.
template <int CPW>
struct QsActs {
    qg_u4 Bh[CPW][8], Bl[CPW][8], Bm[CPW];
    float sx[CPW];
};

// Quantises the wave's columns of one activation row per lane group: lanes with the same `lane & 15`
// share the row `xrow` (null: a row of zeros), lane group kg = lane >> 4 takes 8 of every 32 k.
template <int CPW>
__device__ __forceinline__ void qs_quantise_acts(const float *xrow, int wave, int kg, QsActs<CPW> &A) {
#pragma unroll
    for (int j = 0; j < CPW; j++) {
        const int b = wave * CPW + j;
        float xv[8][8];
        float amax = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 8; ks++) {
            float4 a = float4{0.f, 0.f, 0.f, 0.f}, c = a;
            if (xrow) {
                const float *xp = xrow + 256 * b + 32 * ks + 8 * kg;
                a = *(const float4 *)xp, c = *(const float4 *)(xp + 4);
            }
            xv[ks][0] = a.x, xv[ks][1] = a.y, xv[ks][2] = a.z, xv[ks][3] = a.w;
            xv[ks][4] = c.x, xv[ks][5] = c.y, xv[ks][6] = c.z, xv[ks][7] = c.w;
#pragma unroll
            for (int i = 0; i < 8; i++) amax = fmaxf(amax, mag_or_inf(xv[ks][i]));
        }
        amax = max_xor16(amax);
        amax = max_xor32(amax);
        const bool live = amax > 0.0f && amax < INFINITY;
        const float inv = live ? QG_RANGE / amax : 0.0f;
        A.sx[j] = fixed_scale(amax, QG_RANGE);
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
            A.Bh[j][ks] = qg_u4{qg_pack_h2(hi[0], hi[2]), qg_pack_h2(hi[1], hi[3]), qg_pack_h2(hi[4], hi[6]), qg_pack_h2(hi[5], hi[7])};
            A.Bl[j][ks] = qg_u4{qg_pack_h2(lo[0], lo[2]), qg_pack_h2(lo[1], lo[3]), qg_pack_h2(lo[4], lo[6]), qg_pack_h2(lo[5], lo[7])};
            sum = isum_xor16(sum);
            sum = isum_xor32(sum);
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
        A.Bm[j] = __builtin_bit_cast(qg_u4, pm);
    }
}

// The same operands prepared once per activation row by q4k_acts_prep and read back by every
// workgroup that needs them.  One record of QS_REC bytes per (row, 256-element column):
//   bytes ((ks * 2 + plane) * 4 + kg) * 16 ..+15   the 8 halves of plane `plane` (0 high, 1 low) that
//                                                 lane group kg feeds to the MFMA of 32-element step ks
//   bytes 1024 + kg * 16 ..+15 (kg < 3)            the min operand of lane group kg
//   bytes 1072 ..1075                              the column's scale (f32); 1076 ..1087 zero
// Records sit row after row.  (Laying the 16 rows of a tile side by side, so that a wave's load
// is one contiguous kilobyte, measured slower: every workgroup then reads the same kilobyte at the
// same time, and the requests pile up on one memory channel.)
constexpr int QS_REC = 1088;

__global__ __launch_bounds__(256) void q4k_acts_prep(const float *__restrict__ X, int rows, int k,
                                                      uint8_t *__restrict__ out) {
    const int nb = k >> 8;
    const int unit = (int)((blockIdx.x * 256 + threadIdx.x) >> 5);  // one record per 32 lanes
    if (unit >= rows * nb) return;  // whole half-waves leave; the shuffles below stay within 32 lanes
    const int row = unit / nb, b = unit % nb;
    const int l = threadIdx.x & 31, ks = l >> 2, kg = l & 3;
    const float *xp = X + (size_t)row * k + 256 * b + 32 * ks + 8 * kg;
    const float4 a = *(const float4 *)xp, c = *(const float4 *)(xp + 4);
    const float xv[8] = {a.x, a.y, a.z, a.w, c.x, c.y, c.z, c.w};
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) amax = fmaxf(amax, mag_or_inf(xv[i]));
#pragma unroll
    for (int off = 1; off < 32; off <<= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    const bool live = amax > 0.0f && amax < INFINITY;
    const float inv = live ? QG_RANGE / amax : 0.0f, sx = fixed_scale(amax, QG_RANGE);
    int lo[8], hi[8], sum = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int Xi = __float2int_rn(xv[i] * inv);
        lo[i] = ((Xi + 1024) & 2047) - 1024;
        hi[i] = (Xi - lo[i]) >> 11;
        sum += Xi;
    }
    // slot j (0..16: the 16 operand slots, then the min operand) of this lane group
    uint8_t *base = out + (size_t)unit * QS_REC + kg * 16;
    constexpr int slot_stride = 64;
    // operand order within the 8 k of a lane: 0,2,1,3,4,6,5,7 (what the weight unpack produces)
    *(qg_u4 *)(base + (ks * 2 + 0) * slot_stride) =
        qg_u4{qg_pack_h2(hi[0], hi[2]), qg_pack_h2(hi[1], hi[3]), qg_pack_h2(hi[4], hi[6]), qg_pack_h2(hi[5], hi[7])};
    *(qg_u4 *)(base + (ks * 2 + 1) * slot_stride) =
        qg_u4{qg_pack_h2(lo[0], lo[2]), qg_pack_h2(lo[1], lo[3]), qg_pack_h2(lo[4], lo[6]), qg_pack_h2(lo[5], lo[7])};
    sum += __shfl_xor(sum, 1, 64);
    sum += __shfl_xor(sum, 2, 64);  // the 32-element step's sum, in its four lanes
    _Float16 p0, p1, p2;
    qg_split_sum(sum, p0, p1, p2);
    uint8_t *mslot = base + 16 * slot_stride;
    if (kg < 3) {
        *(_Float16 *)(mslot + ks * 2) = kg == 0 ? p0 : kg == 1 ? p1 : p2;
    } else if (ks == 0) {
        *(uint2 *)mslot = uint2{__float_as_uint(sx), 0u};
    } else if (ks == 1) {
        *(uint2 *)(mslot + 8) = uint2{0u, 0u};
    }
}

// The operands of one column for lane group kg: `base` is the address of the lane group's piece of
// slot 0 in its row's record (null: a row of zeros).
__device__ __forceinline__ void qs_load_acts(const uint8_t *base, int kg, QsActs<1> &A) {
    constexpr int slot_stride = 64;
    if (!base) {
#pragma unroll
        for (int ks = 0; ks < 8; ks++) A.Bh[0][ks] = A.Bl[0][ks] = qg_u4{0, 0, 0, 0};
        A.Bm[0] = qg_u4{0, 0, 0, 0};
        A.sx[0] = 0.0f;
        return;
    }
#pragma unroll
    for (int ks = 0; ks < 8; ks++) {
        A.Bh[0][ks] = *(const qg_u4 *)(base + (ks * 2 + 0) * slot_stride);
        A.Bl[0][ks] = *(const qg_u4 *)(base + (ks * 2 + 1) * slot_stride);
    }
    const qg_u4 bm = *(const qg_u4 *)(base + 16 * slot_stride);
    A.Bm[0] = kg < 3 ? bm : qg_u4{0, 0, 0, 0};
    // the scale sits in the slot's fourth piece
    A.sx[0] = *(const float *)(base + 16 * slot_stride + (3 - kg) * 16);
}

// Rows row0 .. row0 + 15 of W (clamped to n - 1), the wave's columns: header and this lane group's
// nibble bytes of row row0 + col, and d | dmin of the four rows whose results the lane will hold.
template <int CPW>
__device__ __forceinline__ void qs_load_tile(const uint8_t *__restrict__ W, size_t row_bytes, int row0, int n, int col,
                                             int wave, int kg, QsTileRegs (&r)[CPW]) {
    const uint8_t *rp = W + (size_t)min(row0 + col, n - 1) * row_bytes + (size_t)(wave * CPW) * 144;
#pragma unroll
    for (int j = 0; j < CPW; j++) {
        const uint8_t *blk = rp + 144 * j;
        r[j].hdr = *(const qg_u4 *)blk;
#pragma unroll
        for (int c = 0; c < 4; c++) r[j].nib[c] = *(const uint2 *)(blk + 16 + 32 * c + 8 * kg);
#pragma unroll
        for (int jj = 0; jj < 4; jj++)
            r[j].dm[jj] = *(const uint32_t *)(W + (size_t)min(row0 + 4 * kg + jj, n - 1) * row_bytes +
                                              (size_t)(wave * CPW + j) * 144);
    }
}

// The wave's share of a 16-row tile times the activations: acc[jj] belongs to weight row
// 4*kg + jj of the tile and activation row lane & 15.
template <int CPW>
__device__ __forceinline__ void qs_tile_partial(const QsTileRegs (&cur)[CPW], const QsActs<CPW> &A, int kg, float (&acc)[4]) {
    acc[0] = acc[1] = acc[2] = acc[3] = 0.0f;
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
            qg_u4 lo, hi;
            qg_unpack_words(w0, w1, qg_scale_operand_lo(sc[2 * c]), qg_scale_operand_hi(sc[2 * c + 1]), lo, hi);
            const qg_h8 alo = __builtin_bit_cast(qg_h8, lo), ahi = __builtin_bit_cast(qg_h8, hi);
            Ph = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, __builtin_bit_cast(qg_h8, A.Bh[j][2 * c]), Ph, 0, 0, 0);
            Pl = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, __builtin_bit_cast(qg_h8, A.Bl[j][2 * c]), Pl, 0, 0, 0);
            Ph = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, __builtin_bit_cast(qg_h8, A.Bh[j][2 * c + 1]), Ph, 0, 0, 0);
            Pl = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, __builtin_bit_cast(qg_h8, A.Bl[j][2 * c + 1]), Pl, 0, 0, 0);
        }
        qg_u4 am = qg_u4{0, 0, 0, 0};
        if (kg < 3)
            am = qg_u4{qg_pack_h2((int)mn[0], (int)mn[1]), qg_pack_h2((int)mn[2], (int)mn[3]),
                       qg_pack_h2((int)mn[4], (int)mn[5]), qg_pack_h2((int)mn[6], (int)mn[7])};
        const qg_f4 MM = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(qg_h8, am), __builtin_bit_cast(qg_h8, A.Bm[j]),
                                                                qg_f4{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            const float dr = f16_bits(cur[j].dm[jj]), mr = f16_bits(cur[j].dm[jj] >> 16);
            const float f = fmaf(Ph[jj], 2048.0f, Pl[jj]);
            const float tt = fmaf(-4096.0f * mr, MM[jj], dr * f);
            acc[jj] = fmaf(A.sx[j], tt, acc[jj]);
        }
    }
}

template <int CPW>
__global__ __launch_bounds__(64 * QS_MAX_WAVES) void q4k_stream_mfma(const uint8_t *__restrict__ W, size_t row_bytes,
                                                                      const float *__restrict__ X,
                                                                      float *__restrict__ Y, int m, int k, int n) {
    __shared__ qg_f4 red[2][QS_MAX_WAVES][64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
    const int col = lane & 15, kg = lane >> 4;
    const int n_tiles = (n + 15) >> 4;

    QsActs<CPW> A;
    qs_quantise_acts<CPW>(col < m ? X + (size_t)col * k : nullptr, wave, kg, A);

    QsTileRegs cur[CPW], nxt[CPW];
    int t = blockIdx.x;
    if (t < n_tiles) qs_load_tile<CPW>(W, row_bytes, 16 * t, n, col, wave, kg, cur);
    for (int it = 0; t < n_tiles; t += gridDim.x, it++) {
        const int tn = t + gridDim.x;
        if (tn < n_tiles) qs_load_tile<CPW>(W, row_bytes, 16 * tn, n, col, wave, kg, nxt);

        float acc[4];
        qs_tile_partial<CPW>(cur, A, kg, acc);

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
