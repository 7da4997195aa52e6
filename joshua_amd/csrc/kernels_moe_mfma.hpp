// The expert matmuls of a decode-sized mixture-of-experts call (every routed (token, expert) pair reads its
// expert's rows once) on the int8 matrix cores, over the per-format policies of the one-row GEMV
// (kernels_gemv_mfma.hpp): a wave quantises 256 activations once into registers as the block-diagonal A operand
// and multiplies them with one super-block column of 16 weight rows an instruction group, so no activation
// is read a second time and the integer dot products cost four MFMAs a wave and 16 rows.
//
//   moe_gate_up_mfma    G[pair, j] = silu(gate_e[j] . x_t) * (up_e[j] . x_t)    (reference: src/quantized_qwen3_moe.rs:397-401)
//   moe_down_mfma       y[t, r]    = sum_s w[t, s] (down_e(s)[r] . G[pair(t, s)])  (:504-520, src/quantized_deepseek2.rs:553-557)
//
// Both take rows of at most 8 (gate, up) or 16 (down) super-blocks: the waves of a workgroup then cover whole tiles
// of 16 rows at once and every weight byte of the call is asked for in the launch's first microsecond.
#pragma once
#include "kernels_gemv_mfma.hpp"
#include "kernels_valu.hpp"
#include "kernels_moe.hpp"

namespace jq {

// LDS rows 16 bytes past a multiple of 256: the 16 rows a wave's lanes read side by side fall on all banks.
constexpr int moe_mfma_row_lds(int bytes) { return (bytes + 255) / 256 * 256 + 16; }

// The policy of the formats whose 32-element units decode to signed int8 words (Q::decode_i8: IQ2_XXS through its
// codebook, MXFP4 through two byte permutes): a super-block is 256 consecutive elements, 8 units (one IQ2_XXS block,
// eight MXFP4 blocks).  Lane (r, c) decodes units 2c and 2c + 1 of weight row r into the B operands of four MFMAs;
// the activations are 15-bit fixed point a 32-element sub-block in two int8 planes, block-diagonal in A as for
// Q4_K (row 4c + 2p + plane is non-zero in lane group c only), so the lane receives the two planes' sums of both
// its units and   sum = scale(2c) s(2c) (256 Sh + Sl) + scale(2c + 1) s(2c + 1) (256 Sh' + Sl').
// Every integer sum is exact (|w| <= 43, |X| <= 128, 32 terms).
// Formats whose codes are unsigned with an offset (Q4_0 .. Q5_1, Q5_K: w = scale code - offset) add
// - offset(2c) s(2c) sum X - offset(2c + 1) s(2c + 1) sum X'.  Also a policy of the one-row GEMV (gemv_mfma_lds,
// gemv_mfma_cols) for the formats without a lookup table.
template <class Q>
struct QvI8 {
    static_assert(Q::HAS_DECODE_I8, "units that decode to int8 words, a scale and an offset");
    static constexpr int SUB = 256 / Q::BLOCK_ELEMS;   // format blocks a super-block
    static_assert(SUB * Q::I8_UNITS == 8, "eight units of 32 elements a super-block");
    static constexpr int BLOCK = SUB * Q::BLOCK_BYTES, ROW = 16 * BLOCK, ROW_LDS = moe_mfma_row_lds(ROW);
    static constexpr int STAGE_BYTES = 4 * (128 + 8 + 16);  // the two planes, eight zero words, the sub-blocks' scales and scale x sum
    static constexpr bool TAKES_TABLE = true, SIDE_LDS = false;
    // the one-row GEMV's ring: three tiles of 16 rows where they fit beside its partial sums, else two
    static constexpr int COLS = 4096, SLOTS = 3 * 16 * ROW_LDS + 20 * 1024 <= 160 * 1024 ? 3 : 2;
    typedef Q Format;
    struct Acts {
        qv_i4 a_even[2], a_odd[2];
        float s_e, s_o, xs_e, xs_o;
    };
    __device__ static __forceinline__ void scale(Acts &a, float f) { a.s_e *= f, a.s_o *= f, a.xs_e *= f, a.xs_o *= f; }
    __device__ static __forceinline__ Acts prepare(const float4 v, uint32_t *stage, int lane) {
        const int r = lane & 15, c = lane >> 4;
        const QvQuant q = qv_quantise4(v);
        stage[lane] = q.wl, stage[64 + lane] = q.wh;
        if (lane < 8) stage[128 + lane] = 0;
        float *scales = (float *)(stage + 136);
        if ((lane & 7) == 0) scales[lane >> 3] = q.s, scales[8 + (lane >> 3)] = q.s * (float)q.sum;
        // (the words are written as scalars and read back as vectors: the compiler keeps the order only when told)
        asm volatile("" ::: "memory");
        // row m = r of A: lane group (r / 4) only, unit parity (r / 2) % 2, plane r % 2; the others read zeros
        const bool mine = (r >> 2) == c, odd = (r & 2) != 0;
        const uint32_t *pos = stage + 64 * (r & 1) + 16 * c + (odd ? 8 : 0), *zero = stage + 128;
        const uint32_t *ev = mine && !odd ? pos : zero, *od = mine && odd ? pos : zero;
        const uint4 e0 = *(const uint4 *)ev, e1 = *(const uint4 *)(ev + 4), o0 = *(const uint4 *)od, o1 = *(const uint4 *)(od + 4);
        Acts a;
        a.a_even[0] = qv_i4{(int)e0.x, (int)e0.y, (int)e0.z, (int)e0.w};
        a.a_even[1] = qv_i4{(int)e1.x, (int)e1.y, (int)e1.z, (int)e1.w};
        a.a_odd[0] = qv_i4{(int)o0.x, (int)o0.y, (int)o0.z, (int)o0.w};
        a.a_odd[1] = qv_i4{(int)o1.x, (int)o1.y, (int)o1.z, (int)o1.w};
        a.s_e = scales[2 * c], a.s_o = scales[2 * c + 1], a.xs_e = scales[8 + 2 * c], a.xs_o = scales[9 + 2 * c];
        asm volatile("" ::: "memory");
        return a;
    }
    __device__ static __forceinline__ float block_dot_lane(const uint8_t *blk, const Acts &a, int c, const uint64_t *table) {
        int we[8], wo[8];
        float se, so, oe, oo;
        if (SUB == 1) {
            Q::decode_i8(table, blk, 2 * c, we, se, oe);
            Q::decode_i8(table, blk, 2 * c + 1, wo, so, oo);
        } else {
            Q::decode_i8(table, blk + (2 * c) * Q::BLOCK_BYTES, 0, we, se, oe);
            Q::decode_i8(table, blk + (2 * c + 1) * Q::BLOCK_BYTES, 0, wo, so, oo);
        }
        qv_i4 C = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a_even[0], qv_i4{we[0], we[1], we[2], we[3]}, qv_i4{0, 0, 0, 0}, 0, 0, 0);
        C = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a_even[1], qv_i4{we[4], we[5], we[6], we[7]}, C, 0, 0, 0);
        C = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a_odd[0], qv_i4{wo[0], wo[1], wo[2], wo[3]}, C, 0, 0, 0);
        C = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a_odd[1], qv_i4{wo[4], wo[5], wo[6], wo[7]}, C, 0, 0, 0);
        float sum = fmaf(se * a.s_e, (float)((C[1] << 8) + C[0]), so * a.s_o * (float)((C[3] << 8) + C[2]));
        if (Q::I8_HAS_MIN) sum -= fmaf(oe, a.xs_e, oo * a.xs_o);
        return sum;
    }
    __device__ static __forceinline__ float block_dot_lane(const uint8_t *blk, const Acts &a, int c) {
        return block_dot_lane(blk, a, c, nullptr);  // (the formats without a table)
    }
};

// Q3_K on the same activation operands: w = d (sc - 32) (code - 4) with a 6-bit scale per 16 elements, so the four
// MFMAs of a lane's chunk (16 elements each) keep accumulators of their own and each sum meets its scale in f32.
// The 3-bit codes (two bits of qs, the third from hmask) go through one byte permute to the signed values -4 .. 3.
// (layout: vendor/candle-metal-kernels/src/metal_src/quantized.metal:151-156, 6597-6623)
struct QvQ3K {
    typedef QvI8<Q5_K> Side;  // the activation side does not depend on the weights' format
    static constexpr int BLOCK = 110, ROW = 16 * BLOCK, ROW_LDS = moe_mfma_row_lds(ROW), STAGE_BYTES = Side::STAGE_BYTES;
    static constexpr bool SIDE_LDS = false;
    static constexpr int COLS = 4096, SLOTS = 3;
    typedef Side::Acts Acts;
    __device__ static __forceinline__ void scale(Acts &a, float f) { Side::scale(a, f); }
    __device__ static __forceinline__ Acts prepare(const float4 v, uint32_t *stage, int lane) { return Side::prepare(v, stage, lane); }
    __device__ static __forceinline__ float block_dot_lane(const uint8_t *blk, const Acts &a, int c) {
        // sub-blocks j = 2c (h = j / 4, field t = j % 4) and j + 1: the same half h and the field behind
        const int h = c >> 1, t = 2 * (c & 1);
        const uint4 qa = ldw<uint4>(blk + 32 + 32 * h), qb = ldw<uint4>(blk + 48 + 32 * h);   // elements i and 16 + i of a field
        const uint4 ha = ldw<uint4>(blk), hb = ldw<uint4>(blk + 16);
        const uint2 s8 = ldw<uint2>(blk + 96);
        const uint32_t s4 = ldw<uint32_t>(blk + 104);
        const float d = f16_bits(ld<uint16_t>(blk + 108));
        const uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        const uint32_t hm[8] = {ha.x, ha.y, ha.z, ha.w, hb.x, hb.y, hb.z, hb.w};
        const uint64_t lo8 = ((uint64_t)s8.y << 32) | s8.x;
        int w[2][8];
        float sc[2][2];
#pragma unroll
        for (int p = 0; p < 2; p++) {
            const int tt = t + p;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const uint32_t code = ((q[i] >> (2 * tt)) & 0x03030303u) | (((hm[i] >> (4 * h + tt)) & 0x01010101u) << 2);
                w[p][i] = (int)__builtin_amdgcn_perm(0x03020100u, 0xFFFEFDFCu, code);
            }
#pragma unroll
            for (int hf = 0; hf < 2; hf++) {
                const int is = 8 * h + 2 * tt + hf;
                const uint32_t low4 = (uint32_t)(lo8 >> (8 * (is & 7) + (is < 8 ? 0 : 4))) & 0xFu;
                const uint32_t high2 = (s4 >> (8 * (is & 3) + 2 * (is >> 2))) & 3u;
                sc[p][hf] = (float)((int)(low4 | (high2 << 4)) - 32);
            }
        }
        const qv_i4 z = qv_i4{0, 0, 0, 0};
        const qv_i4 C1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a_even[0], qv_i4{w[0][0], w[0][1], w[0][2], w[0][3]}, z, 0, 0, 0);
        const qv_i4 C2 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a_even[1], qv_i4{w[0][4], w[0][5], w[0][6], w[0][7]}, z, 0, 0, 0);
        const qv_i4 C3 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a_odd[0], qv_i4{w[1][0], w[1][1], w[1][2], w[1][3]}, z, 0, 0, 0);
        const qv_i4 C4 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a.a_odd[1], qv_i4{w[1][4], w[1][5], w[1][6], w[1][7]}, z, 0, 0, 0);
        const float even = fmaf(sc[0][0], (float)((C1[1] << 8) + C1[0]), sc[0][1] * (float)((C2[1] << 8) + C2[0]));
        const float odd = fmaf(sc[1][0], (float)((C3[3] << 8) + C3[2]), sc[1][1] * (float)((C4[3] << 8) + C4[2]));
        return d * fmaf(a.s_e, even, a.s_o * odd);
    }
};

// Policies whose block_dot_lane wants the format's lookup table (a copy in LDS) as a fourth argument.
template <class F, class = void>
struct QvTakesTable : std::false_type {};
template <class F>
struct QvTakesTable<F, std::void_t<decltype(F::TAKES_TABLE)>> : std::true_type {};
template <class F>
__host__ __device__ constexpr int qv_table_bytes() {
    if constexpr (QvTakesTable<F>::value) return (table_bytes<typename F::Format>() + 15) / 16 * 16;
    else return 0;
}
template <class F>
__device__ __forceinline__ const uint64_t *qv_stage_table(uint8_t *lds) {  // holds a barrier when there is a table
    if constexpr (QvTakesTable<F>::value) return stage_table<typename F::Format>(lds);
    else return nullptr;
}
template <class F>
__device__ __forceinline__ float qv_dot(const uint8_t *blk, const typename F::Acts &a, int c, const uint64_t *table) {
    if constexpr (QvTakesTable<F>::value) return F::block_dot_lane(blk, a, c, table);
    else return F::block_dot_lane(blk, a, c);
}

// a wave's staging area: what the policy's prepare() uses, and in front of that the wave's 256 raw activations
template <class F>
constexpr int moe_mfma_stage() { return ((F::STAGE_BYTES > 1024 ? F::STAGE_BYTES : 1024) + 15) / 16 * 16; }

// Where the experts of a stacked tensor start: expert e < n_routed at base + e stride, the folded shared expert
// (number n_routed) at `extra`.
struct MoeStack {
    const uint8_t *base;
    size_t stride;
    const uint8_t *extra;
    int n_routed;
};
__device__ __forceinline__ const uint8_t *moe_expert_base(const MoeStack &st, int e) {
    return e < st.n_routed ? st.base + (size_t)e * st.stride : st.extra;
}

// (where the raw activations have a place of their own)
template <class F>
constexpr int moe_mfma_stage_only() { return (F::STAGE_BYTES + 15) / 16 * 16; }

template <class F, int NB>
constexpr int moe_gate_up_mfma_lds() {
    return qv_table_bytes<F>() + 16 * moe_mfma_row_lds(NB * F::BLOCK) + NB * moe_mfma_stage<F>() + 16 * 68 * 4;
}

// One workgroup of NB waves per (pair, 8 rows of gate and the same 8 rows of up): gate and up multiply the same
// activations, so the 16 weight rows of a matrix-core tile are 8 of each, wave w takes super-block column w of all
// 16, and SwiGLU meets both halves where the rows are stored.  With rows of 8 super-blocks a tile is 18 KB and a
// call's tiles (96 a pair at 768 rows) spread evenly over the chip, four workgroups a compute unit, all asked
// for in the launch's first microsecond behind the waves' activations, which are quantised while they land.
// `zero`: zero_n floats the launch also clears, for the kernel behind it that adds into them.
// GATE: the launch runs the gating too.  Every workgroup's first wave picks the token's experts from the router's
// logits (moe_gate_topk_wave's arithmetic, the same bits) while the activations travel, and takes its pair's
// expert from there; the first workgroup of a token's first pair writes ids, weights and pair groups for the down
// projection.  A launch less than gating on its own, which costs 4 us of which 3 are the launch and its wait for
// the router.
struct MoeGateIn {
    const float *logits, *bias;
    MoeGateParams p;
    uint32_t *ids;
    float *wts;
    MoePairGroups pg;
    int T;
};

template <class F, int NB, bool GATE>
__global__ __launch_bounds__(64 * NB) void moe_gate_up_mfma(MoeStack Wa, MoeStack Wb, const float *__restrict__ X,
                                                            const int *__restrict__ gexp, const int *__restrict__ xrow,
                                                            const int *__restrict__ yrow, float *__restrict__ G, int inter,
                                                            MoeClamp cl, float *__restrict__ zero, int zero_n, MoeGateIn gi) {
    static_assert(NB == 1 || NB == 2 || NB == 4 || NB == 8, "a row of 1, 2, 4 or 8 super-blocks");
    constexpr int RB = NB * F::BLOCK, ROW_LDS = moe_mfma_row_lds(RB), LOADS = (RB + 1023) / 1024, STG = moe_mfma_stage<F>();
    constexpr int RPW = 16 / NB;  // tile rows a wave copies
    static_assert(RB % 16 == 0, "rows are copied 16 bytes a lane");
    extern __shared__ __attribute__((aligned(16))) uint8_t moe_mfma_lds[];
    __shared__ int picked;
    const uint64_t *table = qv_stage_table<F>(moe_mfma_lds);
    uint8_t *tile = moe_mfma_lds + qv_table_bytes<F>();                         // [16][ROW_LDS]: 8 gate rows, 8 up rows
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, c = lane >> 4;
    uint32_t *stage = (uint32_t *)(tile + 16 * ROW_LDS + wave * STG);
    float *part = (float *)(tile + 16 * ROW_LDS + NB * STG);                    // [16][68]
    const int p = blockIdx.y;
    int e, t, out_row;
    if (GATE) {  // pair p is slot p % k_used of token p / k_used, or behind the routed pairs the token's shared expert
        const int P = gi.T * gi.p.k_used;
        t = p < P ? p / gi.p.k_used : p - P;
        out_row = p;
    } else {
        e = gexp[p], t = xrow[p], out_row = yrow[p];
    }
    async_load16(X + (size_t)t * (256 * NB) + 256 * wave + 4 * lane, lds_offset_of(stage));
    typename F::Acts acts;
    // the activations are quantised while the tile lands; with the gating in the launch, by the waves that do not
    // run it while it runs (wave 0 follows behind its tile loads)
    auto prepare = [&]() __attribute__((always_inline)) {
        const float4 v = *(const float4 *)((const float *)stage + 4 * lane);
        acts = F::prepare(v, stage, lane);
    };
    if (GATE) {
        const int P = gi.T * gi.p.k_used;
        if (wave == 0) {
            int slot_e;
            moe_gate_topk_wave_body<4>(t, gi.T, lane, gi.logits, gi.bias, gi.p, gi.ids, gi.wts, gi.pg,
                                       blockIdx.x == 0 && p < P && p % gi.p.k_used == 0, &slot_e);
            const int mine = p < P ? __builtin_amdgcn_readlane(slot_e, p % gi.p.k_used) : gi.p.E;
            if (lane == 0) picked = mine;
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            prepare();
        }
        __syncthreads();
        e = __builtin_amdgcn_readfirstlane(picked);
    }
    const uint8_t *wa = moe_expert_base(Wa, e), *wb = moe_expert_base(Wb, e);
    const int j0 = blockIdx.x * 8;
    const uint32_t tile0 = lds_offset_of(tile);
#pragma unroll
    for (int i = 0; i < RPW; i++) {
        const int rr = wave + NB * i, j = min(j0 + (rr & 7), inter - 1);
        const uint8_t *src = (rr < 8 ? wa : wb) + (size_t)j * RB;
        const uint32_t dst = tile0 + (uint32_t)rr * ROW_LDS;
#pragma unroll
        for (int l = 0; l < LOADS; l++) {
            constexpr int full = 64;
            const int lanes = (RB - 1024 * l) / 16 < full ? (RB - 1024 * l) / 16 : full;
            if (lane < lanes) async_load16_s(src + 1024 * l, 16 * lane, dst + 1024 * l);
        }
    }
    if (!GATE || wave == 0) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(RPW * LOADS) : "memory");  // the activations are in
        prepare();
    }
    asm volatile("s_waitcnt vmcnt(0)\n\ts_waitcnt lgkmcnt(0)" ::: "memory");
    if (NB > 1) __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    part[r * 68 + 4 * wave + c] = qv_dot<F>(tile + r * ROW_LDS + wave * F::BLOCK, acts, c, table);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (NB > 1) __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    // wave w adds the 4 NB chunk sums of gate row w (w + NB, ..) and of the up row beside it
#pragma unroll
    for (int q = 0; q < 8 / NB; q++) {
        const int jj = wave + NB * q;
        float g = lane < 4 * NB ? part[jj * 68 + lane] : 0.0f;
        float u = lane < 4 * NB ? part[(jj + 8) * 68 + lane] : 0.0f;
        g = wave_sum(g), u = wave_sum(u);
        if (lane == 0 && j0 + jj < inter) G[(size_t)out_row * inter + j0 + jj] = swiglu(g, u, cl, e);
    }
    if (zero) {
        const int wg = blockIdx.y * gridDim.x + blockIdx.x, n_wg = gridDim.x * gridDim.y;
        for (int i = wg * (64 * NB) + tid; i < zero_n; i += n_wg * 64 * NB) zero[i] = 0.0f;
    }
}

// Gate and up for rows of more than 8 super-blocks (nb <= 16 NG).  A workgroup of 16 waves stays with one pair
// and walks tiles b, b + gridDim.x, .. of it, a tile again 8 rows of gate and the same 8 rows of up: wave w keeps the
// operands of columns w, w + 16, .. for the whole launch, the tiles travel through a ring of SLOTS slots as whole
// rows (8 consecutive rows of a matrix are one span of memory, copied 16 bytes a lane by all 1024 lanes: J
// instructions a span and wave), and a lane adds its chunk sums of its columns in a register.
// The raw activations (1 KB a column) wait in the ring's slots behind the first until they are prepared.
// ROWS: rows that are whole 16-byte pieces (at most 2 J KB long) travel row by row instead, wave w copying row w of
// the 16, and sit in LDS 16 bytes past a multiple of 256 apart, so that the 16 rows a lane group reads side by side
// fall on all banks (MXFP4 rows of 7168: 3808 bytes, where the rows of a span collide two by two).
template <class F, bool ROWS>
constexpr int moe_gate_up_rows_slot(int nb) {
    return ROWS ? 16 * moe_mfma_row_lds(nb * F::BLOCK) : (16 * nb * F::BLOCK + 15) / 16 * 16;
}
template <class F, int NG, int SLOTS, int J, bool ROWS = false>
constexpr int moe_gate_up_rows_mfma_lds(int nb) {
    return qv_table_bytes<F>() + SLOTS * moe_gate_up_rows_slot<F, ROWS>(nb) + 1024 + 16 * moe_mfma_stage_only<F>() + 16 * 68 * 4;
}

template <class F, int NG, int SLOTS, int J, bool GATE, bool ROWS = false>
__global__ __launch_bounds__(1024) void moe_gate_up_rows_mfma(MoeStack Wa, MoeStack Wb, const float *__restrict__ X,
                                                              const int *__restrict__ gexp, const int *__restrict__ xrow,
                                                              const int *__restrict__ yrow, float *__restrict__ G, int inter,
                                                              int nb, MoeClamp cl, MoeGateIn gi) {
    static_assert(NG >= 1 && NG <= 2 && (SLOTS == 2 || SLOTS == 3) && (J == 1 || J == 2), "two columns a wave at most");
    constexpr int STG = moe_mfma_stage_only<F>(), LPF = 2 * J;  // loads a wave and tile: J a span
    extern __shared__ __attribute__((aligned(16))) uint8_t moe_mfma_lds[];
    __shared__ int picked;
    const uint64_t *table = qv_stage_table<F>(moe_mfma_lds);
    const int RB = nb * F::BLOCK, span = 8 * RB;  // 8 RB is a multiple of 16
    const int RS = ROWS ? moe_mfma_row_lds(RB) : RB, slot_bytes = moe_gate_up_rows_slot<F, ROWS>(nb);
    uint8_t *ring = moe_mfma_lds + qv_table_bytes<F>();
    uint8_t *dump = ring + SLOTS * slot_bytes;                       // where a wave without a piece of a span points its load
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, c = lane >> 4;
    uint32_t *stage = (uint32_t *)(dump + 1024 + wave * STG);
    float *part = (float *)(dump + 1024 + 16 * STG);                 // [16][68]
    float *xraw = (float *)(ring + slot_bytes);                      // [nb][256], in the slots behind the first
    const int p = blockIdx.y;
    int e, t, out_row;
    if (GATE) {
        const int P = gi.T * gi.p.k_used;
        t = p < P ? p / gi.p.k_used : p - P;
        out_row = p;
    } else {
        e = gexp[p], t = xrow[p], out_row = yrow[p];
    }
    const int ntiles = inter / 8, b = blockIdx.x, G_ = gridDim.x;
    const int nt = (ntiles - b + G_ - 1) / G_;
    if (nt <= 0) return;  // (whole workgroups: the barriers below see either all waves or none)
#pragma unroll
    for (int cg = 0; cg < NG; cg++)
        async_load16(X + (size_t)t * (256 * nb) + 256 * min(16 * cg + wave, nb - 1) + 4 * lane,
                     lds_offset_of(xraw + min(16 * cg + wave, nb - 1) * 256));
    if (GATE) {
        const int P = gi.T * gi.p.k_used;
        if (wave == 0) {
            int slot_e;
            moe_gate_topk_wave_body<4>(t, gi.T, lane, gi.logits, gi.bias, gi.p, gi.ids, gi.wts, gi.pg,
                                       b == 0 && p < P && p % gi.p.k_used == 0, &slot_e);
            const int mine = p < P ? __builtin_amdgcn_readlane(slot_e, p % gi.p.k_used) : gi.p.E;
            if (lane == 0) picked = mine;
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    typename F::Acts acts[NG];
#pragma unroll
    for (int cg = 0; cg < NG; cg++) {
        const float4 v = *(const float4 *)(xraw + min(16 * cg + wave, nb - 1) * 256 + 4 * lane);
        acts[cg] = F::prepare(v, stage, lane);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __syncthreads();  // the raw activations are read: the slots they waited in are free; the gating's pick is written
    if (GATE) e = __builtin_amdgcn_readfirstlane(picked);
    const uint8_t *wa = moe_expert_base(Wa, e), *wb = moe_expert_base(Wb, e);
    const uint32_t ring0 = lds_offset_of(ring), dump0 = lds_offset_of(dump);
    const int pieces = (ROWS ? RB : span) / 16;
    auto fetch = [&](int i) __attribute__((always_inline)) {
        const size_t row0 = (size_t)8 * (b + (size_t)min(i, nt - 1) * G_);
        const uint32_t slot0 = ring0 + (uint32_t)(i % SLOTS) * slot_bytes;
        if (ROWS) {
            const uint8_t *src = (wave >= 8 ? wb : wa) + (row0 + (size_t)(wave & 7)) * RB;
#pragma unroll
            for (int j = 0; j < 2 * J; j++) {
                const int first = 64 * j, left = pieces - first;  // this instruction's pieces of the wave's row
                if (left > 0) {
                    if (lane < left) async_load16_s(src + 16 * (size_t)first, 16 * lane, slot0 + wave * RS + 16 * first);
                } else if (lane == 0) {
                    async_load16_s(src, 0, dump0 + 16 * wave);  // so that every wave counts the same loads
                }
            }
            return;
        }
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const uint8_t *src = (half ? wb : wa) + row0 * RB;
#pragma unroll
            for (int j = 0; j < J; j++) {
                const int first = 64 * (wave + 16 * j), left = pieces - first;  // this wave's pieces of the span
                if (left > 0) {
                    if (lane < left) async_load16_s(src + 16 * (size_t)first, 16 * lane, slot0 + half * span + 16 * first);
                } else if (lane == 0) {
                    async_load16_s(src, 0, dump0 + 16 * wave);  // so that every wave counts the same loads
                }
            }
        }
    };
    fetch(0);
    if (nt > 1) fetch(1);
    if (SLOTS == 3 && nt > 2) fetch(2);
    for (int i = 0; i < nt; i++) {
        // tile i is in when only the tiles asked for behind it are out
        const int behind = min(SLOTS - 1, nt - 1 - i);
        if (behind >= 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * LPF) : "memory");
        else if (behind == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LPF) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const uint8_t *slot = ring + (i % SLOTS) * slot_bytes;
        float acc = 0.0f;
#pragma unroll
        for (int cg = 0; cg < NG; cg++)
            if (16 * cg + wave < nb) acc += qv_dot<F>(slot + r * RS + (16 * cg + wave) * F::BLOCK, acts[cg], c, table);
        part[r * 68 + 4 * wave + c] = acc;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        // every wave is done with tile i: its slot takes tile i + SLOTS
        if (i + SLOTS < nt) fetch(i + SLOTS);
        if (wave < 8) {
            float g = wave_sum(part[wave * 68 + lane]), u = wave_sum(part[(wave + 8) * 68 + lane]);
            const int j = 8 * (b + i * G_) + wave;
            if (lane == 0) G[(size_t)out_row * inter + j] = swiglu(g, u, cl, e);
        }
    }
}

// A pointer every lane of the wave holds, moved to scalar registers.
__device__ __forceinline__ const uint8_t *uniform_ptr(const uint8_t *p) {
    const uint64_t v = (uint64_t)p;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return (const uint8_t *)(((uint64_t)hi << 32) | lo);
}

// bytes of a ring slot: 16 rows of SPP segments, padded row by row, or (SPAN) the segments' 16 rows as they lie in memory
template <class F, int NB, int SPP, bool SPAN>
constexpr int moe_down_mfma_slot() {
    return SPAN ? SPP * 16 * NB * F::BLOCK : 16 * moe_mfma_row_lds(SPP * NB * F::BLOCK);
}
template <class F, int NB, int SPP, int SLOTS, int XB, bool SPAN = false>
constexpr int moe_down_mfma_lds() {
    return qv_table_bytes<F>() + SLOTS * moe_down_mfma_slot<F, NB, SPP, SPAN>() + XB * 16 * 1024 + 16 * moe_mfma_stage_only<F>() +
           16 * 68 * 4 + (SPAN ? 256 : 0);
}

// One workgroup per (token, 16 rows of the result).  The token's S = k_used + n_extra pairs are the segments of
// one long row, [down_e(0)[r] | down_e(1)[r] | ..] against [w_0 a_0 | w_1 a_1 | ..] with a_s the pair's activation
// row of NB super-blocks: the combine weights ride on the activations and the sum over the pairs is the sum over
// the row.  A pass is SPP segments (NB SPP <= 16 waves at work: wave w takes block w % NB of segment w / NB),
// its 16 rows x SPP segments travel through a ring of SLOTS slots (three: two passes in flight; two where three
// do not fit) with the waves' activations beside them, and a lane adds its chunk sums of all passes in a register.
// XB: buffers of the waves' raw activations (two with three slots; one is enough with two, where the next pass is
// asked for once this one's activations are in registers).
// SPAN: rows that are not a multiple of 16 bytes (Q6_K: 210-byte blocks).  The 16 rows of a segment's tile are one
// span of memory that starts and ends on 16 bytes whatever the row length; all 1024 lanes copy it 16 bytes each and it
// sits in LDS as in memory (n must be a multiple of 16).
template <class F, int NB, int SPP, int SLOTS, int XB, bool SPAN = false>
__global__ __launch_bounds__(1024) void moe_down_mfma(MoeStack Wd, const float *__restrict__ A,
                                                      const int *__restrict__ gexp, const float *__restrict__ wts,
                                                      float *__restrict__ Y, int n, int k_used, int n_extra, int P) {
    static_assert(NB * SPP <= 16, "a pass is at most 16 super-block columns");
    static_assert(SLOTS == 2 || SLOTS == 3, "one or two passes ahead of the arithmetic");
    static_assert(XB == 2 || (XB == 1 && SLOTS == 2), "two passes in flight keep two activation buffers");
    constexpr int RB = NB * F::BLOCK, ROW_LDS = moe_mfma_row_lds(SPP * RB), STG = moe_mfma_stage_only<F>();
    // load instructions a wave and segment: its row's kilobytes, or its share of the 16 RB / 16 pieces of a span
    constexpr int LOADS = SPAN ? (RB + 1023) / 1024 : (RB + 1023) / 1024;
    constexpr int LPF = SPP * LOADS + 1;  // loads a wave and pass: the segments and the wave's activations
    constexpr int SLOT = moe_down_mfma_slot<F, NB, SPP, SPAN>();
    static_assert(SPAN || RB % 16 == 0, "rows are copied 16 bytes a lane");
    constexpr int MAX_S = 64;
    extern __shared__ __attribute__((aligned(16))) uint8_t moe_mfma_lds[];
    __shared__ const uint8_t *seg_base[MAX_S];
    __shared__ float seg_wt[MAX_S];
    __shared__ int seg_pair[MAX_S];
    const uint64_t *table = qv_stage_table<F>(moe_mfma_lds);
    uint8_t *ring = moe_mfma_lds + qv_table_bytes<F>();            // [SLOTS][SLOT]
    float *xbuf = (float *)(ring + SLOTS * SLOT);                  // [XB][16][256]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, c = lane >> 4;
    uint32_t *stage = (uint32_t *)(ring + SLOTS * SLOT + XB * 16 * 1024 + wave * STG);
    float *part = (float *)(ring + SLOTS * SLOT + XB * 16 * 1024 + 16 * STG);  // [16][68]
    const uint32_t dump0 = lds_offset_of(part + 16 * 68);          // (SPAN) where a wave without a piece of a span points its load
    // gridDim.z workgroups share a (token, row tile): number z takes passes z, z + gridDim.z, ..
    const int t = blockIdx.y, S = k_used + n_extra, Z = gridDim.z, z = blockIdx.z;
    const int NP = ((S + SPP - 1) / SPP - z + Z - 1) / Z;
    if (tid < S) {
        const int pair = tid < k_used ? t * k_used + tid : P + t;
        seg_base[tid] = moe_expert_base(Wd, gexp[pair]);
        seg_wt[tid] = tid < k_used ? wts[pair] : 1.0f;
        seg_pair[tid] = pair;
    }
    __syncthreads();
    const int row = min(16 * (int)blockIdx.x + wave, n - 1);
    const int q = wave / NB, blk = wave % NB;       // this wave's segment of a pass and block of the segment
    const bool worker = q < SPP;
    const uint32_t ring0 = lds_offset_of(ring), xbuf0 = lds_offset_of(xbuf);
    const int inter = 256 * NB;
    auto fetch = [&](int i) __attribute__((always_inline)) {
        const uint32_t slot0 = ring0 + (uint32_t)(i % SLOTS) * SLOT;
        const int first = (z + Z * i) * SPP;  // the pass's first segment
#pragma unroll
        for (int qq = 0; qq < SPP; qq++) {
            const int s = min(first + qq, S - 1);
            if (SPAN) {
                const uint8_t *src = uniform_ptr(seg_base[s]) + (size_t)(16 * (int)blockIdx.x) * RB;
#pragma unroll
                for (int j = 0; j < LOADS; j++) {
                    const int p0 = 64 * (wave + 16 * j), left = RB - p0;  // a span is RB pieces of 16 bytes
                    if (left > 0) {
                        if (lane < left) async_load16_s(src + 16 * (size_t)p0, 16 * lane, slot0 + qq * (16 * RB) + 16 * p0);
                    } else if (lane == 0) {
                        async_load16_s(src, 0, dump0 + 16 * wave);  // so that every wave counts the same loads
                    }
                }
            } else {
                const uint8_t *src = uniform_ptr(seg_base[s]) + (size_t)row * RB;
                const uint32_t dst = slot0 + (uint32_t)wave * ROW_LDS;
#pragma unroll
                for (int j = 0; j < LOADS; j++) {
                    constexpr int full = 64;
                    const int lanes = (RB - 1024 * j) / 16 < full ? (RB - 1024 * j) / 16 : full;
                    if (lane < lanes) async_load16_s(src + 1024 * j, 16 * lane, dst + qq * RB + 1024 * j);
                }
            }
        }
        const int s = min(first + min(q, SPP - 1), S - 1);
        async_load16(A + (size_t)seg_pair[s] * inter + 256 * blk + 4 * lane, xbuf0 + (uint32_t)(((i % XB) * 16 + wave) * 1024));
    };
    fetch(0);
    if (SLOTS == 3 && NP > 1) fetch(1);
    float acc = 0.0f;
    for (int i = 0; i < NP; i++) {
        if (SLOTS == 3 && i + 1 < NP) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LPF) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        const int s = (z + Z * i) * SPP + q;
        const bool live = worker && s < S;
        float4 v = *(const float4 *)(xbuf + ((i % XB) * 16 + wave) * 256 + 4 * lane);
        const float w = seg_wt[min(s, S - 1)];
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        // every wave has passed this pass's barrier, so all are done with pass i - 1, whose slot the next pass to
        // ask for takes; this wave's activations of pass i are in registers and make room as well
        if (i + SLOTS - 1 < NP) fetch(i + SLOTS - 1);
        v = float4{v.x * w, v.y * w, v.z * w, v.w * w};
        const typename F::Acts acts = F::prepare(v, stage, lane);
        if (live) {
            const uint8_t *at = SPAN ? ring + (i % SLOTS) * SLOT + q * (16 * RB) + r * RB + blk * F::BLOCK
                                     : ring + (i % SLOTS) * SLOT + r * ROW_LDS + q * RB + blk * F::BLOCK;
            acc += qv_dot<F>(at, acts, c, table);
        }
    }
    part[r * 68 + 4 * wave + c] = acc;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    const float sum = wave_sum(part[wave * 68 + lane]);
    const int out_row = 16 * (int)blockIdx.x + wave;
    if (lane == 0 && out_row < n) {
        // two workgroups a row tile add into a result the launch before cleared: 0 + a + b in either order
        if (Z > 1) atomicAdd(Y + (size_t)t * n + out_row, sum);
        else Y[(size_t)t * n + out_row] = sum;
    }
}

}  // namespace jq
